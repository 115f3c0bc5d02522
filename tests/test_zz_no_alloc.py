"""jpp_norm_bwd_static - the norm backward that allocates nothing and keeps its partial sums in
the library's own static device buffer - against jpp_norm_bwd with a caller-provided
workspace: same kernels, so dx and the accumulated scale / shift gradients must be
bit-identical.  Two calls in a row share the buffer, the second on a smaller input (fewer
rows and columns than the first left behind); a call beyond the buffer's width is refused.
What the entry point is for - callers that cannot allocate - is checked directly: after a first
call it runs under stream capture and replays bit for bit, and the device's free memory is the
same after the calls as before."""
import ctypes as C

import numpy as np
import pytest

from jaxpp_amd import runtime as rt
from oracle import layers as L

pytestmark = pytest.mark.gpu


def _case(rng, ln, rows, cols):
    r = lambda *s, scale=1.0: L.bf16_round((rng.standard_normal(s) * scale).astype(np.float32))
    x, dy, resid = r(rows, cols, scale=2.0), r(rows, cols), r(rows, cols)
    g = L.bf16_round(1 + 0.1 * rng.standard_normal(cols).astype(np.float32))
    b = L.bf16_round(0.1 * rng.standard_normal(cols).astype(np.float32))
    acc_g = rng.standard_normal(cols).astype(np.float32)
    acc_b = rng.standard_normal(cols).astype(np.float32)
    return dict(ln=ln, rows=rows, cols=cols, x=x, dy=dy, resid=resid, g=g, b=b, acc_g=acc_g,
                acc_b=acc_b)


def _run(case, static):
    """Forward (for the row statistics) then the backward through the chosen entry point."""
    lib = rt.load()
    ln, rows, cols = case["ln"], case["rows"], case["cols"]
    up = rt.DeviceBuffer.from_f32_as_bf16
    bx, bg, bb, bdy, br = up(case["x"]), up(case["g"]), up(case["b"]), up(case["dy"]), up(case["resid"])
    by, bdx = rt.DeviceBuffer(rows * cols * 2), rt.DeviceBuffer(rows * cols * 2)
    bmean, brstd = rt.DeviceBuffer(rows * 4), rt.DeviceBuffer(rows * 4)
    bdg, bdb = rt.DeviceBuffer.from_numpy(case["acc_g"]), rt.DeviceBuffer.from_numpy(case["acc_b"])
    part = None if static else rt.DeviceBuffer(2 * rt.NORM_PARTIALS * cols * 4)
    a = rt.NormArgs(bx.ptr, bg.ptr, bb.ptr if ln else None, by.ptr, bmean.ptr if ln else None,
                    brstd.ptr, bdy.ptr, br.ptr, bdx.ptr, bdg.ptr, bdb.ptr if ln else None,
                    None if static else part.ptr, rows, cols, 1e-5)
    rt.check(lib.jpp_norm_fwd(None, C.byref(a)))
    rt.check((lib.jpp_norm_bwd_static if static else lib.jpp_norm_bwd)(None, C.byref(a)))
    rt.sync()
    return (bdx.download(np.uint16, (rows, cols)), bdg.download(np.float32, (cols,)),
            bdb.download(np.float32, (cols,)) if ln else None)


def test_static_scratch_entry_point_matches_the_workspace_one():
    rt.require_gpu()
    rng = np.random.default_rng(11)
    # a LayerNorm over the widest rows the buffer holds, then a smaller RMSNorm and a smaller
    # LayerNorm: stale partial sums of the first call lie beside and behind what they write
    cases = [_case(rng, True, 1030, 8192), _case(rng, False, 140, 4096), _case(rng, True, 70, 256)]
    want = [_run(c, static=False) for c in cases]
    got = [_run(c, static=True) for c in cases]           # back to back on the shared buffer
    for c, g, w in zip(cases, got, want):
        what = f"ln={c['ln']} {c['rows']}x{c['cols']}"
        np.testing.assert_array_equal(g[0], w[0], err_msg=f"dx, {what}")
        np.testing.assert_array_equal(g[1], w[1], err_msg=f"dgamma, {what}")
        if c["ln"]:
            np.testing.assert_array_equal(g[2], w[2], err_msg=f"dbeta, {what}")
    # and the results are right, not merely equal: against the oracle
    c = cases[1]
    _, rstd = L.rmsnorm_fwd(c["x"], c["g"], 1e-5)
    dx_w, dg_w = L.rmsnorm_bwd(c["dy"], c["x"], rstd, c["g"])
    dx = rt.from_bf16_bits(got[1][0])
    assert np.abs(dx - (dx_w + c["resid"])).max() <= 1e-2 * np.abs(dx_w + c["resid"]).max()
    assert np.abs(got[1][1] - (c["acc_g"] + dg_w)).max() <= 1e-3 * np.abs(c["acc_g"] + dg_w).max()


def test_static_scratch_entry_point_rejects_rows_wider_than_its_buffer():
    rt.require_gpu()
    lib = rt.load()
    d = rt.DeviceBuffer(1 << 16)
    a = rt.NormArgs(d.ptr, d.ptr, None, d.ptr, None, d.ptr, d.ptr, None, d.ptr, d.ptr, None, None,
                    1, 8192 + 8, 1e-5)
    assert lib.jpp_norm_bwd_static(None, C.byref(a)) == -1
    assert b"exceed" in lib.jpp_last_error()


def test_static_scratch_entry_point_allocates_nothing_and_runs_under_capture():
    rt.require_gpu()
    lib = rt.load()
    rng = np.random.default_rng(12)
    c = _case(rng, False, 200, 2048)
    want = _run(c, static=False)
    rows, cols = c["rows"], c["cols"]
    up = rt.DeviceBuffer.from_f32_as_bf16
    bx, bg, bdy, br = up(c["x"]), up(c["g"]), up(c["dy"]), up(c["resid"])
    by, bdx = rt.DeviceBuffer(rows * cols * 2), rt.DeviceBuffer(rows * cols * 2)
    brstd = rt.DeviceBuffer(rows * 4)
    bdg = rt.DeviceBuffer.from_numpy(c["acc_g"])
    a = rt.NormArgs(bx.ptr, bg.ptr, None, by.ptr, None, brstd.ptr, bdy.ptr, br.ptr, bdx.ptr,
                    bdg.ptr, None, None, rows, cols, 1e-5)
    rt.check(lib.jpp_norm_fwd(None, C.byref(a)))
    rt.check(lib.jpp_norm_bwd_static(None, C.byref(a)))      # first call on this device: the
    rt.sync()                                                # address lookup happens here
    stream = rt.Stream()
    graph = rt.Graph(stream)
    with graph:                                              # an allocation or a symbol lookup
        rt.check(lib.jpp_norm_bwd_static(stream.ptr, C.byref(a)))   # here would fail the capture
    graph.launch()                                           # (the runtime's own set-up of a
    stream.sync()                                            # first replay is not counted)
    free0, total = C.c_size_t(), C.c_size_t()
    rt.check(lib.jpp_mem_info(C.byref(free0), C.byref(total)))
    for replay in range(3):
        bdg.upload(c["acc_g"])
        bdx.zero()
        rt.sync()
        graph.launch()
        stream.sync()
        np.testing.assert_array_equal(bdx.download(np.uint16, (rows, cols)), want[0],
                                      err_msg=f"dx, replay {replay}")
        np.testing.assert_array_equal(bdg.download(np.float32, (cols,)), want[1],
                                      err_msg=f"dgamma, replay {replay}")
        rt.check(lib.jpp_norm_bwd_static(None, C.byref(a)))  # eager work between the replays
        rt.sync()
    free1 = C.c_size_t()
    rt.check(lib.jpp_mem_info(C.byref(free1), C.byref(total)))
    assert free1.value == free0.value, "the static entry point (or its replays) allocated device memory"
