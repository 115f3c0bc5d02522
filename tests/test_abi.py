"""The C-ABI library: it is built, loads without a GPU, and exports every
symbol include/jaxpp_amd.h declares (no compute calls here)."""
import ctypes
import os
import re

from jaxpp_amd import runtime as rt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "jaxpp_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jpp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(rt.lib_path()):
        from jaxpp_amd.build import build
        build(verbose=False)
    lib = ctypes.CDLL(rt.lib_path())
    names = declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert sorted(rt.EXPORTS) == names, "runtime.EXPORTS and the header disagree"


def test_diagnostics_live_in_a_library_of_their_own():
    """The measurement aids (no counterpart in the reference) are declared in
    include/jaxpp_amd_diag.h and exported by libjaxpp_amd_diag.so, not by the product library;
    their argument checks run on the host."""
    diag_header = os.path.join(ROOT, "include", "jaxpp_amd_diag.h")
    names = sorted(set(re.findall(r"\b(jpp_[a-z0-9_]+)\s*\(", open(diag_header).read())))
    assert names == ["jpp_lds_read_rate", "jpp_mfma_rate"]
    product = ctypes.CDLL(rt.lib_path())
    for name in names:
        assert name not in declared_symbols()
        assert not hasattr(product, name)
        assert hasattr(rt.load_diag(), name)
    diag = rt.load_diag()
    out = ctypes.c_double(0.0)
    assert diag.jpp_mfma_rate(7, 0, 1, ctypes.byref(out)) == -1
    offsets = (ctypes.c_uint32 * 64)(*([0] * 63 + [65536]))        # lane 63 beyond the probe's LDS
    assert diag.jpp_lds_read_rate(offsets, 0, ctypes.byref(out)) == -1
    assert b"lane 63" in rt.load().jpp_last_error()
    offsets[63] = 8                                                # not a multiple of 16
    assert diag.jpp_lds_read_rate(offsets, 0, ctypes.byref(out)) == -1
    assert diag.jpp_lds_read_rate(None, 0, ctypes.byref(out)) == -1


def test_error_convention_without_gpu():
    lib = rt.load()
    assert lib.jpp_version() == 100
    # argument checks happen on the host, before anything touches a device
    assert lib.jpp_gemm_bf16(None, None) == -1
    assert b"null operand" in lib.jpp_last_error()
    assert lib.jpp_stage_create(None, None) == -1
    assert lib.jpp_norm_fwd(None, None) == -1
    assert lib.jpp_grad_accum_f32(None, None, None, 0, 0) == -1
    assert lib.jpp_adam_step(None, None) == -1
    assert lib.jpp_stage_adam_step(None, None, 1, 0.0, 0.0, 0.0, 0.0, 0.0) == -1


def test_workspace_sizes():
    """jpp_workspace_bytes: what the tests allocate by hand for each operator's scratch."""
    lib = rt.load()
    assert lib.jpp_workspace_bytes(0, 8192, 0, 0) == 2 * rt.NORM_PARTIALS * 8192 * 4     # norm backward
    assert lib.jpp_workspace_bytes(1, 1024 + 4096, 0, 0) == rt.NORM_PARTIALS * 5120 * 4  # column sums
    assert lib.jpp_workspace_bytes(2, 2, 32, 4096) == 2 * 2 * 32 * 4096 * 4                  # attention delta
    assert lib.jpp_workspace_bytes(3, 0, 0, 0) == rt.NORM_PARTIALS * 4
    assert lib.jpp_workspace_bytes(4, 8192, 8, 0) == 2 * 32 * 8 * 4
    assert lib.jpp_workspace_bytes(5, 4096, 8, 0) == 64 * 4096 * 8 * 4
    assert lib.jpp_workspace_bytes(6, 4, 1024, 1024) == 4 * 1024 * 1024 * 4
    assert lib.jpp_workspace_bytes(99, 1, 1, 1) == 0 and lib.jpp_workspace_bytes(0, -1, 0, 0) == 0


def test_struct_layouts_match_header_sizes():
    # 7 pointers + 9 int64 + 5 int (+ padding) ; guards against field drift
    assert ctypes.sizeof(rt.GemmArgs) == (7 * 8 + 9 * 8 + 5 * 4 + 4 + 8 + 2 * 4 + 3 * 8 + 8 + 6 * 8 + 8 +
                                          6 * 8 + 3 * 8 + 2 * 4)
    assert ctypes.sizeof(rt.AttnArgs) == 10 * 8 + 8 * 8 + 6 * 4 + 2 * 8
    assert ctypes.sizeof(rt.NormArgs) == 12 * 8 + 2 * 8 + 8
    assert ctypes.sizeof(rt.StageDesc) == 22 * 4
    assert ctypes.sizeof(rt.MoeArgs) == 9 * 8 + 2 * 8 + 3 * 4 + 4      # 3 ints, padded to 8
    assert ctypes.sizeof(rt.AdamArgs) == 8 + 5 * 8 + 8 + 5 * 8 + 8


def test_struct_fields_match_the_header_as_a_c_compiler_sees_it(tmp_path):
    """Every ctypes mirror against the header itself: a C program prints sizeof and the offset of
    every field (a field missing from the header fails to compile, a reordered or retyped one
    changes an offset)."""
    import shutil
    import subprocess
    import pytest
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    pairs = {"jpp_gemm_args": rt.GemmArgs, "jpp_attn_args": rt.AttnArgs, "jpp_norm_args": rt.NormArgs,
             "jpp_moe_args": rt.MoeArgs, "jpp_stage_desc": rt.StageDesc, "jpp_adam_args": rt.AdamArgs,
             "jpp_colsum_item": rt.ColsumItem}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "jaxpp_amd.h"', 'int main(void) {']
    for cname, cls in pairs.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'  printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run([cc, "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True, capture_output=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True,
                                                 text=True).stdout.splitlines())
    for cname, cls in pairs.items():
        assert int(got[cname]) == ctypes.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert int(got[f"{cname}.{fname}"]) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_enum_values_match_the_header(tmp_path):
    import shutil
    import subprocess
    import pytest
    from jaxpp_amd.types import TaskType
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    want = {"JPP_EPI_BF16": rt.EPI_BF16, "JPP_EPI_GELU": rt.EPI_GELU, "JPP_EPI_DGELU": rt.EPI_DGELU,
            "JPP_EPI_ACC_F32": rt.EPI_ACC_F32, "JPP_EPI_F32": rt.EPI_F32, "JPP_EPI_SWIGLU": rt.EPI_SWIGLU,
            "JPP_EPI_DSWIGLU": rt.EPI_DSWIGLU, "JPP_FAMILY_BERT": rt.FAMILY["bert"],
            "JPP_FAMILY_LLAMA": rt.FAMILY["llama"], "JPP_FAMILY_MIXTRAL": rt.FAMILY["mixtral"],
            "JPP_FAMILY_DECODER": rt.FAMILY["decoder"], "JPP_DTYPE_BF16": rt.DTYPE["bf16"],
            "JPP_DTYPE_F32": rt.DTYPE["f32"], "JPP_FWD": TaskType.FWD.value, "JPP_BWD": TaskType.BWD.value,
            "JPP_BWD_I": TaskType.BWD_I.value, "JPP_BWD_W": TaskType.BWD_W.value,
            "JPP_NORM_PARTIALS": rt.NORM_PARTIALS, "JPP_GROUP_M": 1, "JPP_GROUP_K": 2}
    body = "\n".join(f'  printf("{k} %d\\n", (int){k});' for k in want)
    src = tmp_path / "enums.c"
    src.write_text('#include <stdio.h>\n#include "jaxpp_amd.h"\nint main(void) {\n' + body + "\n  return 0;\n}\n")
    exe = tmp_path / "enums"
    subprocess.run([cc, "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True, capture_output=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True,
                                                 text=True).stdout.splitlines())
    assert {k: int(v) for k, v in got.items()} == want
