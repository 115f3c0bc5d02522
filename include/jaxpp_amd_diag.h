/* jaxpp_amd_diag -- measurement aids, built into libjaxpp_amd_diag.so (not into the product
 * library libjaxpp_amd.so, on which it depends for error reporting: load that one first). */
#ifndef JAXPP_AMD_DIAG_H_
#define JAXPP_AMD_DIAG_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference: a measurement aid.  TFLOP/s this device sustains on
 * a register-only loop of bf16 MFMAs on every SIMD (shape 32: 32x32x16, 16: 16x16x32;
 * operands all zero, or random and different from one MFMA to the next as in a GEMM).
 * The clock under load depends on how many operand bits toggle, so the second figure is
 * the ceiling a real GEMM can approach.  Blocks the host (null stream; two runs of about 0.3 us per iteration, the second timed). */
int jpp_mfma_rate(int shape, int random_operands, int64_t iters, double* tflops);

/* No counterpart in the reference: a measurement aid.  Shader clocks per wave-level LDS read
 * when the 8 waves of one workgroup read in a loop, every wave with the per-lane byte offsets
 * lane_offsets[64] (host memory; into 64 KiB of LDS that the probe owns): ds_read_b128 (16
 * bytes per lane; 4.0 when free of bank conflicts: 256 bytes a cycle), or with transposing != 0
 * ds_read_b64_tr_b16 (8 bytes per lane; 2.1 to 2.3 at best).  With it the address patterns of the
 * kernels' fragment reads can be priced one by one.  Blocks the host (null stream). */
int jpp_lds_read_rate(const uint32_t* lane_offsets, int transposing, double* cycles_per_read);

#ifdef __cplusplus
}
#endif

#endif  /* JAXPP_AMD_DIAG_H_ */
