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

#ifdef __cplusplus
}
#endif

#endif  /* JAXPP_AMD_DIAG_H_ */
