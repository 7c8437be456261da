/*
 * The two normalisation operators of the lmdeploy operator set that the gfx950 library implements.
 *
 * reference: proto/include/diopi/functions_lmdeploy.h:31-49.  The reference tree declares these operators and holds
 * neither an implementation nor a test of them; the library follows the header's statement and the published kernels
 * the interface was written for (see diopi_amd/csrc/rmsnorm_inplace.hip for the exact arithmetic).  The other
 * declarations of that header (fused attention blocks, sampling, batch bookkeeping) are not implemented: a caller
 * that tests the weak symbols' addresses gets diopiNoImplement from its adaptor, as for any absent operator.
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_
#define DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_

#include <diopi/diopirt.h>

#if defined(__cplusplus)
extern "C" {
#endif

/*
 * In-place RMS normalisation of every row (reference: functions_lmdeploy.h:31-38).
 *   inoutput [tokens, hidden] float32 / float16 (bfloat16 accepted as an extension), dense, on the device
 *   scale    [hidden], same dtype
 *   inoutput[r, :] <- inoutput[r, :] * rsqrt(mean(inoutput[r, :]^2) + eps) * scale
 * Sums in fp32.  HBM-bound: one read and one write of the matrix.
 */
DIOPI_API diopiError_t diopiRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t scale, float eps);

/*
 * Residual and bias addition fused with the RMS normalisation that follows it (reference: functions_lmdeploy.h:40-49):
 *   residual <- residual + inoutput + bias          (the sum is formed in fp32 and rounded once)
 *   inoutput <- RMSNorm(residual) * scale
 *   residual [tokens, hidden], same dtype as inoutput, a different tensor; bias [hidden] or a null handle
 * HBM-bound: one read and one write of each of the two matrices, instead of the three reads and two writes that an
 * addition followed by diopiRMSNorm costs.
 */
DIOPI_API diopiError_t diopiFusedAddRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiTensorHandle_t residual,
                                                          diopiConstTensorHandle_t bias, diopiConstTensorHandle_t scale, float eps);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_ */
