// Declaration-compatibility probe for the C ABI.  Compiled twice by tests/test_abi.py (syntax only):
// against the reference's headers (-I <reference>/proto/include) and against this repository's.
// Each operator is re-declared below with the signature the gfx950 library defines; with C linkage a
// mismatch with the header's prototype is a compile error ("conflicting declaration").
#ifdef USE_OWN_HEADERS
#include <diopi/diopirt.h>
#include <diopi/functions.h>
#include <diopi/functions_ext.h>
#include <diopi/functions_lmdeploy.h>
#else
#include <diopi/diopirt.h>
#include <diopi/functions.h>
#include <diopi/functions_ext.h>
#include <diopi/functions_lmdeploy.h>
#endif

extern "C" {
diopiError_t diopiRootMeanSquareNormInp(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, float);
diopiError_t diopiFusedAddRootMeanSquareNormInp(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t,
                                                diopiConstTensorHandle_t, float);
const char* diopiGetVendorName();
const char* diopiGetImplVersion();
const char* diopiGetLastErrorString();
diopiError_t diopiRotaryEmbedding(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                  const bool, const bool);
diopiError_t diopiRotaryEmbeddingV2(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, int64_t);
diopiError_t diopiApplyPenalty(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                               diopiConstTensorHandle_t, diopiConstTensorHandle_t, int);
diopiError_t diopiApplyPenaltyV2(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                 diopiConstTensorHandle_t, diopiConstTensorHandle_t);
diopiError_t diopiRMSNorm(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiSize_t, diopiConstTensorHandle_t,
                          diopiConstTensorHandle_t, double);
diopiError_t diopiRMSNormBackward(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t,
                                  diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiSize_t, double);
diopiError_t diopiDestIndexCopyKV(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t);
diopiError_t diopiTokenAttentionInference(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                          diopiConstTensorHandle_t, diopiConstTensorHandle_t, int);
diopiError_t diopiTokenSoftmaxReduceVInference(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                               diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, int, int);
diopiError_t diopiContextAttentionInference(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                            diopiConstTensorHandle_t, diopiConstTensorHandle_t, int);
diopiError_t diopiFlashAttentionVarLen(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiGeneratorHandle_t, diopiConstTensorHandle_t,
                                       diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                       diopiConstTensorHandle_t, int32_t, int32_t, float, float, bool, int32_t, int32_t);
diopiError_t diopiFlashAttention(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiGeneratorHandle_t, diopiConstTensorHandle_t,
                                 diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, float, float, bool, int32_t, int32_t);
diopiError_t diopiMultiHeadAttention(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, double, bool, bool, double,
                                     diopiTensorHandle_t, diopiTensorHandle_t, diopiGeneratorHandle_t, diopiTensorHandle_t);
diopiError_t diopiMultiHeadAttentionVarLen(diopiContextHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t,
                                           diopiConstTensorHandle_t, int64_t, int64_t, double, bool, bool, double, diopiTensorHandle_t, diopiTensorHandle_t,
                                           diopiGeneratorHandle_t, diopiTensorHandle_t);
diopiError_t diopiPagedAttention(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                 diopiConstTensorHandle_t, diopiSize_t, int64_t, int64_t, int64_t, diopiConstTensorHandle_t, int64_t);
diopiError_t diopiPromptFlashAttention(diopiContextHandle_t, diopiTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t, diopiConstTensorHandle_t,
                                       diopiConstTensorHandle_t, diopiSize_t, int64_t, int64_t, int64_t, int64_t);
// the callbacks the library imports
diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t, diopiSize_t*);
diopiError_t diopiGetStream(diopiContextHandle_t, diopiStreamHandle_t*);
diopiError_t diopiRequireTensor(diopiContextHandle_t, diopiTensorHandle_t*, const diopiSize_t*, const diopiSize_t*, const diopiDtype_t, const diopiDevice_t);
diopiError_t diopiRequireBuffer(diopiContextHandle_t, diopiTensorHandle_t*, int64_t, diopiDevice_t);
}

// value types must have the reference's layout
static_assert(sizeof(diopiSize_t) == 16, "diopiSize_t is {const int64_t*, int64_t}");
static_assert(diopiNoImplement == 13 && diopiDtypeNotSupported == 1000, "error codes");
static_assert(diopi_dtype_int32 == 4 && diopi_dtype_int64 == 6 && diopi_dtype_float16 == 8 && diopi_dtype_float32 == 9 && diopi_dtype_float64 == 10 &&
                  diopi_dtype_bfloat16 == 12,
              "dtype codes");
static_assert(diopi_host == 0 && diopi_device == 1, "device codes");
int main() { return 0; }
