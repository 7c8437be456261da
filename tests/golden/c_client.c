/*
 * A host written in plain C that uses the operator library the way a foreign-function binding would: nothing but the
 * public headers, the two shared libraries on the link line (the runtime first: it defines the callbacks the
 * operator library imports), device memory and streams through the harness hooks of conform_test.h.
 *
 *   diopi_c_client          without a GPU: checks that everything links and that the library identifies itself
 *                           with a GPU: runs diopiRMSNorm (fp32) and diopiDestIndexCopyKV (fp16 bytes) on small tensors
 *                           and compares them with a double-precision loop / a byte-exact scatter done here
 * Exit status 0 and a last line "c client ok" on success.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <conform_test.h>
#include <diopi/functions.h>
#include <diopi/functions_ext.h>
#include <diopirt_hip.h>

#define N1 12
#define N2 32
#define ROWS 120
#define TOKENS 5
#define ROW_ELEMS (8 * 16) /* [heads, dim] of one cache row */

static int fail(const char* what) {
    fprintf(stderr, "c client: %s failed: %s\n", what, diopiGetLastErrorString());
    return 1;
}

static uint32_t lcg(uint32_t* s) {
    *s = *s * 1664525u + 1013904223u;
    return *s;
}

int main(void) {
    const char* vendor = diopiGetVendorName();
    if (vendor == NULL || strstr(vendor, "Device") == NULL) {
        fprintf(stderr, "c client: unexpected vendor name\n");
        return 1;
    }
    printf("vendor %s\n%s\n", vendor, diopiGetImplVersion());
    if (initLibrary() != diopiSuccess) return fail("initLibrary");
    if (diopirtDeviceCount() < 1) {
        printf("no device: link and identity checks only\nc client ok\n");
        return 0;
    }

    diopiStreamHandle_t stream = NULL;
    if (device_make_stream(&stream) != diopiSuccess) return fail("device_make_stream");
    diopiContextHandle_t ctx = diopirtContextCreate(stream);
    uint32_t seed = 12345u;

    /* ---- diopiRMSNorm, fp32 [N1, N2] ---- */
    static float x[N1 * N2], w[N2], out[N1 * N2], inv[N1];
    for (int i = 0; i < N1 * N2; ++i) x[i] = (float)(lcg(&seed) >> 8) / 8388608.0f - 1.0f;
    for (int j = 0; j < N2; ++j) w[j] = 0.5f + (float)(lcg(&seed) >> 8) / 16777216.0f;
    void *dx = device_malloc(sizeof x), *dw = device_malloc(sizeof w), *dout = device_malloc(sizeof out), *dinv = device_malloc(sizeof inv);
    if (!dx || !dw || !dout || !dinv) return fail("device_malloc");
    if (device_memcpy_h2d_async(stream, dx, x, sizeof x) != diopiSuccess) return fail("h2d");
    if (device_memcpy_h2d_async(stream, dw, w, sizeof w) != diopiSuccess) return fail("h2d");
    const int64_t shape2[2] = {N1, N2}, shapeW[1] = {N2}, shapeInv[1] = {N1};
    diopiTensorHandle_t tx = diopirtTensorWrap(dx, shape2, NULL, 2, diopi_dtype_float32, diopi_device);
    diopiTensorHandle_t tout = diopirtTensorWrap(dout, shape2, NULL, 2, diopi_dtype_float32, diopi_device);
    diopiTensorHandle_t tw = diopirtTensorWrap(dw, shapeW, NULL, 1, diopi_dtype_float32, diopi_device);
    diopiTensorHandle_t tinv = diopirtTensorWrap(dinv, shapeInv, NULL, 1, diopi_dtype_float32, diopi_device);
    const diopiSize_t normalized = {shapeW, 1};
    const double eps = 1e-6;
    if (diopiRMSNorm(ctx, tout, tinv, tx, normalized, tw, NULL, eps) != diopiSuccess) return fail("diopiRMSNorm");
    if (device_memcpy_d2h_async(stream, out, dout, sizeof out) != diopiSuccess) return fail("d2h");
    if (device_memcpy_d2h_async(stream, inv, dinv, sizeof inv) != diopiSuccess) return fail("d2h");
    if (device_synchronize_stream(stream) != diopiSuccess) return fail("device_synchronize_stream");
    double worst = 0.0;
    for (int r = 0; r < N1; ++r) {
        double ss = 0.0;
        for (int j = 0; j < N2; ++j) ss += (double)x[r * N2 + j] * x[r * N2 + j];
        const double rinv = 1.0 / sqrt(ss / N2 + eps);
        if (fabs(inv[r] - rinv) > 1e-5 * rinv) {
            fprintf(stderr, "c client: inv_rms[%d] = %g, expected %g\n", r, inv[r], rinv);
            return 1;
        }
        for (int j = 0; j < N2; ++j) {
            const double want = w[j] * (rinv * x[r * N2 + j]);
            const double err = fabs(out[r * N2 + j] - want);
            if (err > worst) worst = err;
            if (err > 1e-5 + 1e-5 * fabs(want)) {
                fprintf(stderr, "c client: out[%d,%d] = %g, expected %g\n", r, j, out[r * N2 + j], want);
                return 1;
            }
        }
    }
    printf("diopiRMSNorm fp32 [%d,%d]: max abs error %.3g\n", N1, N2, worst);

    /* ---- diopiDestIndexCopyKV, 16-bit rows: bytes in, bytes out ---- */
    static uint16_t cache[ROWS * ROW_ELEMS], want[ROWS * ROW_ELEMS], k[TOKENS * ROW_ELEMS];
    static const int32_t dest[TOKENS] = {14, 15, 16, 17, 3};
    for (int i = 0; i < ROWS * ROW_ELEMS; ++i) cache[i] = (uint16_t)(lcg(&seed) >> 16);
    for (int i = 0; i < TOKENS * ROW_ELEMS; ++i) k[i] = (uint16_t)(lcg(&seed) >> 16);
    memcpy(want, cache, sizeof cache);
    for (int t = 0; t < TOKENS; ++t) memcpy(want + dest[t] * ROW_ELEMS, k + t * ROW_ELEMS, ROW_ELEMS * sizeof(uint16_t));
    void *dcache = device_malloc(sizeof cache), *dk = device_malloc(sizeof k), *ddest = device_malloc(sizeof dest);
    if (!dcache || !dk || !ddest) return fail("device_malloc");
    if (device_memcpy_h2d_async(stream, dcache, cache, sizeof cache) != diopiSuccess) return fail("h2d");
    if (device_memcpy_h2d_async(stream, dk, k, sizeof k) != diopiSuccess) return fail("h2d");
    if (device_memcpy_h2d_async(stream, ddest, dest, sizeof dest) != diopiSuccess) return fail("h2d");
    const int64_t shapeCache[3] = {ROWS, 8, 16}, shapeK[3] = {TOKENS, 8, 16}, shapeDest[1] = {TOKENS};
    diopiTensorHandle_t tcache = diopirtTensorWrap(dcache, shapeCache, NULL, 3, diopi_dtype_float16, diopi_device);
    diopiTensorHandle_t tk = diopirtTensorWrap(dk, shapeK, NULL, 3, diopi_dtype_float16, diopi_device);
    diopiTensorHandle_t tdest = diopirtTensorWrap(ddest, shapeDest, NULL, 1, diopi_dtype_int32, diopi_device);
    if (diopiDestIndexCopyKV(ctx, tcache, tk, tdest) != diopiSuccess) return fail("diopiDestIndexCopyKV");
    if (device_memcpy_d2h_async(stream, cache, dcache, sizeof cache) != diopiSuccess) return fail("d2h");
    if (device_synchronize_stream(stream) != diopiSuccess) return fail("device_synchronize_stream");
    if (memcmp(cache, want, sizeof cache) != 0) {
        fprintf(stderr, "c client: diopiDestIndexCopyKV: the cache differs from the scatter done on the host\n");
        return 1;
    }
    printf("diopiDestIndexCopyKV fp16 [%d,8,16] -> [%d,8,16]: bytes equal\n", TOKENS, ROWS);

    /* ---- an argument error comes back as a code and a message, not as a crash ---- */
    if (diopiDestIndexCopyKV(ctx, tcache, tk, NULL) == diopiSuccess || strlen(diopiGetLastErrorString()) == 0) {
        fprintf(stderr, "c client: a null handle was not rejected\n");
        return 1;
    }

    diopiTensorHandle_t handles[] = {tx, tout, tw, tinv, tcache, tk, tdest};
    for (size_t i = 0; i < sizeof handles / sizeof handles[0]; ++i) diopirtTensorDestroy(handles[i]);
    diopirtContextDestroy(ctx);
    void* blocks[] = {dx, dw, dout, dinv, dcache, dk, ddest};
    for (size_t i = 0; i < sizeof blocks / sizeof blocks[0]; ++i) device_free(blocks[i]);
    if (device_destroy_stream(stream) != diopiSuccess) return fail("device_destroy_stream");
    if (finalizeLibrary() != diopiSuccess) return fail("finalizeLibrary");
    printf("c client ok\n");
    return 0;
}
