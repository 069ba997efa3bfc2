/*
 * The C-ABI of include/df11.h used from plain C, with no Python and no torch:
 * compress a synthetic BF16 tensor with the host codec, decode it on the GPU,
 * compare with the original words.  This is what a native caller of the
 * reference path (the kernel launch of dfloat11/dfloat11.py:139-151 and the
 * codec of dfloat11/dfloat11_utils.py:24-187) would link against.
 *
 *   abi_roundtrip [n_elements]      exit status 0 = bit-exact
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "df11.h"

#define CHECK_HIP(x)                                                            \
    do {                                                                        \
        hipError_t e_ = (x);                                                    \
        if (e_ != hipSuccess) {                                                 \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));             \
            return 2;                                                           \
        }                                                                       \
    } while (0)
#define CHECK_DF11(x)                                                           \
    do {                                                                        \
        int rc_ = (x);                                                          \
        if (rc_ != DF11_OK) {                                                   \
            fprintf(stderr, "%s: %s (%s)\n", #x, df11_error_string(rc_),        \
                    rc_ == DF11_ERR_HIP ? df11_last_hip_error() : "-");         \
            return 3;                                                           \
        }                                                                       \
    } while (0)

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static double uniform01(void)
{
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    return (double)(rng_state >> 11) / 9007199254740992.0;
}

static uint16_t to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7FFFu + ((u >> 16) & 1u); /* round to nearest even */
    return (uint16_t)(u >> 16);
}

int main(int argc, char **argv)
{
    const int64_t n = argc > 1 ? atoll(argv[1]) : 3000001;
    if (n <= 0) return 2;
    uint16_t *w = malloc((size_t)n * 2);
    for (int64_t i = 0; i < n; ++i) { /* roughly N(0, 0.02), plus a few zeros and large values */
        double g = 0;
        for (int k = 0; k < 12; ++k) g += uniform01();
        float v = (float)((g - 6.0) * 0.02);
        if (i % 1000 == 7) v = 0.0f;
        if (i % 4001 == 11) v *= 3000.0f;
        w[i] = to_bf16(v);
    }

    /* host codec */
    uint64_t hist[256];
    uint8_t code_len[256], luts[18 * 256];
    uint32_t code_val[256], eof_val;
    int32_t eof_len, n_luts;
    int64_t n_bytes, n_blocks;
    CHECK_DF11(df11_histogram(w, n, hist, 0));
    CHECK_DF11(df11_build_code(hist, code_len, code_val, &eof_len, &eof_val));
    CHECK_DF11(df11_build_luts(code_len, code_val, luts, 18, &n_luts));
    uint8_t *exponent = malloc((size_t)n), *sign_mantissa = malloc((size_t)n);
    CHECK_DF11(df11_split(w, n, exponent, sign_mantissa, 0));
    CHECK_DF11(df11_encode_size(exponent, n, code_len, &n_bytes, &n_blocks, 0));
    uint8_t *encoded = malloc((size_t)n_bytes), *gaps = malloc((size_t)n_blocks * DF11_GAP_BYTES_PER_BLOCK);
    uint32_t *positions = malloc((size_t)(n_blocks + 1) * 4);
    CHECK_DF11(df11_encode(exponent, n, code_len, code_val, eof_len, eof_val, encoded, n_bytes, gaps,
                           positions, n_blocks, 0));

    /* device decode */
    void *d_luts, *d_enc, *d_sm, *d_pos, *d_gaps, *d_out, *d_ws;
    const size_t ws_bytes = df11_workspace_bytes(n_bytes);
    CHECK_HIP(hipMalloc(&d_luts, (size_t)n_luts * 256));
    CHECK_HIP(hipMalloc(&d_enc, (size_t)n_bytes));
    CHECK_HIP(hipMalloc(&d_sm, (size_t)n));
    CHECK_HIP(hipMalloc(&d_pos, (size_t)(n_blocks + 1) * 4));
    CHECK_HIP(hipMalloc(&d_gaps, (size_t)n_blocks * DF11_GAP_BYTES_PER_BLOCK));
    CHECK_HIP(hipMalloc(&d_out, (size_t)n * 2));
    CHECK_HIP(hipMalloc(&d_ws, ws_bytes));
    CHECK_HIP(hipMemcpy(d_luts, luts, (size_t)n_luts * 256, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_enc, encoded, (size_t)n_bytes, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_sm, sign_mantissa, (size_t)n, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_pos, positions, (size_t)(n_blocks + 1) * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_gaps, gaps, (size_t)n_blocks * DF11_GAP_BYTES_PER_BLOCK, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemset(d_out, 0xEE, (size_t)n * 2));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    int32_t max_sub = 0;
    CHECK_DF11(df11_prepare(d_luts, d_enc, d_pos, d_gaps, n_luts, n_bytes, n, d_ws, &max_sub, stream));
    for (int pass = 0; pass < 2; ++pass)
        CHECK_DF11(df11_decode(d_luts, d_enc, d_sm, d_pos, d_gaps, d_out, n_luts, n_bytes, n, d_ws, max_sub, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    uint16_t *back = malloc((size_t)n * 2);
    CHECK_HIP(hipMemcpy(back, d_out, (size_t)n * 2, hipMemcpyDeviceToHost));

    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) bad += back[i] != w[i];
    printf("abi_roundtrip: library version %d, %lld elements, %lld bitstream bytes in %lld blocks, %d LUT rows, "
           "compressed/BF16 = %.4f, longest sub-block %d elements, mismatches %lld\n",
           df11_version(), (long long)n, (long long)n_bytes, (long long)n_blocks, n_luts,
           (double)(n_bytes + n + n_blocks * (DF11_GAP_BYTES_PER_BLOCK + 4) + n_luts * 256) / (2.0 * (double)n),
           max_sub, (long long)bad);
    return bad ? 1 : 0;
}
