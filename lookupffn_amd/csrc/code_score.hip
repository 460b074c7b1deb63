// Code + score of the LookupFFN hash, and the gradient of the score, for gfx950.
// One thread per (token, table) group of k consecutive values.  The fused
// projection kernel computes the same quantities for k == 8 without the round trip
// through memory; these kernels serve every other k, the training path (which
// keeps z for the backward) and callers that already hold z.
#include "lffn_common.h"

// d ascending, mul and add kept separate, as in
// compute_code_score/torch_extension.cc:31-37.
#pragma clang fp contract(off)

namespace {

template <int K>   // K > 0: compile-time length (multiple of 4, vector loads); K == 0: runtime k
__global__ __launch_bounds__(256) void code_score_kernel(const float *__restrict__ z, int32_t *__restrict__ codes,
                                                         float *__restrict__ scores, int64_t N, int k_rt) {
    const int64_t n = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (n >= N) return;
    int code = 0;
    float num = 0.f, den = 1.f;
    if constexpr (K > 0) {
        const float4 *p = reinterpret_cast<const float4 *>(z + n * K);
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
            const float4 t = p[q];
            const float v[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float a = fabsf(v[c]);
                code = (code << 1) | (v[c] > 0.f ? 1 : 0);
                num = num + a;
                den = den * (1.0f + expf(-2.0f * a));
            }
        }
    } else {
        const float *p = z + n * k_rt;
        for (int d = 0; d < k_rt; ++d) {
            const float v = p[d];
            const float a = fabsf(v);
            code = (code << 1) | (v > 0.f ? 1 : 0);
            num = num + a;
            den = den * (1.0f + expf(-2.0f * a));
        }
    }
    codes[n] = code;
    scores[n] = num / den;
}

__global__ __launch_bounds__(256) void code_score_bwd_kernel(const float *__restrict__ z, const float *__restrict__ g_score,
                                                             float *__restrict__ g_z, int64_t N, int k) {
    const int64_t n = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (n >= N) return;
    const float *p = z + n * k;
    float S = 0.f, P = 1.f;
    for (int d = 0; d < k; ++d) {
        const float a = fabsf(p[d]);
        S = S + a;
        P = P * (1.0f + expf(-2.0f * a));
    }
    const float g = g_score[n];
    for (int d = 0; d < k; ++d) {
        const float v = p[d];
        const float a = fabsf(v);
        const float e = expf(-2.0f * a);
        const float sg = v > 0.f ? 1.f : (v < 0.f ? -1.f : 0.f);
        g_z[n * k + d] = g * sg * (1.0f + S * 2.0f * e / (1.0f + e)) / P;
    }
}

}  // namespace

extern "C" int lffn_code_score_f32(const float *z, int32_t *codes, float *scores,
                                   int64_t N, int64_t k, void *stream) {
    LFFN_REQUIRE(z && codes && scores, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(N >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(k >= 1 && k <= 24, LFFN_ERR_UNSUPPORTED);
    if (N == 0) return LFFN_OK;
    const int64_t blocks = (N + 255) / 256;
    LFFN_REQUIRE(blocks <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = lffn_aligned16(z);
    if (vec && k == 8)
        hipLaunchKernelGGL((code_score_kernel<8>), dim3((unsigned)blocks), dim3(256), 0, s, z, codes, scores, N, 8);
    else if (vec && k == 4)
        hipLaunchKernelGGL((code_score_kernel<4>), dim3((unsigned)blocks), dim3(256), 0, s, z, codes, scores, N, 4);
    else if (vec && k == 12)
        hipLaunchKernelGGL((code_score_kernel<12>), dim3((unsigned)blocks), dim3(256), 0, s, z, codes, scores, N, 12);
    else if (vec && k == 16)
        hipLaunchKernelGGL((code_score_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, s, z, codes, scores, N, 16);
    else
        hipLaunchKernelGGL((code_score_kernel<0>), dim3((unsigned)blocks), dim3(256), 0, s, z, codes, scores, N, (int)k);
    return lffn_launch_status();
}

extern "C" int lffn_code_score_bwd_f32(const float *z, const float *g_score, float *g_z,
                                       int64_t N, int64_t k, void *stream) {
    LFFN_REQUIRE(z && g_score && g_z, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(N >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(k >= 1 && k <= 24, LFFN_ERR_UNSUPPORTED);
    if (N == 0) return LFFN_OK;
    const int64_t blocks = (N + 255) / 256;
    LFFN_REQUIRE(blocks <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    hipLaunchKernelGGL(code_score_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), z, g_score, g_z, N, (int)k);
    return lffn_launch_status();
}
