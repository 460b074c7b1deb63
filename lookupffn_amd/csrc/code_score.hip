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
                den = den * (1.0f + exp_minus_2a(a));
            }
        }
    } else {
        const float *p = z + n * k_rt;
        for (int d = 0; d < k_rt; ++d) {
            const float v = p[d];
            const float a = fabsf(v);
            code = (code << 1) | (v > 0.f ? 1 : 0);
            num = num + a;
            den = den * (1.0f + exp_minus_2a(a));
        }
    }
    codes[n] = code;
    scores[n] = num / den;
}

// The tail of the BH4 module and the hash in one pass (PL/lookup.py:36-37, then
// compute_code_score): for column col = t*k + d of token b
//   z = decay * y[b, col] + residual * xpad[b, col % D] + bias[col]
// (the two products, their sum, then the bias: the reference's order), followed by the
// code and score of every group of k columns.  y: [B, ldy] (ldy = R*D), x: [B, H] with
// H <= D, zero beyond H.  K > 0: compile-time k, a multiple of 4, 16-byte loads
// (needs D % K == 0 and H % 4 == 0 so that a group neither wraps nor straddles H).
template <int K>
__global__ __launch_bounds__(256) void mix_code_score_kernel(const float *__restrict__ y, const float *__restrict__ x,
                                                             const float *__restrict__ bias,
                                                             int32_t *__restrict__ codes, float *__restrict__ scores,
                                                             int64_t B, int T, int k_rt, int H, int D, int64_t ldy,
                                                             float decay, float residual) {
    const int64_t n = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (n >= B * T) return;
    const int64_t b = n / T;
    const int t = (int)(n % T);
    int code = 0;
    float num = 0.f, den = 1.f;
    auto step = [&](float yv, float xv, float bv) {
        const float v = (decay * yv + residual * xv) + bv;
        const float a = fabsf(v);
        code = (code << 1) | (v > 0.f ? 1 : 0);
        num = num + a;
        den = den * (1.0f + exp_minus_2a(a));
    };
    if constexpr (K > 0) {
        const int col0 = t * K;
        const int xi0 = col0 % D;
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
            const float4 yv = *reinterpret_cast<const float4 *>(y + b * ldy + col0 + 4 * q);
            const float4 xv = (xi0 + 4 * q < H) ? *reinterpret_cast<const float4 *>(x + b * H + xi0 + 4 * q)
                                                : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 bv = bias ? *reinterpret_cast<const float4 *>(bias + col0 + 4 * q)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
            step(yv.x, xv.x, bv.x);
            step(yv.y, xv.y, bv.y);
            step(yv.z, xv.z, bv.z);
            step(yv.w, xv.w, bv.w);
        }
    } else {
        for (int d = 0; d < k_rt; ++d) {
            const int col = t * k_rt + d;
            const int xi = col % D;
            step(y[b * ldy + col], xi < H ? x[b * H + xi] : 0.f, bias ? bias[col] : 0.f);
        }
    }
    codes[n] = code;
    scores[n] = num / den;
}

// K > 0: k == K, z and g_z 16-byte aligned with K % 4 == 0: one hash per lane, its K values in
// registers (one exponential per value).  K == 0: any k, scalar loads.
template <int K>
__global__ __launch_bounds__(256) void code_score_bwd_kernel(const float *__restrict__ z, const float *__restrict__ g_score,
                                                             float *__restrict__ g_z, int64_t N, int k) {
    const int64_t n = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (n >= N) return;
    if constexpr (K > 0) {
        float v[K], e[K];
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
            const float4 t = reinterpret_cast<const float4 *>(z + n * K)[q];
            v[4 * q] = t.x, v[4 * q + 1] = t.y, v[4 * q + 2] = t.z, v[4 * q + 3] = t.w;
        }
        float S = 0.f, P = 1.f;
#pragma unroll
        for (int d = 0; d < K; ++d) {
            const float a = fabsf(v[d]);
            e[d] = expf(-2.0f * a);
            S = S + a;
            P = P * (1.0f + e[d]);
        }
        const float gp = g_score[n] / P;
        float o[K];
#pragma unroll
        for (int d = 0; d < K; ++d) {
            const float sg = v[d] > 0.f ? gp : (v[d] < 0.f ? -gp : 0.f);
            o[d] = sg * (1.0f + S * 2.0f * (e[d] * __builtin_amdgcn_rcpf(1.0f + e[d])));   // hardware reciprocal, 1 ulp
        }
#pragma unroll
        for (int q = 0; q < K / 4; ++q)
            reinterpret_cast<float4 *>(g_z + n * K)[q] = make_float4(o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]);
    } else {
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

extern "C" int lffn_mix_code_score_f32(const float *y, const float *x, const float *bias, int32_t *codes,
                                       float *scores, int64_t B, int64_t T, int64_t k, int64_t H, int64_t D,
                                       int64_t ldy, float decay, float residual, void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && H >= 1 && D >= 1 && H <= D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(k >= 1 && k <= 24, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * k <= ldy && ldy <= (int64_t(1) << 30) && D <= (1 << 24), LFFN_ERR_BAD_ARG);
    if (B * T == 0) return LFFN_OK;
    LFFN_REQUIRE(y && x && codes && scores, LFFN_ERR_BAD_ARG);
    const int64_t blocks = (B * T + 255) / 256;
    LFFN_REQUIRE(blocks <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = lffn_aligned16(y) && lffn_aligned16(x) && (!bias || lffn_aligned16(bias)) && ldy % 4 == 0 &&
                     H % 4 == 0 && D % k == 0;
#define LFFN_MIX_LAUNCH(KK)                                                                                    \
    hipLaunchKernelGGL((mix_code_score_kernel<KK>), dim3((unsigned)blocks), dim3(256), 0, s, y, x, bias, codes, \
                       scores, B, (int)T, (int)k, (int)H, (int)D, ldy, decay, residual)
    if (vec && k == 8) LFFN_MIX_LAUNCH(8);
    else if (vec && k == 4) LFFN_MIX_LAUNCH(4);
    else if (vec && k == 16) LFFN_MIX_LAUNCH(16);
    else LFFN_MIX_LAUNCH(0);
#undef LFFN_MIX_LAUNCH
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
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = lffn_aligned16(z) && lffn_aligned16(g_z);
    if (vec && k == 8)
        hipLaunchKernelGGL((code_score_bwd_kernel<8>), dim3((unsigned)blocks), dim3(256), 0, s, z, g_score, g_z, N, 8);
    else if (vec && k == 4)
        hipLaunchKernelGGL((code_score_bwd_kernel<4>), dim3((unsigned)blocks), dim3(256), 0, s, z, g_score, g_z, N, 4);
    else if (vec && k == 12)
        hipLaunchKernelGGL((code_score_bwd_kernel<12>), dim3((unsigned)blocks), dim3(256), 0, s, z, g_score, g_z, N, 12);
    else if (vec && k == 16)
        hipLaunchKernelGGL((code_score_bwd_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, s, z, g_score, g_z, N, 16);
    else
        hipLaunchKernelGGL((code_score_bwd_kernel<0>), dim3((unsigned)blocks), dim3(256), 0, s, z, g_score, g_z, N, (int)k);
    return lffn_launch_status();
}
