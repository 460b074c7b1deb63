// Weight gradient of the BH4 stages with 64x64 blocks: for every stage s = (r, j) and block n
//
//   g[s][n][o][i] += sum over tokens b of  p[s][b][64n + o] * u[s][b][64n + i]
//
// p[s]: [B, D] the gradient in front of the stage's block product (what lffn_bh4_block_bwd_f32
// writes), u[s]: the stage's input: x [B, H], zero beyond column H, for j = 0, else the saved
// input [B, D] of stage j (what lffn_bh4_block_hash_train_f32 keeps).  With ln_w the stage-0 input is
// LayerNorm(x), formed on load from x and the rows' kept mean and 1/sigma (the forward's LayerNorm ran
// inside its kernel and the normalised rows were never stored).  A batched product
// with a tiny output (64x64 per block) and a long sum (all tokens): one workgroup takes one
// block and a chunk of tokens, each of its four wavefronts sums a quarter of the chunk into a
// full 64x64 tile on the fp32 matrix cores (16 accumulator tiles), the four tiles are added in
// LDS and the workgroup adds its result to g with global atomics (g must hold the value to
// accumulate into, e.g. zero).
//
// Operands: a lane loads 16 bytes of a token's row of the block, lanes 0-15 cover the 256-byte
// row, the four lane groups take four consecutive tokens (the k index of
// v_mfma_f32_16x16x4_f32).  The four values of a lane feed four different output tiles, so
// tile j holds rows/columns 4*c + j (c = lane % 16): a fixed permutation undone when the tile
// is written.
#include "lffn_common.h"

#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

// LayerNorm on load repeats the forward kernel's operations one by one: no fused multiply-add
#pragma clang fp contract(off)

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BS = 64;
constexpr int CHUNK = 512;        // tokens per workgroup
constexpr int DEPTH = 4;          // token quads whose loads are in flight per wavefront

__global__ __launch_bounds__(256) void bh4_wgrad_kernel(const float *__restrict__ stage_grads,
                                                        const float *__restrict__ x,
                                                        const float *__restrict__ stage_inputs,
                                                        float *__restrict__ g, int64_t B, int H, int D, int J,
                                                        const float *__restrict__ ln_w, const float *__restrict__ ln_b,
                                                        const float *__restrict__ row_stats) {
    __shared__ float red[4][BS * BS / 4];          // a quarter of each wavefront's 64x64 tile
    const int n = blockIdx.y;
    const int s = blockIdx.z;                      // stage r * J + j
    const int r = s / J, j = s % J;
    const float *p = stage_grads + (size_t)s * B * D;
    const float *u = j == 0 ? x : stage_inputs + (size_t)(r * (J - 1) + j - 1) * B * D;
    const int Hu = j == 0 ? H : D, ldu = Hu;
    // a block of the first stage that lies wholly in the zero padding beyond column H has a zero input,
    // hence a zero gradient: g keeps what it holds (768 columns padded to 1024: 4 of 16 blocks)
    if (n * BS >= Hu) return;                      // uniform over the workgroup
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int c = lane & 15;
    const int kq = lane >> 4;
    const int64_t tok_lo = int64_t(blockIdx.x) * CHUNK + wave * (CHUNK / 4);
    const int64_t tok_hi = min<int64_t>(tok_lo + CHUNK / 4, B);
    const int ucol = n * BS + 4 * c;
    const bool u_live = ucol < Hu;                 // Hu % 4 == 0: the four columns are all in or all out
    // LayerNorm on load (stage 0 only): this lane's four columns of the weight and bias
    const bool ln = ln_w != nullptr && j == 0;     // uniform over the workgroup
    float4 lw = make_float4(1.f, 1.f, 1.f, 1.f), lb = make_float4(0.f, 0.f, 0.f, 0.f);
    if (ln && u_live) {
        lw = *reinterpret_cast<const float4 *>(ln_w + ucol);
        lb = *reinterpret_cast<const float4 *>(ln_b + ucol);
    }

    f32x4 acc[4][4];                               // [o tile][i tile]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // The loads of the next DEPTH token quads are issued before the products of the current
    // ones, so a wavefront keeps memory requests in flight while its matrix core works.
    float4 pv[DEPTH], uv[DEPTH], pn[DEPTH], un[DEPTH];
    auto fetch = [&](int64_t t0, float4 *pd, float4 *ud) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int64_t tok = t0 + 4 * d + kq;
            const bool live = tok < tok_hi;
            pd[d] = live ? *reinterpret_cast<const float4 *>(p + tok * D + n * BS + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
            ud[d] = (live && u_live) ? *reinterpret_cast<const float4 *>(u + tok * ldu + ucol)
                                     : make_float4(0.f, 0.f, 0.f, 0.f);
            if (ln && live && u_live) {
                // the same operations as the forward's LayerNorm: (x - mean) * (1/sigma) * weight + bias
                const float2 st = *reinterpret_cast<const float2 *>(row_stats + 2 * tok);
                ud[d].x = (ud[d].x - st.x) * st.y * lw.x + lb.x;
                ud[d].y = (ud[d].y - st.x) * st.y * lw.y + lb.y;
                ud[d].z = (ud[d].z - st.x) * st.y * lw.z + lb.z;
                ud[d].w = (ud[d].w - st.x) * st.y * lw.w + lb.w;
            }
        }
    };
    fetch(tok_lo, pv, uv);
    for (int64_t t0 = tok_lo; t0 < tok_hi; t0 += 4 * DEPTH) {
        fetch(t0 + 4 * DEPTH, pn, un);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const float pa[4] = {pv[d].x, pv[d].y, pv[d].z, pv[d].w};
            const float ub[4] = {uv[d].x, uv[d].y, uv[d].z, uv[d].w};
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[a], ub[b], acc[a][b], 0, 0, 0);
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) { pv[d] = pn[d]; uv[d] = un[d]; }
    }

    // Tile (a, b), lane (c, kq), component r holds the sum for row o = 4*(4*kq + r) + a and
    // column i = 4*c + b.  Sum the four wavefronts through LDS, a quarter of the 64x64 block
    // (one value of a) at a time, then add to g.
    float *gb = g + ((size_t)s * (D / BS) + n) * BS * BS;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        __syncthreads();
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[wave][((4 * kq + r) * 16 + c) * 4 + b] = acc[a][b][r];       // [o' = 4kq+r][c][b]
        __syncthreads();
        // 16 rows o' x 64 columns of this quarter: thread t adds element t, t+256, ...
        for (int e = threadIdx.x; e < BS * BS / 4; e += 256) {
            const float sum = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
            const int op = e / 64, i = e % 64;                   // i = 4*c + b already in order
            unsafeAtomicAdd(gb + (4 * op + a) * BS + i, sum);
        }
    }
}

int wgrad_entry(const float *stage_grads, const float *x, const float *ln_weight, const float *ln_bias,
                const float *row_stats, const float *stage_inputs, float *g_folded, int64_t B, int64_t H, int64_t D,
                int64_t R, int64_t J, int64_t block_size, void *stream) {
    LFFN_REQUIRE(B >= 0 && D >= 1 && H >= 1 && H <= D && R >= 1 && J >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(block_size == BS && D % BS == 0 && D <= (1 << 20), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(H % 4 == 0 && B <= (int64_t(1) << 31) - 1 && R * J <= 65535, LFFN_ERR_UNSUPPORTED);
    if (B == 0) return LFFN_OK;
    LFFN_REQUIRE(stage_grads && x && g_folded && (stage_inputs || J == 1), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(stage_grads) && lffn_aligned16(x) && lffn_aligned16(stage_inputs) && lffn_aligned16(g_folded),
                 LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(!ln_weight || (ln_bias && row_stats && lffn_aligned16(ln_weight) && lffn_aligned16(ln_bias) &&
                                (uintptr_t)row_stats % 8 == 0), LFFN_ERR_BAD_ARG);
    const int64_t chunks = (B + CHUNK - 1) / CHUNK;
    LFFN_REQUIRE(chunks <= 0x7fffffff && D / BS <= 65535, LFFN_ERR_UNSUPPORTED);
    hipLaunchKernelGGL(bh4_wgrad_kernel, dim3((unsigned)chunks, (unsigned)(D / BS), (unsigned)(R * J)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), stage_grads, x, stage_inputs, g_folded, B, (int)H, (int)D, (int)J,
                       ln_weight, ln_bias, row_stats);
    return lffn_launch_status();
}

}  // namespace

extern "C" int lffn_bh4_block_wgrad_f32(const float *stage_grads, const float *x, const float *stage_inputs,
                                        float *g_folded, int64_t B, int64_t H, int64_t D, int64_t R, int64_t J,
                                        int64_t block_size, void *stream) {
    return wgrad_entry(stage_grads, x, nullptr, nullptr, nullptr, stage_inputs, g_folded, B, H, D, R, J, block_size, stream);
}

extern "C" int lffn_ln_bh4_block_wgrad_f32(const float *stage_grads, const float *x, const float *ln_weight,
                                           const float *ln_bias, const float *row_stats, const float *stage_inputs,
                                           float *g_folded, int64_t B, int64_t H, int64_t D, int64_t R, int64_t J,
                                           int64_t block_size, void *stream) {
    LFFN_REQUIRE(ln_weight && ln_bias && row_stats, LFFN_ERR_BAD_ARG);
    return wgrad_entry(stage_grads, x, ln_weight, ln_bias, row_stats, stage_inputs, g_folded, B, H, D, R, J, block_size, stream);
}
