// Backward of the layer's LayerNorm (PL/lookup.py:84,99: torch.nn.LayerNorm over the last
// dimension, biased variance, eps inside the square root), one kernel:
//
//   g    = sum_r g_y[r]                       (the projection's R repeats each bring a gradient)
//   x^   = (x - mean) * rstd                  (recomputed from x: nothing is kept from the forward)
//   g_x  = rstd * (g*w - mean_H(g*w) - x^ * mean_H(g*w * x^))
//   g_w  = sum_b g * x^ ,   g_b = sum_b g
//
// One wavefront per row, H / 64 values per lane in registers (H <= 1024, H % 4 == 0), two
// wave reductions per row.  The weight and bias gradients are summed over a workgroup's rows in
// registers, over its four wavefronts in LDS, and written as one partial per workgroup; the
// caller adds the partials (a few hundred rows of H values).  This replaces what autograd runs
// for the reference (two kernels over the rows plus column reductions).
#include "lffn_common.h"

namespace {

constexpr int NJ_MAX = 4;            // float4 per lane: H <= 1024

struct LnBwdArgs {
    const float *x;       // [B, H]
    const float *w;       // [H] or null (no affine: w = 1)
    const float *gy;      // [R, B, H]
    float *gx;            // [B, H]
    float *part_w;        // [num_partials, H] or null
    float *part_b;        // [num_partials, H] or null
    int64_t B;
    int H, R;
    float eps;
};

template <int NJ>
__global__ __launch_bounds__(256) void layer_norm_bwd_kernel(LnBwdArgs a) {
    __shared__ float red[2][4][NJ * 256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float inv_h = 1.0f / float(a.H);

    float4 wv[NJ], aw[NJ], ab[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e = 256 * j + 4 * lane;
        wv[j] = make_float4(1.f, 1.f, 1.f, 1.f);
        if (a.w && e < a.H) wv[j] = *reinterpret_cast<const float4 *>(a.w + e);
        aw[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        ab[j] = aw[j];
    }

    for (int64_t row = int64_t(blockIdx.x) * 4 + wave; row < a.B; row += int64_t(gridDim.x) * 4) {
        float4 xv[NJ], g[NJ];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int e = 256 * j + 4 * lane;
            xv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            g[j] = xv[j];
            if (e < a.H) {
                xv[j] = *reinterpret_cast<const float4 *>(a.x + row * a.H + e);
                for (int r = 0; r < a.R; ++r) {
                    const float4 t = *reinterpret_cast<const float4 *>(a.gy + (int64_t(r) * a.B + row) * a.H + e);
                    g[j].x += t.x; g[j].y += t.y; g[j].z += t.z; g[j].w += t.w;
                }
            }
            s += (xv[j].x + xv[j].y) + (xv[j].z + xv[j].w);
        }
        const float mean = wave_sum(s) * inv_h;
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const bool on = 256 * j + 4 * lane < a.H;
            xv[j].x = on ? xv[j].x - mean : 0.f; xv[j].y = on ? xv[j].y - mean : 0.f;
            xv[j].z = on ? xv[j].z - mean : 0.f; xv[j].w = on ? xv[j].w - mean : 0.f;
            v += (xv[j].x * xv[j].x + xv[j].y * xv[j].y) + (xv[j].z * xv[j].z + xv[j].w * xv[j].w);
        }
        const float rstd = 1.0f / sqrtf(wave_sum(v) * inv_h + a.eps);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            xv[j].x *= rstd; xv[j].y *= rstd; xv[j].z *= rstd; xv[j].w *= rstd;        // x^
            aw[j].x += g[j].x * xv[j].x; aw[j].y += g[j].y * xv[j].y; aw[j].z += g[j].z * xv[j].z; aw[j].w += g[j].w * xv[j].w;
            ab[j].x += g[j].x; ab[j].y += g[j].y; ab[j].z += g[j].z; ab[j].w += g[j].w;
            g[j].x *= wv[j].x; g[j].y *= wv[j].y; g[j].z *= wv[j].z; g[j].w *= wv[j].w;   // g * w
            s1 += (g[j].x + g[j].y) + (g[j].z + g[j].w);
            s2 += (g[j].x * xv[j].x + g[j].y * xv[j].y) + (g[j].z * xv[j].z + g[j].w * xv[j].w);
        }
        const float m1 = wave_sum(s1) * inv_h, m2 = wave_sum(s2) * inv_h;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int e = 256 * j + 4 * lane;
            if (e < a.H)
                *reinterpret_cast<float4 *>(a.gx + row * a.H + e) =
                    make_float4(rstd * (g[j].x - m1 - xv[j].x * m2), rstd * (g[j].y - m1 - xv[j].y * m2),
                                rstd * (g[j].z - m1 - xv[j].z * m2), rstd * (g[j].w - m1 - xv[j].w * m2));
        }
    }

    if (a.part_w) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            *reinterpret_cast<float4 *>(&red[0][wave][256 * j + 4 * lane]) = aw[j];
            *reinterpret_cast<float4 *>(&red[1][wave][256 * j + 4 * lane]) = ab[j];
        }
        __syncthreads();
        for (int e = threadIdx.x; e < a.H; e += 256) {
            a.part_w[(size_t)blockIdx.x * a.H + e] = (red[0][0][e] + red[0][1][e]) + (red[0][2][e] + red[0][3][e]);
            a.part_b[(size_t)blockIdx.x * a.H + e] = (red[1][0][e] + red[1][1][e]) + (red[1][2][e] + red[1][3][e]);
        }
    }
}

// Column sums of up to two arrays of per-workgroup partial sums, parts[p][n] over p, in one launch
// and in a fixed order (p ascending within a lane, then the 16 lanes of a column group ascending):
// what the backward kernels' callers need for the weight and bias gradients.  A workgroup owns 64
// columns; 16 lanes side by side read 256 contiguous bytes of a row, the 16 lane groups take rows
// 16 apart, eight loads in flight each.
struct SumPartialsArgs {
    const float *pa;
    float *oa;
    int64_t na;
    const float *pb;
    float *ob;
    int64_t nb;
    int P;
    int blocks_a;
    int rows_per_chunk;    // blockIdx.y = chunk: rows [y * rows_per_chunk, ...) summed into row y of the outputs
};

__global__ __launch_bounds__(256) void sum_partials_kernel(SumPartialsArgs a) {
    __shared__ float4 red[16][16];
    const bool second = (int)blockIdx.x >= a.blocks_a;
    const float *parts = second ? a.pb : a.pa;
    float *out = second ? a.ob : a.oa;
    const int64_t n = second ? a.nb : a.na;
    const int blk = second ? blockIdx.x - a.blocks_a : blockIdx.x;
    const int c4 = threadIdx.x & 15, rq = threadIdx.x >> 4;
    const int64_t col = int64_t(blk) * 64 + c4 * 4;
    const bool on = col < n;                                  // n % 4 == 0: all four columns or none
    const int64_t colc = on ? col : 0;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    const int p_begin = blockIdx.y * a.rows_per_chunk, p_end = min(a.P, p_begin + a.rows_per_chunk);
    for (int p0 = p_begin + rq; p0 < p_end; p0 += 16 * 8) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {                         // unconditional loads at clamped rows
            const int p = min(p0 + 16 * u, p_end - 1);
            v[u] = *reinterpret_cast<const float4 *>(parts + int64_t(p) * n + colc);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (p0 + 16 * u < p_end) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
        }
    }
    red[rq][c4] = acc;
    __syncthreads();
    if (rq == 0 && on) {
        float4 s = red[0][c4];
#pragma unroll
        for (int r = 1; r < 16; ++r) {
            const float4 q = red[r][c4];
            s.x += q.x; s.y += q.y; s.z += q.z; s.w += q.w;
        }
        *reinterpret_cast<float4 *>(out + int64_t(blockIdx.y) * n + col) = s;
    }
}

}  // namespace

// Scratch of lffn_layer_norm_bwd_noalloc_f32: the per-workgroup partial sums of the weight and bias
// gradients, [2][num_partials][H] with num_partials <= LN_NOALLOC_PARTIALS and H <= 256 * NJ_MAX.  Held
// by every GPU the library runs on until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress, never a device address.
constexpr int LN_NOALLOC_PARTIALS = 512;
constexpr size_t LN_NOALLOC_FLOATS = size_t(2) * LN_NOALLOC_PARTIALS * 256 * NJ_MAX;      // 4 MiB
static __device__ __align__(256) float ln_noalloc_scratch[LN_NOALLOC_FLOATS];

// The device address of ln_noalloc_scratch on the current device, looked up once per device (each GPU
// holds its own copy of the array at its own address).  Null when the lookup fails.
static float *ln_noalloc_scratch_ptr() {
    static std::atomic<float *> known[LFFN_MAX_DEVICES];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LFFN_MAX_DEVICES) {
        (void)hipGetLastError();
        return nullptr;
    }
    float *p = known[dev].load(std::memory_order_acquire);
    if (p) return p;
    void *sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(ln_noalloc_scratch)) != hipSuccess || !sym) {
        (void)hipGetLastError();
        return nullptr;
    }
    known[dev].store(static_cast<float *>(sym), std::memory_order_release);     // two threads racing store the same address
    return static_cast<float *>(sym);
}

extern "C" int lffn_sum_partials_f32(const float *parts_a, float *out_a, int64_t n_a, const float *parts_b,
                                     float *out_b, int64_t n_b, int64_t num_partials, int64_t chunks,
                                     void *stream) {
    LFFN_REQUIRE(n_a >= 0 && n_b >= 0 && num_partials >= 1 && num_partials <= (int64_t(1) << 30), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(chunks >= 1 && chunks <= 65535 && chunks <= num_partials, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(n_a % 4 == 0 && n_b % 4 == 0 && n_a <= (int64_t(1) << 30) && n_b <= (int64_t(1) << 30),
                 LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE((n_a == 0 || (parts_a && out_a)) && (n_b == 0 || (parts_b && out_b)), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(parts_a) && lffn_aligned16(out_a) && lffn_aligned16(parts_b) && lffn_aligned16(out_b),
                 LFFN_ERR_BAD_ARG);
    if (n_a + n_b == 0) return LFFN_OK;
    SumPartialsArgs a{};
    a.pa = parts_a; a.oa = out_a; a.na = n_a; a.pb = parts_b; a.ob = out_b; a.nb = n_b; a.P = (int)num_partials;
    a.blocks_a = (int)((n_a + 63) / 64);
    a.rows_per_chunk = (int)((num_partials + chunks - 1) / chunks);
    const int blocks = a.blocks_a + (int)((n_b + 63) / 64);
    // every chunk has rows: chunks <= num_partials and rows_per_chunk = ceil, so the last chunk may be
    // short but (chunks - 1) * rows_per_chunk < num_partials must hold for it not to be empty
    LFFN_REQUIRE((chunks - 1) * (int64_t)a.rows_per_chunk < num_partials, LFFN_ERR_BAD_ARG);
    hipLaunchKernelGGL(sum_partials_kernel, dim3((unsigned)blocks, (unsigned)chunks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    return lffn_launch_status();
}

extern "C" int lffn_layer_norm_bwd_f32(const float *x, const float *ln_weight, float ln_eps, const float *g_y,
                                       float *g_x, float *part_weight, float *part_bias, int64_t B, int64_t H,
                                       int64_t R, int64_t num_partials, void *stream) {
    LFFN_REQUIRE(B >= 0 && H >= 1 && R >= 1 && ln_eps >= 0.f, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && H <= 256 * NJ_MAX && B <= (int64_t(1) << 31) - 1 && R <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(num_partials >= 1 && num_partials <= 65535, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE((part_weight != nullptr) == (part_bias != nullptr), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE((x && g_y && g_x) || B == 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(g_y) && lffn_aligned16(g_x) &&
                     (!ln_weight || lffn_aligned16(ln_weight)), LFFN_ERR_BAD_ARG);
    LnBwdArgs a{};
    a.x = x; a.w = ln_weight; a.gy = g_y; a.gx = g_x; a.part_w = part_weight; a.part_b = part_bias;
    a.B = B; a.H = (int)H; a.R = (int)R; a.eps = ln_eps;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)num_partials);       // every workgroup writes its partial, rows or not
    if (H <= 256) hipLaunchKernelGGL((layer_norm_bwd_kernel<1>), grid, dim3(256), 0, st, a);
    else if (H <= 512) hipLaunchKernelGGL((layer_norm_bwd_kernel<2>), grid, dim3(256), 0, st, a);
    else if (H <= 768) hipLaunchKernelGGL((layer_norm_bwd_kernel<3>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((layer_norm_bwd_kernel<4>), grid, dim3(256), 0, st, a);
    return lffn_launch_status();
}

extern "C" int lffn_layer_norm_bwd_noalloc_f32(const float *x, const float *ln_weight, float ln_eps, const float *g_y,
                                               float *g_x, float *g_weight, float *g_bias, int64_t B, int64_t H,
                                               int64_t R, void *stream) {
    LFFN_REQUIRE(B >= 0 && H >= 1, LFFN_ERR_BAD_ARG);
    // the array is sized for rows of up to 256 * NJ_MAX columns, whatever the number of rows
    LFFN_REQUIRE(H <= 256 * NJ_MAX, LFFN_ERR_SCRATCH);
    // as many partials as workgroups that have a row, at most LN_NOALLOC_PARTIALS
    const int64_t want = (B + 3) / 4;
    const int64_t num_partials = want < 1 ? 1 : (want > LN_NOALLOC_PARTIALS ? LN_NOALLOC_PARTIALS : want);
    LFFN_REQUIRE(size_t(2) * size_t(num_partials) * size_t(H) <= LN_NOALLOC_FLOATS, LFFN_ERR_SCRATCH);
    LFFN_REQUIRE(g_weight && g_bias && lffn_aligned16(g_weight) && lffn_aligned16(g_bias), LFFN_ERR_BAD_ARG);
    float *scratch = ln_noalloc_scratch_ptr();
    LFFN_REQUIRE(scratch, LFFN_ERR_LAUNCH);
    float *part_w = scratch, *part_b = scratch + num_partials * H;
    // every one of the num_partials workgroups writes its row of both arrays, so nothing of the last
    // call's contents is read and nothing needs clearing
    const int rc = lffn_layer_norm_bwd_f32(x, ln_weight, ln_eps, g_y, g_x, part_w, part_b, B, H, R, num_partials, stream);
    if (rc != LFFN_OK) return rc;
    return lffn_sum_partials_f32(part_w, g_weight, H, part_b, g_bias, H, num_partials, 1, stream);
}
