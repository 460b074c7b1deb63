// Weighted gather-add and its backward for gfx950, token-major form.
//
//   gather_add              out[b,:]  = sum_i w[b,i] * src[idx[b,i],:]
//   indexed_inner_product   out[b,i]  = <g[b,:], src[idx[b,i],:]>
//   scatter_add             out[idx[b,i],:] += w[b,i] * g[b,:]
//
// A token is owned by a group of LPT lanes (64, 32, 16 or 8, the largest that
// divides the row's 16-byte vectors); lane l of the group owns vectors
// l, l+LPT, ... of a column chunk of LPT*NV vectors (blockIdx.y selects the
// chunk).  Every row access is a 16-byte load per lane, LPT lanes side by side:
// whole 128-byte lines.  The (index, weight) pairs of a block's tokens are staged
// in LDS 64 at a time; the row loop is unrolled so that eight rows' loads are in
// flight per lane before the first is consumed.  Accumulation is fp32, index
// ascending: the order of the reference loop (gather_kernel_fp32.cu:41-43).
//
// All blocks walk the index dimension from 0 upwards at the same pace, so when
// the indices are per-table (idx[b,t] in table t, as LookupFFN issues them) the
// rows in use at any moment belong to a few tables and stay in the L2 of each XCD.
#include "lffn_common.h"

#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

namespace {

constexpr int IC = 64;      // (index, weight) pairs staged per token per pass
constexpr int UNROLL = 8;   // rows in flight per lane group

// FMT: the row format, LFFN_ROWS_F32 (0), LFFN_ROWS_BF16 (1) or LFFN_ROWS_F16 (2)
template <int FMT>
struct Row {
    static constexpr int EPV = FMT != LFFN_ROWS_F32 ? 8 : 4;   // elements per 16-byte vector
    static constexpr int ESZ = FMT != LFFN_ROWS_F32 ? 2 : 4;
};

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

template <int FMT>
__device__ __forceinline__ void axpy_vec(float (&acc)[Row<FMT>::EPV], const uint4 &r, float w) {
    if constexpr (FMT == LFFN_ROWS_F16) {
        // (float)half * float + float: one v_fma_mix_f32 per value
        const unsigned q[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half2_t h = __builtin_bit_cast(half2_t, q[i]);
            acc[2 * i] = fmaf((float)h.x, w, acc[2 * i]);
            acc[2 * i + 1] = fmaf((float)h.y, w, acc[2 * i + 1]);
        }
    } else if constexpr (FMT == LFFN_ROWS_BF16) {
        acc[0] = fmaf(bf16_lo(r.x), w, acc[0]);
        acc[1] = fmaf(bf16_hi(r.x), w, acc[1]);
        acc[2] = fmaf(bf16_lo(r.y), w, acc[2]);
        acc[3] = fmaf(bf16_hi(r.y), w, acc[3]);
        acc[4] = fmaf(bf16_lo(r.z), w, acc[4]);
        acc[5] = fmaf(bf16_hi(r.z), w, acc[5]);
        acc[6] = fmaf(bf16_lo(r.w), w, acc[6]);
        acc[7] = fmaf(bf16_hi(r.w), w, acc[7]);
    } else {
        acc[0] = fmaf(__uint_as_float(r.x), w, acc[0]);
        acc[1] = fmaf(__uint_as_float(r.y), w, acc[1]);
        acc[2] = fmaf(__uint_as_float(r.z), w, acc[2]);
        acc[3] = fmaf(__uint_as_float(r.w), w, acc[3]);
    }
}

// d + <g, r> over one 16-byte vector, element ascending; g has the rows' format
template <int FMT>
__device__ __forceinline__ float dot_vec(const uint4 &gq, const uint4 &r, float d) {
    if constexpr (FMT == LFFN_ROWS_F16) {
        // (float)half * (float)half + float: one v_fma_mix_f32 per value, the product exact
        const unsigned a[4] = {gq.x, gq.y, gq.z, gq.w}, b[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half2_t ha = __builtin_bit_cast(half2_t, a[i]), hb = __builtin_bit_cast(half2_t, b[i]);
            d = fmaf((float)ha.x, (float)hb.x, d);
            d = fmaf((float)ha.y, (float)hb.y, d);
        }
    } else if constexpr (FMT == LFFN_ROWS_BF16) {
        d = fmaf(bf16_lo(gq.x), bf16_lo(r.x), d); d = fmaf(bf16_hi(gq.x), bf16_hi(r.x), d);
        d = fmaf(bf16_lo(gq.y), bf16_lo(r.y), d); d = fmaf(bf16_hi(gq.y), bf16_hi(r.y), d);
        d = fmaf(bf16_lo(gq.z), bf16_lo(r.z), d); d = fmaf(bf16_hi(gq.z), bf16_hi(r.z), d);
        d = fmaf(bf16_lo(gq.w), bf16_lo(r.w), d); d = fmaf(bf16_hi(gq.w), bf16_hi(r.w), d);
    } else {
        d = fmaf(__uint_as_float(gq.x), __uint_as_float(r.x), d);
        d = fmaf(__uint_as_float(gq.y), __uint_as_float(r.y), d);
        d = fmaf(__uint_as_float(gq.z), __uint_as_float(r.z), d);
        d = fmaf(__uint_as_float(gq.w), __uint_as_float(r.w), d);
    }
    return d;
}

// the EPV values of one 16-byte vector as fp32
template <int FMT>
__device__ __forceinline__ void widen_vec(float (&v)[Row<FMT>::EPV], const uint4 &r) {
    if constexpr (FMT == LFFN_ROWS_F16) {
        const unsigned q[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half2_t h = __builtin_bit_cast(half2_t, q[i]);
            v[2 * i] = (float)h.x;
            v[2 * i + 1] = (float)h.y;
        }
    } else if constexpr (FMT == LFFN_ROWS_BF16) {
        v[0] = bf16_lo(r.x); v[1] = bf16_hi(r.x); v[2] = bf16_lo(r.y); v[3] = bf16_hi(r.y);
        v[4] = bf16_lo(r.z); v[5] = bf16_hi(r.z); v[6] = bf16_lo(r.w); v[7] = bf16_hi(r.w);
    } else {
        v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y);
        v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
    }
}

struct GatherArgs {
    const int32_t *idx;   // [B, I]  (codes when structured)
    const void *src;      // [source_size, Dv]
    const float *w;       // [B, I]
    const void *g;        // [B, Dv]   (backward kernels; fp32, or the rows' 16-bit format in the 16-bit forms)
    const float *bias;    // [Dv] or null (structured forward)
    const float *residual;// [B, Dv] or null (structured forward): added to the result
    float *out;
    int64_t B;
    int I;
    int64_t source_size;  // rows of src / out
    int Dv;
    int S;                // structured: table size (power of two); 0 = flat indices
};

// Stage the block's (index, weight) pairs [i0, i0+IC) in LDS, resolving the row
// number: flat indices are clamped into [0, source_size); codes are masked into
// their table and offset by i*S (PL/lookup.py:126).
template <int TPB, bool WITH_W>
__device__ __forceinline__ void stage_pairs(const GatherArgs &a, int64_t tok0, int i0,
                                            int (*s_row)[IC], float (*s_w)[IC]) {
    for (int e = threadIdx.x; e < TPB * IC; e += 256) {
        const int tl = e / IC, ii = e % IC;
        const int64_t tok = tok0 + tl;
        const int i = i0 + ii;
        int row = 0;
        float wt = 0.f;
        if (tok < a.B && i < a.I) {
            const int raw = a.idx[tok * a.I + i];
            if (a.S > 0) {
                row = (raw & (a.S - 1)) + i * a.S;
            } else {
                const int64_t hi = a.source_size - 1;
                row = (int)(raw < 0 ? 0 : (raw > hi ? hi : raw));
            }
            if constexpr (WITH_W) wt = a.w[tok * a.I + i];
        }
        s_row[tl][ii] = row;
        if constexpr (WITH_W) s_w[tl][ii] = wt;
    }
}

template <int FMT, int LPT, int NV>
__global__ __launch_bounds__(256) void gather_add_kernel(GatherArgs a) {
    constexpr int TPB = 256 / LPT;
    constexpr int EPV = Row<FMT>::EPV;
    __shared__ int s_row[TPB][IC];
    __shared__ float s_w[TPB][IC];

    const int tl = threadIdx.x / LPT;
    const int ll = threadIdx.x % LPT;
    const int64_t tok0 = int64_t(blockIdx.x) * TPB;
    const int64_t tok = tok0 + tl;
    const int vec0 = blockIdx.y * (LPT * NV) + ll;            // first 16-byte vector of this lane
    const size_t row_bytes = size_t(a.Dv) * Row<FMT>::ESZ;
    const char *base = static_cast<const char *>(a.src) + size_t(vec0) * 16;

    float acc[NV][EPV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        if (a.bias) {
#pragma unroll
            for (int q = 0; q < EPV / 4; ++q) {
                const float4 bb = *reinterpret_cast<const float4 *>(a.bias + (size_t)(vec0 + v * LPT) * EPV + 4 * q);
                acc[v][4 * q + 0] = bb.x; acc[v][4 * q + 1] = bb.y;
                acc[v][4 * q + 2] = bb.z; acc[v][4 * q + 3] = bb.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[v][e] = 0.f;
        }
    }

    for (int i0 = 0; i0 < a.I; i0 += IC) {
        __syncthreads();
        stage_pairs<TPB, true>(a, tok0, i0, s_row, s_w);
        __syncthreads();
        const int n = min(IC, a.I - i0);
        int ii = 0;
        for (; ii + UNROLL <= n; ii += UNROLL) {
            uint4 r[UNROLL][NV];
            float wt[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                int row = s_row[tl][ii + u];
                wt[u] = s_w[tl][ii + u];
                if constexpr (LPT == 64) {   // one token per wavefront: the row address is uniform
                    row = __builtin_amdgcn_readfirstlane(row);
                    wt[u] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(wt[u])));
                }
                const uint4 *p = reinterpret_cast<const uint4 *>(base + size_t(row) * row_bytes);
#pragma unroll
                for (int v = 0; v < NV; ++v) r[u][v] = p[v * LPT];
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                for (int v = 0; v < NV; ++v) axpy_vec<FMT>(acc[v], r[u][v], wt[u]);
        }
        for (; ii < n; ++ii) {
            const int row = s_row[tl][ii];
            const float wt = s_w[tl][ii];
            const uint4 *p = reinterpret_cast<const uint4 *>(base + size_t(row) * row_bytes);
#pragma unroll
            for (int v = 0; v < NV; ++v) axpy_vec<FMT>(acc[v], p[v * LPT], wt);
        }
    }

    if (tok < a.B) {
        float *o = a.out + tok * a.Dv;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int q = 0; q < EPV / 4; ++q) {
                const size_t c0 = (size_t)(vec0 + v * LPT) * EPV + 4 * q;
                float4 r4 = make_float4(acc[v][4 * q + 0], acc[v][4 * q + 1], acc[v][4 * q + 2], acc[v][4 * q + 3]);
                if (a.residual) {
                    const float4 rr = *reinterpret_cast<const float4 *>(a.residual + tok * a.Dv + c0);
                    r4.x += rr.x; r4.y += rr.y; r4.z += rr.z; r4.w += rr.w;
                }
                *reinterpret_cast<float4 *>(o + c0) = r4;
            }
    }
}

// Sum over the LPT lanes of a token group (LPT a power of two, groups aligned).
template <int LPT>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LPT > 1) v += lane_xor<1>(v);
    if constexpr (LPT > 2) v += lane_xor<2>(v);
    if constexpr (LPT > 4) v += lane_xor<4>(v);
    if constexpr (LPT > 8) v += lane_xor<8>(v);
    if constexpr (LPT > 16) v += lane_xor<16>(v);
    if constexpr (LPT > 32) v += lane_xor<32>(v);
    return v;
}

// out[b,i] = <g[b,:], src[idx[b,i],:]>.  Column chunks are walked inside the
// block; the per-chunk partial dot products are summed in LDS in chunk order.
// 16-bit forms: g and the rows in the same 16-bit format, products and sums in fp32.
template <int FMT, int LPT, int NV>
__global__ __launch_bounds__(256) void inner_product_kernel(GatherArgs a, int chunks) {
    constexpr int TPB = 256 / LPT;
    __shared__ int s_row[TPB][IC];
    __shared__ float s_dot[TPB][IC];

    const int tl = threadIdx.x / LPT;
    const int ll = threadIdx.x % LPT;
    const int64_t tok0 = int64_t(blockIdx.x) * TPB;
    const int64_t tok = tok0 + tl;
    const size_t row_bytes = size_t(a.Dv) * Row<FMT>::ESZ;
    const char *grow = static_cast<const char *>(a.g) + size_t(tok) * row_bytes;

    for (int i0 = 0; i0 < a.I; i0 += IC) {
        __syncthreads();
        stage_pairs<TPB, false>(a, tok0, i0, s_row, s_dot);
        for (int e = threadIdx.x; e < TPB * IC; e += 256) s_dot[e / IC][e % IC] = 0.f;
        __syncthreads();
        const int n = min(IC, a.I - i0);
        for (int ch = 0; ch < chunks; ++ch) {
            const int vec0 = ch * (LPT * NV) + ll;
            uint4 gv[NV];
#pragma unroll
            for (int v = 0; v < NV; ++v)
                gv[v] = tok < a.B ? *reinterpret_cast<const uint4 *>(grow + (size_t)(vec0 + v * LPT) * 16)
                                  : make_uint4(0u, 0u, 0u, 0u);
            const char *base = static_cast<const char *>(a.src) + size_t(vec0) * 16;
            int ii = 0;
            for (; ii + 4 <= n; ii += 4) {
                uint4 r[4][NV];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint4 *p = reinterpret_cast<const uint4 *>(base + size_t(s_row[tl][ii + u]) * row_bytes);
#pragma unroll
                    for (int v = 0; v < NV; ++v) r[u][v] = p[v * LPT];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    float d = 0.f;
#pragma unroll
                    for (int v = 0; v < NV; ++v) d = dot_vec<FMT>(gv[v], r[u][v], d);
                    d = group_sum<LPT>(d);
                    if (ll == 0) s_dot[tl][ii + u] += d;
                }
            }
            for (; ii < n; ++ii) {
                const uint4 *p = reinterpret_cast<const uint4 *>(base + size_t(s_row[tl][ii]) * row_bytes);
                float d = 0.f;
#pragma unroll
                for (int v = 0; v < NV; ++v) d = dot_vec<FMT>(gv[v], p[v * LPT], d);
                d = group_sum<LPT>(d);
                if (ll == 0) s_dot[tl][ii] += d;
            }
        }
        __syncthreads();
        for (int e = threadIdx.x; e < TPB * IC; e += 256) {
            const int t2 = e / IC, ii2 = e % IC;
            if (tok0 + t2 < a.B && i0 + ii2 < a.I) a.out[(tok0 + t2) * a.I + i0 + ii2] = s_dot[t2][ii2];
        }
    }
}

// out[idx[b,i],:] += w[b,i] * g[b,:] with hardware fp32 atomics.  16-bit forms: g in the
// 16-bit format, widened once; the products and the sums (out) are fp32.
template <int FMT, int LPT, int NV>
__global__ __launch_bounds__(256) void scatter_add_kernel(GatherArgs a) {
    constexpr int TPB = 256 / LPT;
    constexpr int EPV = Row<FMT>::EPV;
    __shared__ int s_row[TPB][IC];
    __shared__ float s_w[TPB][IC];

    const int tl = threadIdx.x / LPT;
    const int ll = threadIdx.x % LPT;
    const int64_t tok0 = int64_t(blockIdx.x) * TPB;
    const int64_t tok = tok0 + tl;
    const int vec0 = blockIdx.y * (LPT * NV) + ll;

    float gv[NV][EPV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        uint4 q = make_uint4(0u, 0u, 0u, 0u);
        if (tok < a.B)
            q = *reinterpret_cast<const uint4 *>(static_cast<const char *>(a.g) + size_t(tok) * a.Dv * Row<FMT>::ESZ +
                                                 (size_t)(vec0 + v * LPT) * 16);
        widen_vec<FMT>(gv[v], q);
    }

    for (int i0 = 0; i0 < a.I; i0 += IC) {
        __syncthreads();
        stage_pairs<TPB, true>(a, tok0, i0, s_row, s_w);
        __syncthreads();
        if (tok >= a.B) continue;
        const int n = min(IC, a.I - i0);
        for (int ii = 0; ii < n; ++ii) {
            const float wt = s_w[tl][ii];
            float *o = a.out + size_t(s_row[tl][ii]) * a.Dv + size_t(vec0) * EPV;
#pragma unroll
            for (int v = 0; v < NV; ++v)
#pragma unroll
                for (int e = 0; e < EPV; ++e) unsafeAtomicAdd(o + v * LPT * EPV + e, wt * gv[v][e]);
        }
    }
}

// Split a row of `nvec` 16-byte vectors into lanes-per-token, vectors per lane and
// column chunks.  nvec is a multiple of 8 (bf16) or 16 (f32) by the Dv % 64 rule.
struct Tiling {
    int lpt, nv, chunks;
};

Tiling pick_tiling(int nvec) {
    Tiling t{};
    t.lpt = (nvec % 64 == 0) ? 64 : (nvec % 32 == 0) ? 32 : (nvec % 16 == 0) ? 16 : 8;
    const int m = nvec / t.lpt;
    t.nv = (m % 4 == 0) ? 4 : (m % 3 == 0) ? 3 : (m % 2 == 0) ? 2 : 1;
    t.chunks = m / t.nv;
    return t;
}

enum class Op { Gather, Inner, Scatter };

template <int FMT, Op OP, int LPT, int NV>
void launch_one(const GatherArgs &a, const Tiling &t, hipStream_t s) {
    constexpr int TPB = 256 / LPT;
    const unsigned gx = (unsigned)((a.B + TPB - 1) / TPB);
    if constexpr (OP == Op::Gather)
        hipLaunchKernelGGL((gather_add_kernel<FMT, LPT, NV>), dim3(gx, t.chunks), dim3(256), 0, s, a);
    else if constexpr (OP == Op::Inner)
        hipLaunchKernelGGL((inner_product_kernel<FMT, LPT, NV>), dim3(gx), dim3(256), 0, s, a, t.chunks);
    else
        hipLaunchKernelGGL((scatter_add_kernel<FMT, LPT, NV>), dim3(gx, t.chunks), dim3(256), 0, s, a);
}

template <int FMT, Op OP, int LPT>
void launch_nv(const GatherArgs &a, const Tiling &t, hipStream_t s) {
    switch (t.nv) {
        case 1: launch_one<FMT, OP, LPT, 1>(a, t, s); break;
        case 2: launch_one<FMT, OP, LPT, 2>(a, t, s); break;
        case 3: launch_one<FMT, OP, LPT, 3>(a, t, s); break;
        default: launch_one<FMT, OP, LPT, 4>(a, t, s); break;
    }
}

template <int FMT, Op OP>
int launch(const GatherArgs &a, hipStream_t s) {
    if (a.B == 0 || (a.I == 0 && OP != Op::Gather)) return LFFN_OK;
    const Tiling t = pick_tiling(a.Dv / Row<FMT>::EPV);
    switch (t.lpt) {
        case 64: launch_nv<FMT, OP, 64>(a, t, s); break;
        case 32: launch_nv<FMT, OP, 32>(a, t, s); break;
        case 16: launch_nv<FMT, OP, 16>(a, t, s); break;
        default:
            if constexpr (FMT != LFFN_ROWS_F32) { launch_nv<FMT, OP, 8>(a, t, s); break; }
            else return LFFN_ERR_UNSUPPORTED;
    }
    return lffn_launch_status();
}

int check_common(const void *idx, int64_t B, int64_t I, int64_t rows, int64_t Dv) {
    LFFN_REQUIRE(B >= 0 && I >= 0 && rows >= 1 && Dv >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(idx || B * I == 0, LFFN_ERR_BAD_ARG);   // an empty index array may be null
    LFFN_REQUIRE(Dv % 64 == 0, LFFN_ERR_UNSUPPORTED);            // PL/gather/cuda/kernel.py:43
    LFFN_REQUIRE(Dv <= (1 << 20) && I <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(rows <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);      // int32 indices
    LFFN_REQUIRE(B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    return LFFN_OK;
}

template <int FMT>
int gather_entry(const int32_t *idx, const void *src, const float *w, const float *bias, const float *residual,
                 float *out,
                 int64_t B, int64_t I, int64_t rows, int64_t Dv, int64_t S, void *stream) {
    int rc = check_common(idx, B, I, rows, Dv);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(src && out && (w || B * I == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(src) && lffn_aligned16(out) && (!bias || lffn_aligned16(bias)), LFFN_ERR_BAD_ARG);
    GatherArgs a{};
    a.idx = idx; a.src = src; a.w = w; a.g = nullptr; a.bias = bias; a.residual = residual; a.out = out;
    a.B = B; a.I = (int)I; a.source_size = rows; a.Dv = (int)Dv; a.S = (int)S;
    return launch<FMT, Op::Gather>(a, static_cast<hipStream_t>(stream));
}

}  // namespace

extern "C" int lffn_gather_add_f32(const int32_t *idx, const float *src, const float *w, float *out,
                                   int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream) {
    return gather_entry<LFFN_ROWS_F32>(idx, src, w, nullptr, nullptr, out, B, I, source_size, Dv, 0, stream);
}

extern "C" int lffn_gather_add_bf16(const int32_t *idx, const uint16_t *src, const float *w, float *out,
                                    int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream) {
    return gather_entry<LFFN_ROWS_BF16>(idx, src, w, nullptr, nullptr, out, B, I, source_size, Dv, 0, stream);
}

extern "C" int lffn_gather_add_f16(const int32_t *idx, const uint16_t *src, const float *w, float *out,
                                   int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream) {
    return gather_entry<LFFN_ROWS_F16>(idx, src, w, nullptr, nullptr, out, B, I, source_size, Dv, 0, stream);
}

// Token-major kernel on table-local codes (offset i*S and bias folded in): the
// form lookup_gather.hip falls back to for shapes its LDS-tiled kernel is not
// built for.
int lffn_internal_lookup_gather_token_major(const int32_t *code, const float *score, const void *tables,
                                            const float *bias, const float *residual, float *out, int64_t B,
                                            int64_t T, int64_t S, int64_t Do, int fmt, void *stream) {
    const int64_t rows = T * S > 0 ? T * S : 1;
    if (fmt == LFFN_ROWS_F16) return gather_entry<LFFN_ROWS_F16>(code, tables, score, bias, residual, out, B, T, rows, Do, S, stream);
    return fmt == LFFN_ROWS_BF16 ? gather_entry<LFFN_ROWS_BF16>(code, tables, score, bias, residual, out, B, T, rows, Do, S, stream)
                                 : gather_entry<LFFN_ROWS_F32>(code, tables, score, bias, residual, out, B, T, rows, Do, S, stream);
}

// Atomic scatter-add on table-local codes (row = code & (S-1) + t*S), into a buffer
// the caller has zeroed or wants accumulated into: the fallback of lookup_scatter.hip.
int lffn_internal_lookup_scatter_atomic(const int32_t *code, const float *score, const float *g, float *out,
                                        int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    GatherArgs a{};
    a.idx = code; a.src = nullptr; a.w = score; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)T; a.source_size = T * S; a.Dv = (int)Do; a.S = (int)S;
    return launch<LFFN_ROWS_F32, Op::Scatter>(a, static_cast<hipStream_t>(stream));
}

// Token-major inner product on table-local codes: the fallback of lookup_inner.hip.
int lffn_internal_lookup_inner_token_major(const int32_t *code, const float *g, const float *tables,
                                           float *out, int64_t B, int64_t T, int64_t S, int64_t Do,
                                           void *stream) {
    GatherArgs a{};
    a.idx = code; a.src = tables; a.w = nullptr; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)T; a.source_size = T * S; a.Dv = (int)Do; a.S = (int)S;
    return launch<LFFN_ROWS_F32, Op::Inner>(a, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_indexed_inner_product_f32(const int32_t *idx, const float *g, const float *src, float *out,
                                              int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream) {
    int rc = check_common(idx, B, I, source_size, Dv);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(g && src && (out || B * I == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(src) && lffn_aligned16(g), LFFN_ERR_BAD_ARG);
    GatherArgs a{};
    a.idx = idx; a.src = src; a.w = nullptr; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)I; a.source_size = source_size; a.Dv = (int)Dv; a.S = 0;
    return launch<LFFN_ROWS_F32, Op::Inner>(a, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_scatter_add_f32(const int32_t *idx, const float *g, const float *w, float *out,
                                    int64_t B, int64_t I, int64_t out_size, int64_t Dv, void *stream) {
    int rc = check_common(idx, B, I, out_size, Dv);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(g && out && (w || B * I == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(g) && lffn_aligned16(out), LFFN_ERR_BAD_ARG);
    GatherArgs a{};
    a.idx = idx; a.src = nullptr; a.w = w; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)I; a.source_size = out_size; a.Dv = (int)Dv; a.S = 0;
    return launch<LFFN_ROWS_F32, Op::Scatter>(a, static_cast<hipStream_t>(stream));
}

// The reduced-precision calls of the backward: g and the rows are half, the results fp32.
extern "C" int lffn_indexed_inner_product_f16(const int32_t *idx, const uint16_t *g, const uint16_t *src, float *out,
                                              int64_t B, int64_t I, int64_t source_size, int64_t Dv, void *stream) {
    int rc = check_common(idx, B, I, source_size, Dv);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(g && src && (out || B * I == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(src) && lffn_aligned16(g), LFFN_ERR_BAD_ARG);
    GatherArgs a{};
    a.idx = idx; a.src = src; a.w = nullptr; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)I; a.source_size = source_size; a.Dv = (int)Dv; a.S = 0;
    return launch<LFFN_ROWS_F16, Op::Inner>(a, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_scatter_add_f16(const int32_t *idx, const uint16_t *g, const float *w, float *out,
                                    int64_t B, int64_t I, int64_t out_size, int64_t Dv, void *stream) {
    int rc = check_common(idx, B, I, out_size, Dv);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(g && out && (w || B * I == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(g) && lffn_aligned16(out), LFFN_ERR_BAD_ARG);
    GatherArgs a{};
    a.idx = idx; a.src = nullptr; a.w = w; a.g = g; a.bias = nullptr; a.out = out;
    a.B = B; a.I = (int)I; a.source_size = out_size; a.Dv = (int)Dv; a.S = 0;
    return launch<LFFN_ROWS_F16, Op::Scatter>(a, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_version(void) { return LFFN_ABI_VERSION; }

extern "C" const char *lffn_error_string(int code) {
    switch (code) {
        case LFFN_OK: return "ok";
        case LFFN_ERR_BAD_ARG: return "bad argument (null or misaligned pointer, negative or inconsistent size)";
        case LFFN_ERR_UNSUPPORTED: return "shape not supported by the gfx950 kernels";
        case LFFN_ERR_LAUNCH: return "kernel launch failed";
        case LFFN_ERR_SCRATCH: return "the shape needs more scratch memory than the library's static buffer holds";
        default: return "unknown error code";
    }
}
