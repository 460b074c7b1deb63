// Projection kernels of the LookupFFN layer for gfx950: fast Hadamard transform,
// BH4 mixing with block size 1 (diagonal scale + transform, repeated), and the
// fused projection -> mix -> bias -> 8-bit code + score front-end.
//
// One row (or, for D < 256, 256/D rows) lives in the registers of one 64-lane
// wavefront for the whole computation: nothing round-trips through memory between
// the transforms.  The forward kernel's 512- and 1024-point transforms turn the row
// round through the wavefront's own 4 KB of LDS twice per transform, so that the
// upper lane bits become register bits for a while (fht_rows_xl below: 16 % faster
// than six cross-lane stages at D = 1024); everything else stays in registers.
//
// Register layout.  A lane holds NJ float4; value c of float4 j of row-lane lr is
// element  e = 256*j + 4*lr + c.  So bits 0-1 of e are in-register (c), bits 2..
// are the lane, and bits 8-9 are in-register again (j).  Every global access is a
// fully coalesced 16-byte-per-lane access.  A butterfly over an in-register bit is
// two plain adds; over a lane bit it is one cross-lane move (DPP for lane xor
// 1,2,4,8; ds_swizzle for 16; ds_bpermute for 32) plus one fma with +-1.
//
// Stage order is stride D/2 first, stride 1 last, each stage a single rounded
// add/subtract: the same operations in the same order as the reference kernel
// (fast_hadamard_transform/extension/cuda_kernel.cu:235-251), so results agree
// bit for bit with a scalar butterfly in that order.
#include "lffn_common.h"

#include <type_traits>

// Keep mul and add separate where the reference computes them separately (the
// diagonal scale, the decay/residual mix): explicit fmaf calls below stay fused.
#pragma clang fp contract(off)

namespace {

template <int LOGD>
struct FhtCfg {
    static constexpr int D = 1 << LOGD;
    static constexpr int LPR = D >= 256 ? 64 : D / 4;   // lanes per row
    static constexpr int NJ = D >= 256 ? D / 256 : 1;   // float4 per lane
    static constexpr int RPW = 64 / LPR;                // rows per wavefront
    static_assert(LOGD >= 2 && LOGD <= 10, "FHT dims 4..1024");
};

// Butterflies across lanes 16 or 32 apart, two values at a time, with the gfx950 row / half-wave
// swaps: swap(a, b) hands every lane one of the two values together with that value's partner,
// so a plain add and subtract give both results, and a second swap puts them back in place.
// Four vector-ALU instructions per pair of values, no LDS permute and no sign multiply; the
// sums are the same additions as in the one-value form (a + b and a - b are commutative up to
// the sign of b), so results are unchanged bit for bit.
template <int M>
__device__ __forceinline__ void butterfly_swap_pair(float &e0, float &e1) {
    static_assert(M == 16 || M == 32, "swap butterflies: rows (16) or half-waves (32)");
    unsigned a = __float_as_uint(e0), b = __float_as_uint(e1);
    if constexpr (M == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
        a = r[0]; b = r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
        a = r[0]; b = r[1];
    }
    const float s = __uint_as_float(a) + __uint_as_float(b);
    const float d = __uint_as_float(a) - __uint_as_float(b);
    unsigned su = __float_as_uint(s), du = __float_as_uint(d);
    if constexpr (M == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(su, du, false, false);
        su = r[0]; du = r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane16_swap(su, du, false, false);
        su = r[0]; du = r[1];
    }
    e0 = __uint_as_float(su);
    e1 = __uint_as_float(du);
}

// SWAP: lane distances 16 and 32 with the swap butterflies instead of LDS permutes.  The swaps
// cost more vector-ALU time than a permute plus a multiply-add: the forward kernels, which run
// many wavefronts per SIMD and are bound by ALU issue, are faster with the permutes (59 against
// 66 us at 16384 x 1024, four stages); the backward kernel, two wavefronts per SIMD and waiting
// on every permute, is faster with the swaps (178 -> 130 us).
template <int M, int LPR, int NJ, bool SWAP>
__device__ __forceinline__ void lane_stage(float (&v)[NJ][4], int lr) {
    if constexpr (SWAP && (M == 16 || M == 32) && M < LPR) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            butterfly_swap_pair<M>(v[j][0], v[j][1]);
            butterfly_swap_pair<M>(v[j][2], v[j][3]);
        }
    } else if constexpr (M >= 1 && M < LPR) {
        const float sgn = (lr & M) ? -1.0f : 1.0f;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) v[j][c] = butterfly_xor<M>(v[j][c], sgn);
    }
}

template <int LOGD, bool SWAP = false>
__device__ __forceinline__ void fht_rows(float (&v)[FhtCfg<LOGD>::NJ][4], int lr) {
    using C = FhtCfg<LOGD>;
    constexpr int NJ = C::NJ;
    // strides 512 and 256: across the float4s of a lane
    if constexpr (NJ == 4) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float a = v[j][c], b = v[j + 2][c];
                v[j][c] = a + b;
                v[j + 2][c] = a - b;
            }
    }
    if constexpr (NJ >= 2) {
#pragma unroll
        for (int j = 0; j < NJ; j += 2)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float a = v[j][c], b = v[j + 1][c];
                v[j][c] = a + b;
                v[j + 1][c] = a - b;
            }
    }
    // strides 4*32 .. 4*1: across lanes
    lane_stage<32, C::LPR, NJ, SWAP>(v, lr);
    lane_stage<16, C::LPR, NJ, SWAP>(v, lr);
    lane_stage<8, C::LPR, NJ, SWAP>(v, lr);
    lane_stage<4, C::LPR, NJ, SWAP>(v, lr);
    lane_stage<2, C::LPR, NJ, SWAP>(v, lr);
    lane_stage<1, C::LPR, NJ, SWAP>(v, lr);
    // strides 2 and 1: inside a float4
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        float a0 = v[j][0], a1 = v[j][1], a2 = v[j][2], a3 = v[j][3];
        float b0 = a0 + a2, b2 = a0 - a2, b1 = a1 + a3, b3 = a1 - a3;
        v[j][0] = b0 + b1;
        v[j][1] = b0 - b1;
        v[j][2] = b2 + b3;
        v[j][3] = b2 - b3;
    }
}

// The 512- and 1024-point transforms with two trips through LDS instead of cross-lane moves for the
// upper lane bits.  A lane holds NV = 4*NJ values (8 or 16).  Strides >= 256 are register pairs in the
// load layout, as in fht_rows; then the row is written to the wavefront's own LDS region and read back
// with the top log2(NV) lane bits of the element index in registers (element bits 8-KB .. 7; the lane
// is the low 8-KB bits and bits 8-9), strides 128 .. 2^(8-KB) are plain adds, the row goes back the
// same way, the remaining lane strides (lanes 2 and 1 apart at D = 1024; 4, 2, 1 at 512) are DPP
// butterflies and strides 2 and 1 are inside a float4.  Same additions in the same order as fht_rows:
// results are bit-identical.  Each block of 256 floats starts PAD floats after the one before, so that
// the 64 lanes of a transposed access fall on 64 different banks.
template <int LOGD>
struct XlCfg {
    static constexpr int NJ = FhtCfg<LOGD>::NJ, NV = 4 * NJ;
    static constexpr int KB = LOGD - 6;              // element bits 8-KB .. 7 in registers after the first trip
    static constexpr int STEP = 1 << (8 - KB);       // floats between a lane's values in the transposed layout
    static constexpr int BLOCK = 256 + STEP;         // floats from one block of 256 to the next
    static constexpr int ROW = NJ * BLOCK;           // floats per wavefront region
    static_assert(LOGD == 9 || LOGD == 10, "two-trip form: 512 and 1024 points");
};

// Between a phase in which the lanes of a wavefront store to the wavefront's own LDS region and the phase in
// which they load what other lanes stored: the hardware executes a wavefront's LDS operations in order, so
// no instruction is needed, but the compiler must not move or forward accesses across the hand-over.  A
// release/acquire pair at wavefront scope and a wave barrier say so and emit nothing.
__device__ __forceinline__ void wave_lds_handover() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int LOGD>
__device__ __forceinline__ void fht_rows_xl(float (&v)[FhtCfg<LOGD>::NJ][4], int lr, float *wl) {
    using X = XlCfg<LOGD>;
    constexpr int NJ = X::NJ, NV = X::NV, STEP = X::STEP, BLOCK = X::BLOCK;
    if constexpr (NJ == 4) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float a = v[j][c], b = v[j + 2][c];
                v[j][c] = a + b;
                v[j + 2][c] = a - b;
            }
    }
#pragma unroll
    for (int j = 0; j < NJ; j += 2)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float a = v[j][c], b = v[j + 1][c];
            v[j][c] = a + b;
            v[j + 1][c] = a - b;
        }
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        *reinterpret_cast<float4 *>(wl + BLOCK * j + 4 * lr) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
    wave_lds_handover();
    // transposed: lane = (element bits 0 .. 7-KB) | (bits 8-9) << (8-KB); value k = element bits 8-KB .. 7
    float *col = wl + BLOCK * (lr / STEP) + (lr % STEP);
    float w[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) w[k] = col[STEP * k];
#pragma unroll
    for (int bit = NV / 2; bit >= 1; bit >>= 1)
#pragma unroll
        for (int k = 0; k < NV; ++k)
            if (!(k & bit)) {
                float a = w[k], b = w[k | bit];
                w[k] = a + b;
                w[k | bit] = a - b;
            }
#pragma unroll
    for (int k = 0; k < NV; ++k) col[STEP * k] = w[k];
    wave_lds_handover();
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const float4 t = *reinterpret_cast<const float4 *>(wl + BLOCK * j + 4 * lr);
        v[j][0] = t.x; v[j][1] = t.y; v[j][2] = t.z; v[j][3] = t.w;
    }
    // lane strides STEP/8 .. 1 (element strides STEP/2 .. 4)
    if constexpr (STEP / 8 >= 4) lane_stage<4, 64, NJ, false>(v, lr);
    lane_stage<2, 64, NJ, false>(v, lr);
    lane_stage<1, 64, NJ, false>(v, lr);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        float a0 = v[j][0], a1 = v[j][1], a2 = v[j][2], a3 = v[j][3];
        float b0 = a0 + a2, b2 = a0 - a2, b1 = a1 + a3, b3 = a1 - a3;
        v[j][0] = b0 + b1;
        v[j][1] = b0 - b1;
        v[j][2] = b2 + b3;
        v[j][3] = b2 - b3;
    }
}

struct ProjectArgs {
    const float *x;       // [B, H]
    const float *diag;    // [R, J, D] or null (no scale)
    const float *ln_w;    // [H] LayerNorm weight, or null: no LayerNorm
    const float *ln_b;    // [H] LayerNorm bias (with ln_w)
    float ln_eps;
    const float *pbias;   // [out_cols] or null
    float *out;           // [B, out_stride] or null
    int32_t *codes;       // [B, T] (HASH only)
    float *scores;        // [B, T] (HASH only)
    // HASH only, instead of codes and scores: the record stream of the four-lanes-per-token gather
    // (lookup_gather_quad.hip), rec_stride records of three words per table pair: score of the pair's first
    // table, score of its second, row of the first | row of the second << 8, where a token whose index has
    // bit 1 set takes the pair's tables in the order (2k+1, 2k); a token's slot: lffn_quad_record_slot.
    // T even, 8-bit codes.
    uint32_t *records;    // [T/2][rec_stride][3] or null
    int64_t rec_stride;   // record slots per table pair: whole tiles of rec_tile tokens
    int rec_tile;         // tokens per workgroup of the gather the records are written for
    int blocks_per_xcd;   // records: workgroup b takes rows from the range of XCD b % 8 (see project_kernel)
    int64_t B;
    int H;                // valid input columns (<= D)
    int R, J;
    int out_stride;       // row stride of out
    int out_cols;         // columns of the R*D-wide result that exist (T*8 when hashing)
    int T;
    float decay, residual;
    int mix;              // 1: out = decay*y + residual*x (+ bias); 0: out = y
    int vec_in;           // x rows are 16-byte aligned and H % 4 == 0
    int vec_ln;           // and so are ln_w and ln_b: the LayerNorm parameters load as float4
    // GATHER only: the table rows the codes select are added up in the same kernel
    const float *tables;  // [T, S, Do]
    const float *obias;   // [Do] or null
    const float *gres;    // [B, Do] or null: added to the result
    float *gout;          // [B, Do]
    int S, Do;
};

constexpr int FUSED_MAX_T = 512;   // (code, score) pairs a wavefront keeps in LDS for its token
constexpr int FUSED_MAX_NC = 4;    // column passes of 256 the one-launch layer's gather keeps in flight together

// Part of the score recurrence over the four values of one float4:
// s <- s + a_c, p <- p * f_c with a_c = |z_c| and f_c = 1 + exp(-2|z_c|), c ascending.
__device__ __forceinline__ void score_chain(const float (&a)[4], const float (&f)[4], float &s, float &p) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        s = s + a[c];
        p = p * f[c];
    }
}

// The gather-add of one token inside the one-launch layer (PL/lookup.py:120-130, 108): this
// wavefront adds the rows of tables [t_lo, t_hi) that the (code, score) pairs in `mine` select,
// eight tables at a time and all NC column passes of 256 columns of those eight rows in flight
// together (the token's chain of dependent memory round trips is what a small batch waits for:
// 8 * NC row loads per round trip instead of 8); the four wavefronts' partial sums meet in LDS and
// wavefront 0 adds bias and residual and writes the row.  Loads are unconditional at clamped
// columns, so that none of them waits for another; what a clamped lane loaded is never stored.
template <int NC>
__device__ __forceinline__ void fused_gather(const ProjectArgs &a, const uint2 *mine, float4 (*part)[FUSED_MAX_NC][64],
                                             int64_t row, int col0, int t_lo, int t_hi, int wave, int lane) {
    int gc[NC];
    bool on[NC];
    float4 acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        on[c] = col0 + 256 * c + 4 * lane < a.Do;
        gc[c] = on[c] ? col0 + 256 * c + 4 * lane : 0;
        acc[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int t0 = t_lo; t0 < t_hi; t0 += 8) {
        float4 rv[8][NC];
        float sv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int tt = min(t0 + u, t_hi - 1);
            const uint2 pr = mine[tt];
            sv[u] = t0 + u < t_hi ? __uint_as_float(pr.y) : 0.f;
            const float *rowp = a.tables + ((size_t)tt * a.S + pr.x) * a.Do;
#pragma unroll
            for (int c = 0; c < NC; ++c) rv[u][c] = *reinterpret_cast<const float4 *>(rowp + gc[c]);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                acc[c].x = fmaf(sv[u], rv[u][c].x, acc[c].x);
                acc[c].y = fmaf(sv[u], rv[u][c].y, acc[c].y);
                acc[c].z = fmaf(sv[u], rv[u][c].z, acc[c].z);
                acc[c].w = fmaf(sv[u], rv[u][c].w, acc[c].w);
            }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) part[wave][c][lane] = acc[c];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (!on[c]) continue;
            float4 o = part[0][c][lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) {
                const float4 q = part[w][c][lane];
                o.x += q.x; o.y += q.y; o.z += q.z; o.w += q.w;
            }
            if (a.obias) {
                const float4 bb = *reinterpret_cast<const float4 *>(a.obias + gc[c]);
                o.x += bb.x; o.y += bb.y; o.z += bb.z; o.w += bb.w;
            }
            if (a.gres) {
                const float4 rr = *reinterpret_cast<const float4 *>(a.gres + row * a.Do + gc[c]);
                o.x += rr.x; o.y += rr.y; o.z += rr.z; o.w += rr.w;
            }
            *reinterpret_cast<float4 *>(a.gout + row * a.Do + gc[c]) = o;
        }
    }
    __syncthreads();                                         // `part` is free again
}

template <int LOGD, bool HASH, bool GATHER = false>
__global__ __launch_bounds__(256) void project_kernel(ProjectArgs a) {
    using C = FhtCfg<LOGD>;
    constexpr int D = C::D, NJ = C::NJ, LPR = C::LPR, RPW = C::RPW;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lr = lane % LPR;
    // GATHER: one token per workgroup; its four wavefronts each compute the token's codes (no
    // hand-over needed) and then share the gather, a quarter of the tables each
    // Records are written 12 bytes at a time, a token's slot next to its neighbours': a 128-byte line holds
    // about ten consecutive tokens' records of a table pair, and consecutive workgroups run on different
    // XCDs, whose L2s would each write back a sliver of every line.  So with records every XCD takes a
    // contiguous range of rows (workgroup b runs on XCD b % 8 and is that XCD's workgroup number b / 8).
    const int64_t blk = (HASH && !GATHER && a.records)
                            ? int64_t(blockIdx.x % 8) * a.blocks_per_xcd + blockIdx.x / 8 : int64_t(blockIdx.x);
    const int64_t row = GATHER ? int64_t(blockIdx.x) : (blk * 4 + wave) * RPW + lane / LPR;
    const bool live = row < a.B;
    int64_t rec_slot = 0;                  // where this row's records go within a table pair's
    if constexpr (HASH && !GATHER) {
        if (a.records && live) rec_slot = lffn_quad_record_slot(row, a.rec_tile);
    }

    float orig[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e0 = 256 * j + 4 * lr;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            if (a.vec_in) {
                if (e0 < a.H) t = *reinterpret_cast<const float4 *>(a.x + row * a.H + e0);
            } else {
                const float *p = a.x + row * a.H;
                if (e0 + 0 < a.H) t.x = p[e0 + 0];
                if (e0 + 1 < a.H) t.y = p[e0 + 1];
                if (e0 + 2 < a.H) t.z = p[e0 + 2];
                if (e0 + 3 < a.H) t.w = p[e0 + 3];
            }
        }
        orig[j][0] = t.x; orig[j][1] = t.y; orig[j][2] = t.z; orig[j][3] = t.w;
    }

    if (a.ln_w) {
        // LayerNorm over the H valid columns (biased variance, two passes, eps inside the
        // square root: torch.nn.LayerNorm, PL/lookup.py:84,99); padding columns stay zero.
        float s1 = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) s1 += orig[j][c];          // padding contributes 0
        const float mean = lane_group_sum<LPR>(s1) / float(a.H);
        float s2 = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float dlt = (256 * j + 4 * lr + c < a.H) ? orig[j][c] - mean : 0.f;
                s2 += dlt * dlt;
            }
        const float rstd = 1.0f / sqrtf(lane_group_sum<LPR>(s2) / float(a.H) + a.ln_eps);
        if (a.vec_ln) {                                       // H % 4 == 0: a float4 of weights and biases per lane
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int e0 = 256 * j + 4 * lr;
                if (e0 < a.H) {
                    const float4 lw = *reinterpret_cast<const float4 *>(a.ln_w + e0);
                    const float4 lb = *reinterpret_cast<const float4 *>(a.ln_b + e0);
                    orig[j][0] = (orig[j][0] - mean) * rstd * lw.x + lb.x;
                    orig[j][1] = (orig[j][1] - mean) * rstd * lw.y + lb.y;
                    orig[j][2] = (orig[j][2] - mean) * rstd * lw.z + lb.z;
                    orig[j][3] = (orig[j][3] - mean) * rstd * lw.w + lb.w;
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int e = 256 * j + 4 * lr + c;
                    if (e < a.H) orig[j][c] = (orig[j][c] - mean) * rstd * a.ln_w[e] + a.ln_b[e];
                }
        }
    }

    for (int r = 0; r < a.R; ++r) {
        float v[NJ][4];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) v[j][c] = orig[j][c];

        for (int s = 0; s < a.J; ++s) {
            if (a.diag) {
                const float *dg = a.diag + (int64_t(r) * a.J + s) * D;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const float4 w = *reinterpret_cast<const float4 *>(dg + 256 * j + 4 * lr);
                    v[j][0] = v[j][0] * w.x;
                    v[j][1] = v[j][1] * w.y;
                    v[j][2] = v[j][2] * w.z;
                    v[j][3] = v[j][3] * w.w;
                }
            }
            if constexpr ((LOGD == 10 || LOGD == 9) && !GATHER) {
                __shared__ float xl[4 * XlCfg<LOGD>::ROW];
                fht_rows_xl<LOGD>(v, lr, xl + wave * XlCfg<LOGD>::ROW);
            } else {
                fht_rows<LOGD>(v, lr);
            }
        }

#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int e0 = 256 * j + 4 * lr;
            const int col = r * D + e0;            // column in the R*D-wide result
            const bool in_cols = col < a.out_cols; // out_cols % 4 == 0: all four or none
            float z[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) z[c] = v[j][c];
            if (a.mix) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float m0 = a.decay * z[c];
                    const float m1 = a.residual * orig[j][c];
                    z[c] = m0 + m1;
                }
                if (a.pbias && in_cols) {
                    const float4 bb = *reinterpret_cast<const float4 *>(a.pbias + col);
                    z[0] = z[0] + bb.x; z[1] = z[1] + bb.y; z[2] = z[2] + bb.z; z[3] = z[3] + bb.w;
                }
            }
            if (a.out && live && in_cols)
                *reinterpret_cast<float4 *>(a.out + row * a.out_stride + col) =
                    make_float4(z[0], z[1], z[2], z[3]);

            if constexpr (HASH) {
                // An 8-value group is split over a lane pair: the even lane has
                // d = 0..3 (the high nibble), the odd lane d = 4..7.  The odd lane
                // continues the even lane's running sum and product so that the
                // order of operations is d = 0..7, as in
                // compute_code_score/torch_extension.cc:31-37.
                const int nib = (z[0] > 0.f ? 8 : 0) | (z[1] > 0.f ? 4 : 0) |
                                (z[2] > 0.f ? 2 : 0) | (z[3] > 0.f ? 1 : 0);
                float az[4], fz[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    az[c] = fabsf(z[c]);
                    fz[c] = 1.0f + exp_minus_2a(az[c]);
                }
                float s_loc = 0.f, p_loc = 1.f;
                score_chain(az, fz, s_loc, p_loc);                 // what an even lane hands over
                float s_run = lane_xor<1>(s_loc);
                float p_run = lane_xor<1>(p_loc);
                const int nib_hi = __float_as_int(lane_xor<1>(__int_as_float(nib)));
                score_chain(az, fz, s_run, p_run);                 // an odd lane continues from there
                const int t = col >> 3;
                if constexpr (GATHER) {
                    __shared__ uint2 pairs[4][FUSED_MAX_T];
                    static_assert(RPW == 1, "one token per wavefront");
                    if ((lr & 1) && t < a.T)
                        pairs[wave][t] = make_uint2((unsigned)((nib_hi << 4) | nib), __float_as_uint(s_run / p_run));
                    if (r == a.R - 1 && j == NJ - 1) {
                        // Small batches: the gather-add of the token's T rows follows in the same
                        // workgroup: wavefront w takes tables [w*T/4, (w+1)*T/4) (fused_gather).
                        // No codes or scores go to memory and nothing else is launched.
                        __shared__ float4 part[4][FUSED_MAX_NC][64];
                        __syncthreads();                         // the odd lanes' pairs are visible to the whole wavefront
                        const int tq = (a.T + 3) / 4;
                        const int t_lo = min(wave * tq, a.T), t_hi = min(t_lo + tq, a.T);
                        // up to four column passes of 256 in flight together; wider rows in rounds of 1024
                        for (int col0 = 0; col0 < a.Do; col0 += 256 * FUSED_MAX_NC) {
                            switch (min(FUSED_MAX_NC, (a.Do - col0 + 255) / 256)) {
                                case 1: fused_gather<1>(a, pairs[wave], part, row, col0, t_lo, t_hi, wave, lane); break;
                                case 2: fused_gather<2>(a, pairs[wave], part, row, col0, t_lo, t_hi, wave, lane); break;
                                case 3: fused_gather<3>(a, pairs[wave], part, row, col0, t_lo, t_hi, wave, lane); break;
                                default: fused_gather<4>(a, pairs[wave], part, row, col0, t_lo, t_hi, wave, lane); break;
                            }
                        }
                    }
                } else if (a.records) {
                    // Tables t - 1 (even) and t sit in lanes 4m + 1 and 4m + 3: the latter fetches the
                    // former's code and score (quad_perm [1,1,1,1]) and writes the pair's record.
                    const int code_here = (nib_hi << 4) | nib;
                    const float score_here = s_run / p_run;
                    const int code_even = __builtin_amdgcn_update_dpp(0, code_here, 0x55, 0xF, 0xF, true);
                    const float score_even = __int_as_float(
                        __builtin_amdgcn_update_dpp(0, __float_as_int(score_here), 0x55, 0xF, 0xF, true));
                    if (live && (lr & 3) == 3 && t < a.T) {
                        const bool second_first = (row & 2) != 0;
                        uint32_t *dst = a.records + ((size_t)(t >> 1) * a.rec_stride + rec_slot) * LFFN_RECORD_WORDS;
                        dst[0] = __float_as_uint(second_first ? score_here : score_even);
                        dst[1] = __float_as_uint(second_first ? score_even : score_here);
                        dst[2] = second_first ? (unsigned)(code_here | (code_even << 8))
                                              : (unsigned)(code_even | (code_here << 8));
                    }
                } else if (live && (lr & 1) && t < a.T) {
                    a.codes[row * a.T + t] = (nib_hi << 4) | nib;
                    a.scores[row * a.T + t] = s_run / p_run;
                }
            }
        }
    }
}

template <bool HASH>
int launch_project(const ProjectArgs &a, int logd, hipStream_t stream) {
    if (a.B == 0) return LFFN_OK;
    auto go = [&](auto tag) {
        constexpr int L = decltype(tag)::value;
        const int64_t rows_per_block = 4 * FhtCfg<L>::RPW;
        int64_t blocks = (a.B + rows_per_block - 1) / rows_per_block;
        ProjectArgs b = a;
        if (HASH && a.records) {        // whole rounds of eight workgroups, one per XCD
            b.blocks_per_xcd = (int)((blocks + 7) / 8);
            blocks = int64_t(b.blocks_per_xcd) * 8;
        }
        hipLaunchKernelGGL((project_kernel<L, HASH>), dim3((unsigned)blocks), dim3(256), 0, stream, b);
    };
    switch (logd) {
        case 2: if constexpr (!HASH) { go(std::integral_constant<int, 2>{}); break; } else return LFFN_ERR_UNSUPPORTED;
        case 3: go(std::integral_constant<int, 3>{}); break;
        case 4: go(std::integral_constant<int, 4>{}); break;
        case 5: go(std::integral_constant<int, 5>{}); break;
        case 6: go(std::integral_constant<int, 6>{}); break;
        case 7: go(std::integral_constant<int, 7>{}); break;
        case 8: go(std::integral_constant<int, 8>{}); break;
        case 9: go(std::integral_constant<int, 9>{}); break;
        case 10: go(std::integral_constant<int, 10>{}); break;
        default: return LFFN_ERR_UNSUPPORTED;
    }
    return lffn_launch_status();
}

int check_dims(int64_t B, int64_t H, int64_t D, int64_t R, int64_t J) {
    LFFN_REQUIRE(B >= 0 && H >= 1 && R >= 1 && J >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(D) && D >= 4 && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(H <= D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(B * 1 <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R * D <= (int64_t(1) << 24) && J <= 64, LFFN_ERR_UNSUPPORTED);
    return LFFN_OK;
}

// Backward of the fused projection + hash for block size 1 and 8-bit codes, one kernel:
//   z = decay * y + residual * pad(x) (+ bias),  y = FHT(d_{J-1} * ... FHT(d_0 * pad(x)))   per repeat
// Inputs: x, the diagonals, the z kept by the forward and the gradient of the scores.
// Per row (one wavefront, D >= 256): the gradient of z from the closed form of the score
// (PL/compute_code_score/kernel.py:51-53 differentiated; a group of 8 columns sits in a lane
// pair), the forward stages recomputed in registers (u_0 = pad(x), u_{j+1} = FHT(d_j * u_j)),
// then backwards t <- FHT(t); grad d_j += t * u_j; t <- d_j * t, the transform being its own
// transpose.  grad x of this repeat = t + residual * grad z.  The gradients of the diagonals and
// of the bias are summed over the rows of a wavefront in registers, over the four wavefronts
// of the workgroup in LDS, and written as one partial per workgroup; the caller adds the
// partials (and the per-repeat grad x when R > 1).
struct ProjectBwdArgs {
    const float *x;        // [B, H]
    const float *diag;     // [R, J, D]
    const float *z;        // [B, ncols]  (ncols = T*8)
    const float *g_score;  // [B, T]
    float *g_x;            // [R, B, H]
    float *part_d;         // [nblk, R, J, D]
    float *part_b;         // [nblk, R*D]   (columns >= ncols are written as zero)
    int64_t B;
    int H, R, J, T;
    float decay, residual;
    const float *ln_w;     // [H] or null: the projection's input is LayerNorm(x; ln_w, ln_b, ln_eps), formed on
    const float *ln_b;     // load as in the forward; g_x is then the gradient w.r.t. that LayerNorm output
    float ln_eps;
};

template <int LOGD>
__global__ __launch_bounds__(256) void project_hash_bwd_kernel(ProjectBwdArgs a) {
    using C = FhtCfg<LOGD>;
    constexpr int D = C::D, NJ = C::NJ;
    static_assert(C::LPR == 64, "one row per wavefront");
    constexpr int MAXJ = 4;
    __shared__ float red[4][64][NJ * 4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lr = lane;
    const int r = blockIdx.y;
    // Cross-lane swaps, not the two-trip form of the forward kernel: with two wavefronts per SIMD every
    // LDS round trip is waited for (165 us against 117 us at 16384 x 1024, four stages).
    auto transform = [&](float (&t)[NJ][4]) { fht_rows<LOGD, true>(t, lr); };
    const int ncols = a.T * 8;
    const int64_t nwaves = int64_t(gridDim.x) * 4;

    float acc_d[MAXJ][NJ][4], acc_b[NJ][4];
#pragma unroll
    for (int s = 0; s < MAXJ; ++s)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc_d[s][j][c] = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc_b[j][c] = 0.f;

    for (int64_t row = int64_t(blockIdx.x) * 4 + wave; row < a.B; row += nwaves) {
        // forward stages recomputed: u[s] is the input of stage s
        float u[MAXJ][NJ][4], t[NJ][4];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int e0 = 256 * j + 4 * lr;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e0 < a.H) v = *reinterpret_cast<const float4 *>(a.x + row * a.H + e0);
            t[j][0] = v.x; t[j][1] = v.y; t[j][2] = v.z; t[j][3] = v.w;
        }
        if (a.ln_w) {                                         // uniform
            // LayerNorm over the H valid columns exactly as project_kernel forms it (biased variance,
            // two passes, eps inside the square root; padding columns stay zero)
            float s1 = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int c = 0; c < 4; ++c) s1 += t[j][c];
            const float mean = lane_group_sum<64>(s1) / float(a.H);
            float s2 = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float dlt = (256 * j + 4 * lr + c < a.H) ? t[j][c] - mean : 0.f;
                    s2 += dlt * dlt;
                }
            const float rstd = 1.0f / sqrtf(lane_group_sum<64>(s2) / float(a.H) + a.ln_eps);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int e0 = 256 * j + 4 * lr;
                if (e0 < a.H) {                               // H % 4 == 0: all four columns or none
                    const float4 lw = *reinterpret_cast<const float4 *>(a.ln_w + e0);
                    const float4 lb = *reinterpret_cast<const float4 *>(a.ln_b + e0);
                    t[j][0] = (t[j][0] - mean) * rstd * lw.x + lb.x;
                    t[j][1] = (t[j][1] - mean) * rstd * lw.y + lb.y;
                    t[j][2] = (t[j][2] - mean) * rstd * lw.z + lb.z;
                    t[j][3] = (t[j][3] - mean) * rstd * lw.w + lb.w;
                }
            }
        }
#pragma unroll
        for (int s = 0; s < MAXJ; ++s) {
            if (s < a.J) {
                const float *dg = a.diag + (int64_t(r) * a.J + s) * D;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const float4 w = *reinterpret_cast<const float4 *>(dg + 256 * j + 4 * lr);
#pragma unroll
                    for (int c = 0; c < 4; ++c) u[s][j][c] = t[j][c];
                    t[j][0] = t[j][0] * w.x; t[j][1] = t[j][1] * w.y; t[j][2] = t[j][2] * w.z; t[j][3] = t[j][3] * w.w;
                }
                if (s + 1 < a.J) transform(t);                     // the last transform's output is not needed
            }
        }

        // gradient of z for this repeat's columns
        float gz[NJ][4];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int col = r * D + 256 * j + 4 * lr;
            const bool in_cols = col < ncols;
            float4 zv = make_float4(0.f, 0.f, 0.f, 0.f);
            float g = 0.f;
            if (in_cols) {
                zv = *reinterpret_cast<const float4 *>(a.z + row * ncols + col);
                g = a.g_score[row * a.T + (col >> 3)];
            }
            const float zz[4] = {zv.x, zv.y, zv.z, zv.w};
            float az[4], ez[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                az[c] = fabsf(zz[c]);
                ez[c] = expf(-2.0f * az[c]);
            }
            // S and P over the 8 values of the group, d ascending: the even lane starts, the odd
            // lane continues and hands the totals back
            float s_loc = 0.f, p_loc = 1.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) { s_loc = s_loc + az[c]; p_loc = p_loc * (1.0f + ez[c]); }
            float s_run = lane_xor<1>(s_loc), p_run = lane_xor<1>(p_loc);
#pragma unroll
            for (int c = 0; c < 4; ++c) { s_run = s_run + az[c]; p_run = p_run * (1.0f + ez[c]); }
            const float s_back = lane_xor<1>(s_run), p_back = lane_xor<1>(p_run);
            const float S = (lr & 1) ? s_run : s_back;
            const float P = (lr & 1) ? p_run : p_back;
            // one division per group of four (P is the lane pair's), hardware reciprocals (1 ulp) for
            // the per-value quotients: a gradient, compared at 1e-5
            const float g_over_p = g / P;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float sg = zz[c] > 0.f ? 1.f : (zz[c] < 0.f ? -1.f : 0.f);
                const float q = ez[c] * __builtin_amdgcn_rcpf(1.0f + ez[c]);
                gz[j][c] = in_cols ? sg * (1.0f + S * 2.0f * q) * g_over_p : 0.f;
                acc_b[j][c] += gz[j][c];
            }
        }

        // backwards through the stages
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) t[j][c] = a.decay * gz[j][c];
#pragma unroll
        for (int s = MAXJ - 1; s >= 0; --s) {
            if (s < a.J) {
                transform(t);
                const float *dg = a.diag + (int64_t(r) * a.J + s) * D;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const float4 w = *reinterpret_cast<const float4 *>(dg + 256 * j + 4 * lr);
#pragma unroll
                    for (int c = 0; c < 4; ++c) acc_d[s][j][c] += t[j][c] * u[s][j][c];
                    t[j][0] = t[j][0] * w.x; t[j][1] = t[j][1] * w.y; t[j][2] = t[j][2] * w.z; t[j][3] = t[j][3] * w.w;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int e0 = 256 * j + 4 * lr;
            if (e0 < a.H) {
                float4 o;
                o.x = t[j][0] + a.residual * gz[j][0];
                o.y = t[j][1] + a.residual * gz[j][1];
                o.z = t[j][2] + a.residual * gz[j][2];
                o.w = t[j][3] + a.residual * gz[j][3];
                *reinterpret_cast<float4 *>(a.g_x + (int64_t(r) * a.B + row) * a.H + e0) = o;
            }
        }
    }

    // workgroup partials: sum of the four wavefronts, one array at a time through LDS
    auto flush = [&](const float (&acc)[NJ][4], float *dst) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) red[wave][lane][4 * j + c] = acc[j][c];
        __syncthreads();
        // thread (wave, lane) adds float4 number `wave`.. of lane `lane` over the four wavefronts
        for (int j = wave; j < NJ; j += 4) {
            float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                sum.x += red[w][lane][4 * j + 0]; sum.y += red[w][lane][4 * j + 1];
                sum.z += red[w][lane][4 * j + 2]; sum.w += red[w][lane][4 * j + 3];
            }
            *reinterpret_cast<float4 *>(dst + 256 * j + 4 * lane) = sum;
        }
    };
#pragma unroll
    for (int s = 0; s < MAXJ; ++s)
        if (s < a.J) flush(acc_d[s], a.part_d + ((int64_t(blockIdx.x) * a.R + r) * a.J + s) * D);
    flush(acc_b, a.part_b + (int64_t(blockIdx.x) * a.R + r) * D);
}

// The transform on rows stored as 16-bit floats (IEEE half or bfloat16): widened on load,
// every butterfly in fp32 registers exactly as above, one rounding (to nearest even) on the
// store.  The reference's half kernels add in half2 after every stage
// (fast_hadamard_transform/extension/cuda_kernel.cu:47-84); this is the same transform with
// a single rounding.
template <bool BF16>
__device__ __forceinline__ float widen16(uint32_t h) {
    if constexpr (BF16) return __uint_as_float(h << 16);
    else return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

template <bool BF16>
__device__ __forceinline__ uint32_t narrow16(float f) {
    if constexpr (BF16) {
        const uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;      // NaN stays NaN
        return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    } else {
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    }
}

template <int LOGD, bool BF16>
__global__ __launch_bounds__(256) void fht16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                    int64_t B) {
    using C = FhtCfg<LOGD>;
    constexpr int D = C::D, NJ = C::NJ, LPR = C::LPR, RPW = C::RPW;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lr = lane % LPR;
    const int64_t row = (int64_t(blockIdx.x) * 4 + wave) * RPW + lane / LPR;
    const bool live = row < B;
    float v[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        uint2 t = make_uint2(0u, 0u);
        if (live) t = *reinterpret_cast<const uint2 *>(in + row * D + 256 * j + 4 * lr);
        v[j][0] = widen16<BF16>(t.x & 0xffffu);
        v[j][1] = widen16<BF16>(t.x >> 16);
        v[j][2] = widen16<BF16>(t.y & 0xffffu);
        v[j][3] = widen16<BF16>(t.y >> 16);
    }
    if constexpr (LOGD == 10 || LOGD == 9) {
        __shared__ float xl[4 * XlCfg<LOGD>::ROW];
        fht_rows_xl<LOGD>(v, lr, xl + wave * XlCfg<LOGD>::ROW);
    } else {
        fht_rows<LOGD>(v, lr);
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint2 t;
            t.x = narrow16<BF16>(v[j][0]) | (narrow16<BF16>(v[j][1]) << 16);
            t.y = narrow16<BF16>(v[j][2]) | (narrow16<BF16>(v[j][3]) << 16);
            *reinterpret_cast<uint2 *>(out + row * D + 256 * j + 4 * lr) = t;
        }
    }
}

template <bool BF16>
int fht16_entry(const uint16_t *in, uint16_t *out, int64_t B, int64_t D, void *stream) {
    LFFN_REQUIRE(in && out, LFFN_ERR_BAD_ARG);
    int rc = check_dims(B, D, D, 1, 1);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE((reinterpret_cast<uintptr_t>(in) & 7u) == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0,
                 LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto go = [&](auto tag) {
        constexpr int L = decltype(tag)::value;
        const int64_t rows_per_block = 4 * FhtCfg<L>::RPW;
        hipLaunchKernelGGL((fht16_kernel<L, BF16>), dim3((unsigned)((B + rows_per_block - 1) / rows_per_block)),
                           dim3(256), 0, st, in, out, B);
    };
    switch (lffn_log2(D)) {
        case 2: go(std::integral_constant<int, 2>{}); break;
        case 3: go(std::integral_constant<int, 3>{}); break;
        case 4: go(std::integral_constant<int, 4>{}); break;
        case 5: go(std::integral_constant<int, 5>{}); break;
        case 6: go(std::integral_constant<int, 6>{}); break;
        case 7: go(std::integral_constant<int, 7>{}); break;
        case 8: go(std::integral_constant<int, 8>{}); break;
        case 9: go(std::integral_constant<int, 9>{}); break;
        case 10: go(std::integral_constant<int, 10>{}); break;
        default: return LFFN_ERR_UNSUPPORTED;
    }
    return lffn_launch_status();
}

}  // namespace

extern "C" int lffn_fht_f32(const float *in, float *out, int64_t B, int64_t D, void *stream) {
    LFFN_REQUIRE(in && out, LFFN_ERR_BAD_ARG);
    int rc = check_dims(B, D, D, 1, 1);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(lffn_aligned16(out), LFFN_ERR_BAD_ARG);
    ProjectArgs a{};
    a.x = in; a.diag = nullptr; a.pbias = nullptr; a.out = out; a.codes = nullptr; a.scores = nullptr;
    a.B = B; a.H = (int)D; a.R = 1; a.J = 1; a.out_stride = (int)D; a.out_cols = (int)D; a.T = 0;
    a.decay = 1.f; a.residual = 0.f; a.mix = 0; a.vec_in = lffn_aligned16(in) ? 1 : 0;
    return launch_project<false>(a, lffn_log2(D), static_cast<hipStream_t>(stream));
}

extern "C" int lffn_bh4_diag_f32(const float *x, const float *diag, float *out,
                                 int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, void *stream) {
    LFFN_REQUIRE(x && diag && out, LFFN_ERR_BAD_ARG);
    int rc = check_dims(B, H, D, R, J);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(lffn_aligned16(out) && lffn_aligned16(diag), LFFN_ERR_BAD_ARG);
    ProjectArgs a{};
    a.x = x; a.diag = diag; a.pbias = nullptr; a.out = out; a.codes = nullptr; a.scores = nullptr;
    a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J;
    a.out_stride = (int)(R * D); a.out_cols = (int)(R * D); a.T = 0;
    a.decay = 1.f; a.residual = 0.f; a.mix = 0;
    a.vec_in = (lffn_aligned16(x) && H % 4 == 0) ? 1 : 0;
    return launch_project<false>(a, lffn_log2(D), static_cast<hipStream_t>(stream));
}

static int project_hash_impl(const float *x, const float *ln_w, const float *ln_b, float ln_eps,
                             const float *diag, const float *proj_bias,
                             float *z_out, int32_t *codes, float *scores,
                             int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                             float decay, float residual, void *stream, uint32_t *records = nullptr,
                             int64_t record_stride = 0, int record_tile = 0);

extern "C" int lffn_ln_project_hash_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                        const float *diag, const float *proj_bias,
                                        float *z_out, int32_t *codes, float *scores,
                                        int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                        float decay, float residual, void *stream) {
    LFFN_REQUIRE(ln_weight && ln_bias && ln_eps >= 0.f, LFFN_ERR_BAD_ARG);
    return project_hash_impl(x, ln_weight, ln_bias, ln_eps, diag, proj_bias, z_out, codes, scores,
                             B, H, D, R, J, T, decay, residual, stream);
}

extern "C" int lffn_ln_project_hash_records_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                                const float *diag, const float *proj_bias, uint32_t *records,
                                                int64_t record_stride, int32_t tokens_per_workgroup, int64_t B,
                                                int64_t H, int64_t D, int64_t R, int64_t J, int64_t T, float decay,
                                                float residual, void *stream) {
    LFFN_REQUIRE(ln_eps >= 0.f && ((ln_weight && ln_bias) || (!ln_weight && !ln_bias)), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(records && T % 2 == 0 && B >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_record_layout_ok(B, record_stride, tokens_per_workgroup) && (uintptr_t)records % 4 == 0,
                 LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(D >= 16, LFFN_ERR_UNSUPPORTED);           // a table pair's 16 values within an aligned lane quad
    return project_hash_impl(x, ln_weight, ln_bias, ln_eps, diag, proj_bias, nullptr, nullptr, nullptr,
                             B, H, D, R, J, T, decay, residual, stream, records, record_stride, tokens_per_workgroup);
}

extern "C" int lffn_project_hash_f32(const float *x, const float *diag, const float *proj_bias,
                                     float *z_out, int32_t *codes, float *scores,
                                     int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                     float decay, float residual, void *stream) {
    return project_hash_impl(x, nullptr, nullptr, 0.f, diag, proj_bias, z_out, codes, scores,
                             B, H, D, R, J, T, decay, residual, stream);
}

static int project_hash_impl(const float *x, const float *ln_w, const float *ln_b, float ln_eps,
                             const float *diag, const float *proj_bias,
                             float *z_out, int32_t *codes, float *scores,
                             int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                             float decay, float residual, void *stream, uint32_t *records, int64_t record_stride,
                             int record_tile) {
    LFFN_REQUIRE(x && diag && ((codes && scores) || records), LFFN_ERR_BAD_ARG);
    int rc = check_dims(B, H, D, R, J);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(D >= 8, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T >= 1 && T * 8 <= R * D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(diag) && (!proj_bias || lffn_aligned16(proj_bias)) &&
                     (!z_out || lffn_aligned16(z_out)),
                 LFFN_ERR_BAD_ARG);
    ProjectArgs a{};
    a.x = x; a.diag = diag; a.pbias = proj_bias; a.out = z_out; a.codes = codes; a.scores = scores;
    a.records = records; a.rec_stride = record_stride; a.rec_tile = record_tile;
    a.ln_w = ln_w; a.ln_b = ln_b; a.ln_eps = ln_eps;
    a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J;
    a.out_stride = (int)(T * 8); a.out_cols = (int)(T * 8); a.T = (int)T;
    a.decay = decay; a.residual = residual; a.mix = 1;
    a.vec_in = (lffn_aligned16(x) && H % 4 == 0) ? 1 : 0;
    a.vec_ln = (H % 4 == 0 && ln_w && lffn_aligned16(ln_w) && lffn_aligned16(ln_b)) ? 1 : 0;
    return launch_project<true>(a, lffn_log2(D), static_cast<hipStream_t>(stream));
}

extern "C" int lffn_lookup_ffn_fused_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                         const float *diag, const float *proj_bias, const float *tables,
                                         const float *out_bias, const float *residual_in, float *out, int64_t B,
                                         int64_t H, int64_t D, int64_t R, int64_t J, int64_t T, int64_t S,
                                         int64_t Do, float decay, float residual, void *stream) {
    LFFN_REQUIRE(x && diag && tables && out, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE((ln_weight != nullptr) == (ln_bias != nullptr) && ln_eps >= 0.f, LFFN_ERR_BAD_ARG);
    int rc = check_dims(B, H, D, R, J);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(D >= 256 && T <= FUSED_MAX_T && S >= 256 && S * T <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(Do >= 4 && Do % 4 == 0 && Do <= (1 << 20), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T >= 1 && T * 8 <= R * D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(diag) && (!proj_bias || lffn_aligned16(proj_bias)) && lffn_aligned16(tables) &&
                     (!out_bias || lffn_aligned16(out_bias)) && (!residual_in || lffn_aligned16(residual_in)) &&
                     lffn_aligned16(out),
                 LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    ProjectArgs a{};
    a.x = x; a.diag = diag; a.pbias = proj_bias; a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = ln_eps;
    a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J;
    a.out_stride = (int)(T * 8); a.out_cols = (int)(T * 8); a.T = (int)T;
    a.decay = decay; a.residual = residual; a.mix = 1;
    a.vec_in = (lffn_aligned16(x) && H % 4 == 0) ? 1 : 0;
    a.vec_ln = (H % 4 == 0 && ln_weight && lffn_aligned16(ln_weight) && lffn_aligned16(ln_bias)) ? 1 : 0;
    a.tables = tables; a.obias = out_bias; a.gres = residual_in; a.gout = out; a.S = (int)S; a.Do = (int)Do;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)B);                       // one token per workgroup
    switch (lffn_log2(D)) {
        case 8: hipLaunchKernelGGL((project_kernel<8, true, true>), grid, dim3(256), 0, st, a); break;
        case 9: hipLaunchKernelGGL((project_kernel<9, true, true>), grid, dim3(256), 0, st, a); break;
        default: hipLaunchKernelGGL((project_kernel<10, true, true>), grid, dim3(256), 0, st, a); break;
    }
    return lffn_launch_status();
}

extern "C" int lffn_lookup_ffn_fused_layer_f32(const lffn_fused_layer *layer, const float *x, const float *residual_in,
                                               float *out, int64_t B, void *stream) {
    LFFN_REQUIRE(layer, LFFN_ERR_BAD_ARG);
    return lffn_lookup_ffn_fused_f32(x, layer->ln_weight, layer->ln_bias, layer->ln_eps, layer->diag, layer->proj_bias,
                                     layer->tables, layer->out_bias, residual_in, out, B, layer->H, layer->D, layer->R,
                                     layer->J, layer->T, layer->S, layer->Do, layer->decay, layer->residual, stream);
}

extern "C" int lffn_fht_f16(const uint16_t *in, uint16_t *out, int64_t B, int64_t D, void *stream) {
    return fht16_entry<false>(in, out, B, D, stream);
}

extern "C" int lffn_fht_bf16(const uint16_t *in, uint16_t *out, int64_t B, int64_t D, void *stream) {
    return fht16_entry<true>(in, out, B, D, stream);
}

static int project_hash_bwd_impl(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                 const float *diag, const float *z, const float *g_score,
                                 float *g_x, float *part_diag, float *part_bias, int64_t B, int64_t H,
                                 int64_t D, int64_t R, int64_t J, int64_t T, int64_t num_partials,
                                 float decay, float residual, void *stream);

extern "C" int lffn_project_hash_bwd_f32(const float *x, const float *diag, const float *z, const float *g_score,
                                         float *g_x, float *part_diag, float *part_bias, int64_t B, int64_t H,
                                         int64_t D, int64_t R, int64_t J, int64_t T, int64_t num_partials,
                                         float decay, float residual, void *stream) {
    return project_hash_bwd_impl(x, nullptr, nullptr, 0.f, diag, z, g_score, g_x, part_diag, part_bias, B, H, D, R,
                                 J, T, num_partials, decay, residual, stream);
}

extern "C" int lffn_ln_project_hash_bwd_f32(const float *x, const float *ln_weight, const float *ln_bias,
                                            float ln_eps, const float *diag, const float *z,
                                            const float *g_score, float *g_h, float *part_diag, float *part_bias,
                                            int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                            int64_t num_partials, float decay, float residual, void *stream) {
    LFFN_REQUIRE(ln_weight && ln_bias && ln_eps >= 0.f, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(ln_weight) && lffn_aligned16(ln_bias), LFFN_ERR_BAD_ARG);
    return project_hash_bwd_impl(x, ln_weight, ln_bias, ln_eps, diag, z, g_score, g_h, part_diag, part_bias, B, H, D,
                                 R, J, T, num_partials, decay, residual, stream);
}

static int project_hash_bwd_impl(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                 const float *diag, const float *z, const float *g_score,
                                 float *g_x, float *part_diag, float *part_bias, int64_t B, int64_t H,
                                 int64_t D, int64_t R, int64_t J, int64_t T, int64_t num_partials,
                                 float decay, float residual, void *stream) {
    int rc = check_dims(B, H, D, R, J);
    if (rc != LFFN_OK) return rc;
    LFFN_REQUIRE(D >= 256 && J >= 1 && J <= 4 && H % 4 == 0 && R <= 65535, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T >= 1 && T * 8 <= R * D && num_partials >= 1 && num_partials <= 65535, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(x && diag && z && g_score && g_x && part_diag && part_bias, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(diag) && lffn_aligned16(z) && lffn_aligned16(g_x) &&
                     lffn_aligned16(part_diag) && lffn_aligned16(part_bias), LFFN_ERR_BAD_ARG);
    ProjectBwdArgs a{};
    a.x = x; a.diag = diag; a.z = z; a.g_score = g_score; a.g_x = g_x; a.part_d = part_diag; a.part_b = part_bias;
    a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T; a.decay = decay; a.residual = residual;
    a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = ln_eps;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)num_partials, (unsigned)R);
    switch (lffn_log2(D)) {
        case 8: hipLaunchKernelGGL((project_hash_bwd_kernel<8>), grid, dim3(256), 0, st, a); break;
        case 9: hipLaunchKernelGGL((project_hash_bwd_kernel<9>), grid, dim3(256), 0, st, a); break;
        default: hipLaunchKernelGGL((project_hash_bwd_kernel<10>), grid, dim3(256), 0, st, a); break;
    }
    return lffn_launch_status();
}
