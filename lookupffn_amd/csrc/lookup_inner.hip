// Gradient of the layer's gather w.r.t. the scores, table-major with the table in LDS:
//
//   grad_score[b,t] = < g[b,:], tables[t, code[b,t] & (S-1), :] >
//
// This file: the entry point, and the form with atomics that serves the shapes the
// four-lanes-per-token kernel of lookup_inner_quad.hip does not take (S < 256, an odd
// number of tables, too few tokens to fill the chip with 1024-token tiles).
//
// The mirror image of lookup_gather.hip.  A 1024-lane workgroup owns a 256-byte
// column slice (64 fp32 columns) and a tile of 64*NP tokens whose slice of g stays
// in registers for the whole kernel (16 lanes side by side hold a token's 64
// columns, a wavefront holds 4 tokens at a time, NP passes cover the tile).  For
// every table the workgroup copies that table's slice into LDS once (global ->
// LDS directly, double-buffered, one barrier per table); each token reads its row
// with a conflict-free ds_read_b128, multiplies it into its g values and sums
// over its 16 lanes with four DPP row rotations.  Codes reach the lanes with a
// DPP row broadcast.  A lane keeps the result of "its" table of the 16-table
// chunk and, once per chunk, adds it to grad_score with a global atomic: the
// partial sums of the Do/64 slices of a row are combined there, in whatever order
// the workgroups arrive (the reference's kernel, PL/gather/cuda/extension/gather_kernel_fp32.cu:141,
// also combines its partial sums with atomics).  grad_score must be zero when the
// kernel starts; the entry point clears it first.
//
// Measured at 16384 tokens x 128 tables x 256 x 768 (MI355X): 255 us, of which about
// 35 us are the atomics.  Summing four tokens' partial products together with a
// lane-transposing reduction (12 instead of 20 vector instructions per four sums)
// and requesting the LDS rows of the next pass group ahead of time both left the
// time unchanged: with 832 tokens a tile the table time is the slice copy
// (about 1.1 us for 64 KB per compute unit) plus the part of the arithmetic that
// does not overlap with it.
#include "lffn_common.h"

#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

namespace {

constexpr int WG = 1024;
constexpr int SEG_VECS = 16;          // 16-byte vectors per row segment (256 bytes)
constexpr int CHUNK = 16;             // tables per code register set = lanes per token group
constexpr int MAX_S = 256;
constexpr int XCDS = 8;

struct InnerArgs {
    const int32_t *code;   // [B, T]
    const float *g;        // [B, Do]
    const char *tables;    // [T, S, Do] fp32
    float *out;            // [B, T], zeroed
    int64_t B;
    int T, S, Do;
    int ntiles, nslices, per_xcd;
    int row_bytes;
};

// global_load_lds_dwordx4: lane i of the wavefront writes its 16 bytes at the LDS
// address in M0 + 16*i.  Inline assembly so that the compiler does not serialise
// the copy with the LDS reads of the other buffer; the caller waits with vmcnt(0)
// before the barrier that publishes the buffer.
__device__ __forceinline__ void lds_dma16(const char *gptr, uint32_t lds_byte_addr) {
    // M0 is put back: the compiler reserves it for its own use and does not honour a clobber
    // declaration of it, so the statement must leave it as it found it
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(gptr), "s"(lds_byte_addr)
                 : "memory");
}

template <bool FULL>
__device__ __forceinline__ void copy_slice_to_lds(const char *tb, int row_bytes, int tid, int buf_vecs, uint4 *dst) {
    const char *p = tb + (size_t)(tid >> 4) * row_bytes + (tid & 15) * 16;
    const size_t step = (size_t)(WG / SEG_VECS) * row_bytes;   // 64 rows further down
    const uint32_t wbase = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)(dst + (tid & ~63)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (FULL || tid + i * WG < buf_vecs) lds_dma16(p + i * step, wbase + i * (WG * 16));
    }
}

// One step of a sum over the 16 lanes of a row: v + (v rotated right by N lanes
// within the row).  Every lane has a source, so with bound_ctrl and a zero `old`
// the compiler folds the move into the add (v_add_f32 with a DPP operand).
template <int N>
__device__ __forceinline__ float add_row_ror(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + N, 0xF, 0xF, true));
}

template <int NP, bool FULL>
__global__ __launch_bounds__(WG) void lookup_inner_lds_kernel(InnerArgs a) {
    static_assert(MAX_S * SEG_VECS == 4 * WG, "a lane copies four vectors of a slice");
    constexpr int NQ = (NP + 3) / 4;              // four 8-bit codes per register
    extern __shared__ uint4 lds[];                // 2 buffers of S * SEG_VECS vectors

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.ntiles * a.nslices) return;     // uniform over the workgroup
    const int slice = unit / a.ntiles;
    const int tile = unit % a.ntiles;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int grp = lane >> 4;
    const int j = lane & 15;
    const int64_t tok0 = int64_t(tile) * (64 * NP) + wave * 4 + grp;

    // passes p < nvalid of this lane are tokens below B; the others read token tokb and are dropped
    const int nvalid = (int)max(int64_t(0), min(int64_t(NP), (a.B - tok0 + 63) / 64));
    const int64_t tokb = min(tok0, a.B - 1);
    const uint32_t rowoff = (uint32_t)(tokb * a.T);          // B * T < 2^30
    const uint32_t pass_stride = 64u * (uint32_t)a.T;

    float4 gq[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        gq[p] = p < nvalid ? *reinterpret_cast<const float4 *>(a.g + (tok0 + p * 64) * a.Do + (size_t)slice * 64 + j * 4)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    const int buf_vecs = a.S * SEG_VECS;
    const char *slice_base = a.tables + (size_t)slice * (SEG_VECS * 16);
    const size_t table_bytes = (size_t)a.S * a.row_bytes;

    // Team touch (see lookup_gather.hip): the workgroups that share this slice each pull a share of
    // the lines of the table after next into the XCD's L2.
    const int touch_line = team_touch_line(a.S * 2, a.ntiles, tile, tid);
    const uint32_t touch_off = (uint32_t)(touch_line >> 1) * (uint32_t)a.row_bytes + (touch_line & 1) * 128;
    const uint32_t touch_dst = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)(lds + 2 * buf_vecs);

    copy_slice_to_lds<FULL>(slice_base, a.row_bytes, tid, buf_vecs, lds);
    __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
    __syncthreads();

    for (int t0 = 0; t0 < a.T; t0 += CHUNK) {
        // lane j of a token group holds the code of table t0 + j for each of its NP tokens
        uint32_t ro = rowoff;
        asm volatile("" : "+v"(ro));      // recompute the addresses per chunk instead of keeping 2*NP of them
        unsigned cd[NQ];
        {
            const uint32_t cbase = ro + (uint32_t)min(t0 + j, a.T - 1);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                unsigned w = 0u;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int p = q * 4 + i;
                    if (p < NP) {
                        const int c = a.code[cbase + (p < nvalid ? p * pass_stride : 0u)];
                        w |= unsigned(c & (a.S - 1)) << (8 * i);
                    }
                }
                cd[q] = w;
                __builtin_amdgcn_sched_barrier(0);     // four loads in flight at a time: bounds the registers
            }
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) asm volatile("" : "+v"(cd[q]));   // landed before the table loop

        float res[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) res[p] = 0.f;

        const int nt = min(CHUNK, a.T - t0);
        static_for<CHUNK>([&](auto tt_c) {
            constexpr int TT = decltype(tt_c)::value;
            if (TT < nt) {                                     // uniform
                const int t = t0 + TT;
                copy_slice_to_lds<FULL>(slice_base + (size_t)min(t + 1, a.T - 1) * table_bytes, a.row_bytes, tid,
                                        buf_vecs, lds + ((t + 1) & 1) * buf_vecs);
                if constexpr (FULL)
                    l2_touch(slice_base + (size_t)min(t + TOUCH_AHEAD, a.T - 1) * table_bytes, touch_off, touch_dst);
                const uint4 *buf = lds + (t & 1) * buf_vecs + j;
                constexpr int GRP = 4;
#pragma unroll
                for (int g0 = 0; g0 < NP; g0 += GRP) {
                    const unsigned packed = (unsigned)row_broadcast<TT>((int)cd[g0 / 4]);
                    uint4 r[GRP];
#pragma unroll
                    for (int i = 0; i < GRP; ++i) {
                        if (g0 + i < NP) r[i] = buf[((packed >> (8 * i)) & 0xFFu) * SEG_VECS];
                    }
                    float d[GRP];
#pragma unroll
                    for (int i = 0; i < GRP; ++i) {
                        const int p = g0 + i;
                        if (p < NP) {
                            d[i] = gq[p].x * __uint_as_float(r[i].x);
                            d[i] = fmaf(gq[p].y, __uint_as_float(r[i].y), d[i]);
                            d[i] = fmaf(gq[p].z, __uint_as_float(r[i].z), d[i]);
                            d[i] = fmaf(gq[p].w, __uint_as_float(r[i].w), d[i]);
                        }
                    }
                    // the four sums side by side: independent adds fill the DPP wait states
#pragma unroll
                    for (int i = 0; i < GRP; ++i) if (g0 + i < NP) d[i] = add_row_ror<8>(d[i]);
#pragma unroll
                    for (int i = 0; i < GRP; ++i) if (g0 + i < NP) d[i] = add_row_ror<4>(d[i]);
#pragma unroll
                    for (int i = 0; i < GRP; ++i) if (g0 + i < NP) d[i] = add_row_ror<2>(d[i]);
#pragma unroll
                    for (int i = 0; i < GRP; ++i) if (g0 + i < NP) d[i] = add_row_ror<1>(d[i]);
#pragma unroll
                    for (int i = 0; i < GRP; ++i) {
                        if (g0 + i < NP) res[g0 + i] = (j == TT) ? d[i] : res[g0 + i];   // lane TT keeps this table's value
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                __builtin_amdgcn_s_waitcnt(FULL ? WAIT_VMCNT_1 : WAIT_VMCNT_0);     // vmcnt(1): the copy issued above has landed; the touch,
                                                        // issued after it, may still be out
                __syncthreads();
            }
        });

        // add this slice's partial dot products of tables t0 .. t0+15 to grad_score
        if (t0 + j < a.T) {
            float *ob = a.out + (ro + (uint32_t)(t0 + j));
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                if (p < nvalid) unsafeAtomicAdd(ob + p * pass_stride, res[p]);
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);         // nothing may still be writing this workgroup's LDS when it ends
}

__global__ __launch_bounds__(256) void fill_zero_f32_kernel(float *p, int64_t n) {
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += int64_t(gridDim.x) * 256) p[i] = 0.f;
}

template <int NP, bool FULL>
int launch_inner_full(InnerArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + 64 * NP - 1) / (64 * NP));
    const int units = a.ntiles * a.nslices;
    a.per_xcd = (units + XCDS - 1) / XCDS;
    const size_t lds_bytes = size_t(2) * a.S * SEG_VECS * 16 + TOUCH_SINK_BYTES;     // two buffers + the touches' scratch
    auto kern = lookup_inner_lds_kernel<NP, FULL>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

template <int NP>
int launch_inner(const InnerArgs &a, hipStream_t stream) {
    return a.S == MAX_S ? launch_inner_full<NP, true>(a, stream) : launch_inner_full<NP, false>(a, stream);
}

}  // namespace

// The four-lanes-per-token kernel (lookup_inner_quad.hip) where the shape qualifies: S = 256, T even, tiles of
// 1024 tokens x chunks of 4 or 2 table pairs; 4 when that still gives the chip a round of workgroups (the g
// values are fetched once per chunk and slice), 2 otherwise, and not at all when even 2 leaves most of the chip
// idle.  g: token b's 32 columns of slice s at g + b * g_token_stride + s * g_slice_stride floats.  Returns
// false when the shape does not qualify (nothing launched), true with the launch status in *rc otherwise.
bool lffn_internal_lookup_inner_quad_try(const int32_t *code, const float *g, int64_t g_token_stride,
                                         int64_t g_slice_stride, const void *tables, float *grad_score, int64_t B,
                                         int64_t T, int64_t S, int64_t Do, void *stream, int *rc) {
    if (!(S == MAX_S && T % 2 == 0 && Do % 32 == 0 && B >= 1 && reinterpret_cast<uintptr_t>(code) % 8 == 0 &&
          2 * S * Do * 4 < (int64_t(1) << 32)))
        return false;
    const int64_t tiles = (B + 1023) / 1024, pairs = T / 2;
    const int c = tiles * ((pairs + 3) / 4) >= 200 ? 4 : (tiles * ((pairs + 1) / 2) >= 96 ? 2 : 0);
    if (!c || tiles * ((pairs + c - 1) / c) > (int64_t(1) << 30)) return false;
    *rc = lffn_internal_lookup_inner_quad(code, g, g_token_stride, g_slice_stride, tables, grad_score, B, T, S, Do, 4, c, stream);
    return true;
}

extern "C" int lffn_lookup_inner_f32(const int32_t *code, const float *g, const float *tables, float *grad_score,
                                     int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(S) && S <= (1 << 24) && T * S <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(Do % 64 == 0 && Do <= (1 << 20) && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE((code && g && tables && grad_score) || B * T == 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(tables) && lffn_aligned16(g), LFFN_ERR_BAD_ARG);
    if (B * T == 0) return LFFN_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t nslices = Do / 64;
    // Four lanes per token, one owner per (token, table) (lookup_inner_quad.hip): tiles of 1024 tokens x
    // chunks of 4 or 2 table pairs; 4 when that still gives the chip a round of workgroups (the g values are
    // fetched once per chunk and slice), and the form below when even 2 leaves most of it idle.
    {
        int rc = LFFN_OK;
        if (lffn_internal_lookup_inner_quad_try(code, g, Do, 32, tables, grad_score, B, T, S, Do, stream, &rc)) return rc;
    }

    // LDS form: table fits the buffers, and enough (token tile, slice) units to fill most CUs
    const bool lds_ok = S <= MAX_S && T >= 4 && B * T < (int64_t(1) << 30) &&
                        ((B + 255) / 256) * nslices >= 192 && B * nslices <= (int64_t(1) << 30);
    if (!lds_ok) return lffn_internal_lookup_inner_token_major(code, g, tables, grad_score, B, T, S, Do, stream);

    const int64_t n = B * T;
    const int64_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(fill_zero_f32_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, st,
                       grad_score, n);
    int rc = lffn_launch_status();
    if (rc != LFFN_OK) return rc;

    InnerArgs a{};
    a.code = code; a.g = g; a.tables = reinterpret_cast<const char *>(tables); a.out = grad_score;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)nslices;
    a.row_bytes = (int)(Do * 4);
    // tile: fewest rounds of 256 workgroups, then the larger tile (fewer table copies)
    const int nps[] = {13, 8, 4};
    int best = 4;
    int64_t best_cost = INT64_MAX;
    for (int np : nps) {
        const int64_t tiles = (B + 64 * np - 1) / (64 * np);
        const int64_t rounds = (tiles * nslices + 255) / 256;
        const int64_t cost = rounds * (10 + np);
        if (cost < best_cost) { best_cost = cost; best = np; }
    }
    switch (best) {
        case 13: return launch_inner<13>(a, st);
        case 8: return launch_inner<8>(a, st);
        default: return launch_inner<4>(a, st);
    }
}
