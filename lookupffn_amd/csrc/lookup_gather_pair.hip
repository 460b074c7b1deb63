// The layer's weighted gather-add, table-major, two tables per LDS buffer:
//
//   out[b,:] = bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
//
// Same idea as lookup_gather.hip (a workgroup keeps the accumulators of a token
// tile in registers and walks the tables through LDS), different geometry:
//
//   * a workgroup owns a 128-byte column slice (32 fp32 / 64 bf16 columns) and a
//     tile of 128*NP tokens: 8 lanes cover a token's row segment, a wavefront covers
//     8 tokens at a time.  Twice the tokens per staged byte of the 256-byte form,
//     so half the L2 -> LDS copy volume;
//   * an LDS buffer row holds the segments of TWO tables side by side (table 2k in
//     bytes 0..127, table 2k+1 in bytes 128..255).  In one ds_read_b128 the even
//     token groups of a wavefront read their row of table 2k and the odd groups
//     their row of table 2k+1; a second read swaps the roles.  The two tokens that
//     share a 256-byte LDS access window are therefore always in different bank
//     halves: conflict-free whatever the codes are, which plain 128-byte rows
//     (two random rows per window) would not be;
//   * one barrier per table PAIR, and the global -> LDS copy of pair k+1 has the
//     whole of pair k's work to land.
//
// Accumulation order: even token groups add table 2k then 2k+1, odd groups 2k+1
// then 2k (fp32; each token still adds its T rows one at a time).
//
// (code, score) pairs are read 8 tables at a time (one table per lane of the
// 8-lane token group, four 8-bit codes packed per register) and broadcast in the
// group with two DPP row broadcasts (one per half of the 16-lane row: vector-ALU
// moves, no LDS traffic).  (Loading the next 8 tables' pairs one chunk ahead was
// tried: the extra live registers spill and it runs slower.)
#include "lffn_common.h"

namespace {

constexpr int WG = 1024;
constexpr int MAX_S = 256;
constexpr int XCDS = 8;
constexpr int CHUNK = 8;              // tables per (code, score) register set = lanes per token group
constexpr int ROW_VECS = 16;          // 16-byte vectors per LDS row (two tables x 128 bytes)

struct PairArgs {
    const int32_t *code;   // [B, T]
    const float *score;    // [B, T]
    const char *tables;    // [T, S, Do] fp32 or bf16
    const float *bias;     // [Do] or null
    const float *residual; // [B, Do] or null: added to the result (may be the output buffer)
    float *out;            // [B, Do]
    int64_t B;
    int T, S, Do;
    int ntiles, nslices, per_xcd;
    int row_bytes;         // Do * element size
    int touch;             // 1: with the team touch (decided by the host, see launch_pair)
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

// Copy the 128-byte segments of tables ta and tb (rows 0..S-1) into `dst`:
// vector q = tid + 1024*i is piece q%16 of row q/16; pieces 0-7 come from ta, 8-15 from tb.
template <bool FULL>
__device__ __forceinline__ void copy_pair_to_lds(const char *slice_base, size_t table_bytes, int ta, int tb,
                                                 int row_bytes, int tid, int buf_vecs, uint4 *dst) {
    const int piece = tid & 15;
    const int t = piece < 8 ? ta : tb;
    const char *p = slice_base + (size_t)t * table_bytes + (size_t)(tid >> 4) * row_bytes + (piece & 7) * 16;
    const size_t step = (size_t)(WG / ROW_VECS) * row_bytes;   // 64 rows further down
    const uint32_t wbase = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)(dst + (tid & ~63)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (FULL || tid + i * WG < buf_vecs) lds_dma16(p + i * step, wbase + i * (WG * 16));
    }
}

// Lanes 0-7 of each 16-lane row get the value of row lane NLO (< 8), lanes 8-15 that
// of row lane 8 + NHI: each 8-lane token group reads one of its own lanes.
template <int NLO, int NHI>
__device__ __forceinline__ int half_row_broadcast(int v) {
    // all 16 lanes <- lane NLO (every lane has a source, so no `old` value is needed: a bare
    // v_mov_b32_dpp), then banks 2-3 (lanes 8-15) <- lane 8 + NHI on top of that
    const int lo = __builtin_amdgcn_update_dpp(0, v, DPP_ROW_NEWBCAST0 + NLO, 0xF, 0xF, true);
    return __builtin_amdgcn_update_dpp(lo, v, DPP_ROW_NEWBCAST0 + 8 + NHI, 0xF, 0xC, false);
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const u32x4 *lds_vec_ptr;

// TOUCH: with the team touch (a template parameter: a run-time branch in the pair loop, even a uniform
// one, makes the compiler spill hundreds of registers here).
template <bool BF16, int NP, bool FULL, bool TOUCH>
__global__ __launch_bounds__(WG) void lookup_gather_pair_kernel(PairArgs a) {
    constexpr int EPV = BF16 ? 8 : 4;
    // bf16: four 8-bit codes per register.  fp32: two per register, each at bits 8..15 of its
    // 16-bit half, where a row number sits in an LDS byte address (row * 256 + ...): an address
    // is then one OR of a half-word with the lane's base (S is a power of two and the codes are
    // masked, so the buffer offset never overlaps the row field)
    // (at 16 passes the extra code registers of the two-per-register form would spill: four per register there)
    constexpr bool WIDE = !BF16 && NP <= 13;
    constexpr int NQ = WIDE ? (NP + 1) / 2 : (NP + 3) / 4;
    extern __shared__ uint4 lds[];                // 2 buffers of S * ROW_VECS vectors

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.ntiles * a.nslices) return;     // uniform over the workgroup
    const int slice = unit / a.ntiles;
    const int tile = unit % a.ntiles;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int grp = lane >> 3;        // token within the wavefront's eight
    const int j = lane & 7;           // 16-byte vector within the 128-byte row segment
    const int par = grp & 1;          // odd groups take the pair's tables in the other order
    const int64_t tok0 = int64_t(tile) * (128 * NP) + wave * 8 + grp;

    float acc[NP][EPV];
    {
        float b[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) b[e] = 0.f;
        if (a.bias) {
            const float *bp = a.bias + (size_t)slice * (8 * EPV) + j * EPV;
#pragma unroll
            for (int e = 0; e < EPV; ++e) b[e] = bp[e];
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[p][e] = b[e];
    }

    const int buf_vecs = a.S * ROW_VECS;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    const char *slice_base = a.tables + (size_t)slice * 128;
    const size_t table_bytes = (size_t)a.S * a.row_bytes;
    const int npairs = (a.T + 1) / 2;
    const int last_t = a.T - 1;
    // Team touch (see lookup_gather.hip): the workgroups that share this slice each pull a share of
    // the 2*S lines of the pair after next (one line per table row) into the XCD's L2.
    // (Only whole pairs are touched: with an odd number of tables the last one comes untouched.)
    const int touch_line = team_touch_line(a.S * 2, a.ntiles, tile, tid);
    const bool touch_second = touch_line >= a.S;                      // a row of the pair's second table
    const uint32_t touch_off = (touch_second ? (uint32_t)table_bytes : 0u) +
                               (uint32_t)(touch_line - (touch_second ? a.S : 0)) * (uint32_t)a.row_bytes;
    const int last_whole_pair = max(a.T / 2 - 1, 0);
    const uint32_t touch_dst = lds0 + (uint32_t)(2 * buf_vecs) * 16u;

    // (code, score) of tables c*8 + j for this lane's NP tokens; tokens and tables
    // past the end read a valid address and get score 0
    auto load_chunk = [&](int c, unsigned (&cd)[NQ], float (&sc)[NP]) {
        const int tt = c * CHUNK + j;
        const int ttc = min(tt, last_t);
        int craw[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            // B * T < 2^31 is a precondition of this kernel: 32-bit element offsets
            const int off = (int)min(tok0 + p * 128, a.B - 1) * a.T + ttc;
            craw[p] = a.code[off];
            sc[p] = a.score[off];
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) cd[q] = 0u;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const bool ok = (tok0 + p * 128 < a.B) && (tt < a.T);
            if constexpr (WIDE)
                cd[p / 2] |= unsigned(craw[p] & (a.S - 1)) << (8 + 16 * (p % 2));
            else
                cd[p / 4] |= unsigned(craw[p] & (a.S - 1)) << (8 * (p % 4));
            sc[p] = ok ? sc[p] : 0.f;
        }
    };

    unsigned cd[NQ];
    float sc[NP];

    copy_pair_to_lds<FULL>(slice_base, table_bytes, 0, min(1, last_t), a.row_bytes, tid, buf_vecs, lds);
    __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0)
    __syncthreads();

    const int nchunks = (a.T + CHUNK - 1) / CHUNK;
    for (int c = 0; c < nchunks; ++c) {
        load_chunk(c, cd, sc);
        // these must have landed before the pair loop: inside it nothing but the LDS
        // copies is in flight
#pragma unroll
        for (int q = 0; q < NQ; ++q) asm volatile("" : "+v"(cd[q]));
#pragma unroll
        for (int p = 0; p < NP; ++p) asm volatile("" : "+v"(sc[p]));

        const int k0 = c * (CHUNK / 2);
        const int npc = min(CHUNK / 2, npairs - k0);           // pairs in this chunk
        // the four pairs of the chunk, unrolled, so that the broadcast lanes are constants
        static_for<CHUNK / 2>([&](auto kq_c) {
            constexpr int KQ = decltype(kq_c)::value;
            if (KQ < npc) {                                    // uniform
                const int k = k0 + KQ;
                // next pair's segments straight into the other buffer (last read one pair
                // ago, before the previous barrier); the last iteration re-copies the last pair
                {
                    const int kn = min(k + 1, npairs - 1);
                    copy_pair_to_lds<FULL>(slice_base, table_bytes, 2 * kn, min(2 * kn + 1, last_t), a.row_bytes,
                                           tid, buf_vecs, lds + ((k + 1) & 1) * buf_vecs);
                }
                if constexpr (TOUCH)
                    l2_touch(slice_base + (size_t)(2 * min(k + TOUCH_AHEAD, last_whole_pair)) * table_bytes, touch_off, touch_dst);
                const uint4 *buf = lds + (k & 1) * buf_vecs + j;
                static_for<2>([&](auto half_c) {
                    constexpr int HALF = decltype(half_c)::value;
                    // even groups (row lanes 0-7) take table 2*KQ + HALF of the chunk, odd groups
                    // (row lanes 8-15) table 2*KQ + 1 - HALF; table 2k sits in the left 128 bytes
                    constexpr int NLO = 2 * KQ + HALF, NHI = 2 * KQ + 1 - HALF;
                    const uint4 *hbuf = buf + (HALF ^ par) * 8;
                    const unsigned haddr = lds0 + (unsigned)(((k & 1) * buf_vecs + (HALF ^ par) * 8 + j) * 16);
                    unsigned packed[NQ];
#pragma unroll
                    for (int q = 0; q < NQ; ++q) packed[q] = (unsigned)half_row_broadcast<NLO, NHI>((int)cd[q]);
                    constexpr int GRP = BF16 ? 4 : (NP > 8 ? 4 : NP);
#pragma unroll
                    for (int g0 = 0; g0 < NP; g0 += GRP) {
                        if constexpr (BF16) {
                            uint4 r[GRP];
#pragma unroll
                            for (int i = 0; i < GRP; ++i) {
                                const int p = g0 + i;
                                if (p < NP) {
                                    const unsigned row = (packed[p / 4] >> (8 * (p % 4))) & 0xFFu;
                                    r[i] = hbuf[row * ROW_VECS];
                                }
                            }
#pragma unroll
                            for (int i = 0; i < GRP; ++i) {
                                const int p = g0 + i;
                                if (p < NP) {
                                    const float w = __int_as_float(half_row_broadcast<NLO, NHI>(__float_as_int(sc[p])));
                                    acc[p][0] = fmaf(bf16_lo(r[i].x), w, acc[p][0]);
                                    acc[p][1] = fmaf(bf16_hi(r[i].x), w, acc[p][1]);
                                    acc[p][2] = fmaf(bf16_lo(r[i].y), w, acc[p][2]);
                                    acc[p][3] = fmaf(bf16_hi(r[i].y), w, acc[p][3]);
                                    acc[p][4] = fmaf(bf16_lo(r[i].z), w, acc[p][4]);
                                    acc[p][5] = fmaf(bf16_hi(r[i].z), w, acc[p][5]);
                                    acc[p][6] = fmaf(bf16_lo(r[i].w), w, acc[p][6]);
                                    acc[p][7] = fmaf(bf16_hi(r[i].w), w, acc[p][7]);
                                }
                            }
                        } else {
                            u32x4 r[GRP];
#pragma unroll
                            for (int i = 0; i < GRP; ++i) {
                                const int p = g0 + i;
                                if (p < NP) {
                                    if constexpr (WIDE) {
                                        const unsigned half = (p % 2) ? (packed[p / 2] >> 16) : (packed[p / 2] & 0xFFFFu);
                                        r[i] = *(lds_vec_ptr)(uintptr_t)(half | haddr);
                                    } else {
                                        const unsigned row = (packed[p / 4] >> (8 * (p % 4))) & 0xFFu;
                                        r[i] = *(lds_vec_ptr)(uintptr_t)(haddr + row * (ROW_VECS * 16));
                                    }
                                }
                            }
#pragma unroll
                            for (int i = 0; i < GRP; ++i) {
                                const int p = g0 + i;
                                if (p < NP) {
                                    const float w = __int_as_float(half_row_broadcast<NLO, NHI>(__float_as_int(sc[p])));
                                    acc[p][0] = fmaf(__uint_as_float(r[i].x), w, acc[p][0]);
                                    acc[p][1] = fmaf(__uint_as_float(r[i].y), w, acc[p][1]);
                                    acc[p][2] = fmaf(__uint_as_float(r[i].z), w, acc[p][2]);
                                    acc[p][3] = fmaf(__uint_as_float(r[i].w), w, acc[p][3]);
                                }
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
                // the copy issued above has landed; the touch, issued after it, may still be out
                __builtin_amdgcn_s_waitcnt(TOUCH ? WAIT_VMCNT_1 : WAIT_VMCNT_0);
                __syncthreads();
            }
        });
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);         // nothing may still be writing this workgroup's LDS when it ends

#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int64_t tok = tok0 + p * 128;
        if (tok < a.B) {
            const size_t off = tok * a.Do + (size_t)slice * (8 * EPV) + j * EPV;
            float *o = a.out + off;
#pragma unroll
            for (int q = 0; q < EPV / 4; ++q) {
                float4 v = make_float4(acc[p][4 * q], acc[p][4 * q + 1], acc[p][4 * q + 2], acc[p][4 * q + 3]);
                if (a.residual) {
                    const float4 rr = *reinterpret_cast<const float4 *>(a.residual + off + 4 * q);
                    v.x += rr.x; v.y += rr.y; v.z += rr.z; v.w += rr.w;
                }
                *reinterpret_cast<float4 *>(o + 4 * q) = v;
            }
        }
    }
}

template <bool BF16, int NP, bool FULL, bool TOUCH>
int launch_pair_full(PairArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + 128 * NP - 1) / (128 * NP));
    const int units = a.ntiles * a.nslices;
    a.per_xcd = (units + XCDS - 1) / XCDS;
    const size_t lds_bytes = size_t(2) * a.S * ROW_VECS * 16 + TOUCH_SINK_BYTES;     // two buffers + the touches' scratch
    auto kern = lookup_gather_pair_kernel<BF16, NP, FULL, TOUCH>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

template <bool BF16, int NP>
int launch_pair(const PairArgs &a, hipStream_t stream) {
    // The touch: 256-row tables only (as in lookup_gather.hip) and only while the table set fits the
    // 256 MB memory-side cache: beyond that this kernel is bound by HBM traffic and was measured 2-4%
    // slower with it (537 MB of tables).
    if (a.S != MAX_S) return launch_pair_full<BF16, NP, false, false>(a, stream);
    return a.touch ? launch_pair_full<BF16, NP, true, true>(a, stream)
                             : launch_pair_full<BF16, NP, true, false>(a, stream);
}

}  // namespace

// Launch the pair kernel with 128*np tokens per workgroup.  The caller has checked
// that the shape qualifies: S <= 256, Do a multiple of the 128-byte slice width
// (32 fp32 / 64 bf16 columns), B*T < 2^31, np one of {4, 8, 13, 16} (fp32) or {4, 8} (bf16).
int lffn_internal_lookup_gather_pair(const int32_t *code, const float *score, const void *tables,
                                     const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                     int64_t S,
                                     int64_t Do, bool bf16, int np, void *stream) {
    PairArgs a{};
    a.code = code; a.score = score; a.tables = static_cast<const char *>(tables); a.bias = bias; a.residual = residual; a.out = out;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do / (bf16 ? 64 : 32));
    a.row_bytes = (int)(Do * (bf16 ? 2 : 4)); a.touch = T * S * Do * (bf16 ? 2 : 4) <= (int64_t(256) << 20) ? 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (bf16) return np == 8 ? launch_pair<true, 8>(a, st) : launch_pair<true, 4>(a, st);
    switch (np) {
        case 16: return launch_pair<false, 16>(a, st);
        case 13: return launch_pair<false, 13>(a, st);
        case 8: return launch_pair<false, 8>(a, st);
        default: return launch_pair<false, 4>(a, st);
    }
}
