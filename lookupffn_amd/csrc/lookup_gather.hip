// The weighted gather-add as the LookupFFN layer issues it, table-major with the
// table staged in LDS:
//
//   out[b,:] = bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
//
// (PL/lookup.py:120-130 with the index offset of ":126" and the bias of ":108" folded
// in; the accumulation runs t = 0..T-1 as in gather_kernel_fp32.cu:41-43.)
//
// Work decomposition.  A workgroup of 1024 lanes owns a column slice of 256 bytes
// per row (64 fp32 or 128 bf16 columns) and a tile of 64*NP tokens, whose
// accumulators live in registers for the whole kernel (NP float4 per lane: 16
// lanes side by side cover the 256-byte row segment of one token, a wavefront
// covers 4 tokens at a time, NP passes cover the tile).  For every table the
// workgroup copies that table's slice (S rows x 256 bytes, 64 KiB for S = 256)
// into LDS once and all of its tokens read their rows from there: 16 lanes read
// 256 contiguous bytes, one conflict-free ds_read_b128.  The slices are
// double-buffered and copied global -> LDS directly (global_load_lds_dwordx4, no
// registers in between): the copy of table t+1 is issued before the LDS reads of
// table t and lands in the other buffer, one barrier per table.
//
// So each table slice is fetched once per 64*NP tokens instead of once per
// token, and the per-token row reads are LDS reads.  The (code, score) pairs are
// read 16 tables at a time, one table per lane of the 16-lane token group (four
// 8-bit codes packed per register), and handed to the group's lanes with a DPP
// row broadcast when their table comes up.
//
// blockIdx -> (slice, token tile) is XCD-aware: workgroups are dealt round-robin
// to the 8 XCDs, so block b runs on XCD b % 8; units are numbered so that the
// workgroups of one XCD share as few slices as possible and the slice they
// stream stays in that XCD's L2.
#include "lffn_common.h"


namespace {

constexpr int WG = 1024;
constexpr int SEG_VECS = 16;          // 16-byte vectors per row segment (256 bytes)
constexpr int CHUNK = 16;             // tables whose (code, score) a lane group holds at once
constexpr int MAX_S = 256;            // rows per table the LDS buffers are sized for
constexpr int XCDS = 8;

struct LdsGatherArgs {
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
    // Table split: a unit is (slice, part, tile); part p adds tables [p * part_tables, (p+1) * part_tables)
    // and, when nparts > 1, writes its sums without bias and residual to part_out[p][B][Do].
    int nparts, part_tables;
    float *part_out;
};

// Copy this lane's four vectors of a table slice straight from global memory into
// the LDS buffer `dst` (global_load_lds_dwordx4: lane i of a wavefront writes
// 16 bytes at the wavefront-uniform LDS address in M0 + 16*i, so a wavefront fills
// the 1 KiB of vectors q = wave*64 + [0,64) + 1024*i).  Nothing passes through
// registers.  Issued as inline assembly on purpose: the compiler would otherwise
// wait for the copy before the next LDS read of ANY address (it cannot tell the two
// buffers apart), which would serialise the copy with the pass loop.  The caller
// waits with vmcnt(0) before the barrier that publishes the buffer.
__device__ __forceinline__ void lds_dma16(const char *table, uint32_t lane_offset, uint32_t lds_byte_addr) {
    // scalar base + 32-bit lane offset: the lane offsets are the same for every table, so they
    // stay in registers and a table costs no address arithmetic on the vector unit
    // M0 is put back: the compiler reserves it for its own use and does not honour a clobber
    // declaration of it, so the statement must leave it as it found it
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(table), "s"(lds_byte_addr)
                 : "memory");
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const u32x4 *lds_vec_ptr;

// acc += (sc of lane N of the 16-lane row) * r in one instruction: the DPP row broadcast rides
// on the multiply-add's first operand instead of costing a move of its own (the compiler
// keeps the two apart when the broadcast value has several uses).
template <int N>
__device__ __forceinline__ void fmac_row_bcast(float &acc, float sc, float r) {
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(sc), "v"(r), "n"(N));
}

// Byte offsets, from the start of a table's slice, of the four vectors this lane copies.
struct CopyLanes {
    uint32_t off[4];
    uint32_t wbase;      // LDS byte offset of this wavefront's first vector inside a buffer
};

__device__ __forceinline__ CopyLanes copy_lanes(int row_bytes, int tid) {
    CopyLanes c;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        c.off[i] = (uint32_t)((tid >> 4) + i * (WG / SEG_VECS)) * (uint32_t)row_bytes + (tid & 15) * 16;
    c.wbase = (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6) * (64 * 16);      // scalar: never spilled with the vectors
    return c;
}

template <bool FULL>
__device__ __forceinline__ void copy_slice_to_lds(const char *tb, const CopyLanes &c, int tid, int buf_vecs,
                                                  uint32_t dst_byte_addr) {
    const uint32_t wbase = dst_byte_addr + c.wbase;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (FULL || tid + i * WG < buf_vecs) lds_dma16(tb, c.off[i], wbase + i * (WG * 16));
    }
}

template <bool BF16, int NP, bool FULL>
__global__ __launch_bounds__(WG) void lookup_gather_lds_kernel(LdsGatherArgs a) {
    constexpr int EPV = BF16 ? 8 : 4;
    static_assert(MAX_S * SEG_VECS == 4 * WG, "a lane copies four vectors of a slice");
    extern __shared__ uint4 lds[];                // 2 buffers of S * SEG_VECS vectors

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.ntiles * a.nslices * a.nparts) return;     // uniform over the workgroup
    const int slice = unit / (a.ntiles * a.nparts);
    const int part = (unit / a.ntiles) % a.nparts;
    const int tile = unit % a.ntiles;
    const int t_begin = part * a.part_tables;                  // a multiple of CHUNK
    const int t_end = min(a.T, t_begin + a.part_tables);
    const bool whole = a.nparts == 1;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int grp = lane >> 4;        // token within the wavefront's four
    const int j = lane & 15;          // 16-byte vector within the row segment
    const int64_t tok0 = int64_t(tile) * (64 * NP) + wave * 4 + grp;

    float acc[NP][EPV];
    {
        float b[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) b[e] = 0.f;
        if (a.bias && whole) {
            const float *bp = a.bias + (size_t)slice * (SEG_VECS * EPV) + j * EPV;
#pragma unroll
            for (int e = 0; e < EPV; ++e) b[e] = bp[e];
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[p][e] = b[e];
    }

    const int buf_vecs = a.S * SEG_VECS;
    const char *slice_base = a.tables + (size_t)slice * (SEG_VECS * 16);
    const size_t table_bytes = (size_t)a.S * a.row_bytes;

    const CopyLanes cl = copy_lanes(a.row_bytes, tid);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // Team touch.  The workgroups that share this slice (one per token tile, all on this XCD, in
    // step with each other) each pull a share of the 128-byte lines of the table after next into
    // the XCD's L2 while they read the current one: the copy issued one table later then finds the
    // slice in L2, whether it came from the memory-side cache or from HBM.  One 4-byte
    // global -> LDS load per line into a scratch area behind the buffers.  Only the 256-row form does it
    // (with 64-row tables it was measured 15% slower, not faster).
    const int touch_line = team_touch_line(a.S * 2, a.ntiles, tile, tid);
    const uint32_t touch_off = (uint32_t)(touch_line >> 1) * (uint32_t)a.row_bytes + (touch_line & 1) * 128;
    const uint32_t touch_dst = lds0 + (uint32_t)(2 * buf_vecs) * 16u;
    copy_slice_to_lds<FULL>(slice_base + (size_t)t_begin * table_bytes, cl, tid, buf_vecs,
                            lds0 + (uint32_t)((t_begin & 1) * buf_vecs) * 16u);
    __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0): this lane's copies have landed in LDS
    __syncthreads();

    // Codes are 8 bits (S <= 256).  bf16: four passes' codes per register.  fp32: two per
    // register, each already shifted to bits 8..15 of its 16-bit half, which is where a row
    // number sits in an LDS byte address (row * 256 + vector * 16 + buffer offset; S is a power
    // of two and the codes are masked, so the fields do not overlap): an address is then one
    // OR of a half-word with the lane's base, a single SDWA or AND-OR instruction.
    constexpr int NQ = BF16 ? (NP + 3) / 4 : (NP + 1) / 2;
    const unsigned lds_base = lds0 + j * 16;
    for (int t0 = t_begin; t0 < t_end; t0 += CHUNK) {
        // Lane j of a token group holds (code, score) of table t0 + j for each of
        // its NP tokens.  Addresses are clamped into range and the loads are
        // unconditional, so that all 2*NP of them are in flight together; what was
        // loaded from a clamped address is then zeroed.
        unsigned cd[NQ];
        float sc[NP];
        {
            const int tt = t0 + j;
            const int ttc = min(tt, t_end - 1);
            int craw[NP];
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const int64_t tok = min(tok0 + p * 64, a.B - 1);
                craw[p] = a.code[tok * a.T + ttc];
                sc[p] = a.score[tok * a.T + ttc];
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) cd[q] = 0u;
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const bool ok = (tok0 + p * 64 < a.B) && (tt < t_end);
                if constexpr (BF16)
                    cd[p / 4] |= unsigned(craw[p] & (a.S - 1)) << (8 * (p % 4));
                else
                    cd[p / 2] |= unsigned(craw[p] & (a.S - 1)) << (8 + 16 * (p % 2));
                sc[p] = ok ? sc[p] : 0.f;
            }
        }
        // The pairs must have landed before the table loop starts: inside it the
        // only loads in flight are the next table's slice, which is not waited
        // for until it is written to LDS at the end of an iteration.
#pragma unroll
        for (int q = 0; q < NQ; ++q) asm volatile("" : "+v"(cd[q]));
#pragma unroll
        for (int p = 0; p < NP; ++p) asm volatile("" : "+v"(sc[p]));

        const int nt = min(CHUNK, t_end - t0);
        // The 16 tables of the chunk, unrolled: table t0 + TT takes its codes and scores
        // from lane TT of each 16-lane token group with a DPP row broadcast (a vector-ALU
        // move), so that the only LDS traffic of the pass loop is the row reads.
        static_for<CHUNK>([&](auto tt_c) {
            constexpr int TT = decltype(tt_c)::value;
            if (TT < nt) {                                     // uniform
                const int t = t0 + TT;
                // next table's slice goes straight into the other buffer, which was last
                // read one table ago, before the previous barrier (the last iteration
                // re-copies the last table: harmless)
                copy_slice_to_lds<FULL>(slice_base + (size_t)min(t + 1, t_end - 1) * table_bytes, cl, tid, buf_vecs,
                                        lds0 + (uint32_t)(((t + 1) & 1) * buf_vecs) * 16u);
                if constexpr (FULL)
                    l2_touch(slice_base + (size_t)min(t + TOUCH_AHEAD, t_end - 1) * table_bytes, touch_off, touch_dst);
                const uint4 *buf = lds + (t & 1) * buf_vecs + j;
                const unsigned buf_addr = lds_base + (unsigned)((t & 1) * buf_vecs) * 16u;
                unsigned packed[NQ];
#pragma unroll
                for (int q = 0; q < NQ; ++q) packed[q] = (unsigned)row_broadcast<TT>((int)cd[q]);
                // passes in groups of at most GRP: a group's row reads are issued together
                // (GRP rows in flight per lane), then its fmas; the scheduling barriers keep
                // the compiler from merging groups, which would not fit the register file
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
                                r[i] = buf[row * SEG_VECS];
                            }
                        }
#pragma unroll
                        for (int i = 0; i < GRP; ++i) {
                            const int p = g0 + i;
                            if (p < NP) {
                                const float w = __int_as_float(row_broadcast<TT>(__float_as_int(sc[p])));
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
                                const unsigned half = (p % 2) ? (packed[p / 2] >> 16) : (packed[p / 2] & 0xFFFFu);
                                r[i] = *(lds_vec_ptr)(uintptr_t)(half | buf_addr);
                            }
                        }
#pragma unroll
                        for (int i = 0; i < GRP; ++i) {
                            const int p = g0 + i;
                            if (p < NP) {
                                fmac_row_bcast<TT>(acc[p][0], sc[p], __uint_as_float(r[i].x));
                                fmac_row_bcast<TT>(acc[p][1], sc[p], __uint_as_float(r[i].y));
                                fmac_row_bcast<TT>(acc[p][2], sc[p], __uint_as_float(r[i].z));
                                fmac_row_bcast<TT>(acc[p][3], sc[p], __uint_as_float(r[i].w));
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                __builtin_amdgcn_s_waitcnt(FULL ? WAIT_VMCNT_1 : WAIT_VMCNT_0);     // vmcnt(1): the copy issued above has landed; the touch,
                                                        // issued after it, may still be out
                __syncthreads();
            }
        });
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);         // nothing may still be writing this workgroup's LDS when it ends

#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int64_t tok = tok0 + p * 64;
        if (tok < a.B) {
            const size_t off = tok * a.Do + (size_t)slice * (SEG_VECS * EPV) + j * EPV;
            float *o = (whole ? a.out : a.part_out + (size_t)part * a.B * a.Do) + off;
#pragma unroll
            for (int q = 0; q < EPV / 4; ++q) {
                float4 v = make_float4(acc[p][4 * q], acc[p][4 * q + 1], acc[p][4 * q + 2], acc[p][4 * q + 3]);
                if (a.residual && whole) {
                    const float4 rr = *reinterpret_cast<const float4 *>(a.residual + off + 4 * q);
                    v.x += rr.x; v.y += rr.y; v.z += rr.z; v.w += rr.w;
                }
                *reinterpret_cast<float4 *>(o + 4 * q) = v;
            }
        }
    }
}

template <bool BF16, int NP, bool FULL>
int launch_lds_full(LdsGatherArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + 64 * NP - 1) / (64 * NP));
    const int units = a.ntiles * a.nslices * a.nparts;
    a.per_xcd = (units + XCDS - 1) / XCDS;
    const size_t lds_bytes = size_t(2) * a.S * SEG_VECS * 16 + TOUCH_SINK_BYTES;      // two buffers + the touches' scratch
    auto kern = lookup_gather_lds_kernel<BF16, NP, FULL>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

template <bool BF16, int NP>
int launch_lds(const LdsGatherArgs &a, hipStream_t stream) {
    return a.S == MAX_S ? launch_lds_full<BF16, NP, true>(a, stream) : launch_lds_full<BF16, NP, false>(a, stream);
}

// Which kernel a shape gets.
//   kind 0  token-major kernel (gather.hip): small batches, S > 256
//   kind 1  one table per LDS buffer (this file): 256-byte slices, 64*np tokens per workgroup
//   kind 2  two tables per LDS buffer (lookup_gather_pair.hip): 128-byte slices, 128*np tokens
// The LDS forms need the table to fit the buffers (S <= 256), rows that split into
// whole slices, and enough (token tile, slice) units to occupy most of the 256 CUs
// at the smallest tile.  Workgroups run one per CU in ceil(units / 256) rounds; the
// time of a round is T tables times a per-table cost measured on MI355X for each
// built tile size (microseconds, tables that fit the 256 MB Infinity Cache; larger
// table sets cost BIG times more).  The cheapest predicted time wins.
struct GatherPlan {
    int kind, np;
    double us;             // predicted time
    int tile = 0;          // kind 3: tokens per workgroup (a multiple of 16 in (256 * (np - 1), 256 * np])
};

// The four-lanes-per-token kernel: microseconds per table pair of a workgroup = a fixed part (the 64 KB
// copy, the records, the barrier) + a part per pass of 256 tokens, a short last pass counting by its share
// of 256 tokens.  Measured on MI355X with 10 tiles x 24 slices of fp32 rows (128 x 256 x 768 tables, in the
// memory-side cache): 1.23, 1.33, 1.52, 1.68, 1.85 us at 4 .. 8 passes, 1.58 at 6.44, 1.19 at 3.06 (the copies
// bound the step below about 1.19 us); 512 x 256 x 1024 tables (537 MB, beyond the cache) cost 0.13 to 0.3 us
// more per pair.  A pass over 16-bit rows covers twice the columns and is bound by the vector ALU.
constexpr double QUAD_MARGIN = 0.92;      // the form must promise this much to be worth its workspace
// indexed by LFFN_ROWS_*: fp32, bfloat16, half
constexpr double QUAD_US_PER_PAIR[3] = {0.53, 0.56, 0.61};
constexpr double QUAD_US_PER_PAIR_PASS[3] = {0.165, 0.36, 0.275};
constexpr double QUAD_US_PER_PAIR_MIN = 1.19;

template <bool BF16>
GatherPlan plan_gather(int64_t B, int64_t T, int64_t S, int64_t Do) {
    // token-major: every token reads its T rows from L2 / Infinity Cache, measured 9 TB/s
    GatherPlan best{0, 0, double(B) * double(T) * double(Do) * (BF16 ? 2 : 4) / 9e6 + 5.0};
    if (S > MAX_S || T < 4 || B * T >= (int64_t(1) << 31)) return best;
    // us_per_table: tables that fit the cache (measured at 128 x 256 x 768 fp32, 16384 tokens); us_big:
    // table sets beyond it (512 x 256 x 1024: 537 MB fp32, 268 MB bf16).  All with the team touch in the kernels.
    struct Option { int kind, np; double us_per_table, us_big; };
    static const Option f32_opts[] = {{1, 4, 1.16, 1.45}, {1, 8, 1.05, 1.13}, {1, 13, 1.29, 1.48}, {1, 16, 1.50, 1.56},
                                      {2, 4, 0.74, 1.00}, {2, 8, 0.98, 1.31}, {2, 13, 1.41, 1.31}, {2, 16, 1.77, 1.77}};
    static const Option bf16_opts[] = {{1, 4, 1.10, 1.51}, {1, 8, 1.24, 1.34}, {2, 4, 0.87, 0.88}, {2, 8, 1.44, 1.37}};
    const Option *opts = BF16 ? bf16_opts : f32_opts;
    const int nopts = BF16 ? 4 : 8;
    const bool big = double(T) * double(S) * double(Do) * (BF16 ? 2 : 4) > 200e6;
    double best_us = 1e300;
    for (int k = 0; k < nopts; ++k) {
        const Option &o = opts[k];
        const int cols = (o.kind == 1 ? 256 : 128) / (BF16 ? 2 : 4);
        const int tok = (o.kind == 1 ? 64 : 128) * o.np;
        if (Do % cols != 0) continue;
        const int64_t nslices = Do / cols;
        // enough units at the smallest tile of this form to be worth staging tables at all
        if (((B + tok / o.np * 4 - 1) / (tok / o.np * 4)) * nslices < 192) continue;
        if (B * nslices > (int64_t(1) << 30)) continue;
        const int64_t tiles = (B + tok - 1) / tok;
        const int64_t rounds = (tiles * nslices + 255) / 256;
        const double us = double(rounds) * double(T) * (big ? o.us_big : o.us_per_table);
        if (us < best_us) { best_us = us; best = GatherPlan{o.kind, o.np, us}; }
    }
    return best;
}

// The four-lanes-per-token form (lookup_gather_quad.hip; needs a workspace for its record stream): 128-byte
// slices, 256*np tokens per workgroup, one round of 256 workgroups costs T/2 pairs x the measured cost of a
// pair at np passes; plus the packing kernel when the records come from [B, T] codes and scores (`pack`).
// 256-row tables and an even number of them only.
GatherPlan plan_quad(int fmt, int64_t B, int64_t T, int64_t S, int64_t Do, bool pack = true) {
    GatherPlan best{0, 0, 1e300};
    const int esz = fmt == LFFN_ROWS_F32 ? 4 : 2;
    const int cols = 128 / esz;
    if (S != MAX_S || T < 8 || T % 2 != 0 || T > (1 << 20) || Do % cols != 0 || B * T >= (int64_t(1) << 31) ||
        2 * S * Do * esz >= (int64_t(1) << 32))
        return best;
    const int64_t nslices = Do / cols;
    if (((B + 1023) / 1024) * nslices < 192 || B * nslices > (int64_t(1) << 30)) return best;
    const double per_pass = QUAD_US_PER_PAIR_PASS[fmt], fixed = QUAD_US_PER_PAIR[fmt];
    for (int np : {4, 5, 6, 7, 8}) {
        if (!lffn_internal_quad_np_built(fmt, np)) continue;
        // Tiles of np passes, the tokens spread evenly over them in groups of 16: from as few tiles as np full
        // passes allow up to as many as still need np passes.  The last pass is then short for some of a
        // workgroup's wavefronts, which leave it out: it costs its share of a pass.  More, shorter tiles can
        // fill workgroup slots that fewer, fuller ones leave
        // idle (16384 tokens x 12 slices of 16-bit rows: 21 tiles of 784 tokens = 252 workgroups, not 16 x 12 = 192).
        const int64_t tiles_min = (B + 256 * np - 1) / (256 * np);
        for (int64_t tiles = tiles_min; tiles <= tiles_min + 32; ++tiles) {       // (filling a round of 256 workgroups never takes more)
            const int64_t tile = (((B + tiles - 1) / tiles) + 15) & ~int64_t(15);
            if (tile <= 256 * (np - 1)) break;
            const int64_t rem = tile - 256 * (np - 1);                                 // tokens in the last pass: 16 .. 256
            const double passes = double(np - 1) + double(rem) / 256.0;
            const int64_t rounds = (tiles * nslices + 255) / 256;
            const double pair_us = fixed + passes * per_pass;
            const double us = double(rounds) * double(T / 2) * (pair_us > QUAD_US_PER_PAIR_MIN ? pair_us : QUAD_US_PER_PAIR_MIN) +
                              (pack ? double(B) * double(T) * 14.0 / 3e6 + 4.0 : 0.0);     // packing: 8 bytes read, 6 written per (token, table)
            if (us < best.us) best = GatherPlan{3, np, us, (int)tile};
        }
    }
    return best;
}

// Table split (needs a workspace): for a few thousand tokens there are too few (tile, slice) units
// to fill the chip at the large tiles that make the staging pay, and the token-major kernel reads
// every row from L2.  nparts workgroups share a unit, each adding a range of part_tables tables
// (a multiple of the 16-table chunk) into its own partial output; a second kernel adds the
// partials in a fixed order together with bias and residual.
struct SplitPlan {
    int np, nparts, part_tables;
    double us;
};

template <bool BF16>
SplitPlan plan_split(int64_t B, int64_t T, int64_t S, int64_t Do) {
    SplitPlan best{0, 1, (int)T, 1e300};
    const int cols = BF16 ? 128 : 64;
    if (S > MAX_S || T < 32 || Do % cols != 0 || B < 256 || B * T >= (int64_t(1) << 31)) return best;
    struct Option { int np; double us_per_table; };
    static const Option f32_opts[] = {{4, 1.16}, {8, 1.05}, {13, 1.29}};
    static const Option bf16_opts[] = {{4, 1.10}, {8, 1.24}};
    const Option *opts = BF16 ? bf16_opts : f32_opts;
    const int nopts = BF16 ? 2 : 3;
    const int64_t nslices = Do / cols;
    const bool big = double(T) * double(S) * double(Do) * (BF16 ? 2 : 4) > 200e6;
    for (int k = 0; k < nopts; ++k) {
        const int64_t tiles = (B + 64 * opts[k].np - 1) / (64 * opts[k].np);
        for (int nparts = 2; nparts <= 16; nparts *= 2) {
            const int64_t part_tables = ((T + nparts - 1) / nparts + CHUNK - 1) / CHUNK * CHUNK;
            if (part_tables * (nparts - 1) >= T) continue;            // the last part would be empty
            const int64_t units = tiles * nslices * nparts;
            if (units > (int64_t(1) << 24)) continue;
            const int64_t rounds = (units + 255) / 256;
            // partials written and read once, the result written: about 4 TB/s for buffers of this size
            const double reduce_us = double(2 * nparts + 1) * double(B) * double(Do) * 4.0 / 4e6 + 6.0;
            const double us = double(rounds) * double(part_tables) * opts[k].us_per_table * (big ? 1.3 : 1.0) + reduce_us;
            if (us < best.us) best = SplitPlan{opts[k].np, nparts, (int)part_tables, us};
        }
    }
    return best;
}

__global__ __launch_bounds__(256) void gather_parts_reduce_kernel(const float *parts, int nparts, const float *bias,
                                                                  const float *residual, float *out, int64_t B, int Do) {
    const int64_t n4 = B * Do / 4;
    const int q = Do / 4;
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < n4; i += int64_t(gridDim.x) * 256) {
        float4 v = bias ? reinterpret_cast<const float4 *>(bias)[i % q] : make_float4(0.f, 0.f, 0.f, 0.f);
        for (int p = 0; p < nparts; ++p) {                       // parts in table order, as the one-part kernel adds them
            const float4 t = reinterpret_cast<const float4 *>(parts)[(int64_t)p * n4 + i];
            v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
        }
        if (residual) {
            const float4 r = reinterpret_cast<const float4 *>(residual)[i];
            v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
        }
        reinterpret_cast<float4 *>(out)[i] = v;
    }
}

// Is (kind, np) a kernel that is built, and does the shape meet its preconditions?
// Many tokens and tables that fit the 256 MB Infinity Cache are taken in pieces: in one launch over
// all tokens the outputs, codes and scores streaming through push the tables out of the caches and
// every round of workgroups fetches its slices from further away (131072 tokens at 128 x 256 x 768
// fp32: 1745 us in one launch, 1357 in pieces).  A piece is what one round of 256 workgroups takes at
// the tile size that is cheapest for the whole batch: 21 tiles of 832 tokens at 768 columns, 32
// tiles of 1024 tokens at 512 columns (32768 tokens: 295 -> 211 us against pieces of 16384).
// Returns the tokens per piece (a multiple of 64), or B when the batch goes in one launch.
template <bool BF16>
int64_t gather_pieces(int64_t B, int64_t T, int64_t S, int64_t Do) {
    if (B < 2 * 16384 || double(T) * double(S) * double(Do) * (BF16 ? 2 : 4) > double(int64_t(192) << 20)) return B;
    const GatherPlan whole = plan_gather<BF16>(B, T, S, Do);
    if (whole.kind == 0) return B;
    double best_us = 1e300;
    int64_t best_each = B;
    for (int kind = 1; kind <= 2; ++kind) {
        const int cols = (kind == 1 ? 256 : 128) / (BF16 ? 2 : 4);
        if (Do % cols != 0) continue;
        const int64_t nslices = Do / cols;
        if (nslices > 256) continue;
        for (int np : {4, 8, 13, 16}) {
            if (BF16 && np > 8) continue;
            const int64_t piece = (256 / nslices) * int64_t(kind == 1 ? 64 : 128) * np;     // one round
            const int64_t n = (B + piece - 1) / piece;
            const int64_t each = ((B + n - 1) / n + 63) & ~int64_t(63);
            const GatherPlan p = plan_gather<BF16>(each, T, S, Do);                        // what a piece will run as
            const double us = double(n) * (p.us + 4.0);                                    // + a launch
            if (us < best_us) { best_us = us; best_each = each; }
        }
    }
    // two rounds still go faster in one launch (32768 tokens, bf16 rows of 1024: 339 us against 382 in two
    // pieces; fp32 rows of 768: 345 either way); from three rounds on the pieces win (65536 tokens: 693
    // against 735, 131072: 1357 against 1745)
    if ((B + best_each - 1) / best_each <= 2) return B;
    return best_each;
}

// The four-lanes-per-token form over the whole batch (one launch, however many tokens: its tables come
// through the touch by turns, so it has no use for pieces), if it promises to beat what the other forms
// get for the batch by QUAD_MARGIN: pieces, the one-launch LDS forms, the table split.  kind 0 otherwise.
template <bool BF16>
GatherPlan choose_quad(int64_t B, int64_t T, int64_t S, int64_t Do, bool pack = true) {
    const GatherPlan none{0, 0, 1e300};
    const GatherPlan qp = plan_quad(BF16 ? LFFN_ROWS_BF16 : LFFN_ROWS_F32, B, T, S, Do, pack);
    if (qp.kind != 3) return none;
    double other;
    const int64_t each = gather_pieces<BF16>(B, T, S, Do);
    if (each < B) {
        other = double((B + each - 1) / each) * (plan_gather<BF16>(each, T, S, Do).us + 4.0);
    } else {
        other = plan_gather<BF16>(B, T, S, Do).us;
        const SplitPlan sp = plan_split<BF16>(B, T, S, Do);
        if (sp.nparts > 1 && sp.us < other) other = sp.us;
    }
    return qp.us < QUAD_MARGIN * other ? qp : none;
}

// four lanes per token: a tile (tokens per workgroup: whole groups of 16, its last pass not empty) whose number
// of passes is built for the row format, 256-row tables, an even number of them, whole 128-byte slices, 32-bit
// offsets inside a table pair
bool quad_plan_is_valid(int fmt, int64_t tile, int64_t B, int64_t T, int64_t S, int64_t Do) {
    const int esz = fmt == LFFN_ROWS_F32 ? 4 : 2;
    const int cols = 128 / esz;
    const int np = lffn_internal_quad_passes(fmt, tile);
    return np != 0 && tile > 256 * (np - 1) && S == MAX_S && T >= 2 && T % 2 == 0 && T <= (1 << 20) &&
           Do % cols == 0 && B * T < (int64_t(1) << 31) && 2 * S * Do * esz < (int64_t(1) << 32) &&
           B * (Do / cols) <= (int64_t(1) << 30);
}

template <bool BF16>
bool plan_is_valid(const GatherPlan &p, int64_t B, int64_t T, int64_t S, int64_t Do) {
    if (p.kind == 0) return true;
    if (p.kind == 3)        // four lanes per token
        return quad_plan_is_valid(BF16 ? LFFN_ROWS_BF16 : LFFN_ROWS_F32, p.tile, B, T, S, Do);
    if (p.kind != 1 && p.kind != 2) return false;
    const bool np_ok = BF16 ? (p.np == 4 || p.np == 8) : (p.np == 4 || p.np == 8 || p.np == 13 || p.np == 16);
    const int cols = (p.kind == 1 ? 256 : 128) / (BF16 ? 2 : 4);
    return np_ok && S <= MAX_S && T >= 1 && Do % cols == 0 && B * T < (int64_t(1) << 31) &&
           B * (Do / cols) <= (int64_t(1) << 30);
}

// kind_req < 0: choose the kernel with plan_gather; otherwise run exactly the
// requested kernel (kind_req tables per buffer, tokens_req tokens per workgroup).
template <bool BF16>
int lookup_gather_entry(const int32_t *code, const float *score, const void *tables, const float *bias,
                        const float *residual, float *out, int64_t B, int64_t T, int64_t S, int64_t Do, int kind_req, int tokens_req,
                        void *stream, void *workspace = nullptr, int64_t workspace_bytes = 0) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(S) && S <= (1 << 24) && T * S <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(Do % 64 == 0 && Do <= (1 << 20) && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(tables && out && ((code && score) || B * T == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(tables) && lffn_aligned16(out) && (!bias || lffn_aligned16(bias)) &&
                     (!residual || lffn_aligned16(residual)), LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    if (kind_req < 0 && workspace) {
        // (the packing kernel reads a table pair's codes and scores as 8-byte vectors)
        const GatherPlan qp = choose_quad<BF16>(B, T, S, Do);
        if (qp.kind == 3 && workspace_bytes >= lffn_internal_quad_stream_bytes(B, T) && (uintptr_t)code % 8 == 0 &&
            (uintptr_t)score % 8 == 0) {
            LFFN_REQUIRE(lffn_aligned16(workspace), LFFN_ERR_BAD_ARG);
            return lffn_internal_lookup_gather_quad(code, score, tables, bias, residual, out, B, T, S, Do,
                                                    BF16 ? LFFN_ROWS_BF16 : LFFN_ROWS_F32, qp.tile, workspace, stream);
        }
    }
    // Many tokens, tables that fit the 256 MB Infinity Cache: take the tokens in pieces, one launch
    // after the other (gather_pieces).
    const int64_t each = kind_req < 0 ? gather_pieces<BF16>(B, T, S, Do) : B;
    if (each < B) {
        for (int64_t b0 = 0; b0 < B; b0 += each) {
            // (a workspace serves every piece in turn: the launches are ordered on the stream)
            const int rc = lookup_gather_entry<BF16>(code + b0 * T, score + b0 * T, tables, bias,
                                                     residual ? residual + b0 * Do : nullptr, out + b0 * Do,
                                                     B - b0 < each ? B - b0 : each, T, S, Do, -1, 0, stream, workspace,
                                                     workspace_bytes);
            if (rc != LFFN_OK) return rc;
        }
        return LFFN_OK;
    }
    GatherPlan plan;
    void *quad_ws = nullptr;
    if (kind_req < 0) {
        plan = plan_gather<BF16>(B, T, S, Do);
        if (workspace) {
            const SplitPlan sp = plan_split<BF16>(B, T, S, Do);
            if (sp.nparts > 1 && sp.us < 0.85 * plan.us && workspace_bytes >= int64_t(sp.nparts) * B * Do * 4) {
                LFFN_REQUIRE(lffn_aligned16(workspace), LFFN_ERR_BAD_ARG);
                LdsGatherArgs a{};
                a.code = code; a.score = score; a.tables = static_cast<const char *>(tables); a.bias = nullptr;
                a.residual = nullptr; a.out = out;
                a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
                a.nslices = (int)(Do / (BF16 ? 128 : 64));
                a.row_bytes = (int)(Do * (BF16 ? 2 : 4));
                a.nparts = sp.nparts; a.part_tables = sp.part_tables; a.part_out = static_cast<float *>(workspace);
                hipStream_t st = static_cast<hipStream_t>(stream);
                int rc;
                if constexpr (BF16) {
                    rc = sp.np == 8 ? launch_lds<true, 8>(a, st) : launch_lds<true, 4>(a, st);
                } else {
                    rc = sp.np == 13 ? launch_lds<false, 13>(a, st)
                                     : (sp.np == 8 ? launch_lds<false, 8>(a, st) : launch_lds<false, 4>(a, st));
                }
                if (rc != LFFN_OK) return rc;
                const int64_t blocks = (B * Do / 4 + 255) / 256;
                hipLaunchKernelGGL(gather_parts_reduce_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, st,
                                   a.part_out, sp.nparts, bias, residual, out, B, (int)Do);
                return lffn_launch_status();
            }
        }
    } else {
        plan.kind = kind_req;
        if (kind_req == 3) {          // any whole number of 16-token groups; the passes follow from it
            LFFN_REQUIRE(tokens_req > 0 && tokens_req % 16 == 0, LFFN_ERR_BAD_ARG);
            plan.tile = tokens_req;
            plan.np = lffn_internal_quad_passes(BF16 ? LFFN_ROWS_BF16 : LFFN_ROWS_F32, tokens_req);
        } else {
            const int per_np = kind_req == 1 ? 64 : 128;
            plan.np = kind_req == 0 ? 0 : tokens_req / per_np;
            LFFN_REQUIRE(kind_req == 0 || (tokens_req > 0 && tokens_req % per_np == 0), LFFN_ERR_BAD_ARG);
        }
        LFFN_REQUIRE(plan_is_valid<BF16>(plan, B, T, S, Do), LFFN_ERR_UNSUPPORTED);
        if (plan.kind == 3) {       // needs the record stream's workspace
            LFFN_REQUIRE(workspace && workspace_bytes >= lffn_internal_quad_stream_bytes(B, T), LFFN_ERR_UNSUPPORTED);
            LFFN_REQUIRE(lffn_aligned16(workspace) && (uintptr_t)code % 8 == 0 && (uintptr_t)score % 8 == 0, LFFN_ERR_BAD_ARG);
            quad_ws = workspace;
        }
    }
    if (plan.kind == 0)
        return lffn_internal_lookup_gather_token_major(code, score, tables, bias, residual, out, B, T, S, Do, BF16, stream);
    if (plan.kind == 3)
        return lffn_internal_lookup_gather_quad(code, score, tables, bias, residual, out, B, T, S, Do,
                                                BF16 ? LFFN_ROWS_BF16 : LFFN_ROWS_F32, plan.tile, quad_ws, stream);
    if (plan.kind == 2)
        return lffn_internal_lookup_gather_pair(code, score, tables, bias, residual, out, B, T, S, Do, BF16, plan.np, stream);
    const int np = plan.np;
    LdsGatherArgs a{};
    a.code = code; a.score = score; a.tables = static_cast<const char *>(tables); a.bias = bias; a.residual = residual; a.out = out;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do / (BF16 ? 128 : 64));
    a.row_bytes = (int)(Do * (BF16 ? 2 : 4));
    a.nparts = 1; a.part_tables = (int)T; a.part_out = nullptr;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if constexpr (BF16) {
        return np == 8 ? launch_lds<true, 8>(a, st) : launch_lds<true, 4>(a, st);
    } else {
        switch (np) {
            case 16: return launch_lds<false, 16>(a, st);
            case 13: return launch_lds<false, 13>(a, st);
            case 8: return launch_lds<false, 8>(a, st);
            default: return launch_lds<false, 4>(a, st);
        }
    }
}

// Half rows (the row format of the reference's reduced-precision gather, gather_kernel_fp16.cu:6-62; fp32
// sums here): the four-lanes-per-token kernel where the shape qualifies and the caller brings a workspace for
// the records, the token-major kernel otherwise.  kind_req < 0: choose; 0 or 3: exactly that kernel.
int lookup_gather_entry_f16(const int32_t *code, const float *score, const void *tables, const float *bias,
                            const float *residual, float *out, int64_t B, int64_t T, int64_t S, int64_t Do, int kind_req,
                            int tokens_req, void *stream, void *workspace, int64_t workspace_bytes) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(S) && S <= (1 << 24) && T * S <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(Do % 64 == 0 && Do <= (1 << 20) && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(tables && out && ((code && score) || B * T == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(tables) && lffn_aligned16(out) && (!bias || lffn_aligned16(bias)) &&
                     (!residual || lffn_aligned16(residual)), LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    int tile = 0;
    if (kind_req < 0) {
        const GatherPlan qp = plan_quad(LFFN_ROWS_F16, B, T, S, Do);
        const double token_major_us = double(B) * double(T) * double(Do) * 2 / 9e6 + 5.0;
        if (qp.kind == 3 && qp.us < QUAD_MARGIN * token_major_us && workspace &&
            workspace_bytes >= lffn_internal_quad_stream_bytes(B, T) && lffn_aligned16(workspace) &&
            (uintptr_t)code % 8 == 0 && (uintptr_t)score % 8 == 0)
            tile = qp.tile;
    } else if (kind_req == 3) {
        LFFN_REQUIRE(tokens_req > 0 && tokens_req % 16 == 0, LFFN_ERR_BAD_ARG);
        tile = tokens_req;
        LFFN_REQUIRE(quad_plan_is_valid(LFFN_ROWS_F16, tile, B, T, S, Do), LFFN_ERR_UNSUPPORTED);
        LFFN_REQUIRE(workspace && workspace_bytes >= lffn_internal_quad_stream_bytes(B, T), LFFN_ERR_UNSUPPORTED);
        LFFN_REQUIRE(lffn_aligned16(workspace) && (uintptr_t)code % 8 == 0 && (uintptr_t)score % 8 == 0, LFFN_ERR_BAD_ARG);
    } else {
        LFFN_REQUIRE(kind_req == 0, LFFN_ERR_UNSUPPORTED);       // the 16- and 8-lane LDS kernels are not built for half rows
    }
    if (tile)
        return lffn_internal_lookup_gather_quad(code, score, tables, bias, residual, out, B, T, S, Do, LFFN_ROWS_F16, tile,
                                                workspace, stream);
    return lffn_internal_lookup_gather_token_major(code, score, tables, bias, residual, out, B, T, S, Do, LFFN_ROWS_F16, stream);
}

}  // namespace

extern "C" int lffn_lookup_gather_f32(const int32_t *code, const float *score, const float *tables,
                                      const float *bias, float *out,
                                      int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    return lookup_gather_entry<false>(code, score, tables, bias, nullptr, out, B, T, S, Do, -1, 0, stream);
}

extern "C" int lffn_lookup_gather_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                       const float *bias, float *out,
                                       int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    return lookup_gather_entry<true>(code, score, tables, bias, nullptr, out, B, T, S, Do, -1, 0, stream);
}

extern "C" int lffn_lookup_gather_residual_f32(const int32_t *code, const float *score, const float *tables,
                                               const float *bias, const float *residual, float *out,
                                               int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    return lookup_gather_entry<false>(code, score, tables, bias, residual, out, B, T, S, Do, -1, 0, stream);
}

extern "C" int lffn_lookup_gather_residual_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                                const float *bias, const float *residual, float *out,
                                                int64_t B, int64_t T, int64_t S, int64_t Do, void *stream) {
    return lookup_gather_entry<true>(code, score, tables, bias, residual, out, B, T, S, Do, -1, 0, stream);
}

extern "C" int lffn_lookup_gather_workspace_bytes(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format,
                                                  int64_t *bytes) {
    LFFN_REQUIRE(bytes && row_format >= 0 && row_format <= 2, LFFN_ERR_BAD_ARG);
    *bytes = 0;
    if (B < 1 || T < 1 || Do < 1 || !lffn_is_pow2(S) || Do % 64 != 0 || B * T >= (int64_t(1) << 31)) return LFFN_OK;
    if (row_format == LFFN_ROWS_F16) {
        const GatherPlan qp = plan_quad(LFFN_ROWS_F16, B, T, S, Do);
        if (qp.kind == 3 && qp.us < QUAD_MARGIN * (double(B) * double(T) * double(Do) * 2 / 9e6 + 5.0))
            *bytes = lffn_internal_quad_stream_bytes(B, T);
        return LFFN_OK;
    }
    const bool bf16 = row_format == LFFN_ROWS_BF16;
    if ((bf16 ? choose_quad<true>(B, T, S, Do) : choose_quad<false>(B, T, S, Do)).kind == 3) {
        *bytes = lffn_internal_quad_stream_bytes(B, T);
        return LFFN_OK;
    }
    const int64_t each = bf16 ? gather_pieces<true>(B, T, S, Do) : gather_pieces<false>(B, T, S, Do);
    if (each < B) return LFFN_OK;                              // taken in pieces, none of which is split
    const GatherPlan plan = bf16 ? plan_gather<true>(B, T, S, Do) : plan_gather<false>(B, T, S, Do);
    const SplitPlan sp = bf16 ? plan_split<true>(B, T, S, Do) : plan_split<false>(B, T, S, Do);
    if (sp.nparts > 1 && sp.us < 0.85 * plan.us) *bytes = int64_t(sp.nparts) * B * Do * 4;
    return LFFN_OK;
}

// What the workspace entry points run for a shape when given a workspace of workspace_bytes: the tokens per
// workgroup, and in *form 0 (token-major), 1 or 2 (tables per LDS buffer), 3 (four lanes per token, record
// stream in the workspace) or 4 (table split: partial outputs in the workspace, 64-token passes of form 1).
// A batch that is taken in pieces reports the form of a piece.
extern "C" int lffn_lookup_gather_ws_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format,
                                          int64_t workspace_bytes, int32_t *form) {
    if (B < 0 || T < 0 || Do < 1 || !lffn_is_pow2(S) || Do % 64 != 0 || row_format < 0 || row_format > 2 || workspace_bytes < 0)
        return LFFN_ERR_BAD_ARG;
    int kind = 0, tokens = 0;
    if (B >= 1 && T >= 1 && B * T < (int64_t(1) << 31)) {
        const bool room = workspace_bytes >= lffn_internal_quad_stream_bytes(B, T);
        if (row_format == LFFN_ROWS_F16) {
            const GatherPlan qp = plan_quad(LFFN_ROWS_F16, B, T, S, Do);
            if (qp.kind == 3 && room && qp.us < QUAD_MARGIN * (double(B) * double(T) * double(Do) * 2 / 9e6 + 5.0)) {
                kind = 3; tokens = qp.tile;
            }
        } else {
            const bool bf16 = row_format == LFFN_ROWS_BF16;
            const GatherPlan qp = bf16 ? choose_quad<true>(B, T, S, Do) : choose_quad<false>(B, T, S, Do);
            if (qp.kind == 3 && room) {
                kind = 3; tokens = qp.tile;
            } else {
                int64_t each = bf16 ? gather_pieces<true>(B, T, S, Do) : gather_pieces<false>(B, T, S, Do);
                if (each > B) each = B;
                const GatherPlan plan = bf16 ? plan_gather<true>(each, T, S, Do) : plan_gather<false>(each, T, S, Do);
                const SplitPlan sp = bf16 ? plan_split<true>(each, T, S, Do) : plan_split<false>(each, T, S, Do);
                if (each == B && sp.nparts > 1 && sp.us < 0.85 * plan.us && workspace_bytes >= int64_t(sp.nparts) * B * Do * 4) {
                    kind = 4; tokens = 64 * sp.np;
                } else {
                    kind = plan.kind;
                    tokens = plan.kind == 0 ? 0 : (plan.kind == 1 ? 64 : 128) * plan.np;
                }
            }
        }
    }
    if (form) *form = kind;
    return tokens;
}

extern "C" int lffn_lookup_gather_ws_f32(const int32_t *code, const float *score, const float *tables,
                                         const float *bias, const float *residual, float *out, void *workspace,
                                         int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                         void *stream) {
    LFFN_REQUIRE(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), LFFN_ERR_BAD_ARG);
    return lookup_gather_entry<false>(code, score, tables, bias, residual, out, B, T, S, Do, -1, 0, stream, workspace,
                                      workspace_bytes);
}

extern "C" int lffn_lookup_gather_ws_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                          const float *bias, const float *residual, float *out, void *workspace,
                                          int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                          void *stream) {
    LFFN_REQUIRE(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), LFFN_ERR_BAD_ARG);
    return lookup_gather_entry<true>(code, score, tables, bias, residual, out, B, T, S, Do, -1, 0, stream, workspace,
                                     workspace_bytes);
}

extern "C" int lffn_lookup_gather_ws_f16(const int32_t *code, const float *score, const uint16_t *tables,
                                         const float *bias, const float *residual, float *out, void *workspace,
                                         int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                         void *stream) {
    LFFN_REQUIRE(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), LFFN_ERR_BAD_ARG);
    return lookup_gather_entry_f16(code, score, tables, bias, residual, out, B, T, S, Do, -1, 0, stream, workspace,
                                   workspace_bytes);
}

extern "C" int lffn_lookup_gather_ws_planned_rows(const int32_t *code, const float *score, const void *tables,
                                                  const float *bias, const float *residual, float *out, void *workspace,
                                                  int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                                  int32_t row_format, int32_t tables_per_buffer,
                                                  int32_t tokens_per_workgroup, void *stream) {
    LFFN_REQUIRE(tables_per_buffer >= 0 && row_format >= 0 && row_format <= 2, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), LFFN_ERR_BAD_ARG);
    if (row_format == LFFN_ROWS_F16)
        return lookup_gather_entry_f16(code, score, tables, bias, residual, out, B, T, S, Do, tables_per_buffer,
                                       tokens_per_workgroup, stream, workspace, workspace_bytes);
    if (row_format == LFFN_ROWS_BF16)
        return lookup_gather_entry<true>(code, score, tables, bias, residual, out, B, T, S, Do, tables_per_buffer,
                                         tokens_per_workgroup, stream, workspace, workspace_bytes);
    return lookup_gather_entry<false>(code, score, tables, bias, residual, out, B, T, S, Do, tables_per_buffer,
                                      tokens_per_workgroup, stream, workspace, workspace_bytes);
}

extern "C" int lffn_lookup_gather_planned_f32(const int32_t *code, const float *score, const float *tables,
                                              const float *bias, float *out,
                                              int64_t B, int64_t T, int64_t S, int64_t Do,
                                              int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream) {
    LFFN_REQUIRE(tables_per_buffer >= 0, LFFN_ERR_BAD_ARG);
    return lookup_gather_entry<false>(code, score, tables, bias, nullptr, out, B, T, S, Do, tables_per_buffer,
                                      tokens_per_workgroup, stream);
}

extern "C" int lffn_lookup_gather_ws_planned_f32(const int32_t *code, const float *score, const float *tables,
                                                 const float *bias, const float *residual, float *out, void *workspace,
                                                 int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                                 int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream) {
    LFFN_REQUIRE(tables_per_buffer >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), LFFN_ERR_BAD_ARG);
    return lookup_gather_entry<false>(code, score, tables, bias, residual, out, B, T, S, Do, tables_per_buffer,
                                      tokens_per_workgroup, stream, workspace, workspace_bytes);
}

extern "C" int lffn_lookup_gather_planned_bf16(const int32_t *code, const float *score, const uint16_t *tables,
                                               const float *bias, float *out,
                                               int64_t B, int64_t T, int64_t S, int64_t Do,
                                               int32_t tables_per_buffer, int32_t tokens_per_workgroup, void *stream) {
    LFFN_REQUIRE(tables_per_buffer >= 0, LFFN_ERR_BAD_ARG);
    return lookup_gather_entry<true>(code, score, tables, bias, nullptr, out, B, T, S, Do, tables_per_buffer,
                                     tokens_per_workgroup, stream);
}

extern "C" int lffn_lookup_gather_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t bf16,
                                       int32_t *tables_per_buffer) {
    if (B < 0 || T < 0 || Do < 1 || !lffn_is_pow2(S) || Do % 64 != 0) return LFFN_ERR_BAD_ARG;
    const GatherPlan plan = bf16 ? plan_gather<true>(B, T, S, Do) : plan_gather<false>(B, T, S, Do);
    if (tables_per_buffer) *tables_per_buffer = plan.kind;
    return plan.kind == 0 ? 0 : (plan.kind == 1 ? 64 : 128) * plan.np;
}

// ---------------------------------------------------------------- gather from a record stream

extern "C" int lffn_lookup_gather_records_plan_rows(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t row_format,
                                                    int32_t *tokens_per_workgroup, int64_t *record_stride, int64_t *bytes) {
    LFFN_REQUIRE(tokens_per_workgroup && record_stride && bytes && row_format >= 0 && row_format <= 2, LFFN_ERR_BAD_ARG);
    *tokens_per_workgroup = 0; *record_stride = 0; *bytes = 0;
    if (B < 1 || T < 1 || Do < 1 || !lffn_is_pow2(S) || Do % 64 != 0 || B * T >= (int64_t(1) << 31)) return LFFN_OK;
    GatherPlan qp;
    if (row_format == LFFN_ROWS_F16) {
        qp = plan_quad(LFFN_ROWS_F16, B, T, S, Do, false);
        if (qp.kind == 3 && !(qp.us < QUAD_MARGIN * (double(B) * double(T) * double(Do) * 2 / 9e6 + 5.0))) qp.kind = 0;
    } else {
        // (the records are written by the projection kernel: no packing kernel to pay for)
        qp = row_format == LFFN_ROWS_BF16 ? choose_quad<true>(B, T, S, Do, false) : choose_quad<false>(B, T, S, Do, false);
    }
    if (qp.kind != 3) return LFFN_OK;
    *tokens_per_workgroup = qp.tile;
    *record_stride = lffn_internal_quad_record_stride(B, row_format, qp.tile);
    *bytes = (T / 2) * 3 * *record_stride * 4;
    return LFFN_OK;
}

extern "C" int lffn_lookup_gather_records_plan(int64_t B, int64_t T, int64_t S, int64_t Do, int32_t *tokens_per_workgroup,
                                               int64_t *record_stride, int64_t *bytes) {
    return lffn_lookup_gather_records_plan_rows(B, T, S, Do, LFFN_ROWS_F32, tokens_per_workgroup, record_stride, bytes);
}

extern "C" int lffn_lookup_gather_records_rows(const uint32_t *records, int64_t record_stride, const void *tables,
                                               const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                               int64_t S, int64_t Do, int32_t row_format, int32_t tokens_per_workgroup,
                                               void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && Do >= 1 && tokens_per_workgroup > 0 && row_format >= 0 && row_format <= 2, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(tokens_per_workgroup % 16 == 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(S) && Do % 64 == 0 && quad_plan_is_valid(row_format, tokens_per_workgroup, B, T, S, Do),
                 LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(tables && out && (records || B == 0), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(tables) && lffn_aligned16(out) && (!bias || lffn_aligned16(bias)) &&
                     (!residual || lffn_aligned16(residual)) && lffn_aligned16(records) && record_stride % 4 == 0,
                 LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    return lffn_internal_lookup_gather_quad_records(records, record_stride, tables, bias, residual, out, B, T, S, Do,
                                                    row_format, tokens_per_workgroup, stream);
}

extern "C" int lffn_lookup_gather_records_f32(const uint32_t *records, int64_t record_stride, const float *tables,
                                              const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                              int64_t S, int64_t Do, int32_t tokens_per_workgroup, void *stream) {
    return lffn_lookup_gather_records_rows(records, record_stride, tables, bias, residual, out, B, T, S, Do, LFFN_ROWS_F32,
                                           tokens_per_workgroup, stream);
}
