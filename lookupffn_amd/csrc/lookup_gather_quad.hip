// The layer's weighted gather-add, table-major, two tables per LDS buffer, FOUR lanes per token:
//
//   out[b,:] = bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
//
// (PL/lookup.py:120-130 with the index offset of ":126" and the bias of ":108" folded in.)
//
// Same idea as lookup_gather.hip (a workgroup keeps the accumulators of a token tile in registers
// and walks the tables through LDS) and the same LDS layout as lookup_gather_pair.hip (a buffer row
// holds the 128-byte segments of tables 2k and 2k+1 side by side), with a geometry chosen for the
// vector ALU, which is what limits the eight-lanes-per-token form:
//
//   * a workgroup owns a 128-byte column slice (32 fp32 columns) and a tile of 256*NP tokens: the
//     four lanes of a quad cover a token, a lane owns 8 columns (two 16-byte pieces 64 bytes apart),
//     a wavefront covers 16 tokens at a time.  Per staged byte four times the tokens of the
//     256-byte-slice form: a quarter of the L2 -> LDS copy volume per token;
//   * (code, score) pairs reach the quad's lanes by DPP quad_perm, which rides on the
//     multiply-add itself (v_fmac_f32_dpp) at full rate and needs no bank masks: no broadcast
//     instruction is spent on the scores at all, and a row address costs one SDWA byte move into a
//     persistent address register (row number = byte 1 of an LDS address: rows are 256 bytes apart);
//   * bank conflicts: the LDS serves 64 banks (256 bytes) per clock to 16 lanes = four quads.  In every
//     read the four quads of a 16-lane group take four different 64-byte columns of the 256-byte row
//     window (table 2k or 2k+1, first or second half of the segment), whatever rows their codes
//     select, and rotate through the four columns over the four reads of a table pair.  So the
//     order in which a quad adds the pair's two tables depends on the quad (2k then 2k+1, or the
//     reverse); each token still adds its T rows one at a time in fp32.
//
// One barrier per table pair; the global -> LDS copy of pair k+1 has the whole of pair k's work to land.
#include "lffn_common.h"

namespace {

constexpr int WG = 1024;
constexpr int MAX_S = 256;
constexpr int XCDS = 8;
constexpr int CHUNK = 8;                    // tables per (code, score) register set: lane j of a quad holds pair j
constexpr int BUF_BYTES = MAX_S * 256;      // one table pair: S rows of 2 x 128 bytes; a power of two (bit 16)
constexpr int SLICE_COLS = 32;
constexpr int QUAD_TOUCH_AHEAD = 3;         // pairs between the one being read and the one being touched

// (code, score) of one token and one table pair in the order the token's quad takes the pair's tables
// (tokens whose index has bit 1 set take table 2k+1 first), 12 bytes.  The kernels that read the
// caller's [B, T] arrays directly fetch 32 bytes per token and chunk of 8 tables from rows T*4 bytes
// apart, sixteen cache lines per wavefront load, and that alone cost a third of the kernel's time; a
// stream of these records, [chunk of 8 tables][token][pair within the chunk], puts what a wavefront
// loads at once (16 tokens x 4 pairs) in 768 contiguous bytes.
struct PairRecord {
    float score_first, score_second;
    uint32_t rows;         // row of the first table | row of the second table << 8
};

struct QuadArgs {
    const int32_t *code;   // [B, T]
    const float *score;    // [B, T]
    const char *tables;    // [T, S, Do] fp32
    const float *bias;     // [Do] or null
    const float *residual; // [B, Do] or null: added to the result (may be the output buffer)
    float *out;            // [B, Do]
    int64_t B;
    int T, S, Do;          // T even
    int ntiles, nslices, per_xcd;
    int row_bytes;         // Do * 4
    const PairRecord *stream;   // PACKED kernels: [ceil(T/8)][B][4] records written by pack_pairs_kernel
};

// global_load_lds_dwordx4 with a scalar base and a 32-bit lane offset: lane i of the wavefront writes
// its 16 bytes at the LDS address in M0 + 16*i.  Inline assembly so that the compiler does not
// serialise the copy with the LDS reads of the other buffer; the caller waits (vmcnt) before the
// barrier that publishes the buffer.  M0 is put back: the compiler reserves it for its own use and
// does not honour a clobber declaration of it.
__device__ __forceinline__ void lds_dma16(const char *base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(base), "s"(lds_byte_addr)
                 : "memory");
}

// Byte offsets, from the start of table 2k's slice, of the four vectors this lane copies of a pair:
// vector q = tid + 1024*i is piece q%16 of LDS row q/16; pieces 0-7 come from table 2k, 8-15 from 2k+1.
struct CopyLanes {
    uint32_t off[4];
    uint32_t wbase;      // LDS byte offset of this wavefront's first vector inside a buffer
};

__device__ __forceinline__ CopyLanes copy_lanes(int row_bytes, uint32_t table_bytes, int tid) {
    CopyLanes c;
    const int piece = tid & 15;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        c.off[i] = (piece < 8 ? 0u : table_bytes) + (uint32_t)((tid >> 4) + i * (WG / 16)) * (uint32_t)row_bytes +
                   (uint32_t)(piece & 7) * 16u;
    c.wbase = (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6) * (64 * 16);
    return c;
}

__device__ __forceinline__ void copy_pair_to_lds(const char *pair_base, const CopyLanes &c, int tid, int buf_vecs,
                                                 uint32_t dst_byte_addr) {
    const uint32_t wbase = dst_byte_addr + c.wbase;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        lds_dma16(pair_base, c.off[i], wbase + i * (WG * 16));
    }
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const u32x4 *lds_vec_ptr;

// Value held by lane N of the caller's quad, in every lane of the quad (one DPP move).  DPP and SDWA
// forms of vector instructions issue at half the rate of plain ones on this part (4.4 against 2.5 clocks
// per wavefront instruction, measured), so a score is broadcast once and then feeds plain multiply-adds
// instead of riding on each multiply-add as a DPP operand.
template <int N>
__device__ __forceinline__ unsigned quad_broadcast(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, N * 0x55, 0xF, 0xF, true);     // quad_perm [N,N,N,N]
}
template <int N>
__device__ __forceinline__ float quad_broadcast(float v) {
    return __uint_as_float(quad_broadcast<N>(__float_as_uint(v)));
}

// An LDS byte address whose rows are 256 bytes apart: byte 1 (the row number) from byte BYTE of
// `packed`, the other three bytes from `base`.  One v_perm_b32 (a plain, full-rate instruction).
template <int BYTE>
__device__ __forceinline__ unsigned with_row(unsigned base, unsigned packed) {
    // selector bytes 0-3 name bytes of the second operand, 4-7 bytes of the first
    return __builtin_amdgcn_perm(packed, base, 0x03020000u | ((4u + BYTE) << 8));
}

// One record per thread: thread i writes stream[i], i = (chunk * B + token) * 4 + pair within the chunk.
__global__ __launch_bounds__(256) void pack_pairs_kernel(const int32_t *code, const float *score, PairRecord *stream,
                                                         int64_t B, int T, int S, int64_t total) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int l = (int)(i & 3);
    const int64_t cb = i >> 2;
    const int64_t b = cb % B;
    const int t = (int)(cb / B) * CHUNK + 2 * l;
    PairRecord r{0.f, 0.f, 0u};
    if (t < T) {                                               // T is even: both tables of the pair or none
        const int2 c = *reinterpret_cast<const int2 *>(code + b * T + t);
        const float2 w = *reinterpret_cast<const float2 *>(score + b * T + t);
        const uint32_t ca = uint32_t(c.x & (S - 1)), cb2 = uint32_t(c.y & (S - 1));
        const bool second_first = (b & 2) != 0;
        r.score_first = second_first ? w.y : w.x;
        r.score_second = second_first ? w.x : w.y;
        r.rows = second_first ? (cb2 | (ca << 8)) : (ca | (cb2 << 8));
    }
    stream[i] = r;
}

// PACKED: (code, score) come from the record stream pack_pairs_kernel writes instead of the [B, T] arrays.
template <int NP, bool TOUCH, bool PACKED>
__global__ __launch_bounds__(WG) void lookup_gather_quad_kernel(QuadArgs a) {
    constexpr int NQ = (NP + 1) / 2;              // code registers: two tokens' (first, second) rows per register
    extern __shared__ uint4 lds[];                // 2 buffers of BUF_BYTES + the touches' sink

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.ntiles * a.nslices) return;     // uniform over the workgroup
    const int slice = unit / a.ntiles;
    const int tile = unit % a.ntiles;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int quad = lane >> 2;       // token within the wavefront's sixteen
    const int l = lane & 3;           // lane within the quad: 16-byte piece l of each 64-byte column
    // the quad's place among the four quads of its 16-lane group decides which 64-byte column of the
    // row window it starts on: bit 1 = which table of the pair comes first, bit 0 = which half of the
    // 128-byte segment comes first
    const bool second_first = (quad & 2) != 0;
    const int half0 = quad & 1;
    const int64_t tok0 = int64_t(tile) * (256 * NP) + wave * 16 + quad;

    // acc[p][h][e]: token tok0 + 256 p, column (half0 ^ h) * 16 + 4 l + e of the slice
    float acc[NP][2][4];
    {
        float b[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) b[h][e] = 0.f;
        if (a.bias) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float *bp = a.bias + (size_t)slice * SLICE_COLS + (half0 ^ h) * 16 + l * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) b[h][e] = bp[e];
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[p][h][e] = b[h][e];
    }

    const int buf_vecs = a.S * 16;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // Where pair k's 2 x S x 128 bytes of this slice start, and which bytes of them this lane copies.
    // Rows are Do*4 bytes apart, the second table S rows further down.
    const size_t table_bytes = (size_t)a.S * a.row_bytes;
    const char *slice_base = a.tables + (size_t)slice * 128;
    const size_t pair_stride = 2 * table_bytes;
    const int npairs = a.T / 2;
    const CopyLanes cl = copy_lanes(a.row_bytes, (uint32_t)table_bytes, tid);

    // Touch by turns.  A slice's next blocks have to come into this XCD's L2 from the memory-side cache
    // or from HBM before the copies ask for them, or every copy waits out that latency.  But the vector
    // memory path of a CU returns data in order: a request that misses L2 holds up everything the CU
    // issues after it, the copies included, so a workgroup that touches a few lines of the next pair in
    // every step (as the team touch of lookup_gather.hip does) stalls its own copies once per step.  Here
    // the workgroups that share the slice (one per token tile, all on this XCD, in step with each other)
    // take turns instead: in step k the workgroup whose tile number is k mod ntiles touches ALL 2*S lines
    // of pair k + QUAD_TOUCH_AHEAD (lanes 0..2S-1 one 128-byte line each), the others touch nothing
    // (their instruction reads a line of the pair they are on: a hit).  Every CU then takes the latency
    // once in ntiles steps.
    const int my_line = tid < 2 * a.S ? tid : 0;
    const bool line_second = my_line >= a.S;
    const uint32_t touch_off_on = (line_second ? (uint32_t)table_bytes : 0u) +
                                  (uint32_t)(my_line - (line_second ? a.S : 0)) * (uint32_t)a.row_bytes;
    int turn = 0;                                   // k mod ntiles, kept without a division
    const uint32_t touch_dst = lds0 + 2u * BUF_BYTES;

    // LDS byte addresses of this lane's four reads of a pair, row field (byte 1) still empty: read i
    // takes table (i >> 1) of the quad's order, half (i & 1) of its order.  Bit 16 selects the buffer and
    // is flipped after every pair.
    unsigned base[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int table_sel = (i >> 1) ^ (second_first ? 1 : 0);
        const int half = (i & 1) ^ half0;
        base[i] = lds0 + (unsigned)(table_sel * 128 + half * 64 + l * 16);
    }

    copy_pair_to_lds(slice_base, cl, tid, buf_vecs, lds0);
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);
    __syncthreads();

    unsigned cd[NQ];
    float sc[NP][2];
    const int nchunks = (a.T + CHUNK - 1) / CHUNK;
    for (int c = 0; c < nchunks; ++c) {
        // Lane l of a quad holds (code, score) of the chunk's pair l (tables 8c + 2l, 8c + 2l + 1) for
        // each of its NP tokens, already in the quad's order (first, second).  Addresses are clamped
        // into range and the loads are unconditional, so that all of them are in flight together; what
        // was loaded from a clamped address gets score 0.
        if constexpr (PACKED) {
            PairRecord rec[NP];
#pragma unroll
            for (int p = 0; p < NP; ++p)
                rec[p] = a.stream[((int64_t)c * a.B + min(tok0 + p * 256, a.B - 1)) * 4 + l];
#pragma unroll
            for (int q = 0; q < NQ; ++q) cd[q] = 0u;
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const bool ok = tok0 + p * 256 < a.B;
                cd[p / 2] |= (p % 2) ? (rec[p].rows << 16) : rec[p].rows;
                sc[p][0] = ok ? rec[p].score_first : 0.f;
                sc[p][1] = ok ? rec[p].score_second : 0.f;
            }
        } else {
            const int tt = c * CHUNK + 2 * l;
            const int ttc = min(tt, a.T - 2);
            int2 craw[NP];
            float2 sraw[NP];
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                // B * T < 2^31 is a precondition of this kernel: 32-bit element offsets (even: 8-byte aligned)
                const int off = (int)min(tok0 + p * 256, a.B - 1) * a.T + ttc;
                craw[p] = *reinterpret_cast<const int2 *>(a.code + off);
                sraw[p] = *reinterpret_cast<const float2 *>(a.score + off);
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) cd[q] = 0u;
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const bool ok = (tok0 + p * 256 < a.B) && (tt < a.T);
                const unsigned ca = unsigned(craw[p].x & (a.S - 1)), cb = unsigned(craw[p].y & (a.S - 1));
                const unsigned first = second_first ? cb : ca, second = second_first ? ca : cb;
                cd[p / 2] |= (first | (second << 8)) << (16 * (p % 2));
                const float sa = ok ? sraw[p].x : 0.f, sb = ok ? sraw[p].y : 0.f;
                sc[p][0] = second_first ? sb : sa;
                sc[p][1] = second_first ? sa : sb;
            }
        }
        // these must have landed before the pair loop: inside it nothing but the LDS copies is in flight
#pragma unroll
        for (int q = 0; q < NQ; ++q) asm volatile("" : "+v"(cd[q]));
#pragma unroll
        for (int p = 0; p < NP; ++p) asm volatile("" : "+v"(sc[p][0]), "+v"(sc[p][1]));

        const int k0 = c * (CHUNK / 2);
        const int npc = min(CHUNK / 2, npairs - k0);           // pairs in this chunk
        // the four pairs of the chunk, unrolled, so that the broadcast lane is a constant
        static_for<CHUNK / 2>([&](auto kq_c) {
            constexpr int KQ = decltype(kq_c)::value;
            if (KQ < npc) {                                    // uniform
                const int k = k0 + KQ;
                // next pair's segments straight into the other buffer (last read one pair ago, before
                // the previous barrier); the last iteration re-copies the last pair
                copy_pair_to_lds(slice_base + (size_t)min(k + 1, npairs - 1) * pair_stride, cl, tid, buf_vecs,
                                       lds0 + (uint32_t)((k + 1) & 1) * BUF_BYTES);
                if constexpr (TOUCH)
                {
                    const bool mine = turn == tile;                              // uniform
                    const int kt = mine ? min(k + QUAD_TOUCH_AHEAD, npairs - 1) : k;
                    l2_touch(slice_base + (size_t)kt * pair_stride, mine ? touch_off_on : 0u, touch_dst);
                    turn = turn + 1 == a.ntiles ? 0 : turn + 1;
                }
                unsigned packed[NQ];
#pragma unroll
                for (int q = 0; q < NQ; ++q) packed[q] = quad_broadcast<KQ>(cd[q]);
                // Software pipeline over the passes: a pass's four rows are requested while the pass before
                // is still being added (its first table's two rows are consumed, their registers take the
                // next pass's first two reads; likewise the second table's), so a wavefront always has
                // two to four row reads in flight behind its multiply-adds.
                auto row_addr = [&](auto p_c, auto i_c) -> unsigned {
                    constexpr int P = decltype(p_c)::value, I = decltype(i_c)::value;
                    return with_row<2 * (P % 2) + (I >> 1)>(base[I], packed[P / 2]);
                };
                auto fma4 = [&](float (&ac)[4], float w, const u32x4 &v) {
                    ac[0] = fmaf(__uint_as_float(v.x), w, ac[0]);
                    ac[1] = fmaf(__uint_as_float(v.y), w, ac[1]);
                    ac[2] = fmaf(__uint_as_float(v.z), w, ac[2]);
                    ac[3] = fmaf(__uint_as_float(v.w), w, ac[3]);
                };
                using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
                using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
                u32x4 r[4];
                r[0] = *(lds_vec_ptr)(uintptr_t)row_addr(I0{}, I0{});
                r[1] = *(lds_vec_ptr)(uintptr_t)row_addr(I0{}, I1{});
                r[2] = *(lds_vec_ptr)(uintptr_t)row_addr(I0{}, I2{});
                r[3] = *(lds_vec_ptr)(uintptr_t)row_addr(I0{}, I3{});
                static_for<NP>([&](auto p_c) {
                    constexpr int P = decltype(p_c)::value;
                    constexpr bool MORE = P + 1 < NP;
                    using PN = std::integral_constant<int, MORE ? P + 1 : P>;
                    const float w0 = quad_broadcast<KQ>(sc[P][0]);
                    fma4(acc[P][0], w0, r[0]);
                    fma4(acc[P][1], w0, r[1]);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (MORE) {
                        r[0] = *(lds_vec_ptr)(uintptr_t)row_addr(PN{}, I0{});
                        r[1] = *(lds_vec_ptr)(uintptr_t)row_addr(PN{}, I1{});
                    }
                    const float w1 = quad_broadcast<KQ>(sc[P][1]);
                    __builtin_amdgcn_sched_barrier(0);
                    fma4(acc[P][0], w1, r[2]);
                    fma4(acc[P][1], w1, r[3]);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (MORE) {
                        r[2] = *(lds_vec_ptr)(uintptr_t)row_addr(PN{}, I2{});
                        r[3] = *(lds_vec_ptr)(uintptr_t)row_addr(PN{}, I3{});
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
                // the other buffer for the next pair
#pragma unroll
                for (int i = 0; i < 4; ++i) base[i] ^= (unsigned)BUF_BYTES;
                // the copy issued above has landed; the touch, issued after it, may still be out
                __builtin_amdgcn_s_waitcnt(TOUCH ? WAIT_VMCNT_1 : WAIT_VMCNT_0);
                __syncthreads();
            }
        });
    }
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);         // nothing may still be writing this workgroup's LDS when it ends

#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int64_t tok = tok0 + p * 256;
        if (tok < a.B) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const size_t off = tok * a.Do + (size_t)slice * SLICE_COLS + (half0 ^ h) * 16 + l * 4;
                float4 v = make_float4(acc[p][h][0], acc[p][h][1], acc[p][h][2], acc[p][h][3]);
                if (a.residual) {
                    const float4 rr = *reinterpret_cast<const float4 *>(a.residual + off);
                    v.x += rr.x; v.y += rr.y; v.z += rr.z; v.w += rr.w;
                }
                *reinterpret_cast<float4 *>(a.out + off) = v;
            }
        }
    }
}

template <int NP, bool TOUCH, bool PACKED>
int launch_quad_full(QuadArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + 256 * NP - 1) / (256 * NP));
    const int units = a.ntiles * a.nslices;
    a.per_xcd = (units + XCDS - 1) / XCDS;
    const size_t lds_bytes = size_t(2) * BUF_BYTES + TOUCH_SINK_BYTES;     // two buffers + the touches' scratch
    auto kern = lookup_gather_quad_kernel<NP, TOUCH, PACKED>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

template <int NP, bool PACKED>
int launch_quad(const QuadArgs &a, bool touch, hipStream_t stream) {
    return touch ? launch_quad_full<NP, true, PACKED>(a, stream) : launch_quad_full<NP, false, PACKED>(a, stream);
}

template <bool PACKED>
int launch_quad_np(const QuadArgs &a, int np, bool touch, hipStream_t st) {
    switch (np) {
        case 8: return launch_quad<8, PACKED>(a, touch, st);
        case 7: return launch_quad<7, PACKED>(a, touch, st);
        case 6: return launch_quad<6, PACKED>(a, touch, st);
        default: return launch_quad<4, PACKED>(a, touch, st);
    }
}

}  // namespace

// Bytes of the record stream for a shape (whole chunks of 8 tables).
int64_t lffn_internal_quad_stream_bytes(int64_t B, int64_t T) {
    return ((T + CHUNK - 1) / CHUNK) * B * 4 * (int64_t)sizeof(PairRecord);
}

// Launch the quad kernel with 256*np tokens per workgroup.  The caller has checked that the shape
// qualifies: fp32 rows, S = 256 (a table pair fills an LDS buffer), T even, Do a multiple of 32, B*T < 2^31, 2*S*Do*4 < 2^32 (32-bit
// lane offsets from a table pair's base), np one of {4, 6, 7, 8}.  With a workspace of at least
// lffn_internal_quad_stream_bytes(B, T) bytes (16-byte aligned) the (code, score) pairs are first
// packed into the record stream there (one more small kernel); with a null workspace the gather kernel
// reads the [B, T] arrays itself.
int lffn_internal_lookup_gather_quad(const int32_t *code, const float *score, const void *tables,
                                     const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                     int64_t S, int64_t Do, int np, void *workspace, void *stream) {
    QuadArgs a{};
    a.code = code; a.score = score; a.tables = static_cast<const char *>(tables); a.bias = bias; a.residual = residual; a.out = out;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do / SLICE_COLS);
    a.row_bytes = (int)(Do * 4);
    // the touch pays while the table set fits the 256 MB memory-side cache (as in lookup_gather_pair.hip)
    const bool touch = T * S * Do * 4 <= (int64_t(256) << 20);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!workspace) return launch_quad_np<false>(a, np, touch, st);
    PairRecord *recs = static_cast<PairRecord *>(workspace);
    const int64_t total = ((T + CHUNK - 1) / CHUNK) * B * 4;
    hipLaunchKernelGGL(pack_pairs_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, code, score, recs, B,
                       (int)T, (int)S, total);
    if (hipGetLastError() != hipSuccess) return LFFN_ERR_LAUNCH;
    a.stream = recs;
    return launch_quad_np<true>(a, np, touch, st);
}
