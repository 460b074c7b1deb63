// Gradient of the layer's gather w.r.t. the scores, table-major, two tables per LDS buffer, four lanes
// per token, every (token, table) owned by one workgroup:
//
//   grad_score[b,t] = < g[b,:], tables[t, code[b,t] & (S-1), :] >
//
// (the score gradient of PL/lookup.py:120-130's gather; the reference's kernel,
// PL/gather/cuda/extension/gather_kernel_fp32.cu:141, combines per-warp partial sums with atomics).
//
// The mirror image of lookup_gather_quad.hip with the loop nest turned round.  A workgroup owns a
// tile of 256*NP tokens and a chunk of C table pairs and walks the Do/32 column slices itself:
//
//   for slice:                       g[tile, slice] -> registers (8 values per lane and pass)
//     for pair of the chunk:         the pair's 2 x S x 128 bytes of this slice -> LDS (double buffered,
//                                    global -> LDS directly, one barrier per step)
//       for pass:                    a quad reads its token's row of both tables (4 x ds_read_b128,
//                                    bank-conflict-free as in the gather), multiplies into its g values
//                                    and sums over its four lanes
//
// The sums of a (token, table) stay in a register of one lane across the slices and are stored once:
// no atomics, no zero-fill, a fixed order of additions (slice by slice).  The four-lane sum transposes
// as it goes: the two values of a pass (first and second table of the pair) end up in the even and the
// odd lanes of the quad, three DPP operations and two selects for both.
//
// Per (256 tokens, table pair, slice) a workgroup moves 64 KB / NP of table bytes and 32 KB / C of g
// from L2.  The g values of the next slice are requested by each pass as it finishes with the current
// ones, in the slice's last step, and stay in flight across that step's barrier (they are needed a whole
// step later); everything else that is in flight inside the loop is a global -> LDS copy the compiler
// does not know of, so the loop is laid out for the compiler's own waits to fall where they cost nothing:
//   * the chunk size is a compile-time constant of the loop (a chunk of fewer pairs runs another copy
//     of it), so the step with the loads is always the loop body's last and only its first step has
//     waits for them;
//   * the step exists twice, with and without the loads, each with its own wait before the barrier:
//     loads and wait under separate conditions would leave a path with loads and no wait, and the
//     compiler, which places waits by the worst path, would then wait for everything (the copies just
//     issued included) at the top of every step: measured, 30 % of the kernel's time.
// Measured at 16384 tokens x 128 tables x 256 x 768 (MI355X, NP = 4, C = 4): 140-150 us against 234 us
// for the form with atomics in lookup_inner.hip; 130-140 us with g slice-major ([Do/32][B][32]: a
// tile's slice contiguous instead of one 128-byte line per 3 KB).  Without the g loads the loop runs
// in 113 us.  Pulling the next slice of g into L2 ahead of the loads (a share per step) and issuing a
// step's four copies one per pass instead of together both cost more instructions on the vector
// memory path than they saved in waiting (173 against 161 us; no change).  NP = 6 and 8 (fewer table
// bytes per token) need more than the 128 registers a 16-wavefront workgroup leaves a lane.
#include "lffn_common.h"

namespace {

constexpr int WG = 1024;
constexpr int MAX_S = 256;
constexpr int XCDS = 8;
constexpr int BUF_BYTES = MAX_S * 256;      // one table pair: S rows of 2 x 128 bytes; a power of two (bit 16)
constexpr int SLICE_COLS = 32;
constexpr int TOUCH_AHEAD = 3;              // steps between the one being read and the one being touched

struct InnerQuadArgs {
    const int32_t *code;   // [B, T]
    const float *g;        // token b, slice s (32 columns) at g + b * g_token_stride + s * g_slice_stride
    int64_t g_token_stride, g_slice_stride;     // floats: Do and 32 for [B, Do]; 32 and B * 32 for [Do/32][B][32]
    const char *tables;    // [T, S, Do] fp32
    float *out;            // [B, T]
    int64_t B;
    int T, S, Do;          // T even, S = 256
    int ntiles, nchunks, nslices, per_xcd;
    int group_tiles;       // tiles per tile group (see the unit order in the kernel)
    int row_bytes;         // Do * 4
};

// global_load_lds_dwordx4 with a scalar base and a 32-bit lane offset: lane i of the wavefront writes
// its 16 bytes at the LDS address in M0 + 16*i.  M0 is put back: the compiler reserves it for its own
// use and does not honour a clobber declaration of it.
__device__ __forceinline__ void lds_dma16(const char *base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(base), "s"(lds_byte_addr)
                 : "memory");
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const u32x4 *lds_vec_ptr;

// Value held by lane N of the caller's quad, in every lane of the quad (one DPP move).
template <int N>
__device__ __forceinline__ unsigned quad_broadcast(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, N * 0x55, 0xF, 0xF, true);     // quad_perm [N,N,N,N]
}

// An LDS byte address whose rows are 256 bytes apart: byte 1 (the row number) from byte BYTE of
// `packed`, the other three bytes from `base`.  One v_perm_b32.
template <int BYTE>
__device__ __forceinline__ unsigned with_row(unsigned base, unsigned packed) {
    return __builtin_amdgcn_perm(packed, base, 0x03020000u | ((4u + BYTE) << 8));
}

// v of another lane of the quad (CTRL: a quad_perm pattern).  Every lane has a source, so with bound_ctrl
// and a zero `old` the compiler folds the move into the add that uses it.
template <int CTRL>
__device__ __forceinline__ float quad_swap(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// A pointer that is the same in every lane, in scalar registers (where the compiler's own analysis does
// not conclude that, an inline-assembly operand that has to be scalar would not assemble).
__device__ __forceinline__ const char *uniform_ptr(const char *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const char *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ float dot4(const float4 &g, const u32x4 &v, float acc) {
    acc = fmaf(g.x, __uint_as_float(v.x), acc);
    acc = fmaf(g.y, __uint_as_float(v.y), acc);
    acc = fmaf(g.z, __uint_as_float(v.z), acc);
    return fmaf(g.w, __uint_as_float(v.w), acc);
}

template <int NP, int C>
__global__ __launch_bounds__(WG) void lookup_inner_quad_kernel(InnerQuadArgs a) {
    static_assert(NP >= 4 && NP <= 8, "lane l of a quad holds the row numbers of passes l and l + 4");
    static_assert(1 + 2 * NP <= 15, "the wait before the barrier names 1 + 2*NP operations in the 4-bit vmcnt field");
    // (NP = 4 is what is built: 6 and 8 passes need more than the 128 registers of a 16-wavefront workgroup)
    static_assert(C >= 1 && C <= 4, "row numbers of a chunk: two registers per lane");
    constexpr int W = (C + 1) / 2;                // words of row numbers per pass: two pairs (4 bytes) a word
    extern __shared__ uint4 lds[];                // 2 buffers of BUF_BYTES, the touches' sink

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    // Units in the order (tile group, chunk, tile of the group), consecutive units on one XCD: an XCD then
    // works on group_tiles tiles x a few chunks, and what it pulls through the fabric is those chunks'
    // tables once and those tiles' rows of g once per chunk group (every tile's workgroups of a chunk run in
    // step and share the copies in L2).  The launch picks group_tiles to make the sum smallest.
    const int group_units = a.nchunks * a.group_tiles;
    const int group = unit / group_units, in_group = unit % group_units;
    const int chunk = in_group / a.group_tiles;
    const int tile_in_group = in_group % a.group_tiles;
    const int tile = group * a.group_tiles + tile_in_group;
    if (tile >= a.ntiles) return;                 // uniform over the workgroup (ragged last group; also past the last group)
    const int team = min(a.group_tiles, a.ntiles - group * a.group_tiles);     // workgroups that share this chunk's copies
    const int npairs = a.T / 2;
    const int k0 = chunk * C;
    const int nk = min(C, npairs - k0);           // table pairs in this chunk

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int quad = lane >> 2;       // token within the wavefront's sixteen
    const int l = lane & 3;           // lane within the quad: 16-byte piece l of each 64-byte column
    // as in the gather: bit 1 of the quad number = which table of a pair comes first, bit 0 = which half
    // of the 128-byte segment comes first
    const bool second_first = (quad & 2) != 0;
    const int half0 = quad & 1;
    const int64_t tok0 = int64_t(tile) * (256 * NP) + wave * 16 + quad;
    // passes whose token is beyond B compute on the last token's data and store nothing
    auto token_of = [&](int p) { return min(tok0 + int64_t(p) * 256, a.B - 1); };

    // Row numbers: lane l holds those of passes l and l + 4 (clamped), byte 2 (kk % 2) of word kk / 2 =
    // row in the pair's first table, the next byte = row in its second (first, second in the quad's order).
    unsigned rows[2][W];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int32_t *cp = a.code + token_of(min(l + 4 * j, NP - 1)) * a.T + 2 * k0;
#pragma unroll
        for (int w = 0; w < W; ++w) rows[j][w] = 0u;
#pragma unroll
        for (int kk = 0; kk < C; ++kk) {
            if (kk < nk) {
                const int2 c = *reinterpret_cast<const int2 *>(cp + 2 * kk);
                const unsigned ca = unsigned(c.x) & unsigned(a.S - 1), cb = unsigned(c.y) & unsigned(a.S - 1);
                const unsigned both = second_first ? (cb | (ca << 8)) : (ca | (cb << 8));
                rows[j][kk / 2] |= both << (16 * (kk % 2));
            }
        }
    }

    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // Where a step's 2 x S x 128 bytes start, and which bytes of them this lane copies: vector
    // q = tid + 1024*i is piece q%16 of LDS row q/16; pieces 0-7 come from table 2k, 8-15 from 2k+1.
    const size_t table_bytes = (size_t)a.S * a.row_bytes;
    const size_t pair_stride = 2 * table_bytes;
    const char *chunk_base = a.tables + (size_t)k0 * pair_stride;
    auto step_base = [&](int slice, int kk) { return chunk_base + (size_t)kk * pair_stride + (size_t)slice * 128; };
    const size_t quarter = (size_t)(WG / 16) * a.row_bytes;
    const uint32_t copy_off = ((tid & 15) < 8 ? 0u : (uint32_t)table_bytes) + (uint32_t)(tid >> 4) * (uint32_t)a.row_bytes +
                              (uint32_t)(tid & 7) * 16u;
    const uint32_t copy_dst = (uint32_t)wave * (64 * 16);
    auto copy_pair_to_lds = [&](const char *pair_base, uint32_t dst_byte_addr) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_dma16(pair_base + i * quarter, copy_off, dst_byte_addr + copy_dst + i * (WG * 16));
    };

    // Touch by turns (see lookup_gather_quad.hip): the workgroups of a chunk run in step; in step n the one
    // whose number among the chunk's workgroups on this XCD is n mod their count pulls all 2*S lines of the step TOUCH_AHEAD further on into the
    // XCD's L2, the others touch a line of the step they are on.
    const int my_line = tid < 2 * a.S ? tid : 0;
    const bool line_second = my_line >= a.S;
    const uint32_t touch_off_on = (line_second ? (uint32_t)table_bytes : 0u) +
                                  (uint32_t)(my_line - (line_second ? a.S : 0)) * (uint32_t)a.row_bytes;
    int turn = 0;
    const uint32_t touch_dst = lds0 + 2u * BUF_BYTES;

    // LDS byte addresses of this lane's four reads of a pair, row field (byte 1) still empty
    unsigned base[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int table_sel = (i >> 1) ^ (second_first ? 1 : 0);
        const int half = (i & 1) ^ half0;
        base[i] = lds0 + (unsigned)(table_sel * 128 + half * 64 + l * 16);
    }

    // gq[p][h]: g of token tok0 + 256 p, columns (half0 ^ h) * 16 + 4 l .. + 3 of the current slice
    float4 gq[NP][2];
    const int g_col = l * 4;
    int tok_low = (int)tok0;          // B < 2^31
    auto load_g = [&](int slice, int p) {
        // the address is formed afresh at every use (an empty statement the compiler cannot see through):
        // hoisted out of the slice loop the NP row pointers would cost 2*NP registers
        asm volatile("" : "+v"(tok_low));
        const int64_t tok = min(int64_t(tok_low) + int64_t(p) * 256, a.B - 1);
        const float *gp = a.g + tok * a.g_token_stride + (size_t)slice * a.g_slice_stride + g_col;
        gq[p][0] = *reinterpret_cast<const float4 *>(gp + half0 * 16);
        gq[p][1] = *reinterpret_cast<const float4 *>(gp + (half0 ^ 1) * 16);
    };
#pragma unroll
    for (int p = 0; p < NP; ++p) load_g(0, p);

    // res[p][kk], even lanes of the quad: the sum for (token of pass p, first table of pair kk in the
    // quad's order); odd lanes: the second table
    float res[NP][C];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int kk = 0; kk < C; ++kk) res[p][kk] = 0.f;

    copy_pair_to_lds(step_base(0, 0), lds0);
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);
    __syncthreads();

    const bool odd = (l & 1) != 0;
    int parity = 0;                               // buffer that holds the current step

    // One step: the passes over pair KK of the chunk in the current slice, while the next step's segments
    // are copied into the other buffer.  RELOAD (the slice's last step when another slice follows): each
    // pass fetches its g values of the next slice as soon as it is done with this slice's; they are needed
    // again a whole step later, so the wait at the end of the step leaves them in flight.
    auto step = [&](int slice, auto kk_c, auto nk_c, auto reload_c, bool more_slices) {
        constexpr int KK = decltype(kk_c)::value, NK = decltype(nk_c)::value;
        constexpr bool RELOAD = decltype(reload_c)::value;
        constexpr bool LAST_OF_SLICE = KK + 1 == NK;
        auto rows_of = [&](auto p_c) {
            constexpr int P = decltype(p_c)::value;
            return quad_broadcast<P % 4>(rows[P / 4][KK / 2]);
        };
        constexpr int B0 = 2 * (KK % 2);               // byte of the first table's row number
        using I0 = std::integral_constant<int, 0>;
        u32x4 r[4];
        unsigned pk = rows_of(I0{});
        r[0] = *(lds_vec_ptr)(uintptr_t)with_row<B0>(base[0], pk);
        r[1] = *(lds_vec_ptr)(uintptr_t)with_row<B0>(base[1], pk);
        r[2] = *(lds_vec_ptr)(uintptr_t)with_row<B0 + 1>(base[2], pk);
        r[3] = *(lds_vec_ptr)(uintptr_t)with_row<B0 + 1>(base[3], pk);
        __builtin_amdgcn_sched_barrier(0);
        // the next step's segments go into the other buffer: the next pair of the chunk, or the chunk's
        // first pair in the next slice (after the very last step the last one is copied again)
        {
            const int nslice = LAST_OF_SLICE ? (more_slices ? slice + 1 : slice) : slice;
            const int nkk = LAST_OF_SLICE ? (more_slices ? 0 : KK) : KK + 1;
            copy_pair_to_lds(uniform_ptr(step_base(nslice, nkk)), lds0 + (uint32_t)(parity ^ 1) * BUF_BYTES);
            // touch by turns: the step TOUCH_AHEAD further on (the last step, beyond it)
            const bool mine = turn == tile_in_group;                     // uniform
            int ts = slice, tk = KK + TOUCH_AHEAD;
#pragma unroll
            for (int i = 0; i < TOUCH_AHEAD; ++i) {
                if (tk >= NK) { tk -= NK; ts += 1; }
            }
            if (ts >= a.nslices) { ts = a.nslices - 1; tk = NK - 1; }
            l2_touch(uniform_ptr(mine ? step_base(ts, tk) : step_base(slice, KK)), mine ? touch_off_on : 0u, touch_dst);
            turn = turn + 1 == team ? 0 : turn + 1;
        }
        __builtin_amdgcn_sched_barrier(0);
        static_for<NP>([&](auto p_c) {
            constexpr int P = decltype(p_c)::value;
            constexpr bool MORE = P + 1 < NP;
            using PN = std::integral_constant<int, MORE ? P + 1 : P>;
            if constexpr (MORE) pk = rows_of(PN{});
            float d0 = dot4(gq[P][0], r[0], 0.f);
            d0 = dot4(gq[P][1], r[1], d0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MORE) {
                r[0] = *(lds_vec_ptr)(uintptr_t)with_row<B0>(base[0], pk);
                r[1] = *(lds_vec_ptr)(uintptr_t)with_row<B0>(base[1], pk);
            }
            float d1 = dot4(gq[P][0], r[2], 0.f);
            d1 = dot4(gq[P][1], r[3], d1);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MORE) {
                r[2] = *(lds_vec_ptr)(uintptr_t)with_row<B0 + 1>(base[2], pk);
                r[3] = *(lds_vec_ptr)(uintptr_t)with_row<B0 + 1>(base[3], pk);
            }
            // sum over the quad: even lanes collect the first table's value, odd lanes the second's
            const float give = odd ? d0 : d1;
            float keep = odd ? d1 : d0;
            keep += quad_swap<DPP_QUAD_XOR1>(give);
            keep += quad_swap<DPP_QUAD_XOR2>(keep);
            res[P][KK] += keep;
            if constexpr (RELOAD) load_g(slice + 1, P);
            __builtin_amdgcn_sched_barrier(0);
        });
        // the other buffer for the next step
#pragma unroll
        for (int i = 0; i < 4; ++i) base[i] ^= (unsigned)BUF_BYTES;
        parity ^= 1;
        if constexpr (RELOAD) {
            // The copies and the touch came first, then the 2*NP loads of g, in that order: loads cannot move
            // below a statement that may write memory, and none of them can be merged or dropped.  With at
            // most 2*NP + 1 operations still out, the copies have landed (more operations than that, such as
            // a register spill, only make the wait stricter; FEWER than 2*NP loads after the copies would
            // leave a copy in flight at the barrier, which is why load_g issues exactly two loads per pass
            // and this kernel must not spill: the test suite checks the compiler's resource report).
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0 | (1 + 2 * NP));
        } else {
            // the copies issued above have landed; the touch, issued after them, may still be out
            __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_1);
        }
        __syncthreads();
    };
    // The slice loop for a chunk of NK pairs, NK a compile-time constant: the step with the g loads is then
    // always the last one of the loop body, and only the first step of the body (where loads may still be
    // in flight) carries the compiler's own waits for them.
    auto run = [&](auto nk_c) {
        constexpr int NK = decltype(nk_c)::value;
        for (int slice = 0; slice < a.nslices; ++slice) {
            const bool more_slices = slice + 1 < a.nslices;
            static_for<NK - 1>([&](auto kk_c) { step(slice, kk_c, nk_c, std::false_type{}, more_slices); });
            using Last = std::integral_constant<int, NK - 1>;
            if (more_slices) step(slice, Last{}, nk_c, std::true_type{}, true);
            else step(slice, Last{}, nk_c, std::false_type{}, false);
        }
    };
    static_for<C>([&](auto i_c) {
        constexpr int NK = decltype(i_c)::value + 1;
        if (nk == NK) run(std::integral_constant<int, NK>{});      // uniform
    });
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);         // nothing may still be writing this workgroup's LDS when it ends

    // lanes 0, 1 of a quad store the even pairs of the chunk, lanes 2, 3 the odd ones (lanes l and l ^ 2
    // hold the same sums)
    const int which = (odd ? 1 : 0) ^ (second_first ? 1 : 0);      // table of the pair this lane's sums belong to
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int64_t tok = tok0 + int64_t(p) * 256;
        if (tok < a.B) {
#pragma unroll
            for (int kk = 0; kk < C; ++kk) {
                if (kk < nk && (l >> 1) == (kk & 1)) a.out[tok * a.T + 2 * (k0 + kk) + which] = res[p][kk];
            }
        }
    }
}

template <int NP, int C>
int launch_inner_quad(InnerQuadArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + 256 * NP - 1) / (256 * NP));
    a.nchunks = (a.T / 2 + C - 1) / C;
    // tile groups: with per_xcd units on an XCD, group_tiles tiles and per_xcd / group_tiles chunks meet there;
    // bytes through the fabric per XCD = chunks x (C pairs of tables) + tiles x (1024 rows of g)
    {
        const int per_xcd0 = (a.ntiles * a.nchunks + XCDS - 1) / XCDS;
        const double chunk_bytes = double(C) * 2 * a.S * a.row_bytes, tile_bytes = 256.0 * NP * a.row_bytes;
        int best = a.ntiles;
        double best_bytes = 1e300;
        for (int gt = a.ntiles; gt >= 1; gt = (gt + 1) / 2) {
            const double bytes = double((per_xcd0 + gt - 1) / gt) * chunk_bytes + double(gt) * tile_bytes;
            const int idle_tiles = (a.ntiles + gt - 1) / gt * gt - a.ntiles;          // of a ragged last group
            if (bytes < best_bytes && idle_tiles * 8 <= a.ntiles) { best_bytes = bytes; best = gt; }
            if (gt == 1) break;
        }
        a.group_tiles = best;
    }
    const int groups = (a.ntiles + a.group_tiles - 1) / a.group_tiles;
    const int units = groups * a.nchunks * a.group_tiles;       // the last group's missing tiles included
    a.per_xcd = (units + XCDS - 1) / XCDS;
    const size_t lds_bytes = size_t(2) * BUF_BYTES + TOUCH_SINK_BYTES;
    auto kern = lookup_inner_quad_kernel<NP, C>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

}  // namespace

// The caller has checked that the shape qualifies: S = 256 (a table pair fills an LDS buffer), T even,
// Do a multiple of 32, 2*S*Do*4 < 2^32 (32-bit lane offsets from a table pair's base), 1 <= B < 2^31, code
// aligned to 8 bytes, g to 16.  g: token b's 32 columns of slice s start at g + b * g_token_stride +
// s * g_slice_stride floats (both multiples of 4).  256 * np tokens and c table pairs per workgroup.
int lffn_internal_lookup_inner_quad(const int32_t *code, const float *g, int64_t g_token_stride, int64_t g_slice_stride,
                                    const void *tables, float *grad_score, int64_t B, int64_t T, int64_t S, int64_t Do,
                                    int np, int c, void *stream) {
    if (S != MAX_S || T % 2 != 0 || T < 2 || Do % SLICE_COLS != 0 || B < 1) return LFFN_ERR_BAD_ARG;
    InnerQuadArgs a{};
    a.code = code; a.g = g; a.tables = static_cast<const char *>(tables); a.out = grad_score;
    a.g_token_stride = g_token_stride; a.g_slice_stride = g_slice_stride;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do / SLICE_COLS);
    a.row_bytes = (int)(Do * 4);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (np * 10 + c) {
        case 44: return launch_inner_quad<4, 4>(a, st);
        case 42: return launch_inner_quad<4, 2>(a, st);
        default: return LFFN_ERR_BAD_ARG;
    }
}
