// The layer's weighted gather-add, table-major, two tables per LDS buffer, FOUR lanes per token:
//
//   out[b,:] = bias + sum_t score[b,t] * tables[t, code[b,t] & (S-1), :]
//
// (PL/lookup.py:120-130 with the index offset of ":126" and the bias of ":108" folded in.)
//
// Same idea as lookup_gather.hip (a workgroup keeps the accumulators of a token tile in registers
// and walks the tables through LDS) and the same LDS layout as lookup_gather_pair.hip (a buffer row
// holds the 128-byte segments of tables 2k and 2k+1 side by side), with a geometry chosen so that a
// staged table byte serves four times as many tokens:
//
//   * a workgroup owns a 128-byte column slice (32 fp32 columns) and a tile of 256*NP tokens: the
//     four lanes of a quad cover a token, a lane owns 8 columns (two 16-byte pieces 64 bytes apart),
//     a wavefront covers 16 tokens at a time.  Per staged byte four times the tokens of the
//     256-byte-slice form: a quarter of the L2 -> LDS copy volume per token;
//   * bank conflicts: the LDS serves 64 banks (256 bytes) per clock to 16 lanes = four quads.  In every
//     read the four quads of a 16-lane group take four different 64-byte columns of the 256-byte row
//     window (table 2k or 2k+1, first or second half of the segment), whatever rows their codes
//     select, and rotate through the four columns over the four reads of a table pair.  So the
//     order in which a quad adds the pair's two tables depends on the quad (2k then 2k+1, or the
//     reverse); each token still adds its T rows one at a time in fp32;
//   * (code, score) pairs come from a stream of records, three words per (table pair, token), that a
//     small kernel packs first (the caller's [B, T] arrays have a token's pair 8 bytes wide in rows
//     T*4 bytes apart: sixteen cache lines per wavefront load).  The stream keeps, per table pair, the
//     records in the order the wavefronts use them (lffn_quad_record_slot in lffn_common.h): all the
//     records a wavefront needs for a pair, 16 tokens x its passes, are one contiguous run of 192
//     bytes per pass.  A wavefront copies that run for the NEXT table pair straight from global
//     memory into its own corner of LDS while it works on the current one (one or two 16-byte-per-
//     lane copy instructions, no registers, nothing to wait for), reads its records from there at the
//     start of the step, two per lane, and hands them round the quad with DPP quad_perm moves.  Six
//     registers hold a lane's records, against 3*NP when they were loaded a chunk of tables ahead.
//     (As three planes indexed by token, which is how the stream was laid out first, the same copy
//     took six one-word-per-lane instructions, and the vector memory path is as busy as the LDS:
//     105 -> 100 us at 16384 tokens x 128 tables x 768.)
//
// One barrier per table pair; the global -> LDS copy of pair k+1 has the whole of pair k's work to land.
//
// Row formats.  fp32 rows: the slice is 32 columns and a lane owns 8 of them.  16-bit rows (bfloat16, and
// half, the format of the reference's own reduced-precision kernels, PL/gather/cuda/extension/
// gather_kernel_fp16.cu:6-62): the slice is still 128 bytes = 64 columns, a lane owns 16 of them, and the
// sums stay fp32 (the reference accumulates in half).  The LDS side is the same bytes either way; what
// differs is the vector-ALU work per 16-byte piece: 4 multiply-adds (fp32), 8 widenings + 8 multiply-adds
// (bfloat16: a shift or a mask per value), 8 v_fma_mix_f32 (half: the instruction widens its operand).
#include "lffn_common.h"

namespace {

constexpr int WG = 1024;
constexpr int NWAVES = WG / 64;
constexpr int MAX_S = 256;
constexpr int XCDS = 8;
constexpr int BUF_BYTES = MAX_S * 256;      // one table pair: S rows of 2 x 128 bytes; a power of two (bit 16)
constexpr int SLICE_BYTES = 128;            // a slice of a row: 32 fp32 columns or 64 16-bit columns
constexpr int FMT_F32 = LFFN_ROWS_F32, FMT_BF16 = LFFN_ROWS_BF16, FMT_F16 = LFFN_ROWS_F16;
constexpr int fmt_bytes(int fmt) { return fmt == FMT_F32 ? 4 : 2; }
constexpr int QUAD_TOUCH_AHEAD = 3;         // pairs between the one being read and the one being touched

// (code, score) of one token and one table pair in the order the token's quad takes the pair's tables
// (tokens whose index has bit 1 set take table 2k+1 first): three words, word 0 = score of the first
// table, 1 = score of the second, 2 = row of the first table | row of the second << 8; where a token's
// record sits among its pair's: lffn_quad_record_slot.
struct PairRecord {
    float score_first, score_second;
    uint32_t rows;
};
constexpr int REC_WORDS = LFFN_RECORD_WORDS;

struct QuadArgs {
    const char *tables;    // [T, S, Do] fp32, bfloat16 or half
    const float *bias;     // [Do] or null
    const float *residual; // [B, Do] or null: added to the result (may be the output buffer)
    float *out;            // [B, Do]
    int64_t B;
    int T, S, Do;          // T even, S = 256
    int ntiles, nslices, per_xcd;
    int tile_tokens;       // tokens per tile: a multiple of 16 in ((NP - 1) * 256, NP * 256]
    int row_bytes;         // Do * bytes per element
    const uint32_t *stream;     // [T/2][Bpad][3] record words written by pack_pairs_kernel
    int64_t Bpad;               // record slots per table pair: every tile's tile_tokens (lffn_internal_quad_record_stride)
};

// global_load_lds_dwordx4 / _dword with a scalar base and a 32-bit lane offset: lane i of the
// wavefront writes its 16 (4) bytes at the LDS address in M0 + 16*i (4*i).  Inline assembly so that
// the compiler does not serialise the copy with the LDS reads of the other buffer; the caller waits
// (vmcnt) before the data is read.  M0 is put back: the compiler reserves it for its own use and
// does not honour a clobber declaration of it.
__device__ __forceinline__ void lds_dma16(const char *base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(base), "s"(lds_byte_addr)
                 : "memory");
}
__device__ __forceinline__ void lds_dma4(const char *base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(base), "s"(lds_byte_addr)
                 : "memory");
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x3 __attribute__((ext_vector_type(3)));
typedef __attribute__((address_space(3))) const u32x4 *lds_vec_ptr;
// a record in LDS: three consecutive words
struct LdsRecord { unsigned x, y, z; };
typedef __attribute__((address_space(3))) const unsigned *lds_word_ptr;
__device__ __forceinline__ LdsRecord read_record(unsigned lds_byte_addr) {
    lds_word_ptr p = (lds_word_ptr)(uintptr_t)lds_byte_addr;
    return LdsRecord{p[0], p[1], p[2]};
}

// Value held by lane N of the caller's quad, in every lane of the quad (one DPP move).
template <int N>
__device__ __forceinline__ unsigned quad_broadcast(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, N * 0x55, 0xF, 0xF, true);     // quad_perm [N,N,N,N]
}

// An LDS byte address whose rows are 256 bytes apart: byte 1 (the row number) from byte BYTE of
// `packed`, the other three bytes from `base`.  One v_perm_b32 (a plain, full-rate instruction).
template <int BYTE>
__device__ __forceinline__ unsigned with_row(unsigned base, unsigned packed) {
    // selector bytes 0-3 name bytes of the second operand, 4-7 bytes of the first
    return __builtin_amdgcn_perm(packed, base, 0x03020000u | ((4u + BYTE) << 8));
}

// Packs the caller's [B, T] codes and scores into the record stream [T/2][Bpad][3].  A workgroup takes 64
// tokens x 32 table pairs: it reads them pair-fastest (a token's 32 pairs are 256 contiguous bytes),
// turns them round in LDS and writes them token-fastest (16 consecutive tokens' records of a pair are 192
// contiguous bytes).  Slots of tokens from B on are left as they are: the gather reads them (their row
// numbers are bytes, always inside the LDS buffer) and does not store their sums.
__global__ __launch_bounds__(256) void pack_pairs_kernel(const int32_t *code, const float *score, uint32_t *stream,
                                                         int64_t B, int64_t Bpad, int T, int S, int tile_tokens) {
    __shared__ PairRecord tile[32][64 + 1];
    const int npairs = T / 2;
    const int64_t tok0 = int64_t(blockIdx.x) * 64;
    const int k0 = blockIdx.y * 32;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int item = threadIdx.x + 256 * i;
        const int kk = item & 31, row = item >> 5;
        const int64_t b = tok0 + row;
        PairRecord r{0.f, 0.f, 0u};
        if (b < B && k0 + kk < npairs) {
            const int2 c = *reinterpret_cast<const int2 *>(code + b * T + 2 * (k0 + kk));
            const float2 w = *reinterpret_cast<const float2 *>(score + b * T + 2 * (k0 + kk));
            const uint32_t ca = uint32_t(c.x & (S - 1)), cb = uint32_t(c.y & (S - 1));
            const bool second_first = (b & 2) != 0;
            r.score_first = second_first ? w.y : w.x;
            r.score_second = second_first ? w.x : w.y;
            r.rows = second_first ? (cb | (ca << 8)) : (ca | (cb << 8));
        }
        tile[kk][row] = r;
    }
    __syncthreads();
    const int row = threadIdx.x & 63;
    const int64_t slot = tok0 + row < B ? lffn_quad_record_slot(tok0 + row, tile_tokens) : 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int kk = (threadIdx.x >> 6) + 4 * i;
        if (tok0 + row < B && k0 + kk < npairs) {
            uint32_t *dst = stream + (int64_t(k0 + kk) * Bpad + slot) * REC_WORDS;
            const PairRecord r = tile[kk][row];
            dst[0] = __float_as_uint(r.score_first);
            dst[1] = __float_as_uint(r.score_second);
            dst[2] = r.rows;
        }
    }
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// acc += w * (the EPV values of one 16-byte piece of a row)
template <int FMT, int EPV>
__device__ __forceinline__ void fma_piece(float (&ac)[EPV], float w, const u32x4 &v) {
    if constexpr (FMT == FMT_F32) {
        ac[0] = fmaf(__uint_as_float(v.x), w, ac[0]);
        ac[1] = fmaf(__uint_as_float(v.y), w, ac[1]);
        ac[2] = fmaf(__uint_as_float(v.z), w, ac[2]);
        ac[3] = fmaf(__uint_as_float(v.w), w, ac[3]);
    } else {
        const unsigned q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (FMT == FMT_BF16) {
                ac[2 * i] = fmaf(bf16_lo(q[i]), w, ac[2 * i]);
                ac[2 * i + 1] = fmaf(bf16_hi(q[i]), w, ac[2 * i + 1]);
            } else {
                // (float)half * float + float: one v_fma_mix_f32 each
                const half2_t h = __builtin_bit_cast(half2_t, q[i]);
                ac[2 * i] = fmaf((float)h.x, w, ac[2 * i]);
                ac[2 * i + 1] = fmaf((float)h.y, w, ac[2 * i + 1]);
            }
        }
    }
}

template <int FMT, int NP, bool TOUCH>
__global__ __launch_bounds__(WG) void lookup_gather_quad_kernel(QuadArgs a) {
    static_assert(NP >= 4 && NP <= 8, "a lane reads the records of passes l and l + 4");
    constexpr int EPV = 16 / fmt_bytes(FMT);              // columns in a 16-byte piece
    constexpr int SLICE_COLS = SLICE_BYTES / fmt_bytes(FMT);
    constexpr int WAVE_RECS = 16 * NP;                    // records a wavefront uses per table pair, at most
    extern __shared__ uint4 lds[];                // 2 buffers of BUF_BYTES, the touches' sink, the wavefronts' records

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.ntiles * a.nslices) return;     // uniform over the workgroup
    const int slice = unit / a.ntiles;
    const int tile = unit % a.ntiles;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int quad = lane >> 2;       // token within the wavefront's sixteen
    const int l = lane & 3;           // lane within the quad: 16-byte piece l of each 64-byte column
    // the quad's place among the four quads of its 16-lane group decides which 64-byte column of the
    // row window it starts on: bit 1 = which table of the pair comes first, bit 0 = which half of the
    // 128-byte segment comes first
    const bool second_first = (quad & 2) != 0;
    const int half0 = quad & 1;
    // Tile `tile` holds tokens [tile * tile_tokens, (tile + 1) * tile_tokens), in groups of 16: group p * 16 + wave
    // is pass p of wavefront `wave`.  tile_tokens need not fill the last pass: the wavefronts whose group of that
    // pass lies beyond the tile leave the pass out (the launch balances the tiles: 16384 tokens over 10 workgroups
    // are 1648 each, six passes and seven of sixteen wavefronts in the seventh, instead of nine full tiles of
    // 1792 and a tenth that is mostly padding).
    const int64_t tok0 = int64_t(tile) * a.tile_tokens + wave * 16 + quad;
    const int n_last = a.tile_tokens / 16 - 16 * (NP - 1);                     // wavefronts that have the last pass
    const bool last_pass = wave < n_last;                                      // uniform over the wavefront

    // acc[p][h][e]: token tok0 + 256 p, column ((half0 ^ h) * 4 + l) * EPV + e of the slice
    float acc[NP][2][EPV];
    {
        float b[2][EPV];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < EPV; ++e) b[h][e] = 0.f;
        if (a.bias) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float *bp = a.bias + (size_t)slice * SLICE_COLS + ((half0 ^ h) * 4 + l) * EPV;
#pragma unroll
                for (int e = 0; e < EPV; ++e) b[h][e] = bp[e];
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[p][h][e] = b[h][e];
    }

    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // Where pair k's 2 x S x 128 bytes of this slice start, and which bytes of them this lane copies:
    // vector q = tid + 1024*i is piece q%16 of LDS row q/16; pieces 0-7 come from table 2k, 8-15 from
    // 2k+1; rows are Do*4 bytes apart, the second table S rows further down.  The four vectors of a lane
    // are 64 rows apart: one lane offset, four uniform bases.
    const size_t table_bytes = (size_t)a.S * a.row_bytes;
    const char *slice_base = a.tables + (size_t)slice * SLICE_BYTES;
    const size_t pair_stride = 2 * table_bytes;
    const size_t quarter = (size_t)(WG / 16) * a.row_bytes;
    const int npairs = a.T / 2;
    const uint32_t copy_off = ((tid & 15) < 8 ? 0u : (uint32_t)table_bytes) + (uint32_t)(tid >> 4) * (uint32_t)a.row_bytes +
                              (uint32_t)(tid & 7) * 16u;
    const uint32_t copy_dst = (uint32_t)wave * (64 * 16);       // LDS byte offset of this wavefront's first vector in a buffer
    auto copy_pair_to_lds = [&](const char *pair_base, uint32_t dst_byte_addr) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_dma16(pair_base + i * quarter, copy_off, dst_byte_addr + copy_dst + i * (WG * 16));
    };

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

    // This wavefront's records of a table pair: 16 per pass, record r = pass r/16, quad r%16, 12 bytes each,
    // one contiguous run in the stream (lffn_quad_record_slot) and, copied as it is, at rec_lds + 12 r in
    // LDS.  12 NPW lanes copy 16 bytes each: one instruction up to five passes, two beyond.
    const uint32_t rec_lds = lds0 + 2u * BUF_BYTES + TOUCH_SINK_BYTES + (uint32_t)wave * (WAVE_RECS * REC_WORDS * 4);
    const int wave_slot = 16 * ((NP - 1) * wave + min(wave, n_last));
    const char *rec_base = reinterpret_cast<const char *>(a.stream + (int64_t(tile) * a.tile_tokens + wave_slot) * REC_WORDS);
    const size_t pair_rec_bytes = (size_t)a.Bpad * (REC_WORDS * 4);
    auto copy_records_to_lds = [&](int k, auto npw_c) {
        constexpr int NV = 12 * decltype(npw_c)::value;         // 16-byte vectors
        const char *src = rec_base + (size_t)k * pair_rec_bytes;
        if (NV >= 64 || lane < NV) lds_dma16(src, (uint32_t)lane * 16u, rec_lds);
        if constexpr (NV > 64) {
            if (lane < NV - 64) lds_dma16(src + 1024, (uint32_t)lane * 16u, rec_lds + 1024u);
        }
    };
    // lane l of a quad reads the records of passes l and l + 4 (clamped: NP = 4..7 have fewer than 8)
    const uint32_t rec_read0 = rec_lds + (uint32_t)((l * 16 + quad) * (REC_WORDS * 4));
    const uint32_t rec_read1 = rec_lds + (uint32_t)((min(l + 4, NP - 1) * 16 + quad) * (REC_WORDS * 4));

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

    // The loop over the table pairs for a wavefront that takes NPW of the NP passes (NP, or NP - 1 when its group
    // of the last pass lies beyond the tile): two copies of the loop, chosen once, so that neither has a branch
    // inside (a conditional in the loop body, even a uniform one, costs this kernel hundreds of spilled
    // registers).  Both copies meet at the same barriers.
    auto run_pairs = [&](auto npw_c) {
    constexpr int NPW = decltype(npw_c)::value;
    copy_records_to_lds(0, npw_c);
    copy_pair_to_lds(slice_base, lds0);
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);
    // A pair's records: x, y = the scores and z = the row numbers (first | second << 8), in the order the
    // quad takes the pair's tables.  They sit in this wavefront's own corner of LDS and it has just waited
    // for its own copies, so they are read BEFORE the barrier: their latency is out of the way when the
    // barrier opens and the first row reads go out at once.  (The copies are inline assembly: the compiler
    // does not know that they write LDS nor that the wait is what completes them, so an ordering point it
    // does honour keeps the reads below the wait.)  A lane whose pass l + 4 is beyond NPW reads a record
    // that is not this step's (or not written at all): it is never used.
    asm volatile("" ::: "memory");
    LdsRecord rec0 = read_record(rec_read0);
    LdsRecord rec1 = read_record(rec_read1);
    __syncthreads();
    for (int k = 0; k < npairs; ++k) {

        // Software pipeline over the passes: a pass's four rows are requested while the pass before
        // is still being added (its first table's two rows are consumed, their registers take the
        // next pass's first two reads; likewise the second table's), so a wavefront always has
        // two to four row reads in flight behind its multiply-adds.
        auto fma4 = [&](float (&ac)[EPV], float w, const u32x4 &v) { fma_piece<FMT, EPV>(ac, w, v); };
        // the record of pass P sits in lane P % 4 of the quad, in rec0 (P < 4) or rec1
        auto rows_of = [&](auto p_c) {
            constexpr int P = decltype(p_c)::value;
            return quad_broadcast<P % 4>(P < 4 ? rec0.z : rec1.z);
        };
        auto score_of = [&](auto p_c, auto which_c) {
            constexpr int P = decltype(p_c)::value, W = decltype(which_c)::value;
            return __uint_as_float(quad_broadcast<P % 4>(P < 4 ? (W ? rec0.y : rec0.x) : (W ? rec1.y : rec1.x)));
        };
        using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
        // the first pass's rows are asked for before anything else ...
        u32x4 r[4];
        unsigned pk = rows_of(I0{});
        r[0] = *(lds_vec_ptr)(uintptr_t)with_row<0>(base[0], pk);
        r[1] = *(lds_vec_ptr)(uintptr_t)with_row<0>(base[1], pk);
        r[2] = *(lds_vec_ptr)(uintptr_t)with_row<1>(base[2], pk);
        r[3] = *(lds_vec_ptr)(uintptr_t)with_row<1>(base[3], pk);
        __builtin_amdgcn_sched_barrier(0);
        // ... and the copies are issued while they are on their way.  The records have been read (the row
        // numbers above came from them), so the next pair's may overwrite them in LDS; the next pair's
        // segments go straight into the other buffer (last read one pair ago, before the previous
        // barrier); the last step copies the last pair's again.
        asm volatile("" : "+v"(rec0.x), "+v"(rec0.y), "+v"(rec0.z), "+v"(rec1.x), "+v"(rec1.y), "+v"(rec1.z));
        const int kn = min(k + 1, npairs - 1);
        copy_records_to_lds(kn, npw_c);
        copy_pair_to_lds(slice_base + (size_t)kn * pair_stride, lds0 + (uint32_t)((k + 1) & 1) * BUF_BYTES);
        if constexpr (TOUCH) {
            const bool mine = turn == tile;                              // uniform
            const int kt = mine ? min(k + QUAD_TOUCH_AHEAD, npairs - 1) : k;
            l2_touch(slice_base + (size_t)kt * pair_stride, mine ? touch_off_on : 0u, touch_dst);
            turn = turn + 1 == a.ntiles ? 0 : turn + 1;
        }
        __builtin_amdgcn_sched_barrier(0);
        static_for<NPW>([&](auto p_c) {
            constexpr int P = decltype(p_c)::value;
            constexpr bool MORE = P + 1 < NPW;
            using PN = std::integral_constant<int, MORE ? P + 1 : P>;
            if constexpr (MORE) pk = rows_of(PN{});
            const float w0 = score_of(p_c, I0{});
            fma4(acc[P][0], w0, r[0]);
            fma4(acc[P][1], w0, r[1]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MORE) {
                r[0] = *(lds_vec_ptr)(uintptr_t)with_row<0>(base[0], pk);
                r[1] = *(lds_vec_ptr)(uintptr_t)with_row<0>(base[1], pk);
            }
            const float w1 = score_of(p_c, I1{});
            __builtin_amdgcn_sched_barrier(0);
            fma4(acc[P][0], w1, r[2]);
            fma4(acc[P][1], w1, r[3]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MORE) {
                r[2] = *(lds_vec_ptr)(uintptr_t)with_row<1>(base[2], pk);
                r[3] = *(lds_vec_ptr)(uintptr_t)with_row<1>(base[3], pk);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // the other buffer for the next pair
#pragma unroll
        for (int i = 0; i < 4; ++i) base[i] ^= (unsigned)BUF_BYTES;
        // the copies issued above have landed (records and segments); the touch, issued after them, may still be out
        __builtin_amdgcn_s_waitcnt(TOUCH ? WAIT_VMCNT_1 : WAIT_VMCNT_0);
        // the next pair's records (this wavefront's own, just landed; kept below the wait by the ordering
        // point), then the barrier for the segments
        asm volatile("" ::: "memory");
        rec0 = read_record(rec_read0);
        rec1 = read_record(rec_read1);
        __syncthreads();
    }
    };
    if (last_pass) run_pairs(std::integral_constant<int, NP>{});
    else run_pairs(std::integral_constant<int, NP - 1>{});
    __builtin_amdgcn_s_waitcnt(WAIT_VMCNT_0);         // nothing may still be writing this workgroup's LDS when it ends

#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int64_t tok = tok0 + p * 256;
        if (tok < a.B && (p < NP - 1 || last_pass)) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < EPV / 4; ++q) {
                    const size_t off = tok * a.Do + (size_t)slice * SLICE_COLS + ((half0 ^ h) * 4 + l) * EPV + 4 * q;
                    float4 v = make_float4(acc[p][h][4 * q], acc[p][h][4 * q + 1], acc[p][h][4 * q + 2], acc[p][h][4 * q + 3]);
                    if (a.residual) {
                        const float4 rr = *reinterpret_cast<const float4 *>(a.residual + off);
                        v.x += rr.x; v.y += rr.y; v.z += rr.z; v.w += rr.w;
                    }
                    *reinterpret_cast<float4 *>(a.out + off) = v;
                }
        }
    }
}

template <int FMT, int NP, bool TOUCH>
int launch_quad(QuadArgs a, hipStream_t stream) {
    a.ntiles = (int)((a.B + a.tile_tokens - 1) / a.tile_tokens);
    const int units = a.ntiles * a.nslices;
    a.per_xcd = (units + XCDS - 1) / XCDS;
    // two buffers, the touches' scratch, every wavefront's records of one table pair
    const size_t lds_bytes = size_t(2) * BUF_BYTES + TOUCH_SINK_BYTES + size_t(NWAVES) * 16 * NP * REC_WORDS * 4;
    auto kern = lookup_gather_quad_kernel<FMT, NP, TOUCH>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, stream, a);
    return lffn_launch_status();
}

}  // namespace

// Bytes of the record stream for a shape: T/2 table pairs x the token slots of all tiles (fewer than 2048
// more than B, whatever the tile size).
int64_t lffn_internal_quad_stream_bytes(int64_t B, int64_t T) {
    return (T / 2) * (B + 2048) * (int64_t)(REC_WORDS * 4);
}

// Which tile sizes (passes of 256 tokens per workgroup) are built for a row format: the accumulators, 8 per
// pass and lane for fp32 rows and 16 for 16-bit rows, must fit the 128 registers a lane of a 1024-lane
// workgroup can have.
bool lffn_internal_quad_np_built(int fmt, int np) {
    if (fmt == FMT_F32) return np >= 4 && np <= 8;
    return (fmt == FMT_BF16 || fmt == FMT_F16) && np == 4;
}

// Passes a tile of `tokens` tokens takes: the smallest built number that covers it, or 0 (tokens: a multiple
// of 16 in [16, 2048]).
int lffn_internal_quad_passes(int fmt, int64_t tokens) {
    if (tokens < 16 || tokens > 2048 || tokens % 16 != 0) return 0;
    const int need = (int)((tokens + 255) / 256);
    for (int np = need; np <= 8; ++np)
        if (lffn_internal_quad_np_built(fmt, np)) return np;
    return 0;
}

// Record slots per table pair for B tokens in tiles of `tokens`: whole tiles (a multiple of 16, fewer than
// B + 2048).
int64_t lffn_internal_quad_record_stride(int64_t B, int fmt, int64_t tokens) {
    (void)fmt;
    return (B + tokens - 1) / tokens * tokens;
}

// Run the gather from a record stream [T/2][record_stride][3] (pack_pairs_kernel's layout; the projection
// kernels of fht.hip and bh4_block.hip write the same) with `tokens` tokens per workgroup, the tile size
// the stream was written for.  The caller has checked that the
// shape qualifies: S = 256 (a table pair fills an LDS buffer), T even, Do a multiple of the slice's columns
// (32 for fp32 rows, 64 for 16-bit rows), 2*S*Do*element bytes < 2^32 (32-bit lane offsets from a table
// pair's base), a tile size the format is built for.  record_stride: at least
// lffn_internal_quad_record_stride(B, fmt, tokens); what the records of tokens from B on hold does not matter
// (their row numbers are bytes, always inside the LDS buffer, and their sums are not stored).
int lffn_internal_lookup_gather_quad_records(const uint32_t *records, int64_t record_stride, const void *tables,
                                             const float *bias, const float *residual, float *out, int64_t B,
                                             int64_t T, int64_t S, int64_t Do, int fmt, int tokens, void *stream) {
    const int np = lffn_internal_quad_passes(fmt, tokens);
    if (!records || S != MAX_S || T % 2 != 0 || np == 0 || tokens <= 256 * (np - 1)) return LFFN_ERR_BAD_ARG;
    // 16-byte copies: the stream and every table pair's part of it on 16-byte boundaries
    if (record_stride < lffn_internal_quad_record_stride(B, fmt, tokens) || record_stride % 4 != 0 ||
        !lffn_aligned16(records))
        return LFFN_ERR_BAD_ARG;
    const int esz = fmt_bytes(fmt);
    if (Do % (SLICE_BYTES / esz) != 0) return LFFN_ERR_BAD_ARG;
    QuadArgs a{};
    a.tables = static_cast<const char *>(tables); a.bias = bias; a.residual = residual; a.out = out;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do * esz / SLICE_BYTES);
    a.row_bytes = (int)(Do * esz);
    a.tile_tokens = tokens;
    a.Bpad = record_stride;
    a.stream = records;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the touch by turns, always: tables beyond the 256 MB memory-side cache need it most (984 -> 736 us
    // at 512 tables x 256 x 1024 and 1024 tokens per workgroup)
    if (fmt == FMT_BF16) return launch_quad<FMT_BF16, 4, true>(a, st);
    if (fmt == FMT_F16) return launch_quad<FMT_F16, 4, true>(a, st);
    switch (np) {
        case 8: return launch_quad<FMT_F32, 8, true>(a, st);
        case 7: return launch_quad<FMT_F32, 7, true>(a, st);
        case 6: return launch_quad<FMT_F32, 6, true>(a, st);
        case 5: return launch_quad<FMT_F32, 5, true>(a, st);
        default: return launch_quad<FMT_F32, 4, true>(a, st);
    }
}

// Pack the (code, score) pairs into the record stream in `workspace` (at least
// lffn_internal_quad_stream_bytes(B, T) bytes, 16-byte aligned) and run the gather from it.
int lffn_internal_lookup_gather_quad(const int32_t *code, const float *score, const void *tables,
                                     const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                     int64_t S, int64_t Do, int fmt, int tokens, void *workspace, void *stream) {
    if (!workspace || S != MAX_S || T % 2 != 0 || lffn_internal_quad_passes(fmt, tokens) == 0) return LFFN_ERR_BAD_ARG;
    if (B == 0) return LFFN_OK;
    uint32_t *recs = static_cast<uint32_t *>(workspace);
    const int64_t stride = lffn_internal_quad_record_stride(B, fmt, tokens);
    const dim3 grid((unsigned)((B + 63) / 64), (unsigned)((T / 2 + 31) / 32));
    hipLaunchKernelGGL(pack_pairs_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), code, score, recs, B,
                       stride, (int)T, (int)S, tokens);
    if (hipGetLastError() != hipSuccess) return LFFN_ERR_LAUNCH;
    return lffn_internal_lookup_gather_quad_records(recs, stride, tables, bias, residual, out, B, T, S, Do, fmt, tokens, stream);
}
