// Table gradient of the lookup layer without atomics on the accumulators:
//
//   grad_tables[t][code[b][t]][:] += score[b][t] * g[b][:]        (PL/gather/cuda/kernel.py:190-202,
//                                                                   PL/gather/cuda/extension/gather_kernel_fp32.cu:49)
//
// Three launches and a workspace.
//
// lookup_prep_kernel: code and score are [B, T]; a table's column is one value per 4*T bytes,
// and 64 lanes reading it are 64 separate requests, which made the sort four times slower
// than it is.  The kernel writes them transposed, [T, B] (codes masked, as 16-bit values).
//
// lookup_sort_pack_kernel: two jobs in one launch, by workgroup number.  The sort occupies one
// workgroup per table (128 of the 256 compute units at 128 tables) and is bound by latency; the
// copy of g to a slice-major layout [Do/32][B][32] (in which the 128-byte row pieces of a slice
// are contiguous: with rows 4*Do bytes apart the pieces of one slice fall on a quarter of the L2
// channels) is pure memory traffic and depends on nothing: its workgroups fill the rest of the
// chip while the sort runs (23 + 25 us as two launches at 16384 tokens x 128 tables x 768).
//
// The sort: one workgroup per table sorts the tokens by their code for that
// table (a stable counting sort: per-wavefront histograms over contiguous token ranges,
// ranks inside a 64-token batch from ballots over the code bits) and writes (token, score)
// pairs bucket by bucket: into LDS first (a 16-bit token and a score per entry: at most 18432
// entries, 108 KB), from where the list goes to memory in whole lines; written straight
// from the ranks, every wavefront store was 64 separate 8-byte requests.  Every bucket is padded to a multiple of eight entries with
// (first token of the bucket, 0.0f), so that eight consecutive entries always belong to
// one code, and the bucket boundaries are stored in units of eight entries.
//
// lookup_scatter_sorted_kernel: one workgroup per (table, 32-column slice).  The sorted
// list is cut into equal pieces, one per wavefront, whatever the bucket sizes (a skewed code
// distribution costs nothing).  A wavefront walks its piece eight tokens at a time: lane
// group q = lane / 8 takes token q of the step, its eight lanes load the token's 128-byte
// piece of g and multiply-add it into registers; at a bucket boundary (wave-uniform,
// because of the padding) the eight partial sums are added across the lane groups and the
// row is stored.  Buckets cut by a piece boundary go to LDS and one wavefront adds the
// pieces in order after a barrier.  Every row of the slice is written exactly once with
// plain stores: no zero-fill, no atomics, and the sum order is fixed (run-to-run
// reproducible).  The slices are dealt to the XCDs so that the workgroups running on one
// XCD read the same 32 columns of g (2 MB at 16384 tokens), which then stay in its L2.
#include "lffn_common.h"

namespace {

constexpr int SORT_WG = 1024;
constexpr int SORT_WAVES = SORT_WG / 64;
constexpr int MAX_S = 512;
constexpr int XCDS = 8;
constexpr int SORT_DEPTH = 16;      // batches of 64 tokens whose loads are in flight per wavefront

constexpr int MWG = 512;             // main kernel: threads per workgroup
constexpr int MWAVES = MWG / 64;
constexpr int SC = 32;               // columns per slice: 8 lanes x float4
constexpr int U = 8;                 // steps (of eight tokens) per batch = one 64-entry load of pairs

struct PrepArgs {
    const int32_t *code;   // [B, T]
    const float *score;    // [B, T]
    const float *g;        // [B, Do]
    uint16_t *code_t;      // [T, Bp]
    float *score_t;        // [T, Bp]
    float *g_packed;       // [Do / SC][B][SC]
    int64_t B, Bp;
    int T, S, Do, tiles_t;
};

// one 64 x 64 tile of code and score per workgroup
__global__ __launch_bounds__(256) void lookup_prep_kernel(PrepArgs a) {
    __shared__ int sc[64][65];
    __shared__ float ss[64][65];
    const int tid = threadIdx.x, lane = tid & 63, row0 = tid >> 6;
    const int64_t b0 = int64_t(blockIdx.x / a.tiles_t) * 64;
    const int t0 = (blockIdx.x % a.tiles_t) * 64;
    const int mask = a.S - 1;
    // all sixteen rows of a thread are requested before the first is used
    int cv[16];
    float sv[16];
    const int t_in = t0 + lane;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t b = b0 + row0 + 4 * i;
        const bool live = b < a.B && t_in < a.T;
        cv[i] = live ? a.code[b * a.T + t_in] : 0;
        sv[i] = live ? a.score[b * a.T + t_in] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        sc[row0 + 4 * i][lane] = cv[i] & mask;
        ss[row0 + 4 * i][lane] = sv[i];
    }
    __syncthreads();
    const int64_t b_out = b0 + lane;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = row0 + 4 * i, t = t0 + r;
        if (b_out < a.B && t < a.T) {
            a.code_t[(size_t)t * a.Bp + b_out] = (uint16_t)sc[lane][r];
            a.score_t[(size_t)t * a.Bp + b_out] = ss[lane][r];
        }
    }
}

constexpr int PACK_TOKENS = 32;      // rows of g per workgroup of the slice-major copy

// PACK_TOKENS rows of g, copied to the slice-major layout (workgroup `blk` of the copy)
__device__ __forceinline__ void pack_rows(const PrepArgs &a, int64_t blk) {
    const int64_t b0 = blk * PACK_TOKENS;
    const int q = a.Do / 4;
    // eight loads per thread in flight before the first store (a store must not overtake a load the compiler
    // cannot prove independent of it, so load-store pairs one after the other would each wait out a round trip)
    constexpr int DEPTH = 8;
    for (int e0 = threadIdx.x; e0 < PACK_TOKENS * q; e0 += SORT_WG * DEPTH) {
        float4 v[DEPTH];
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) {
            const int e = e0 + i * SORT_WG;
            const int64_t b = b0 + e / q;
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < PACK_TOKENS * q && b < a.B) v[i] = *reinterpret_cast<const float4 *>(a.g + (size_t)b * a.Do + (e % q) * 4);
        }
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) {
            const int e = e0 + i * SORT_WG;
            const int64_t b = b0 + e / q;
            const int col = (e % q) * 4;
            if (e < PACK_TOKENS * q && b < a.B)
                *reinterpret_cast<float4 *>(a.g_packed + ((size_t)(col / SC) * a.B + b) * SC + col % SC) = v[i];
        }
    }
}

struct SortArgs {
    const uint16_t *code;  // [T, Bp], masked
    const float *score;    // [T, Bp]
    uint2 *pairs;          // [T, stride] (token, score bits)
    int32_t *off8;         // [T, S + 1] bucket starts, in units of eight entries
    int64_t B, Bp, stride;
    int T, S, nbits;
    int stage;             // the sorted list is collected in LDS and written out in whole lines (it fits: S <= 256)
};

__device__ __forceinline__ void sort_table(const SortArgs &a, const int t) {
    extern __shared__ int sm[];
    const int S = a.S;
    int *hist = sm;                    // [SORT_WAVES][S]: counts, then running write positions
    int *count = hist + SORT_WAVES * S;
    int *start = count + S;            // padded bucket starts (entries)
    int *first = start + S;            // lowest token of the bucket
    int *total = first + S;
    float *sc_s = reinterpret_cast<float *>(total + 4);                       // [stride] scores of the sorted list
    unsigned short *tok_s = reinterpret_cast<unsigned short *>(sc_s + a.stride);   // [stride] tokens

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint16_t *code = a.code + (size_t)t * a.Bp;
    const float *score = a.score + (size_t)t * a.Bp;
    for (int q = tid; q < SORT_WAVES * S; q += SORT_WG) hist[q] = 0;
    for (int q = tid; q < S; q += SORT_WG) first[q] = 0x7fffffff;
    __syncthreads();

    // A wavefront takes up to SORT_DEPTH batches of 64 consecutive tokens (the launch keeps B within 1024 * SORT_DEPTH).
    // Their codes and scores are loaded once, all loads in flight together, and stay in registers through both
    // passes, as does every token's rank among the tokens of its batch with the same code (from ballots over
    // the code bits): the first pass counts a batch's codes once per code (the lowest lane of each adds the
    // whole count: no two lanes of an instruction touch one counter, however skewed the codes are), the
    // second turns ranks into positions.
    const int64_t per = ((a.B + SORT_WG - 1) / SORT_WG) * 64;       // tokens per wavefront, whole batches
    const int64_t lo = min<int64_t>(a.B, wave * per), hi = min<int64_t>(a.B, lo + per);
    int *myh = hist + wave * S;
    int cv[SORT_DEPTH], rk[SORT_DEPTH];
    float sv[SORT_DEPTH];
#pragma unroll
    for (int k = 0; k < SORT_DEPTH; ++k) {
        const int64_t b = lo + 64 * k + lane;                    // loads are unconditional (clamped), so none waits for another
        const int64_t bc = min<int64_t>(b, a.B - 1);
        const int c = code[bc];
        sv[k] = score[bc];
        cv[k] = b < hi ? c : -1;
    }
#pragma unroll
    for (int k = 0; k < SORT_DEPTH; ++k) {
        rk[k] = 0;
        if (lo + 64 * k >= hi) continue;                         // uniform
        const bool live = cv[k] >= 0;
        const int c = live ? cv[k] : 0;
        unsigned long long m = __ballot(live);
        for (int bit = 0; bit < a.nbits; ++bit) {
            const bool mine = (c >> bit) & 1;
            const unsigned long long bb = __ballot(mine);
            m &= mine ? bb : ~bb;
        }
        const int rank = __popcll(m & ((1ull << lane) - 1ull));
        const int cnt = __popcll(m);
        rk[k] = rank | (cnt << 8);
        if (live && rank == 0) {
            myh[c] += cnt;
            atomicMin(&first[c], (int)(lo + 64 * k + lane));
        }
    }
    __syncthreads();
    for (int c = tid; c < S; c += SORT_WG) {
        int sum = 0;
        for (int w = 0; w < SORT_WAVES; ++w) {
            const int v = hist[w * S + c];
            hist[w * S + c] = sum;
            sum += v;
        }
        count[c] = sum;
        start[c] = (sum + 7) & ~7;
    }
    __syncthreads();
    if (wave == 0) {                   // exclusive scan of the padded counts
        const int per_lane = (S + 63) / 64;
        int loc = 0;
        for (int k = 0; k < per_lane; ++k) {
            const int i = lane * per_lane + k;
            if (i < S) loc += start[i];
        }
        int inc = loc;
        for (int d = 1; d < 64; d <<= 1) {
            const int v = __shfl_up(inc, d);
            if (lane >= d) inc += v;
        }
        int run = inc - loc;
        for (int k = 0; k < per_lane; ++k) {
            const int i = lane * per_lane + k;
            if (i < S) {
                const int v = start[i];
                start[i] = run;
                run += v;
            }
        }
        if (lane == 63) *total = inc;
    }
    __syncthreads();
    for (int c = tid; c < S; c += SORT_WG) {
        const int o = start[c];
        a.off8[(size_t)t * (S + 1) + c] = o >> 3;
        for (int w = 0; w < SORT_WAVES; ++w) hist[w * S + c] += o;
    }
    if (tid == 0) a.off8[(size_t)t * (S + 1) + S] = *total >> 3;
    __syncthreads();

    uint2 *out = a.pairs + (size_t)t * a.stride;
#pragma unroll
    for (int k = 0; k < SORT_DEPTH; ++k) {
        if (lo + 64 * k >= hi) continue;                         // uniform
        if (cv[k] >= 0) {
            const int c = cv[k], rank = rk[k] & 0xff, cnt = rk[k] >> 8;
            const int base = myh[c];                              // all lanes of a code read before its last lane writes
            if (a.stage) {                                        // uniform
                tok_s[base + rank] = (unsigned short)(lo + 64 * k + lane);
                sc_s[base + rank] = sv[k];
            } else {
                out[base + rank] = make_uint2((unsigned)(lo + 64 * k + lane), __float_as_uint(sv[k]));
            }
            if (rank == cnt - 1) myh[c] = base + cnt;
        }
    }
    __syncthreads();
    for (int c = tid; c < S; c += SORT_WG) {
        const int n = count[c], o = start[c];
        for (int p = n; p < ((n + 7) & ~7); ++p) {
            if (a.stage) {
                tok_s[o + p] = (unsigned short)first[c];
                sc_s[o + p] = 0.f;
            } else {
                out[o + p] = make_uint2((unsigned)first[c], 0u);
            }
        }
    }
    if (!a.stage) return;                                     // uniform
    __syncthreads();
    const int n_out = *total;
    for (int i = tid; i < n_out; i += SORT_WG) out[i] = make_uint2((unsigned)tok_s[i], __float_as_uint(sc_s[i]));
}

// workgroups [0, nsort): the sort of one table each; the others: PACK_TOKENS rows of the copy of g each
__global__ __launch_bounds__(SORT_WG) void lookup_sort_pack_kernel(SortArgs sa, PrepArgs pa, int nsort) {
    if ((int)blockIdx.x < nsort) sort_table(sa, (int)blockIdx.x);      // uniform over the workgroup
    else pack_rows(pa, int64_t(blockIdx.x) - nsort);
}

struct SortedArgs {
    const uint2 *pairs;
    const int32_t *off8;
    const float *g;        // [Do / SC][B][SC]
    float *out;            // [T, S, Do]
    int64_t stride;
    unsigned last_token;   // B - 1
    int T, S, Do, nslices, accumulate;
};

__device__ __forceinline__ float4 add4(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }

// v + (v of the lane 16 / 32 positions away): gfx950's row and half-wave swaps, no LDS traffic
__device__ __forceinline__ float add_xor16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float add_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// v + (v of lane ^ 8): a DPP rotation by eight inside the 16-lane row
__device__ __forceinline__ float add_xor8(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));
}

// sum over the eight lane groups; afterwards every lane holds the total of its column group
__device__ __forceinline__ float4 sum_groups(float4 v) {
    v.x = add_xor32(add_xor16(add_xor8(v.x)));
    v.y = add_xor32(add_xor16(add_xor8(v.y)));
    v.z = add_xor32(add_xor16(add_xor8(v.z)));
    v.w = add_xor32(add_xor16(add_xor8(v.w)));
    return v;
}

__global__ __launch_bounds__(MWG) void lookup_scatter_sorted_kernel(SortedArgs a) {
    extern __shared__ int sm[];
    const int S = a.S;
    int *off = sm;                                            // [S + 1]
    int *flag = off + ((S + 1 + 3) & ~3);                     // [MWAVES][4]: head code, head closes, tail code
    float *slot = reinterpret_cast<float *>(flag + MWAVES * 4);   // [MWAVES][2][SC]

    const int xcd = blockIdx.x % XCDS, idx = blockIdx.x / XCDS;
    const int slice = xcd + XCDS * (idx / a.T);
    const int t = idx % a.T;
    if (slice >= a.nslices) return;                           // uniform over the workgroup

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = lane >> 3, j = lane & 7;
    for (int q = tid; q <= S; q += MWG) off[q] = a.off8[(size_t)t * (S + 1) + q];
    if (tid < MWAVES * 4) flag[tid] = -1;
    __syncthreads();

    float *orow = a.out + (size_t)t * S * a.Do + (size_t)slice * SC + j * 4;     // + code * Do
    if (!a.accumulate)                                        // rows no token points at
        for (int q = tid; q < S * 8; q += MWG) {
            const int c = q >> 3;
            if (off[c + 1] == off[c])
                *reinterpret_cast<float4 *>(a.out + ((size_t)t * S + c) * a.Do + (size_t)slice * SC + (q & 7) * 4) =
                    make_float4(0.f, 0.f, 0.f, 0.f);
        }

    const int n8 = off[S];
    const int s_lo = (int)((int64_t)wave * n8 / MWAVES), s_hi = (int)((int64_t)(wave + 1) * n8 / MWAVES);
    if (s_lo < s_hi) {
        // the bucket holding step s_lo: the last c with off[c] <= s_lo
        int lo = 0, hi = S;                                   // invariant: off[lo] <= s_lo < off[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (off[mid] <= s_lo) lo = mid; else hi = mid;
        }
        int cur = __builtin_amdgcn_readfirstlane(lo);
        int next_b = __builtin_amdgcn_readfirstlane(off[cur + 1]);
        bool head = off[cur] < s_lo;                          // the bucket began in an earlier piece
        const uint2 *pp = a.pairs + (size_t)t * a.stride;
        const float *gcol = a.g + (size_t)slice * SC * (size_t(a.last_token) + 1) + j * 4;
        const int last_entry = s_hi * 8 - 1;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);

        auto flush = [&](bool continues) {
            const float4 v = sum_groups(acc);
            if (head) {
                if (lane < 8) *reinterpret_cast<float4 *>(slot + (wave * 2 + 0) * SC + j * 4) = v;
                if (lane == 0) { flag[wave * 4 + 0] = cur; flag[wave * 4 + 1] = continues ? 0 : 1; }
            } else if (continues) {
                if (lane < 8) *reinterpret_cast<float4 *>(slot + (wave * 2 + 1) * SC + j * 4) = v;
                if (lane == 0) flag[wave * 4 + 2] = cur;
            } else if (lane < 8) {
                float4 *dst = reinterpret_cast<float4 *>(orow + (size_t)cur * a.Do);
                *dst = a.accumulate ? add4(*dst, v) : v;
            }
            head = false;
            acc = make_float4(0.f, 0.f, 0.f, 0.f);
        };

        uint2 pr = pp[min(s_lo * 8 + lane, last_entry)];
        for (int step0 = s_lo; step0 < s_hi; step0 += U) {
            float4 gv[U];
            float sc[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const unsigned tok = min(__shfl(pr.x, u * 8 + grp), a.last_token);
                sc[u] = __uint_as_float(__shfl(pr.y, u * 8 + grp));
                gv[u] = *reinterpret_cast<const float4 *>(gcol + (size_t)tok * SC);
            }
            if (step0 + U < s_hi) pr = pp[min((step0 + U) * 8 + lane, last_entry)];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int step = step0 + u;
                if (step < s_hi) {                            // uniform
                    if (step == next_b) {                     // uniform: the bucket ended with the step before
                        flush(false);
                        do {
                            ++cur;
                            next_b = __builtin_amdgcn_readfirstlane(off[cur + 1]);
                        } while (next_b == step && cur < S - 1);   // skip codes without tokens
                    }
                    acc.x = fmaf(sc[u], gv[u].x, acc.x);
                    acc.y = fmaf(sc[u], gv[u].y, acc.y);
                    acc.z = fmaf(sc[u], gv[u].z, acc.z);
                    acc.w = fmaf(sc[u], gv[u].w, acc.w);
                }
            }
        }
        flush(next_b > s_hi);
    }
    __syncthreads();

    // buckets cut by piece boundaries: add their parts in order
    if (tid < 8) {
        float4 pend = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int w = 0; w < MWAVES; ++w) {
            const int hc = flag[w * 4 + 0];
            if (hc >= 0) {
                pend = add4(pend, *reinterpret_cast<const float4 *>(slot + (w * 2 + 0) * SC + j * 4));
                if (flag[w * 4 + 1] == 1) {
                    float4 *dst = reinterpret_cast<float4 *>(orow + (size_t)hc * a.Do);
                    *dst = a.accumulate ? add4(*dst, pend) : pend;
                    pend = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            if (flag[w * 4 + 2] >= 0) pend = *reinterpret_cast<const float4 *>(slot + (w * 2 + 1) * SC + j * 4);
        }
    }
}

inline int64_t pair_stride(int64_t B, int64_t S) { return ((B + 7) & ~int64_t(7)) + 8 * S; }

inline bool sorted_supported(int64_t B, int64_t T, int64_t S, int64_t Do) {
    return B >= 1 && T >= 1 && lffn_is_pow2(S) && S <= MAX_S && Do % SC == 0 && Do <= (1 << 20) &&
           B <= (int64_t(1) << 31) - 1 && T <= (1 << 20) && T * ((Do / SC + XCDS - 1) / XCDS) * XCDS <= 0x7fffffff;
}

inline int64_t round16(int64_t v) { return (v + 15) & ~int64_t(15); }
inline int64_t padded_tokens(int64_t B) { return (B + 63) & ~int64_t(63); }

// Tokens are taken CHUNK at a time (later chunks add to the result of the earlier ones): a
// 32-column slice of 16384 rows of g is 2 MB and stays in an XCD's 4 MB L2 while the
// workgroups of that XCD walk it in 128 different orders; twice that no longer does.
constexpr int64_t CHUNK = 16384;

struct Workspace {
    int64_t pairs, off8, code_t, score_t, g_packed, total;    // byte offsets
};

inline Workspace workspace_layout(int64_t B, int64_t T, int64_t S, int64_t Do) {
    Workspace w{};
    const int64_t Bc = B < CHUNK ? B : CHUNK, Bp = padded_tokens(Bc);
    w.pairs = 0;
    w.off8 = w.pairs + T * pair_stride(Bc, S) * 8;
    w.code_t = w.off8 + round16(T * (S + 1) * 4);
    w.score_t = w.code_t + round16(T * Bp * 2);
    w.g_packed = w.score_t + round16(T * Bp * 4);
    w.total = w.g_packed + round16(Bc * Do * 4);
    return w;
}

}  // namespace

extern "C" int lffn_lookup_scatter_workspace_bytes(int64_t B, int64_t T, int64_t S, int64_t Do, int64_t *bytes) {
    LFFN_REQUIRE(bytes, LFFN_ERR_BAD_ARG);
    *bytes = sorted_supported(B, T, S, Do) ? workspace_layout(B, T, S, Do).total : 0;
    return LFFN_OK;
}

namespace {

// The sorted scatter over chunks of CHUNK tokens and, when grad_score is given, the score gradient of each
// chunk from the same slice-major copy of g the scatter reads (lookup_prep_kernel writes it once per chunk).
// grad_tables may be null (score gradient only).
int sorted_backward(const int32_t *code, const float *score, const float *g, const float *tables, float *grad_score,
                    float *grad_tables, void *workspace, int64_t workspace_bytes, int64_t B, int64_t T, int64_t S,
                    int64_t Do, int32_t accumulate, void *stream) {
    const Workspace w = workspace_layout(B, T, S, Do);
    LFFN_REQUIRE(workspace_bytes >= w.total, LFFN_ERR_BAD_ARG);
    hipStream_t st = static_cast<hipStream_t>(stream);
    char *base = static_cast<char *>(workspace);
    uint2 *pairs = reinterpret_cast<uint2 *>(base + w.pairs);
    int32_t *off8 = reinterpret_cast<int32_t *>(base + w.off8);

    for (int64_t c0 = 0; c0 < B; c0 += CHUNK) {
        const int64_t Bc = B - c0 < CHUNK ? B - c0 : CHUNK;
        const int64_t stride = pair_stride(Bc, S), Bp = padded_tokens(Bc);

        PrepArgs pa{};
        pa.code = code + c0 * T; pa.score = score + c0 * T; pa.g = g + c0 * Do;
        pa.code_t = reinterpret_cast<uint16_t *>(base + w.code_t);
        pa.score_t = reinterpret_cast<float *>(base + w.score_t);
        pa.g_packed = reinterpret_cast<float *>(base + w.g_packed);
        pa.B = Bc; pa.Bp = Bp; pa.T = (int)T; pa.S = (int)S; pa.Do = (int)Do;
        pa.tiles_t = (int)((T + 63) / 64);
        // (score gradient only: the codes and scores need no transposing or sorting, only g its slice-major copy)
        const int64_t transpose_blocks = grad_tables ? (Bp / 64) * pa.tiles_t : 0;
        const int64_t pack_blocks = (Bc + PACK_TOKENS - 1) / PACK_TOKENS;
        const int64_t nsort = grad_tables ? T : 0;
        LFFN_REQUIRE(transpose_blocks <= 0x7fffffff && nsort + pack_blocks <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
        int rc = LFFN_OK;
        if (transpose_blocks > 0) {
            hipLaunchKernelGGL(lookup_prep_kernel, dim3((unsigned)transpose_blocks), dim3(256), 0, st, pa);
            rc = lffn_launch_status();
            if (rc != LFFN_OK) return rc;
        }
        SortArgs sa{};
        sa.code = pa.code_t; sa.score = pa.score_t; sa.pairs = pairs; sa.off8 = off8;
        sa.B = Bc; sa.Bp = Bp; sa.stride = stride; sa.T = (int)T; sa.S = (int)S; sa.nbits = lffn_log2(S);
        // histograms and bucket tables, then the sorted list itself (4 + 2 bytes per entry; tokens of a chunk fit 16 bits)
        static_assert(CHUNK <= 65536, "tokens of a chunk are staged as 16-bit values");
        static_assert(CHUNK <= int64_t(SORT_WG) * SORT_DEPTH, "a wavefront of the sort holds its tokens in registers");
        const size_t tables_lds = (size_t(SORT_WAVES) * S + 3 * S + 4 + 4) * sizeof(int);
        const size_t staged_lds = tables_lds + size_t(stride) * 6 + 16;
        sa.stage = staged_lds <= 160 * 1024 ? 1 : 0;            // 512-row tables: the list goes straight to memory
        const size_t sort_lds = nsort ? (sa.stage ? staged_lds : tables_lds) : 0;
        static LdsGrant granted;
        if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(lookup_sort_pack_kernel), sort_lds, granted))
            return LFFN_ERR_LAUNCH;
        hipLaunchKernelGGL(lookup_sort_pack_kernel, dim3((unsigned)(nsort + pack_blocks)), dim3(SORT_WG), sort_lds, st, sa, pa,
                           (int)nsort);
        rc = lffn_launch_status();
        if (rc != LFFN_OK) return rc;

        if (grad_score) {
            // token b's 32 columns of slice s sit at g_packed + (s * Bc + b) * 32
            if (!lffn_internal_lookup_inner_quad_try(pa.code, pa.g_packed, SC, Bc * SC, tables, grad_score + c0 * T, Bc, T, S,
                                                     Do, stream, &rc))
                rc = lffn_lookup_inner_f32(pa.code, pa.g, tables, grad_score + c0 * T, Bc, T, S, Do, stream);
            if (rc != LFFN_OK) return rc;
        }
        if (!grad_tables) continue;

        SortedArgs ma{};
        ma.pairs = pairs; ma.off8 = off8; ma.g = pa.g_packed; ma.out = grad_tables; ma.stride = stride;
        ma.last_token = (unsigned)(Bc - 1);
        ma.T = (int)T; ma.S = (int)S; ma.Do = (int)Do; ma.nslices = (int)(Do / SC);
        ma.accumulate = (accumulate || c0 > 0) ? 1 : 0;
        const int64_t per_xcd = (ma.nslices + XCDS - 1) / XCDS * T;
        const size_t main_lds = (((S + 1 + 3) & ~int64_t(3)) + MWAVES * 4) * sizeof(int) + size_t(MWAVES) * 2 * SC * sizeof(float);
        hipLaunchKernelGGL(lookup_scatter_sorted_kernel, dim3((unsigned)(per_xcd * XCDS)), dim3(MWG), main_lds, st, ma);
        rc = lffn_launch_status();
        if (rc != LFFN_OK) return rc;
    }
    return LFFN_OK;
}

}  // namespace

extern "C" int lffn_lookup_scatter_sorted_f32(const int32_t *code, const float *score, const float *g,
                                              float *grad_tables, void *workspace, int64_t workspace_bytes,
                                              int64_t B, int64_t T, int64_t S, int64_t Do, int32_t accumulate,
                                              void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && S >= 1 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(sorted_supported(B, T, S, Do), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(code && score && g && grad_tables && workspace, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(grad_tables) && lffn_aligned16(g) && lffn_aligned16(workspace), LFFN_ERR_BAD_ARG);
    return sorted_backward(code, score, g, nullptr, nullptr, grad_tables, workspace, workspace_bytes, B, T, S, Do, accumulate,
                           stream);
}

// Both gradients of the layer's gather in one call with one workspace (lffn_lookup_scatter_workspace_bytes):
//   grad_score[b,t]  = < g[b,:], tables[t, code[b,t], :] >           (overwritten)
//   grad_tables[t,s] = sum over b with code[b,t] = s of score[b,t] * g[b,:]   (overwritten, or added to)
// Per chunk of 16384 tokens: one kernel transposes code and score and copies g slice-major, the score-gradient
// kernel and the sorted scatter both read that copy.
extern "C" int lffn_lookup_backward_f32(const int32_t *code, const float *score, const float *g, const float *tables,
                                        float *grad_score, float *grad_tables, void *workspace,
                                        int64_t workspace_bytes, int64_t B, int64_t T, int64_t S, int64_t Do,
                                        int32_t accumulate, void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && S >= 1 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(sorted_supported(B, T, S, Do) && Do % 64 == 0, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(code && g && workspace && (grad_score || grad_tables), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE((!grad_score || tables) && (!grad_tables || score), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(g) && lffn_aligned16(workspace) && (!grad_tables || lffn_aligned16(grad_tables)) &&
                     (!tables || lffn_aligned16(tables)), LFFN_ERR_BAD_ARG);
    return sorted_backward(code, score, g, tables, grad_score, grad_tables, workspace, workspace_bytes, B, T, S, Do,
                           accumulate, stream);
}
