// BH4 with 64x64 blocks (PL/bh4/kernel.py:23-36), all stages of a repeat in one kernel:
//
//   y <- pad(x);  for s < J:  y <- FHT_D( blockdiag(W[r,s]) y );   out[:, r*D:(r+1)*D] = y
//
// D = 64*NB.  In natural (Sylvester) order H_D = H_NB (x) H_64 with the block number
// as the high index bits, so a stage is  (H_NB (x) I_64) * blockdiag(H_64 W[r,s,n]):
// the 64-point part of the transform is folded into the weights once per call
// (lffn_bh4_fold_f32, a 64-point transform down the output index of every 64x64
// block), and the part across blocks is NB-point butterflies between accumulators.
//
// One workgroup = 4 wavefronts = 32 tokens, whose rows stay in LDS between the
// stages ((D+4)-float rows: conflict-free 16-byte accesses down a column of
// tokens).  Wavefront w owns output columns [16w, 16w+16) of every block for both
// 16-token halves, so a weight fragment fetched from L2 is used for 32 tokens.  The
// products run on v_mfma_f32_16x16x4_f32 with the weights as the A operand
// (rows = output columns) and the tokens as the B operand, which leaves each lane
// with four consecutive output columns of one token: one 16-byte LDS store per
// (block, half).  2*NB accumulator tiles per wavefront; the butterflies across
// blocks are register adds.
//
// Rounding differs from doing the product first and the full transform after it
// (the reference's order): the 64-point part is applied to the weights, in fp32,
// before the product.  Results agree to fp32 rounding (1e-5 of the row's largest
// magnitude), not bit for bit.
//
// The same kernel also runs the layer's whole hashing front end for 8-bit codes
// (lffn_ln_bh4_block_hash_f32): LayerNorm while the token tile is loaded (a wavefront
// owns 8 rows, a row is spread over its 64 lanes; mean and 1/sigma are kept in LDS),
// and after the last stage, instead of storing y, z = decay*y + residual*LN(x) + bias
// on the accumulators (x is read again and normalised with the kept statistics) and
// the code and score of every 8 columns: a group is split over the lane pair
// (l, l+16), whose second lane continues the first lane's running sum and product so
// that the operations run in column order.
#include "lffn_common.h"

// the mix and the score keep the reference's operation order: no fused multiply-add
#pragma clang fp contract(off)

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BS = 64;          // block size this file is built for
constexpr int PAD = 4;          // floats of padding per LDS row

// 64-point unnormalised Hadamard transform down the output index o of every block:
// wf[blk]{o', i} = sum_o H64[o'][o] * w[blk][o][i], stored in the order the product kernel's
// lanes fetch it.  One lane per (blk, i).
// MODE 0: the order the forward product fetches (below).  MODE 1: the order the backward
// product fetches, whose A operand is the transposed block: rows = input index i, k = output
// index o'.  MODE 2: natural [o'][i] order (turns a gradient w.r.t. the folded weights into the
// gradient w.r.t. the weights: H64 is symmetric).
template <int MODE>
__global__ __launch_bounds__(256) void bh4_fold_kernel(const float *w, float *wf, int64_t nblk) {
    const int64_t gid = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (gid >= nblk * BS) return;
    const int64_t blk = gid / BS;
    const int i = (int)(gid % BS);
    const float *src = w + blk * (BS * BS) + i;
    float v[BS];
#pragma unroll
    for (int o = 0; o < BS; ++o) v[o] = src[o * BS];
#pragma unroll
    for (int h = BS / 2; h >= 1; h >>= 1) {
#pragma unroll
        for (int o = 0; o < BS; ++o) {
            if ((o & h) == 0) {
                const float lo = v[o], hi = v[o + h];
                v[o] = lo + hi;
                v[o + h] = lo - hi;
            }
        }
    }
    if constexpr (MODE == 0) {
        // fragment order: [wavefront = o/16][q = (i%16)/4][lane = 16*(i/16) + o%16][i%4], so that a
        // wavefront's load of (block, q) is 1 KB of contiguous memory, 16 bytes per lane
        float *dst = wf + blk * (BS * BS) + ((i % 16) / 4) * 256 + (i / 16) * 64 + (i % 4);
#pragma unroll
        for (int o = 0; o < BS; ++o) dst[(o / 16) * 1024 + (o % 16) * 4] = v[o];
    } else if constexpr (MODE == 1) {
        // the same with the roles of o and i exchanged: [i/16][(o%16)/4][16*(o/16) + i%16][o%4]
        float *dst = wf + blk * (BS * BS) + (i / 16) * 1024 + (i % 16) * 4;
#pragma unroll
        for (int o = 0; o < BS; ++o) dst[((o % 16) / 4) * 256 + (o / 16) * 64 + (o % 4)] = v[o];
    } else {
        float *dst = wf + blk * (BS * BS) + i;
#pragma unroll
        for (int o = 0; o < BS; ++o) dst[o * BS] = v[o];
    }
}

#define LFFN_MFMA(acc, a, b) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0)

struct BlockArgs {
    const float *x;        // [B, H]
    const float *ln_w;     // [H] LayerNorm weight, or null: no LayerNorm
    const float *ln_b;     // [H]
    float ln_eps;
    const float *wf;       // folded weights
    float *out;            // [B, R*D]            (plain form)
    const float *pbias;    // [T*8] or null       (hash form)
    int32_t *codes;        // [B, T]              (hash form)
    float *scores;         // [B, T]              (hash form)
    uint32_t *records;     // hash form, instead of codes and scores: the record stream of the
    int64_t rec_stride;    // four-lanes-per-token gather, [T/2][rec_stride][3] (lffn_quad_record_slot)
    int rec_tile;          // tokens per workgroup of the gather the records are written for
    float *z_out;          // [B, T*8] or null    (hash form: z kept for the backward)
    float *row_stats;      // [B, 2] or null: LayerNorm's mean and 1/sigma of every row, kept for the backward
    float *stage_save;     // forward: [R, J-1, B, D] inputs of stages 1..J-1, or null;
                           // backward: [R, J, B, D] gradient before the product of each stage
    const float *gz;       // [B, T*8]            (backward form: gradient of z)
    int64_t B;
    int H, R, J, T;
    float decay, residual;
};

// NH = token halves per wavefront.  NH == 2: 4 wavefronts, each both 16-token halves (a weight
// fragment is fetched once per workgroup).  NH == 1: 8 wavefronts, wavefront w and w+4 own the
// same output columns for one half each (the fragment is fetched twice, the second time mostly
// from the L1), two wavefronts per SIMD: the phases that are not products (tile load and
// LayerNorm, butterflies, stage hand-over, hash) run on twice the wavefronts.
//
// BWD: the backward through the stages with the same machinery.  With G_{s+1} the gradient of a
// stage's output, the gradient of its input is  W'_s^T (H_NB (x) I_64) G_{s+1}  (H_64 is
// symmetric and already inside W' = H_64 W): the butterflies across blocks run BEFORE the
// product, as a pass over the LDS tile, the product takes the folded weights in transposed
// fragment order (bh4_fold_kernel<1>), and nothing follows it.  The butterflied gradient
// P_s = (H_NB (x) I) G_{s+1} is also written to memory: the gradient w.r.t. the folded
// weights is the per-block product P_s^T U_s over all tokens (U_s = the stage's input, which
// the forward saved), formed by the caller.  Tile load: decay * grad z; result: grad x of
// this repeat = G_0[:, :H] + residual * grad z[:, :H].
// Lanes 16-31 and 48-63 get the value of the lane 16 below; the other lanes keep their own.
__device__ __forceinline__ float from_row_below(float v) {
    const unsigned u = __float_as_uint(v);
    return __uint_as_float(__builtin_amdgcn_permlane16_swap(u, u, false, false)[0]);
}

// HV = 16-token halves per workgroup: 2 (32 tokens, one workgroup per CU at D = 1024) or 1 (16
// tokens, half the LDS, so that two workgroups share a CU and the load, hand-over and hash phases
// of one run under the products of the other).
template <int NB, bool HASH, int NH, bool BWD = false, int HV = 2>
__global__ __launch_bounds__(256 * HV / NH, HV == 1 ? 2 : 1) void bh4_block_kernel(BlockArgs a) {
    static_assert(!(HASH && BWD), "one form at a time");
    static_assert(NH <= HV, "a wavefront cannot hold more halves than the tile has");
    constexpr int TOK = 16 * HV;                  // tokens per workgroup
    constexpr int NWAVE = 4 * (HV / NH);
    const float *__restrict__ x = a.x;
    const float *__restrict__ wf = a.wf;
    const int64_t B = a.B;
    const int H = a.H, R = a.R, J = a.J;
    constexpr int D = BS * NB;
    constexpr int LDR = D + PAD;
    constexpr int G = NB >= 2 ? 2 : 1;            // blocks worked on together
    constexpr int NS = 2 * G;                     // register slots: block n sits in slot n % NS
    constexpr bool AHEAD = NB >= NS;              // first blocks of a stage fetched during the previous one
    extern __shared__ __attribute__((aligned(16))) float xs[];   // TOK rows of LDR floats, then the row statistics
    float *stats = xs + TOK * LDR;                // [TOK][2]: mean and 1/sigma of LayerNorm
    float *lnw_s = stats + 2 * TOK;               // [D] LayerNorm weight and bias (hash form, for the epilogue)
    float *lnb_s = lnw_s + D;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ow = wave & 3;                      // output columns [16*ow, 16*ow + 16) of each block
    const int hg = wave >> 2;                     // NH == 1: the token half of this wavefront
    const int c = lane & 15;                      // A operand: output column; B operand and result: token
    const int kq = lane >> 4;                     // k index inside an MFMA; result: output columns 4*kq .. 4*kq+3
    const int64_t tok_base = int64_t(blockIdx.x) * TOK;
    if (HASH && a.ln_w) {
        for (int e = tid * 4; e < D; e += 256 * NWAVE) {
            const bool in = e < H;
            *reinterpret_cast<float4 *>(lnw_s + e) = in ? *reinterpret_cast<const float4 *>(a.ln_w + e)
                                                        : make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4 *>(lnb_s + e) = in ? *reinterpret_cast<const float4 *>(a.ln_b + e)
                                                        : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }

    // this lane's weight fragment of block n, quarter q (input columns 16*kq + 4*q .. +3 of output
    // column 16*wave + c): wf[..][n][wave][q][lane][0..3]
    const int w_lane_off = ow * 1024 + lane * 4;
    // this lane's token values of block n, half h: xs[(16*h + c) * LDR + 64*n + 16*kq ..]
    const int x_lane_off = c * LDR + 16 * kq;
    // where this lane's results of block n, half h go: xs[(16*h + c) * LDR + 64*n + 16*wave + 4*kq ..]
    const int y_lane_off = c * LDR + 16 * ow + 4 * kq;

    auto load_w = [&](const float *wst, int n, int q) {
        return *reinterpret_cast<const float4 *>(wst + n * (BS * BS) + q * 256);
    };
    auto read_x = [&](int h, int n, int q) {
        return *reinterpret_cast<const float4 *>(xs + h * 16 * LDR + x_lane_off + n * BS + q * 4);
    };

    for (int r = 0; r < R; ++r) {
        __syncthreads();                          // the previous repeat's last stage has been read
        {
            // A wavefront loads TOK/NWAVE rows, 16 bytes per lane and 1 KB of a row per instruction, all
            // loads in flight before the first use (one at a time, each would pay the full
            // memory latency).  Columns at or beyond H are zero.
            constexpr int RPW = TOK / NWAVE;
            constexpr int NQ = D >= 256 ? D / 256 : 1;
            float4 v[RPW][NQ];
#pragma unroll
            for (int i = 0; i < RPW; ++i) {
                const int64_t tok = tok_base + wave * RPW + i;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const int col = (q * 64 + lane) * 4;
                    if constexpr (BWD) {
                        const int gcol = r * D + col;
                        float4 g4 = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (tok < B && col < D && gcol < a.T * 8)
                            g4 = *reinterpret_cast<const float4 *>(a.gz + tok * (a.T * 8) + gcol);
                        v[i][q] = make_float4(a.decay * g4.x, a.decay * g4.y, a.decay * g4.z, a.decay * g4.w);
                    } else {
                        v[i][q] = (tok < B && col < H) ? *reinterpret_cast<const float4 *>(x + tok * H + col)
                                                       : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                }
            }
            if (!BWD && a.ln_w) {
                // LayerNorm over the H valid columns (biased variance, two passes, eps inside the
                // square root: torch.nn.LayerNorm, PL/lookup.py:84,99)
                float4 lw[NQ], lb[NQ];
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const int col = (q * 64 + lane) * 4;
                    lw[q] = col < H ? *reinterpret_cast<const float4 *>(a.ln_w + col) : make_float4(0.f, 0.f, 0.f, 0.f);
                    lb[q] = col < H ? *reinterpret_cast<const float4 *>(a.ln_b + col) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int i = 0; i < RPW; ++i) {
                    float s1 = 0.f;
#pragma unroll
                    for (int q = 0; q < NQ; ++q) s1 += (v[i][q].x + v[i][q].y) + (v[i][q].z + v[i][q].w);
                    const float mean = wave_sum(s1) / float(H);
                    float s2 = 0.f;
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        if ((q * 64 + lane) * 4 < H) {
                            const float d0 = v[i][q].x - mean, d1 = v[i][q].y - mean;
                            const float d2 = v[i][q].z - mean, d3 = v[i][q].w - mean;
                            s2 += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
                        }
                    }
                    const float rstd = 1.0f / sqrtf(wave_sum(s2) / float(H) + a.ln_eps);
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        if ((q * 64 + lane) * 4 < H) {
                            v[i][q].x = (v[i][q].x - mean) * rstd * lw[q].x + lb[q].x;
                            v[i][q].y = (v[i][q].y - mean) * rstd * lw[q].y + lb[q].y;
                            v[i][q].z = (v[i][q].z - mean) * rstd * lw[q].z + lb[q].z;
                            v[i][q].w = (v[i][q].w - mean) * rstd * lw[q].w + lb[q].w;
                        }
                    }
                    if (lane == 0) {
                        stats[2 * (wave * RPW + i)] = mean;
                        stats[2 * (wave * RPW + i) + 1] = rstd;
                        const int64_t tok = tok_base + wave * RPW + i;
                        if (a.row_stats && r == 0 && tok < B) *reinterpret_cast<float2 *>(a.row_stats + 2 * tok) = make_float2(mean, rstd);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < RPW; ++i)
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const int col = (q * 64 + lane) * 4;
                    if (col < D) *reinterpret_cast<float4 *>(xs + (wave * RPW + i) * LDR + col) = v[i][q];
                }
        }
        __syncthreads();

        float4 wq[NS][4];                         // weight fragments
        if constexpr (AHEAD) {
            const float *w0 = wf + (size_t)((r * J + (BWD ? J - 1 : 0)) * NB) * (BS * BS) + w_lane_off;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int g = 0; g < G; ++g) wq[g][q] = load_w(w0, g, q);
        }
#pragma unroll 1
        for (int si = 0; si < J; ++si) {
            const int s = BWD ? J - 1 - si : si;                  // the backward walks the stages down
            const float *wst = wf + (size_t)((r * J + s) * NB) * (BS * BS) + w_lane_off;
            if constexpr (BWD) {
                // butterflies across the blocks on the LDS tile, 16 bytes of every block per thread;
                // the result is this stage's P, kept for the weight gradient
                for (int e = tid; e < TOK * 16; e += 64 * NWAVE) {
                    const int row = e / 16, c4 = (e % 16) * 4;
                    f32x4 pv[NB];
#pragma unroll
                    for (int n = 0; n < NB; ++n) pv[n] = *reinterpret_cast<const f32x4 *>(xs + row * LDR + n * BS + c4);
#pragma unroll
                    for (int h = NB / 2; h >= 1; h >>= 1) {
#pragma unroll
                        for (int n = 0; n < NB; ++n) {
                            if ((n & h) == 0) {
                                const f32x4 lo = pv[n], hi = pv[n + h];
                                pv[n] = lo + hi;
                                pv[n + h] = lo - hi;
                            }
                        }
                    }
                    const int64_t tok = tok_base + row;
                    float *ps = a.stage_save + ((size_t(r) * J + s) * B + tok) * D + c4;
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        *reinterpret_cast<f32x4 *>(xs + row * LDR + n * BS + c4) = pv[n];
                        if (tok < B) *reinterpret_cast<f32x4 *>(ps + n * BS) = pv[n];
                    }
                }
                __syncthreads();
            }
            f32x4 acc[NH][NB];
#pragma unroll
            for (int n = 0; n < NB; ++n)
#pragma unroll
                for (int t = 0; t < NH; ++t) acc[t][n] = (f32x4){0.f, 0.f, 0.f, 0.f};
            if constexpr (!AHEAD) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int g = 0; g < G; ++g) wq[g][q] = load_w(wst, g, q);
            }
            float4 xv[NH][NS][4];                 // token values of this wavefront's halves
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int g = 0; g < G; ++g)
#pragma unroll
                    for (int t = 0; t < NH; ++t) xv[t][g][q] = read_x(hg * NH + t, g, q);

            // Wavefronts issue in order and there are one or two per SIMD: the loads for the next
            // pair of blocks are spread between the products instead of queueing in a burst at the
            // LDS and the texture unit, and two blocks are worked on together (2*NH independent
            // accumulation chains).
            static_for<NB / G>([&](auto p_c) {
                constexpr int n0 = decltype(p_c)::value * G;
                constexpr int n1 = n0 + G - 1;                  // == n0 when G == 1
                constexpr bool more = n0 + G < NB;              // another pair follows in this stage
                constexpr int m0 = (n0 + G) % NS, m1 = (n1 + G) % NS;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 w0v = wq[n0 % NS][q], w1v = wq[n1 % NS][q];
                    if constexpr (more) wq[m0][q] = load_w(wst, n0 + G, q);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n0], w0v.x, xv[t][n0 % NS][q].x);
                    if constexpr (G == 2) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n1], w1v.x, xv[t][n1 % NS][q].x);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (more) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) xv[t][m0][q] = read_x(hg * NH + t, n0 + G, q);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n0], w0v.y, xv[t][n0 % NS][q].y);
                    if constexpr (G == 2) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n1], w1v.y, xv[t][n1 % NS][q].y);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (more && G == 2) wq[m1][q] = load_w(wst, n1 + G, q);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n0], w0v.z, xv[t][n0 % NS][q].z);
                    if constexpr (G == 2) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n1], w1v.z, xv[t][n1 % NS][q].z);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (more && G == 2) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) xv[t][m1][q] = read_x(hg * NH + t, n1 + G, q);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n0], w0v.w, xv[t][n0 % NS][q].w);
                    if constexpr (G == 2) {
#pragma unroll
                        for (int t = 0; t < NH; ++t) LFFN_MFMA(acc[t][n1], w1v.w, xv[t][n1 % NS][q].w);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            // the next stage's first blocks (a harmless re-read after the last stage): every product
            // that read slots 0 .. G-1 was issued at least one pair ago
            if constexpr (AHEAD) {
                const int sn = BWD ? max(s - 1, 0) : min(s + 1, J - 1);
                const float *wnx = wf + (size_t)((r * J + sn) * NB) * (BS * BS) + w_lane_off;
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int g = 0; g < G; ++g) wq[g][q] = load_w(wnx, g, q);
                __builtin_amdgcn_sched_barrier(0);
            }

            // H_NB across the blocks (the backward did it before the product)
            if constexpr (!BWD) {
#pragma unroll
                for (int h = NB / 2; h >= 1; h >>= 1) {
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        if ((n & h) == 0) {
#pragma unroll
                            for (int t = 0; t < NH; ++t) {
                                const f32x4 lo = acc[t][n], hi = acc[t][n + h];
                                acc[t][n] = lo + hi;
                                acc[t][n + h] = lo - hi;
                            }
                        }
                    }
                }
            }

            __syncthreads();                      // every wavefront has read this stage's input
            if (si + 1 < J) {
#pragma unroll
                for (int n = 0; n < NB; ++n)
#pragma unroll
                    for (int t = 0; t < NH; ++t)
                        *reinterpret_cast<f32x4 *>(xs + (hg * NH + t) * 16 * LDR + y_lane_off + n * BS) = acc[t][n];
                if (!BWD && a.stage_save) {
                    // the input of stage s+1, kept for the weight gradient of the backward
#pragma unroll
                    for (int t = 0; t < NH; ++t) {
                        const int64_t tok = tok_base + 16 * (hg * NH + t) + c;
                        if (tok < B) {
                            float *o = a.stage_save + ((size_t(r) * (J - 1) + s) * B + tok) * D + 16 * ow + 4 * kq;
#pragma unroll
                            for (int n = 0; n < NB; ++n) *reinterpret_cast<f32x4 *>(o + n * BS) = acc[t][n];
                        }
                    }
                }
                __syncthreads();
            } else if constexpr (BWD) {
                // grad x of this repeat: the first H columns, plus the residual path of the mix
                const int ncols = a.T * 8;
#pragma unroll
                for (int t = 0; t < NH; ++t) {
                    const int64_t tok = tok_base + 16 * (hg * NH + t) + c;
                    if (tok < B) {
#pragma unroll
                        for (int n = 0; n < NB; ++n) {
                            const int xc = n * BS + 16 * ow + 4 * kq;
                            if (xc < H) {
                                f32x4 o = acc[t][n];
                                if (r * D + xc < ncols) {
                                    const f32x4 g4 = *reinterpret_cast<const f32x4 *>(a.gz + tok * ncols + r * D + xc);
                                    o.x = o.x + a.residual * g4.x; o.y = o.y + a.residual * g4.y;
                                    o.z = o.z + a.residual * g4.z; o.w = o.w + a.residual * g4.w;
                                }
                                *reinterpret_cast<f32x4 *>(a.out + (size_t(r) * B + tok) * H + xc) = o;
                            }
                        }
                    }
                }
            } else if constexpr (!HASH) {
                const int64_t ld_out = int64_t(R) * D;
#pragma unroll
                for (int t = 0; t < NH; ++t) {
                    const int64_t tok = tok_base + 16 * (hg * NH + t) + c;
                    if (tok < B) {
                        float *o = a.out + tok * ld_out + (size_t)r * D + 16 * ow + 4 * kq;
#pragma unroll
                        for (int n = 0; n < NB; ++n) *reinterpret_cast<f32x4 *>(o + n * BS) = acc[t][n];
                    }
                }
            } else {
                const int ncols = a.T * 8;
                constexpr int CROW = D / 8 + 1;                // padded: tokens down a column hit different banks
                int *cs = reinterpret_cast<int *>(xs);         // [TOK][CROW] codes of this repeat
                float *ss = xs + TOK * CROW;                   // [TOK][CROW] scores
                // the addresses below do not change from stage to stage; computed from an opaque
                // zero they are formed here instead of being kept in registers through the stages
                int opq = 0;
                asm volatile("" : "+v"(opq));
                int64_t tokv[NH];
                bool livev[NH];
                float meanv[NH], rstdv[NH];
                // the tokens' input values for every block, all requested before the first use
                float4 xin[NH][NB];
#pragma unroll
                for (int t = 0; t < NH; ++t) {
                    const int trow = 16 * (hg * NH + t) + c + opq;     // token within the tile
                    tokv[t] = tok_base + trow;
                    livev[t] = tokv[t] < B;
                    meanv[t] = a.ln_w ? stats[2 * trow] : 0.f;
                    rstdv[t] = a.ln_w ? stats[2 * trow + 1] : 1.f;
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        const int xc = n * BS + 16 * ow + 4 * kq + opq;
                        xin[t][n] = (livev[t] && xc < H) ? *reinterpret_cast<const float4 *>(x + tokv[t] * H + xc)
                                                         : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int n = 0; n < NB; ++n) {
                    const int xc = n * BS + 16 * ow + 4 * kq + opq;        // column of the padded input
                    const int col = r * D + xc;                            // column of z
                    const bool in_cols = col < ncols;                      // whole groups of 8: all or nothing
                    float4 lw = make_float4(0.f, 0.f, 0.f, 0.f), lb = lw, bb = lw;
                    if (a.ln_w && xc < H) {
                        lw = *reinterpret_cast<const float4 *>(lnw_s + xc);
                        lb = *reinterpret_cast<const float4 *>(lnb_s + xc);
                    }
                    if (a.pbias && in_cols) bb = *reinterpret_cast<const float4 *>(a.pbias + col);
                    // the token halves of this wavefront side by side: independent work
#pragma unroll
                    for (int t = 0; t < NH; ++t) {
                        float4 xv = xin[t][n];
                        if (a.ln_w && xc < H) {
                            xv.x = (xv.x - meanv[t]) * rstdv[t] * lw.x + lb.x;
                            xv.y = (xv.y - meanv[t]) * rstdv[t] * lw.y + lb.y;
                            xv.z = (xv.z - meanv[t]) * rstdv[t] * lw.z + lb.z;
                            xv.w = (xv.w - meanv[t]) * rstdv[t] * lw.w + lb.w;
                        }
                        float z[4];
                        z[0] = a.decay * acc[t][n].x + a.residual * xv.x;
                        z[1] = a.decay * acc[t][n].y + a.residual * xv.y;
                        z[2] = a.decay * acc[t][n].z + a.residual * xv.z;
                        z[3] = a.decay * acc[t][n].w + a.residual * xv.w;
                        if (a.pbias && in_cols) {
                            z[0] = z[0] + bb.x; z[1] = z[1] + bb.y; z[2] = z[2] + bb.z; z[3] = z[3] + bb.w;
                        }
                        if (a.z_out && in_cols && livev[t])
                            *reinterpret_cast<float4 *>(a.z_out + tokv[t] * ncols + col) = make_float4(z[0], z[1], z[2], z[3]);
                        // columns 8g .. 8g+3 sit in the lane with even kq (the high nibble),
                        // 8g+4 .. 8g+7 in lane + 16, which continues the sum and the product
                        // (d = 0..7 in order, compute_code_score/torch_extension.cc:31-37)
                        const int nib = (z[0] > 0.f ? 8 : 0) | (z[1] > 0.f ? 4 : 0) | (z[2] > 0.f ? 2 : 0) |
                                        (z[3] > 0.f ? 1 : 0);
                        float az[4], fz[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            az[i] = fabsf(z[i]);
                            fz[i] = 1.0f + exp_minus_2a(az[i]);
                        }
                        float s_loc = 0.f, p_loc = 1.f;
#pragma unroll
                        for (int i = 0; i < 4; ++i) { s_loc = s_loc + az[i]; p_loc = p_loc * fz[i]; }
                        // odd rows of 16 lanes take over from the lane 16 below (a row swap on the vector
                        // ALU: with two wavefronts per SIMD an LDS permute here is waited for every time)
                        float s_run = from_row_below(s_loc);
                        float p_run = from_row_below(p_loc);
                        const int nib_hi = __float_as_int(from_row_below(__int_as_float(nib)));
#pragma unroll
                        for (int i = 0; i < 4; ++i) { s_run = s_run + az[i]; p_run = p_run * fz[i]; }
                        // staged in LDS (the stage buffer is free now), written out row by row below:
                        // straight from here a store would scatter 4-byte pieces over 32 rows
                        if (kq & 1) {
                            cs[(16 * (hg * NH + t) + c) * CROW + (xc >> 3)] = (nib_hi << 4) | nib;
                            ss[(16 * (hg * NH + t) + c) * CROW + (xc >> 3)] = s_run / p_run;
                        }
                    }
                }
                __syncthreads();
                if (a.records) {
                    // records: per table pair three words per token, the workgroup's TOK tokens (whole
                    // groups of 16: 192 contiguous bytes each) side by side; a token whose index has bit 1
                    // set takes the pair's tables in the order (2k+1, 2k)
                    static_assert((64 * NWAVE) % TOK == 0, "a thread stays on one token");
                    const int row = tid % TOK;
                    const int64_t tok = tok_base + row;
                    const int64_t slot = tok < B ? lffn_quad_record_slot(tok, a.rec_tile) : 0;
                    for (int kk = tid / TOK; kk < D / 16; kk += 64 * NWAVE / TOK) {
                        const int pair = r * (D / 16) + kk;
                        if (tok < B && 2 * pair + 1 < a.T) {
                            const int ca = cs[row * CROW + 2 * kk], cb = cs[row * CROW + 2 * kk + 1];
                            const float sa = ss[row * CROW + 2 * kk], sb = ss[row * CROW + 2 * kk + 1];
                            const bool second_first = (tok & 2) != 0;
                            uint32_t *dst = a.records + ((size_t)pair * a.rec_stride + slot) * LFFN_RECORD_WORDS;
                            dst[0] = __float_as_uint(second_first ? sb : sa);
                            dst[1] = __float_as_uint(second_first ? sa : sb);
                            dst[2] = second_first ? (unsigned)(cb | (ca << 8)) : (unsigned)(ca | (cb << 8));
                        }
                    }
                } else {
                    // every wavefront writes the D/8 codes and scores of TOK/NWAVE tokens
#pragma unroll 1
                    for (int i = 0; i < TOK / NWAVE; ++i) {
                        const int row = wave * (TOK / NWAVE) + i;
                        const int64_t tok = tok_base + row;
                        if (tok >= B) break;
#pragma unroll
                        for (int e0 = 0; e0 < D / 8; e0 += 64) {
                            const int e = e0 + lane;
                            const int tt = r * (D / 8) + e;
                            if (e < D / 8 && tt < a.T) {
                                a.codes[tok * a.T + tt] = cs[row * CROW + e];
                                a.scores[tok * a.T + tt] = ss[row * CROW + e];
                            }
                        }
                    }
                }
            }
        }
    }
}

template <int NB, bool HASH, int NH, bool BWD = false, int HV = 2>
int launch_block(const BlockArgs &a, hipStream_t st) {
    constexpr int TOK = 16 * HV;
    const size_t lds_bytes = (size_t(TOK) * (BS * NB + PAD) + 2 * TOK + (HASH ? 2 * BS * NB : 0)) * sizeof(float);
    auto kern = bh4_block_kernel<NB, HASH, NH, BWD, HV>;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(kern), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.B + TOK - 1) / TOK)), dim3(256 * HV / NH), lds_bytes, st, a);
    return lffn_launch_status();
}

int dispatch_block_bwd(const BlockArgs &a, int64_t D, hipStream_t st) {
    switch (D / BS) {
        case 1: return launch_block<1, false, 2, true>(a, st);
        case 2: return launch_block<2, false, 2, true>(a, st);
        case 4: return launch_block<4, false, 2, true>(a, st);
        case 8: return launch_block<8, false, 2, true>(a, st);
        default: return launch_block<16, false, 1, true>(a, st);
    }
}

template <bool HASH>
int dispatch_block(const BlockArgs &a, int64_t D, hipStream_t st) {
    switch (D / BS) {
        // The hash form as 16-token workgroups of 4 wavefronts where that measured faster (more workgroups
        // per compute unit: the vector work of one hides behind the products of the others): 32768 tokens,
        // D = 512, two repeats 268 -> 212 us; D = 128 74 -> 70 us; D = 64 44 -> 41 us; D = 256 65 -> 69 us
        // (kept on 32 tokens); the plain form is as fast or faster with 32 tokens everywhere.
        case 1: return HASH ? launch_block<1, HASH, 1, false, 1>(a, st) : launch_block<1, HASH, 2>(a, st);
        case 2: return HASH ? launch_block<2, HASH, 1, false, 1>(a, st) : launch_block<2, HASH, 2>(a, st);
        case 4: return launch_block<4, HASH, 2>(a, st);
        case 8: return HASH ? launch_block<8, HASH, 1, false, 1>(a, st) : launch_block<8, HASH, 2>(a, st);
        // measured at 16384 x 1024: the plain form 110 us with 4 wavefronts, 118 us with 8 (the
        // second fetch of the weight fragments costs more than the other phases gain); the hash
        // form 141 us with 4, 133 us with 8 (LayerNorm and the hash are vector-ALU work), 118 us
        // (124 before: both with the later epilogue changes) as two 16-token workgroups per CU.
        // Eight wavefronts that hold one token half each fetch 4 KB of weight fragments per 16
        // products, 31 of the compute unit's 64 bytes per clock of memory pipeline; starting every
        // other workgroup late so that the two on a compute unit run out of phase gained nothing.
        default: return HASH ? launch_block<16, HASH, 1, false, 1>(a, st) : launch_block<16, HASH, 2>(a, st);
    }
}

}  // namespace

extern "C" int lffn_bh4_fold_f32(const float *w, float *w_folded, int64_t R, int64_t stages, int64_t num_block,
                                 int64_t block_size, void *stream) {
    LFFN_REQUIRE(R >= 1 && stages >= 1 && num_block >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(block_size == BS, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(w && w_folded && w != w_folded, LFFN_ERR_BAD_ARG);
    const int64_t nblk = R * stages * num_block;
    LFFN_REQUIRE(nblk <= (int64_t(1) << 24), LFFN_ERR_UNSUPPORTED);
    hipLaunchKernelGGL(bh4_fold_kernel<0>, dim3((unsigned)((nblk * BS + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), w, w_folded, nblk);
    return lffn_launch_status();
}

extern "C" int lffn_bh4_fold_mode_f32(const float *w, float *out, int64_t num_blocks, int64_t block_size,
                                      int32_t mode, void *stream) {
    LFFN_REQUIRE(num_blocks >= 0 && num_blocks <= (int64_t(1) << 24), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(block_size == BS && mode >= 0 && mode <= 2, LFFN_ERR_UNSUPPORTED);
    if (num_blocks == 0) return LFFN_OK;
    LFFN_REQUIRE(w && out && w != out, LFFN_ERR_BAD_ARG);
    const dim3 grid((unsigned)((num_blocks * BS + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == 0) hipLaunchKernelGGL(bh4_fold_kernel<0>, grid, dim3(256), 0, st, w, out, num_blocks);
    else if (mode == 1) hipLaunchKernelGGL(bh4_fold_kernel<1>, grid, dim3(256), 0, st, w, out, num_blocks);
    else hipLaunchKernelGGL(bh4_fold_kernel<2>, grid, dim3(256), 0, st, w, out, num_blocks);
    return lffn_launch_status();
}

extern "C" int lffn_bh4_block_f32(const float *x, const float *w_folded, float *out, int64_t B, int64_t H,
                                  int64_t D, int64_t R, int64_t J, int64_t block_size, void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    if (B == 0) return LFFN_OK;
    LFFN_REQUIRE(x && w_folded && out, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(w_folded) && lffn_aligned16(out), LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.x = x; a.wf = w_folded; a.out = out; a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J;
    return dispatch_block<false>(a, D, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_ln_bh4_block_hash_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                          const float *w_folded, const float *proj_bias, int32_t *codes,
                                          float *scores, int64_t B, int64_t H, int64_t D, int64_t R, int64_t J,
                                          int64_t T, int64_t block_size, float decay, float residual,
                                          void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D && T >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1 && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * 8 <= R * D, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(!ln_weight || (ln_bias && ln_eps >= 0.f), LFFN_ERR_BAD_ARG);
    if (B == 0 || T == 0) return LFFN_OK;
    LFFN_REQUIRE(x && w_folded && codes && scores, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(w_folded) && (!proj_bias || lffn_aligned16(proj_bias)) &&
                     (!ln_weight || (lffn_aligned16(ln_weight) && lffn_aligned16(ln_bias))),
                 LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = ln_eps; a.wf = w_folded; a.pbias = proj_bias;
    a.codes = codes; a.scores = scores; a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T;
    a.decay = decay; a.residual = residual;
    return dispatch_block<true>(a, D, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_ln_bh4_block_hash_records_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                                  const float *w_folded, const float *proj_bias, uint32_t *records,
                                                  int64_t record_stride, int32_t tokens_per_workgroup, int64_t B,
                                                  int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                                  int64_t block_size, float decay, float residual, void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D && T >= 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1 && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * 8 <= R * D && T % 2 == 0 && lffn_record_layout_ok(B, record_stride, tokens_per_workgroup),
                 LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(!ln_weight || (ln_bias && ln_eps >= 0.f), LFFN_ERR_BAD_ARG);
    if (B == 0 || T == 0) return LFFN_OK;
    LFFN_REQUIRE(x && w_folded && records, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(w_folded) && (!proj_bias || lffn_aligned16(proj_bias)) &&
                     (!ln_weight || (lffn_aligned16(ln_weight) && lffn_aligned16(ln_bias))) && (uintptr_t)records % 4 == 0,
                 LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = ln_eps; a.wf = w_folded; a.pbias = proj_bias;
    a.records = records; a.rec_stride = record_stride; a.rec_tile = tokens_per_workgroup; a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T;
    a.decay = decay; a.residual = residual;
    return dispatch_block<true>(a, D, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_bh4_block_hash_train_f32(const float *x, const float *w_folded, const float *proj_bias,
                                             int32_t *codes, float *scores, float *z, float *stage_inputs,
                                             int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                             int64_t block_size, float decay, float residual, void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D && T >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1 && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * 8 <= R * D, LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    LFFN_REQUIRE(x && w_folded && codes && scores && z && (stage_inputs || J == 1), LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(w_folded) && lffn_aligned16(z) &&
                     (!proj_bias || lffn_aligned16(proj_bias)) && (!stage_inputs || lffn_aligned16(stage_inputs)),
                 LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.x = x; a.wf = w_folded; a.pbias = proj_bias; a.codes = codes; a.scores = scores; a.z_out = z;
    a.stage_save = stage_inputs; a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T;
    a.decay = decay; a.residual = residual;
    return dispatch_block<true>(a, D, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_ln_bh4_block_hash_train_f32(const float *x, const float *ln_weight, const float *ln_bias, float ln_eps,
                                                const float *w_folded, const float *proj_bias, int32_t *codes,
                                                float *scores, float *z, float *stage_inputs, float *row_stats,
                                                int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                                int64_t block_size, float decay, float residual, void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D && T >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1 && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * 8 <= R * D && ln_eps >= 0.f, LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    LFFN_REQUIRE(x && ln_weight && ln_bias && w_folded && codes && scores && z && row_stats && (stage_inputs || J == 1),
                 LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(x) && lffn_aligned16(w_folded) && lffn_aligned16(z) && lffn_aligned16(ln_weight) &&
                     lffn_aligned16(ln_bias) && (uintptr_t)row_stats % 8 == 0 &&
                     (!proj_bias || lffn_aligned16(proj_bias)) && (!stage_inputs || lffn_aligned16(stage_inputs)),
                 LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.x = x; a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = ln_eps; a.wf = w_folded; a.pbias = proj_bias;
    a.codes = codes; a.scores = scores; a.z_out = z; a.row_stats = row_stats;
    a.stage_save = stage_inputs; a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T;
    a.decay = decay; a.residual = residual;
    return dispatch_block<true>(a, D, static_cast<hipStream_t>(stream));
}

extern "C" int lffn_bh4_block_bwd_f32(const float *g_z, const float *w_folded_t, float *g_x, float *stage_grads,
                                      int64_t B, int64_t H, int64_t D, int64_t R, int64_t J, int64_t T,
                                      int64_t block_size, float decay, float residual, void *stream) {
    LFFN_REQUIRE(B >= 0 && R >= 1 && J >= 1 && D >= 1 && H >= 1 && H <= D && T >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(H % 4 == 0 && J <= 64, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(block_size == BS && lffn_is_pow2(D) && D >= BS && D <= 1024, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(R <= 4096 && B <= (int64_t(1) << 31) - 1 && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(T * 8 <= R * D, LFFN_ERR_BAD_ARG);
    if (B == 0) return LFFN_OK;
    LFFN_REQUIRE(g_z && w_folded_t && g_x && stage_grads, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(g_z) && lffn_aligned16(w_folded_t) && lffn_aligned16(g_x) &&
                     lffn_aligned16(stage_grads), LFFN_ERR_BAD_ARG);
    BlockArgs a{};
    a.gz = g_z; a.wf = w_folded_t; a.out = g_x; a.stage_save = stage_grads;
    a.B = B; a.H = (int)H; a.R = (int)R; a.J = (int)J; a.T = (int)T; a.decay = decay; a.residual = residual;
    return dispatch_block_bwd(a, D, static_cast<hipStream_t>(stream));
}
