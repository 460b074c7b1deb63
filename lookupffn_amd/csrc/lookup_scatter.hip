// Gradient of the layer's gather w.r.t. the tables, table-major with the
// gradient slice accumulated in LDS:
//
//   grad_tables[t, s, :] (+)= sum over tokens b with (code[b,t] & (S-1)) == s of score[b,t] * g[b,:]
//
// The reference computes this with one global fp32 atomicAdd per (token, table,
// column) (gather_kernel_fp32.cu:83-91).  Here a 1024-lane workgroup owns one
// table and a 64-column slice: their gradient (S rows x 64 columns) lives in LDS
// as DOUBLES (128 KiB for S = 256), zeroed at the start.  The workgroup streams
// over ALL tokens; a wavefront takes one token at a time, lane l holding column l
// of the slice, and adds score * g into the row the token's code selects with one
// ds_add_f64: 64 lanes hit 64 consecutive doubles, so an instruction never has a
// bank conflict or two lanes on one address, however skewed the code distribution
// is.  At the end the slice is rounded to fp32 and written to HBM with plain
// coalesced stores: no global atomics, and the output needs no zero-fill.
//
// Why doubles: on gfx950 the LDS fp32 atomic add is processed lane by lane (192
// clocks per 64-lane instruction measured), while the fp64 atomic add runs at the
// rate of an LDS integer atomic (under 10 clocks).  Accumulating in fp64 also makes
// the sum independent of the order in which wavefronts reach a row up to one fp32
// rounding at the end, so results repeat from run to run except where that final
// rounding sits on a tie.
//
// (row offset, score) pairs of 64 tokens are fetched by the 64 lanes at once (one
// token per lane), parked in a wavefront-private LDS strip and read back as a
// broadcast ds_read_b64 when their token comes up.
#include "lffn_common.h"

#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

namespace {

constexpr int WG = 1024;
constexpr int WAVES = WG / 64;
constexpr int COLS = 64;           // columns per slice = lanes per token
constexpr int MAX_S = 256;
constexpr int XCDS = 8;
constexpr int GDEPTH = 16;         // gradient rows in flight per wavefront

struct ScatterArgs {
    const int32_t *code;   // [B, T]
    const float *score;    // [B, T]
    const float *g;        // [B, Do]
    float *out;            // [T, S, Do]
    int64_t B;
    int T, S, Do;
    int nslices, per_xcd;
    int accumulate;
};

__global__ __launch_bounds__(WG) void lookup_scatter_lds_kernel(ScatterArgs a) {
    extern __shared__ double lds[];                // [S][COLS] doubles, then [WAVES][64] uint2
    const int tab_elems = a.S * COLS;
    uint2 *strip = reinterpret_cast<uint2 *>(lds + tab_elems) + (threadIdx.x >> 6) * 64;

    const int xcd = blockIdx.x % XCDS;
    const int unit = xcd * a.per_xcd + blockIdx.x / XCDS;
    if (unit >= a.T * a.nslices) return;           // uniform over the workgroup
    // units that share a slice of g are neighbours, so they land on one XCD
    const int slice = unit / a.T;
    const int t = unit % a.T;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    for (int q = tid; q < tab_elems / 2; q += WG)
        reinterpret_cast<double2 *>(lds)[q] = make_double2(0.0, 0.0);
    __syncthreads();

    const int mask = a.S - 1;
    const float *gcol = a.g + (size_t)slice * COLS + lane;
    double *my_col = lds + lane;

    // The wavefront's token stream: batch k covers tokens wave*64 + k*1024 + [0, 64).
    // The wavefront number is made scalar so that all per-token address arithmetic
    // runs on the scalar unit; only the lane's column offset is a vector value.
    const int swave = __builtin_amdgcn_readfirstlane(wave);
    const int64_t first = int64_t(swave) * 64;
    const int64_t nbatch = first < a.B ? (a.B - first + WG - 1) / WG : 0;
    const int64_t last = a.B - 1;

    auto load_pair = [&](int64_t batch) {
        const int64_t tok = min<int64_t>(first + batch * WG + lane, last);
        uint2 pr;
        pr.x = (unsigned)((a.code[tok * a.T + t] & mask) * COLS);
        pr.y = __float_as_uint(a.score[tok * a.T + t]);
        return pr;
    };

    uint2 pr_next = make_uint2(0u, 0u);
    if (nbatch > 0) pr_next = load_pair(0);
    for (int64_t batch = 0; batch < nbatch; ++batch) {
        const int64_t base = first + batch * WG;
        strip[lane] = pr_next;     // wavefront-private: ordered by the LDS queue, no barrier needed
        pr_next = load_pair(batch + 1 < nbatch ? batch + 1 : batch);   // pairs run one batch ahead
        const int n = (int)min<int64_t>(64, a.B - base);
        const float *gp = gcol + base * a.Do;
        if (n == 64) {
#pragma unroll
            for (int i0 = 0; i0 < 64; i0 += GDEPTH) {
                float gv[GDEPTH];
                uint2 pr[GDEPTH];
#pragma unroll
                for (int u = 0; u < GDEPTH; ++u) gv[u] = gp[(size_t)(i0 + u) * a.Do];
#pragma unroll
                for (int u = 0; u < GDEPTH; ++u) pr[u] = strip[i0 + u];   // broadcast reads
#pragma unroll
                for (int u = 0; u < GDEPTH; ++u)
                    unsafeAtomicAdd(my_col + pr[u].x, (double)(__uint_as_float(pr[u].y) * gv[u]));
            }
        } else {
            for (int i = 0; i < n; ++i) {
                const uint2 pr = strip[i];
                unsafeAtomicAdd(my_col + pr.x, (double)(__uint_as_float(pr.y) * gp[(size_t)i * a.Do]));
            }
        }
    }
    __syncthreads();

    // flush: rows of table t x this slice, 16 lanes per 256-byte row segment
    for (int q = tid; q < a.S * (COLS / 4); q += WG) {
        const int row = q / (COLS / 4);
        const int v = q % (COLS / 4);
        const double2 lo = reinterpret_cast<double2 *>(lds)[2 * q];
        const double2 hi = reinterpret_cast<double2 *>(lds)[2 * q + 1];
        float4 val = make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
        float *dst = a.out + ((size_t)t * a.S + row) * a.Do + (size_t)slice * COLS + v * 4;
        if (a.accumulate) {
            const float4 old = *reinterpret_cast<const float4 *>(dst);
            val.x += old.x; val.y += old.y; val.z += old.z; val.w += old.w;
        }
        *reinterpret_cast<float4 *>(dst) = val;
    }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float4 *p, int64_t n4) {
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < n4; i += int64_t(gridDim.x) * 256)
        p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

}  // namespace

extern "C" int lffn_lookup_scatter_f32(const int32_t *code, const float *score, const float *g,
                                       float *grad_tables, int64_t B, int64_t T, int64_t S, int64_t Do,
                                       int32_t accumulate, void *stream) {
    LFFN_REQUIRE(B >= 0 && T >= 0 && Do >= 1, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_is_pow2(S) && S <= (1 << 24) && T * S <= 0x7fffffff, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(Do % 64 == 0 && Do <= (1 << 20) && T <= (1 << 24), LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(B <= (int64_t(1) << 31) - 1, LFFN_ERR_UNSUPPORTED);
    LFFN_REQUIRE(grad_tables || T == 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE((code && score && g) || B * T == 0, LFFN_ERR_BAD_ARG);
    LFFN_REQUIRE(lffn_aligned16(grad_tables) && lffn_aligned16(g), LFFN_ERR_BAD_ARG);
    if (T == 0) return LFFN_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t units = T * (Do / COLS);
    if (S > MAX_S || units > (int64_t(1) << 24)) {
        // tables too large for the LDS slice: zero-fill, then global atomics
        if (!accumulate) {
            const int64_t n4 = T * S * Do / 4;
            hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n4 + 255) / 256 < 65536 ? (n4 + 255) / 256 : 65536)), dim3(256), 0,
                               st, reinterpret_cast<float4 *>(grad_tables), n4);
            int rc = lffn_launch_status();
            if (rc != LFFN_OK) return rc;
        }
        if (B == 0) return LFFN_OK;
        return lffn_internal_lookup_scatter_atomic(code, score, g, grad_tables, B, T, S, Do, stream);
    }
    ScatterArgs a{};
    a.code = code; a.score = score; a.g = g; a.out = grad_tables;
    a.B = B; a.T = (int)T; a.S = (int)S; a.Do = (int)Do;
    a.nslices = (int)(Do / COLS);
    a.per_xcd = (int)((units + XCDS - 1) / XCDS);
    a.accumulate = accumulate;
    const size_t lds_bytes = size_t(S) * COLS * 8 + size_t(WAVES) * 64 * 8;
    static LdsGrant granted;      // one record per kernel instantiation
    if (!lffn_grant_dynamic_lds(reinterpret_cast<const void *>(lookup_scatter_lds_kernel), lds_bytes, granted)) return LFFN_ERR_LAUNCH;
    hipLaunchKernelGGL(lookup_scatter_lds_kernel, dim3(a.per_xcd * XCDS), dim3(WG), lds_bytes, st, a);
    return lffn_launch_status();
}
