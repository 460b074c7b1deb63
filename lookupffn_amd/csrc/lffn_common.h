// Shared device helpers and host-side argument checks for the gfx950 LookupFFN kernels.
// wave64 is assumed everywhere: this code is built for gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "../../include/lookupffn_hip.h"

#define LFFN_WAVE 64

#define LFFN_REQUIRE(cond, code) \
    do {                         \
        if (!(cond)) return (code); \
    } while (0)

static inline bool lffn_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool lffn_is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
static inline int lffn_log2(int64_t v) {
    int l = 0;
    while ((int64_t(1) << l) < v) ++l;
    return l;
}

// Row formats of the gather's tables: the values of the C ABI's row_format arguments.
constexpr int LFFN_ROWS_F32 = 0, LFFN_ROWS_BF16 = 1, LFFN_ROWS_F16 = 2;

// gather.hip: token-major gather on table-local codes (not exported); fmt is one of LFFN_ROWS_*
__attribute__((visibility("hidden")))
int lffn_internal_lookup_gather_token_major(const int32_t *code, const float *score, const void *tables,
                                            const float *bias, const float *residual, float *out, int64_t B,
                                            int64_t T, int64_t S, int64_t Do, int fmt, void *stream);

// gather.hip: atomic scatter-add on table-local codes (not exported)
__attribute__((visibility("hidden")))
int lffn_internal_lookup_scatter_atomic(const int32_t *code, const float *score, const float *g, float *out,
                                        int64_t B, int64_t T, int64_t S, int64_t Do, void *stream);

// gather.hip: token-major indexed inner product on table-local codes (not exported)
__attribute__((visibility("hidden")))
int lffn_internal_lookup_inner_token_major(const int32_t *code, const float *g, const float *tables,
                                           float *out, int64_t B, int64_t T, int64_t S, int64_t Do,
                                           void *stream);

// lookup_gather_pair.hip: the two-tables-per-buffer LDS gather (not exported)
__attribute__((visibility("hidden")))
int lffn_internal_lookup_gather_pair(const int32_t *code, const float *score, const void *tables,
                                     const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                     int64_t S, int64_t Do, bool bf16, int np, void *stream);

// Dynamic LDS beyond the default limit has to be granted to a kernel once per device
// (hipFuncAttributeMaxDynamicSharedMemorySize).  `granted` is the caller's record for ONE kernel
// instantiation (a function-local static array, zero-initialised): the largest size granted so far
// on each device, so that the attribute call is made when a launch needs more than that and not on
// every launch.  Devices beyond the record ask every time.
constexpr int LFFN_MAX_DEVICES = 16;
struct LdsGrant {
    std::atomic<int> bytes[LFFN_MAX_DEVICES];
};
static inline bool lffn_grant_dynamic_lds(const void *kernel, size_t lds_bytes, LdsGrant &granted) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    const bool recorded = dev >= 0 && dev < LFFN_MAX_DEVICES;
    if (recorded && granted.bytes[dev].load(std::memory_order_acquire) >= (int)lds_bytes) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (recorded) {
        int seen = granted.bytes[dev].load(std::memory_order_relaxed);
        while (seen < (int)lds_bytes &&
               !granted.bytes[dev].compare_exchange_weak(seen, (int)lds_bytes, std::memory_order_release)) {
        }
    }
    return true;
}

// lookup_gather_quad.hip: the two-tables-per-buffer LDS gather with four lanes per token (not exported);
// fmt is one of LFFN_ROWS_*, tokens the tokens per workgroup (a multiple of 16)
__attribute__((visibility("hidden")))
int lffn_internal_lookup_gather_quad(const int32_t *code, const float *score, const void *tables,
                                     const float *bias, const float *residual, float *out, int64_t B, int64_t T,
                                     int64_t S, int64_t Do, int fmt, int tokens, void *workspace, void *stream);
__attribute__((visibility("hidden")))
bool lffn_internal_quad_np_built(int fmt, int np);
__attribute__((visibility("hidden")))
int lffn_internal_quad_passes(int fmt, int64_t tokens);
__attribute__((visibility("hidden")))
int64_t lffn_internal_quad_stream_bytes(int64_t B, int64_t T);
__attribute__((visibility("hidden")))
int64_t lffn_internal_quad_record_stride(int64_t B, int fmt, int64_t tokens);
__attribute__((visibility("hidden")))
int lffn_internal_lookup_gather_quad_records(const uint32_t *records, int64_t record_stride, const void *tables,
                                             const float *bias, const float *residual, float *out, int64_t B,
                                             int64_t T, int64_t S, int64_t Do, int fmt, int tokens, void *stream);

// The record stream of the four-lanes-per-token gather (lookup_gather_quad.hip), as its writers address it.
// A record is three words: score of the pair's first table, score of its second, row of the first | row of
// the second << 8, where token b takes the tables of pair k in the order (2k, 2k+1) when bit 1 of b is clear
// and (2k+1, 2k) when it is set.  Records are kept per table pair, record_stride slots of 12 bytes each, in
// the order the gather's wavefronts copy them: a tile of tile_tokens tokens (a multiple of 16 in
// (256 (np-1), 256 np]) is np passes of 16 wavefronts x 16 tokens, group p*16 + w of the tile being pass p of
// wavefront w; a wavefront's records of all its passes are contiguous (pass-major), the wavefronts follow each
// other, the tiles follow each other: slot = tile * tile_tokens + first slot of the wavefront + pass * 16 +
// token within the group.  Wavefronts below n_last = tile_tokens/16 - 16 (np-1) have np passes, the others np-1.
__host__ __device__ __forceinline__ int64_t lffn_quad_record_slot(int64_t token, int tile_tokens) {
    const int npm1 = (tile_tokens - 1) >> 8;                  // passes - 1
    const int n_last = (tile_tokens >> 4) - 16 * npm1;
    const int64_t tile = token / tile_tokens;
    const int r = (int)(token - tile * tile_tokens);
    const int group = r >> 4, wave = group & 15, pass = group >> 4;
    return tile * tile_tokens + 16 * (npm1 * wave + (wave < n_last ? wave : n_last)) + pass * 16 + (r & 15);
}
constexpr int LFFN_RECORD_WORDS = 3;
// what a writer of records checks: a tile size the slots are defined for and room for every tile
static inline bool lffn_record_layout_ok(int64_t B, int64_t record_stride, int64_t tile_tokens) {
    return tile_tokens >= 16 && tile_tokens <= 2048 && tile_tokens % 16 == 0 &&
           record_stride >= (B + tile_tokens - 1) / tile_tokens * tile_tokens;
}

// lookup_inner.hip: the four-lanes-per-token score gradient where the shape qualifies (not exported)
__attribute__((visibility("hidden")))
bool lffn_internal_lookup_inner_quad_try(const int32_t *code, const float *g, int64_t g_token_stride,
                                         int64_t g_slice_stride, const void *tables, float *grad_score, int64_t B,
                                         int64_t T, int64_t S, int64_t Do, void *stream, int *rc);

// lookup_inner_quad.hip: the score gradient with four lanes per token and one owner per (token, table) (not exported)
__attribute__((visibility("hidden")))
int lffn_internal_lookup_inner_quad(const int32_t *code, const float *g, int64_t g_token_stride, int64_t g_slice_stride,
                                    const void *tables, float *grad_score, int64_t B, int64_t T, int64_t S, int64_t Do,
                                    int np, int c, void *stream);

static inline int lffn_launch_status() {
    return hipGetLastError() == hipSuccess ? LFFN_OK : LFFN_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------
// Cross-lane moves.  dpp_mov<CTRL>: lanes whose source is outside the row, or
// that the bank mask switches off, keep `old`.
// ---------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ float dpp_mov(float old, float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL,
                                                      ROW_MASK, BANK_MASK, false));
}

constexpr int DPP_QUAD_XOR1 = 0xB1;   // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;   // quad_perm [2,3,0,1]
constexpr int DPP_ROW_SHL4 = 0x104;   // lane i <- lane i+4
constexpr int DPP_ROW_SHR4 = 0x114;   // lane i <- lane i-4
constexpr int DPP_ROW_ROR8 = 0x128;   // lane i <- lane (i-8) mod 16 == i xor 8
constexpr int DPP_ROW_NEWBCAST0 = 0x150;   // + n: every lane of a 16-lane row <- lane n of that row

// Value held by lane N of the caller's 16-lane row, in every lane of the row (one
// vector-ALU move, no LDS traffic).  N is a compile-time constant.
template <int N>
__device__ __forceinline__ int row_broadcast(int v) {
    static_assert(N >= 0 && N < 16, "row_broadcast: lane within the row");
    // every lane has a source inside its row, so `old` is never used: 0 with bound_ctrl lets the
    // compiler emit the bare v_mov_b32_dpp without first copying v into the destination
    return __builtin_amdgcn_update_dpp(0, v, DPP_ROW_NEWBCAST0 + N, 0xF, 0xF, true);
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, typename F, int I = 0>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, F, I + 1>(static_cast<F &&>(f));
    }
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov_all(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Value held by lane (lane ^ M), for M a power of two below 64.
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
    // Where every lane has a source, `old` is never used: 0 with bound_ctrl gives the bare
    // v_mov_b32_dpp, without a copy of v into the destination first.
    if constexpr (M == 1) {
        return dpp_mov_all<DPP_QUAD_XOR1>(v);
    } else if constexpr (M == 2) {
        return dpp_mov_all<DPP_QUAD_XOR2>(v);
    } else if constexpr (M == 4) {
        float r = dpp_mov_all<DPP_ROW_SHL4>(v);            // lane+4 (banks 0,2 keep it; lanes 12-15 read 0)
        return dpp_mov<DPP_ROW_SHR4, 0xF, 0xA>(r, v);      // banks 1,3 take lane-4
    } else if constexpr (M == 8) {
        return dpp_mov_all<DPP_ROW_ROR8>(v);
    } else if constexpr (M == 16) {
        // ds_swizzle, bit-mask mode inside 32 lanes: and 0x1F, or 0, xor 0x10
        return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
    } else {
        static_assert(M == 32, "lane_xor: M must be a power of two below 64");
        return __shfl_xor(v, 32, 64);
    }
}

// One butterfly across lanes: the lane whose M bit is clear gets own + partner,
// the other gets partner - own.  `sgn` is +1 / -1 for the two cases.
// (The gfx950 v_permlane16_swap / v_permlane32_swap instructions can do the M = 16 and M = 32
// exchanges on the vector ALU; the kernels that wait on LDS permutes use them, see fht.hip.)
template <int M>
__device__ __forceinline__ float butterfly_xor(float v, float sgn) {
    return fmaf(v, sgn, lane_xor<M>(v));   // (+-1)*v is exact: one rounding, like a plain add
}

// Sum over the LPR lanes of an aligned lane group (LPR a power of two <= 64).
template <int LPR>
__device__ __forceinline__ float lane_group_sum(float v) {
    if constexpr (LPR > 1) v += lane_xor<1>(v);
    if constexpr (LPR > 2) v += lane_xor<2>(v);
    if constexpr (LPR > 4) v += lane_xor<4>(v);
    if constexpr (LPR > 8) v += lane_xor<8>(v);
    if constexpr (LPR > 16) v += lane_xor<16>(v);
    if constexpr (LPR > 32) v += lane_xor<32>(v);
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
    v += lane_xor<1>(v);
    v += lane_xor<2>(v);
    v += lane_xor<4>(v);
    v += lane_xor<8>(v);
    v += lane_xor<16>(v);
    v += lane_xor<32>(v);
    return v;
}

// One 4-byte global -> LDS load per active lane into a scratch area nobody reads (256 bytes at
// lds_byte_addr, shared by all wavefronts): pulls the lane's 128-byte line into L2 and writes no
// register.  As with every global -> LDS copy the workgroup must wait (vmcnt) before it ends.
constexpr int TOUCH_SINK_BYTES = 256;
// s_waitcnt immediates (vmcnt in bits 3:0, the other counters left alone)
constexpr int WAIT_VMCNT_0 = 0x0F70;
constexpr int WAIT_VMCNT_1 = 0x0F71;
__device__ __forceinline__ void l2_touch(const char *base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    // M0 is put back: the compiler reserves it for its own use and does not honour a clobber
    // declaration of it, so the statement must leave it as it found it
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(lane_offset), "s"(base), "s"(lds_byte_addr)
                 : "memory");
}

// The line of a region of `nlines` 128-byte lines that lane `tid` of workgroup `member` of a team of
// `nteam` workgroups touches: the team splits the lines evenly and a workgroup's first lanes take
// its share one each; the other lanes repeat the workgroup's first line (one address per
// wavefront costs next to nothing), so that every wavefront issues the same instruction and
// waits the same way: no branch, no lane mask.  (Spreading the share over the wavefronts instead was
// measured worse with cold tables, 196 -> 214 us at 16384 tokens: the first wavefront's touch leaves
// right behind its own four copies, the later wavefronts' would queue behind everybody's.)
__device__ __forceinline__ int team_touch_line(int nlines, int nteam, int member, int tid) {
    const int share = (nlines + nteam - 1) / nteam;
    const int first = member * share;
    const int line = first + (tid < share ? tid : 0);
    return min(line, nlines - 1);
}

// How far ahead of the table being read the team touches: the copy of table t+1 is issued with the
// reads of table t, the touch of table t+2 with it (3 or 4 ahead measured no better).
constexpr int TOUCH_AHEAD = 2;

// exp(-2a) for a >= 0 in the hash kernels' scores: the hardware exp2 (v_exp_f32, 1 ulp) on
// a * (-2 log2 e) instead of the library's expf, which costs ten times the instructions in kernels that
// are bound by instruction issue.  The rounding of the scaled argument adds a relative error of
// about |argument| * 4e-8, i.e. 1e-6 at a = 8, where the value is 1e-7 beside the 1 it is added to:
// the scores agree with the float64 oracle as before (2e-6).
__device__ __forceinline__ float exp_minus_2a(float a) { return __builtin_amdgcn_exp2f(-2.885390081777927f * a); }

__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xFFFF0000u); }
