// Shared device-side helpers for the gfx950 kernels of libsfbert_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sfbert_hip.h"

namespace sfb {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
// Seed of the running row maximum, in raw-score units (ewops.h:70 of the reference CPU path).
constexpr float kMaxSeed = -1000000.0f;
// Score given to a masked key: far below any real score, finite so that (s - max) never makes NaN.
constexpr float kMaskedScore = -3.0e38f;
// Probabilities are kept relative to a reference maximum that may lag the true one by this many
// powers of two before the accumulators are rescaled.
constexpr float kLazyRescaleLog2 = 8.0f;

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// fp32 pair -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// acc + lo(pair) + hi(pair) for a packed bf16 pair (v_dot2c_f32_bf16 against packed ones).
__device__ __forceinline__ float dot2_bf16_ones(uint32_t pair, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair),
                                           __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __builtin_bit_cast(float, bits16 << 16);
}

// Element offset of (b, token, h, 0) in a [B, L, H, d] tensor.
__device__ __forceinline__ size_t token_offset(uint32_t b, uint32_t token, uint32_t h, uint32_t L,
                                               uint32_t H, uint32_t d) {
    return (((size_t)b * L + token) * H + h) * (size_t)d;
}

// Work-group id -> (batch*head index, rank of the work item in the launch order).
// Hardware deals consecutive work-group ids round-robin to the 8 XCDs, each with its own L2.  All
// work items of one (batch, head) are given ids of the same residue mod 8, so the K/V blocks they
// share (window neighbours, global and random blocks) are fetched into one L2 only.  Within an XCD
// the ranks of one (batch, head) are consecutive and the heads follow one another, so that only a
// couple of heads' K and V (about 1 MiB each at L = 4096) are live in the 4 MiB L2 at any time.
struct WorkId {
    uint32_t bh;
    uint32_t rank;
    bool valid;
};

// The first `heavy` ranks (items much longer than the rest, sorted to the front) are the exception:
// they are issued for all heads before anything else, so that they overlap with the short items
// instead of forming the tail of the launch.
__device__ __forceinline__ WorkId decode_work(uint32_t wg, uint32_t num_bh, uint32_t ranks,
                                              uint32_t heavy = 0) {
    constexpr uint32_t kXcds = 8;
    const uint32_t xcd = wg % kXcds;
    uint32_t q = wg / kXcds;
    const uint32_t groups = (num_bh + kXcds - 1) / kXcds;
    WorkId w;
    uint32_t group;
    if (q < heavy * groups) {
        w.rank = q / groups;
        group = q % groups;
    } else {
        q -= heavy * groups;
        const uint32_t light = ranks - heavy;
        w.rank = heavy + q % light;
        group = q / light;
    }
    w.bh = group * kXcds + xcd;
    w.valid = w.bh < num_bh;
    return w;
}

inline uint32_t bh_groups(uint32_t num_bh) { return (num_bh + 7u) / 8u; }

// A launcher reports only its own launch: the thread's last-error state may still hold an error left by
// an unrelated earlier HIP call of the process, so it is cleared before the launch and read after it.
inline void clear_stale_error() { (void)hipGetLastError(); }
inline int launch_status() { return hipGetLastError() == hipSuccess ? SFB_OK : SFB_ERR_LAUNCH; }

}  // namespace sfb
