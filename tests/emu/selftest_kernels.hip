// Kernels with deliberate mistakes (selected by arguments), for the test that the host model notices them: a read of
// an LDS-direct load that nobody waited for, a read of another wave's LDS data without a barrier, a buffer refilled
// while another wave still reads it, a wave-wide operation under divergent control flow.  Built into the host model's
// library only; nothing here is part of the product.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t __attribute__((address_space(3)))* lds_u32_ptr;

__device__ __forceinline__ uint32_t lds_address(const void* p) { return (uint32_t)(uintptr_t)(lds_u32_ptr)p; }

__device__ __forceinline__ void load_1k(uint32_t lds_dst, const uint8_t* src, uint32_t lane) {
    const uint64_t base = (uint64_t)src;
    const uint32_t off = lane * 16u;
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(off), "s"(base) : "memory");
}

// 128 threads.  Each wave brings 1 KiB of src into its half of a 2 KiB tile; every lane then copies 16 bytes of the
// *other* wave's half to dst.
__global__ __launch_bounds__(128) void exchange_kernel(const uint8_t* src, uint8_t* dst, int with_wait, int with_barrier) {
    __shared__ __attribute__((aligned(1024))) uint8_t tile[2048];
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    load_1k(lds_address(tile) + wave * 1024u, src + wave * 1024u, lane);
    if (with_wait) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (with_barrier) __syncthreads();
    const uint32_t other = (wave ^ 1u) * 1024u + lane * 16u;
    *(u32x4*)(dst + other) = *(const u32x4*)(tile + other);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// 128 threads.  Both waves fill their halves (correctly); wave 0 copies wave 1's half to dst[0..1023]; wave 1 then
// refills its half with the third KiB of src and copies that to dst[1024..2047] -- with or without a barrier between
// wave 0's reads and the refill.
__global__ __launch_bounds__(128) void refill_kernel(const uint8_t* src, uint8_t* dst, int with_barrier) {
    __shared__ __attribute__((aligned(1024))) uint8_t tile[2048];
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    load_1k(lds_address(tile) + wave * 1024u, src + wave * 1024u, lane);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (wave == 0) *(u32x4*)(dst + lane * 16u) = *(const u32x4*)(tile + 1024u + lane * 16u);
    if (with_barrier) __syncthreads();
    if (wave == 1) {
        load_1k(lds_address(tile) + 1024u, src + 2048u, lane);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        *(u32x4*)(dst + 1024u + lane * 16u) = *(const u32x4*)(tile + 1024u + lane * 16u);
    }
}

// The lower half of the wave takes a wave-wide operation that the upper half does not reach.
__global__ __launch_bounds__(64) void diverged_kernel(uint32_t* out) {
    const uint32_t lane = threadIdx.x;
    uint32_t v = 1000u + lane;
    if (lane >= 8 && lane < 32) v = __builtin_amdgcn_readfirstlane(v);
    out[lane] = v;
}

__global__ __launch_bounds__(64) void mfma_kernel(const uint16_t* a, const uint16_t* b, float* d) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x16 __attribute__((ext_vector_type(16)));
    const uint32_t lane = threadIdx.x, r = lane % 32, h = lane / 32;
    bf16x8 av, bv;
    // A [32][16] row-major, B [16][32] row-major
    for (int e = 0; e < 8; ++e) {
        av[e] = __builtin_bit_cast(__bf16, a[r * 16 + 8 * h + e]);
        bv[e] = __builtin_bit_cast(__bf16, b[(8 * h + e) * 32 + r]);
    }
    f32x16 acc;
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    for (int i = 0; i < 16; ++i) d[(8 * (i / 4) + 4 * h + i % 4) * 32 + r] = acc[i];
}

}  // namespace

extern "C" int emu_selftest_exchange(const uint8_t* src, uint8_t* dst, int with_wait, int with_barrier) {
    (void)hipGetLastError();
    exchange_kernel<<<dim3(1), dim3(128), 0, nullptr>>>(src, dst, with_wait, with_barrier);
    return (int)hipGetLastError();
}
extern "C" int emu_selftest_refill(const uint8_t* src, uint8_t* dst, int with_barrier) {
    (void)hipGetLastError();
    refill_kernel<<<dim3(1), dim3(128), 0, nullptr>>>(src, dst, with_barrier);
    return (int)hipGetLastError();
}
extern "C" int emu_selftest_diverged(uint32_t* out) {
    (void)hipGetLastError();
    diverged_kernel<<<dim3(1), dim3(64), 0, nullptr>>>(out);
    return (int)hipGetLastError();
}
extern "C" int emu_selftest_mfma(const uint16_t* a, const uint16_t* b, float* d) {
    (void)hipGetLastError();
    mfma_kernel<<<dim3(1), dim3(64), 0, nullptr>>>(a, b, d);
    return (int)hipGetLastError();
}
