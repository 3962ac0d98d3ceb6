// Host stand-in for <hip/hip_runtime.h>, for the CPU tests that run the library's kernel sources as they are.
//
// Test infrastructure, not a product path: nothing under sf-bert_amd/ includes or links this.  The kernel sources are
// compiled as plain C++ for the host (tests/emu_lib.py rewrites only what is not C++: kernel launches, __shared__
// declarations and inline assembly).  Every thread of a work-group is a fiber with its own stack; fibers run one at a
// time until they reach an operation that involves other lanes, and the scheduler (emu_runtime.cpp) executes such an
// operation for the whole wave once every live lane of the wave has arrived at it:
//   * v_mfma_f32_32x32x16_bf16, v_mfma_f32_32x32x2_f32: lane l supplies A[l % 32][k-slots of half l / 32] and
//     B[the same k-slots][l % 32] and receives D[8 (i / 4) + 4 (l / 32) + i % 4][l % 32] in element i;
//   * ds_read_b64_tr_b16, v_readlane, v_readfirstlane, ballot, shuffles, DPP moves, wave and work-group barriers.
// Between such points the lanes of a work-group run in an order the test chooses (ascending, descending, shuffled), so
// code that needs a barrier it does not have reads stale or unwritten LDS under some order.
// LDS-direct loads (global_load_lds_dwordx4) are kept in a per-lane queue and land either when issued or only when an
// s_waitcnt asks for them (the test chooses), so both a missing wait and a tile overwritten while it is still read
// show up as wrong results.  __shared__ memory comes from a per-work-group arena below 4 GiB (its 32-bit addresses
// are the LDS addresses the kernels compute), filled with NaN patterns at the start of every work-group.
#pragma once

#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <functional>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

struct dim3 {
    uint32_t x, y, z;
    dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorLaunchFailure = 719 };
enum { hipMemcpyDeviceToHost = 2, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToDevice = 3 };
typedef enum { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 } hipStreamCaptureStatus;
typedef void* hipEvent_t;
enum { hipDeviceAttributeMultiprocessorCount = 63 };

namespace emu {

enum OpKind {
    OP_NONE = 0, OP_BLOCK_BARRIER, OP_BLOCK_AND, OP_WAVE_BARRIER, OP_MFMA_BF16, OP_MFMA_F32, OP_READFIRSTLANE,
    OP_READLANE, OP_BALLOT, OP_SHFL_XOR, OP_DS_READ_TR16, OP_DPP, OP_YIELD, OP_KINDS
};

struct Pending {
    uint8_t* dst;
    const uint8_t* src;
};

struct Block;
struct Lane {
    void* sp;
    uint8_t* stack;
    Block* block;
    uint32_t tid, lane, wave;
    bool done;
    int op;
    // operands and results of the operation the lane waits at
    float acc[16];
    uint16_t a16[8], b16[8];
    float a32, b32;
    uint32_t value, index, result;
    uint64_t result64;
    int pred, ctrl;
    const void* addr;
    uint16_t tr[4];
    Pending vm[256];
    uint32_t vm_head, vm_count;
};

extern Lane* cur;
dim3 thread_idx();
dim3 block_idx();
dim3 block_dim();
dim3 grid_dim();
void wait(int op);   // gives the processor back until the scheduler has executed the lane's operation
void* lds_alloc(const void* site, size_t bytes, size_t align);
void launch(dim3 grid, dim3 block, size_t shared, hipStream_t stream, const std::function<void()>& body);
hipError_t last_error();

void global_load_lds_dwordx4(uint32_t m0, uint32_t voffset, uint64_t sbase, int inst_offset);
// complete this lane's LDS-direct loads except the `in_flight` newest
void s_waitcnt_vmcnt(int in_flight);

}  // namespace emu

#define threadIdx (emu::thread_idx())
#define blockIdx (emu::block_idx())
#define blockDim (emu::block_dim())
#define gridDim (emu::grid_dim())

inline hipError_t hipGetLastError() { return emu::last_error(); }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = 256; return hipSuccess; }   // compute units, as on the device
template <typename F>
inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* n, F, int, size_t) { *n = 2; return hipSuccess; }
inline hipError_t hipMemcpy(void* dst, const void* src, size_t n, int) { memcpy(dst, src, n); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, int, hipStream_t) { memcpy(dst, src, n); return hipSuccess; }
inline hipError_t hipMemcpy2DAsync(void* dst, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, int,
                                   hipStream_t) {
    for (size_t r = 0; r < height; ++r) memcpy((uint8_t*)dst + r * dpitch, (const uint8_t*)src + r * spitch, width);
    return hipSuccess;
}
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* s) { *s = hipStreamCaptureStatusNone; return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = (void*)1; return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 1.0f; return hipSuccess; }
// memory of host programs built against this header: host memory, aligned as device allocations are
template <typename T>
inline hipError_t hipMalloc(T** p, size_t bytes) {
    *p = (T*)aligned_alloc(256, (bytes + 255) / 256 * 256);
    return *p ? hipSuccess : 2;
}
inline hipError_t hipFree(void* p) { free(p); return hipSuccess; }
inline hipError_t hipMemset(void* p, int value, size_t bytes) { memset(p, value, bytes); return hipSuccess; }
inline hipError_t hipStreamCreate(hipStream_t* s) { *s = nullptr; return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "error of the host model"; }
template <typename T>
inline hipError_t hipGetSymbolAddress(void** p, T* symbol) { *p = (void*)symbol; return hipSuccess; }

// ---------------------------------------------------------------------------------------------------------------
// device functions
// ---------------------------------------------------------------------------------------------------------------
inline void __syncthreads() { emu::wait(emu::OP_BLOCK_BARRIER); }
inline int __syncthreads_and(int pred) {
    emu::cur->pred = pred;
    emu::wait(emu::OP_BLOCK_AND);
    return (int)emu::cur->result;
}
inline float __shfl_xor(float v, int mask) {
    emu::cur->value = __builtin_bit_cast(uint32_t, v);
    emu::cur->index = (uint32_t)mask;
    emu::wait(emu::OP_SHFL_XOR);
    return __builtin_bit_cast(float, emu::cur->result);
}

typedef float emu_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 emu_bf16x8 __attribute__((ext_vector_type(8)));
typedef short emu_s16x4 __attribute__((ext_vector_type(4)));

inline emu_f32x16 emu_mfma_f32_32x32x16_bf16(emu_bf16x8 a, emu_bf16x8 b, emu_f32x16 c, int, int, int) {
    emu::Lane* l = emu::cur;
    memcpy(l->a16, &a, 16);
    memcpy(l->b16, &b, 16);
    memcpy(l->acc, &c, 64);
    emu::wait(emu::OP_MFMA_BF16);
    emu_f32x16 d;
    memcpy(&d, l->acc, 64);
    return d;
}
inline emu_f32x16 emu_mfma_f32_32x32x2f32(float a, float b, emu_f32x16 c, int, int, int) {
    emu::Lane* l = emu::cur;
    l->a32 = a;
    l->b32 = b;
    memcpy(l->acc, &c, 64);
    emu::wait(emu::OP_MFMA_F32);
    emu_f32x16 d;
    memcpy(&d, l->acc, 64);
    return d;
}
template <typename T>
inline T emu_readfirstlane(T v) {
    static_assert(sizeof(T) == 4, "32-bit values");
    emu::cur->value = __builtin_bit_cast(uint32_t, v);
    emu::wait(emu::OP_READFIRSTLANE);
    return __builtin_bit_cast(T, emu::cur->result);
}
template <typename T>
inline T emu_readlane(T v, uint32_t lane) {
    static_assert(sizeof(T) == 4, "32-bit values");
    emu::cur->value = __builtin_bit_cast(uint32_t, v);
    emu::cur->index = lane;
    emu::wait(emu::OP_READLANE);
    return __builtin_bit_cast(T, emu::cur->result);
}
inline uint64_t emu_ballot_w64(bool pred) {
    emu::cur->pred = pred;
    emu::wait(emu::OP_BALLOT);
    return emu::cur->result64;
}
template <typename P>
inline emu_s16x4 emu_ds_read_tr16_b64(P p) {
    emu::cur->addr = (const void*)(uintptr_t)p;
    emu::wait(emu::OP_DS_READ_TR16);
    emu_s16x4 r;
    memcpy(&r, emu::cur->tr, 8);
    return r;
}
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    (void)old; (void)row_mask; (void)bank_mask; (void)bound_ctrl;
    emu::cur->value = (uint32_t)src;
    emu::cur->ctrl = ctrl;
    emu::wait(emu::OP_DPP);
    return (int)emu::cur->result;
}
inline void emu_wave_barrier() { emu::wait(emu::OP_WAVE_BARRIER); }
inline void emu_s_sleep(int) { emu::wait(emu::OP_YIELD); }
inline float emu_fdot2_f32_bf16(__attribute__((ext_vector_type(2))) __bf16 a, __attribute__((ext_vector_type(2))) __bf16 b,
                                float c, bool) {
    return c + (float)a.x * (float)b.x + (float)a.y * (float)b.y;
}

#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 emu_mfma_f32_32x32x16_bf16
#define __builtin_amdgcn_mfma_f32_32x32x2f32 emu_mfma_f32_32x32x2f32
#define __builtin_amdgcn_readfirstlane emu_readfirstlane
#define __builtin_amdgcn_readlane emu_readlane
#define __builtin_amdgcn_ballot_w64 emu_ballot_w64
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16 emu_ds_read_tr16_b64
#define __builtin_amdgcn_update_dpp emu_update_dpp
#define __builtin_amdgcn_wave_barrier emu_wave_barrier
#define __builtin_amdgcn_s_sleep emu_s_sleep
#define __builtin_amdgcn_fdot2_f32_bf16 emu_fdot2_f32_bf16
#define __builtin_amdgcn_exp2f exp2f
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_sched_barrier(...) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(...) ((void)0)

#define __HIP_MEMORY_SCOPE_AGENT 0
template <typename T>
inline T emu_atomic_load(const T* p) {
    T v;
    __atomic_load(p, &v, __ATOMIC_RELAXED);
    return v;
}
template <typename T, typename V>
inline void emu_atomic_store(T* p, V v) {
    T w = (T)v;
    __atomic_store(p, &w, __ATOMIC_RELAXED);
}
#define __hip_atomic_load(p, order, scope) emu_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu_atomic_store(p, v)
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add(p, v, order)
