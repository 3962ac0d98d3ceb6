// Host-surface types of the block-sparse attention path (counterpart of the reference's gpu_types.h:
// bhalf storage structs :48-76, NT_OP/NN_OP/TN_OP :135-137, CEIL_DIV / THREAD_POW2 :213-215,
// magicu64 declaration :226).  Plain C++: usable from TUs compiled by g++ or hipcc.
#ifndef SFB_HOST_GPU_TYPES_H
#define SFB_HOST_GPU_TYPES_H

#include <stdint.h>

#include "../../include/sfbert_hip.h"

typedef unsigned int uint;
typedef unsigned short ushort;
typedef unsigned long long uint64;

// The LUT entry type of the launchers.  With the HIP headers present uint2 is HIP's own vector type
// (same layout: two 32-bit words); otherwise a plain struct stands in.
#if defined(__HIPCC__) || defined(HIP_INCLUDE_HIP_HIP_RUNTIME_H)
#include <hip/hip_runtime.h>
#else
struct uint2 { uint x, y; };
#endif
static_assert(sizeof(uint2) == sizeof(sfb_uint2), "LUT entries are two 32-bit words");

// bf16 storage: the high 16 bits of a float (gpu_types.h:48-52).
struct bhalf { ushort x; };
struct bhalf2 { uint x; };

// The reference passes a CUstream; here it is the HIP stream handle.
typedef void* CUstream;

#define NT_OP SFB_NT_OP
#define NN_OP SFB_NN_OP
#define TN_OP SFB_TN_OP

#define CEIL_DIV(x, y) (((x) + (y)-1) / (y))
#define THREAD_POW2(x) (x <= 32 ? 32 : x <= 64 ? 64 : x <= 128 ? 128 : x <= 256 ? 256 : x <= 512 ? 512 : 1024)

inline void magicu64(uint d, uint& magic, uint& shift) { sfb_magicu64(d, &magic, &shift); }

namespace sfb_host {
template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static const int value = SFB_F32; };
template <> struct dtype_of<bhalf> { static const int value = SFB_BF16; };
inline const sfb_uint2* lut_cast(const uint2* p) { return reinterpret_cast<const sfb_uint2*>(p); }
// Last status returned by a wrapped launcher on this thread (the reference's launchers return only bool).
inline int& last_status() { static thread_local int status = SFB_OK; return status; }
inline bool ok(int status) { last_status() = status; return status == SFB_OK; }
}  // namespace sfb_host

#endif
