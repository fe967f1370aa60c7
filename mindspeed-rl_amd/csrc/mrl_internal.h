// Shared host-side helpers of libmrl_hip.so: status codes, the per-thread error message,
// argument checks and launch checking.  Not part of the public ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "mrl_hip.h"

// 16-byte vector usable with the nontemporal load/store builtins.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace mrl {

__host__ __device__ inline u32x4 make_u32x4(unsigned a, unsigned b, unsigned c, unsigned d) {
    u32x4 v = {a, b, c, d};
    return v;
}

// Raw buffer access with hardware range checking: a load at a byte offset at or beyond `bytes`
// returns zero and a store there is dropped, so the tail of a row needs no branch.  Branch-free
// bodies matter on gfx9: with a branch around every access the compiler can no longer count the
// accesses in flight and waits for ALL of them (vmcnt(0)) before each use - and stores count too.
// `base` must be uniform over the wavefront.  Accesses carry the non-temporal hint.
#if defined(__HIP_DEVICE_COMPILE__)
using rsrc_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load_nt(rsrc_t r, uint32_t byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 2);
}
// a vector at lane offset + wavefront-uniform offset, default cache policy (data that other CUs read too)
__device__ __forceinline__ u32x4 buf_load(rsrc_t r, uint32_t lane_byte_off, uint32_t uniform_byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_byte_off, (int)uniform_byte_off, 0);
}
__device__ __forceinline__ void buf_store_nt(u32x4 v, rsrc_t r, uint32_t byte_off) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)byte_off, 0, 2);
}
// single entries, same cache policy as the vectors
__device__ __forceinline__ void buf_store_b16(uint16_t v, rsrc_t r, uint32_t byte_off) {
    __builtin_amdgcn_raw_buffer_store_b16((short)v, r, (int)byte_off, 0, 2);
}
__device__ __forceinline__ void buf_store_b32(uint32_t v, rsrc_t r, uint32_t byte_off) {
    __builtin_amdgcn_raw_buffer_store_b32(v, r, (int)byte_off, 0, 2);
}
// device-scope fetch-and-add through a descriptor: lanes whose offset is outside the range take no
// part (and get 0 back), so "one lane of the workgroup" needs no branch around the instruction
__device__ __forceinline__ uint32_t buf_atomic_add_u32(rsrc_t r, uint32_t byte_off, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32((int)v, r, (int)byte_off, 0, 0);
}
#else   // the host pass only has to parse the kernels
struct rsrc_t {};
__device__ inline rsrc_t make_rsrc(const void*, uint32_t) { return rsrc_t(); }
__device__ inline u32x4 buf_load_nt(rsrc_t, uint32_t) { return make_u32x4(0, 0, 0, 0); }
__device__ inline u32x4 buf_load(rsrc_t, uint32_t, uint32_t) { return make_u32x4(0, 0, 0, 0); }
__device__ inline void buf_store_nt(u32x4, rsrc_t, uint32_t) {}
__device__ inline void buf_store_b16(uint16_t, rsrc_t, uint32_t) {}
__device__ inline void buf_store_b32(uint32_t, rsrc_t, uint32_t) {}
__device__ inline uint32_t buf_atomic_add_u32(rsrc_t, uint32_t, uint32_t) { return 0; }
#endif

// Single IEEE operations that stay single: HIP compiles with floating-point contraction on, and its
// __fadd_rn / __fmul_rn are plain operators, so `a + b * c` (also across inlined calls) becomes one
// fused multiply-add with a single rounding.  Where a kernel has to reproduce the separately rounded
// arithmetic of numpy or of a torch CPU loop bit for bit, it goes through these.
template <typename F>
__host__ __device__ __forceinline__ F add_rn(F a, F b) {
#pragma clang fp contract(off)
    return a + b;
}
template <typename F>
__host__ __device__ __forceinline__ F sub_rn(F a, F b) {
#pragma clang fp contract(off)
    return a - b;
}
template <typename F>
__host__ __device__ __forceinline__ F mul_rn(F a, F b) {
#pragma clang fp contract(off)
    return a * b;
}

// Stores a printf-style message for mrl_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int float_dtype_bytes(int dt) {
    switch (dt) {
        case MRL_F32: return 4;
        case MRL_BF16: return 2;
        case MRL_F16: return 2;
        default: return 0;
    }
}

inline int int_dtype_bytes(int dt) {
    switch (dt) {
        case MRL_I32: return 4;
        case MRL_I64: return 8;
        default: return 0;
    }
}

inline int mask_dtype_bytes(int dt) {
    switch (dt) {
        case MRL_F32: return 4;
        case MRL_I32: return 4;
        case MRL_I64: return 8;
        case MRL_U8: return 1;
        default: return 0;
    }
}

// Call right after a kernel launch: turns a rejected launch into MRL_ERR_LAUNCH.
inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MRL_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return MRL_OK;
}

}  // namespace mrl

#define MRL_REQUIRE(cond, code, ...)                   \
    do {                                               \
        if (!(cond)) return mrl::fail(code, __VA_ARGS__); \
    } while (0)
