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
