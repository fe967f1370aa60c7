// Device-side building blocks shared by the vocabulary sweeps: element traits of the three
// logits dtypes (16-byte vector unpack / pack), the online-softmax statistics and their merge.
#pragma once

#include "mrl_internal.h"

namespace mrl_vocab {

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;
// Start value of the running maximum: finite, so that (z - max) never becomes inf - inf.
constexpr float kMaxInit = -1.0e30f;

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));

template <int DT>
struct Elem;

template <>
struct Elem<MRL_F32> {
    using T = float;
    static constexpr int kVec = 4;
    static __device__ __forceinline__ void unpack(const u32x4& v, float (&z)[kVec]) {
        z[0] = __uint_as_float(v.x);
        z[1] = __uint_as_float(v.y);
        z[2] = __uint_as_float(v.z);
        z[3] = __uint_as_float(v.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&z)[kVec]) {
        return mrl::make_u32x4(__float_as_uint(z[0]), __float_as_uint(z[1]), __float_as_uint(z[2]),
                          __float_as_uint(z[3]));
    }
    static __device__ __forceinline__ float load(const T* p) { return *p; }
    // the entry as loaded and its conversion, separately: a kernel that requests an entry long
    // before it needs it converts at the use, so that nothing waits at the request
    static __device__ __forceinline__ uint32_t load_bits(const T* p) { return __float_as_uint(*p); }
    static __device__ __forceinline__ float from_bits(uint32_t b) { return __uint_as_float(b); }
    static __device__ __forceinline__ void store(T* p, float v) { *p = v; }
    static __device__ __forceinline__ void buf_store(mrl::rsrc_t r, uint32_t byte_off, float v) {
        mrl::buf_store_b32(__float_as_uint(v), r, byte_off);
    }
};

template <>
struct Elem<MRL_BF16> {
    using T = uint16_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ void unpack(const u32x4& v, float (&z)[kVec]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            z[2 * i] = __uint_as_float(w[i] << 16);
            z[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        floatx2 f = {a, b};
        bf16x2 h = __builtin_convertvector(f, bf16x2);  // round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&z)[kVec]) {
        return mrl::make_u32x4(pack2(z[0], z[1]), pack2(z[2], z[3]), pack2(z[4], z[5]), pack2(z[6], z[7]));
    }
    static __device__ __forceinline__ float load(const T* p) { return __uint_as_float((uint32_t)(*p) << 16); }
    static __device__ __forceinline__ uint32_t load_bits(const T* p) { return *p; }
    static __device__ __forceinline__ float from_bits(uint32_t b) { return __uint_as_float(b << 16); }
    static __device__ __forceinline__ void store(T* p, float v) {
        __bf16 h = (__bf16)v;
        *p = __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ void buf_store(mrl::rsrc_t r, uint32_t byte_off, float v) {
        __bf16 h = (__bf16)v;
        mrl::buf_store_b16(__builtin_bit_cast(uint16_t, h), r, byte_off);
    }
};

template <>
struct Elem<MRL_F16> {
    using T = uint16_t;
    static constexpr int kVec = 8;
    static __device__ __forceinline__ void unpack(const u32x4& v, float (&z)[kVec]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            halfx2 h = __builtin_bit_cast(halfx2, w[i]);
            z[2 * i] = (float)h[0];
            z[2 * i + 1] = (float)h[1];
        }
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        floatx2 f = {a, b};
        halfx2 h = __builtin_convertvector(f, halfx2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&z)[kVec]) {
        return mrl::make_u32x4(pack2(z[0], z[1]), pack2(z[2], z[3]), pack2(z[4], z[5]), pack2(z[6], z[7]));
    }
    static __device__ __forceinline__ float load(const T* p) {
        return (float)__builtin_bit_cast(_Float16, *p);
    }
    static __device__ __forceinline__ uint32_t load_bits(const T* p) { return *p; }
    static __device__ __forceinline__ float from_bits(uint32_t b) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
    }
    static __device__ __forceinline__ void store(T* p, float v) {
        _Float16 h = (_Float16)v;
        *p = __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ void buf_store(mrl::rsrc_t r, uint32_t byte_off, float v) {
        _Float16 h = (_Float16)v;
        mrl::buf_store_b16(__builtin_bit_cast(uint16_t, h), r, byte_off);
    }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Online softmax statistics of a set of raw logits z (before temperature), with k = inv_T*log2e:
//   m = max z,  s = sum 2^((z-m) k),  u = sum 2^((z-m) k) z
struct Stats {
    float m, s, u;
};

template <bool kEntropy>
__device__ __forceinline__ void grow_max(Stats& st, float new_max, float k) {
    if (new_max > st.m) {
        const float scale = fast_exp2((st.m - new_max) * k);
        st.s *= scale;
        if (kEntropy) st.u *= scale;
        st.m = new_max;
    }
}

template <bool kEntropy>
__device__ __forceinline__ void add_one(Stats& st, float z, float k, float mk) {
    const float e = fast_exp2(__builtin_fmaf(z, k, -mk));
    st.s += e;
    if (kEntropy) st.u = __builtin_fmaf(e, z, st.u);
}

template <bool kEntropy>
__device__ __forceinline__ Stats merge(const Stats& a, const Stats& b, float k) {
    Stats r;
    r.m = fmaxf(a.m, b.m);
    const float fa = fast_exp2((a.m - r.m) * k);
    const float fb = fast_exp2((b.m - r.m) * k);
    r.s = a.s * fa + b.s * fb;
    r.u = kEntropy ? a.u * fa + b.u * fb : 0.f;
    return r;
}

// Wavefront shuffle reduction, then a cross-wavefront combine through LDS (kWaves entries).
// Every thread of the workgroup must call it; all return the workgroup total.
template <bool kEntropy, int kWaves>
__device__ __forceinline__ Stats block_reduce(Stats st, float k, Stats* lds) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        Stats o;
        o.m = __shfl_xor(st.m, off, 64);
        o.s = __shfl_xor(st.s, off, 64);
        o.u = kEntropy ? __shfl_xor(st.u, off, 64) : 0.f;
        st = merge<kEntropy>(st, o, k);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = st;
    __syncthreads();
    Stats r = lds[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) r = merge<kEntropy>(r, lds[w], k);
    return r;
}

}  // namespace mrl_vocab
