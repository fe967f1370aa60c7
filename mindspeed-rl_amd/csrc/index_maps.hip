// Remove-padding index maps for gfx950: sequence-length scan, pack / unpack gathers, the
// padded-layout response window and the length mask.  Integer results are bit-exact with the
// per-sequence Python loops they replace; payloads are copied verbatim.
//
// Every map is written as a GATHER over the destination (each output element finds its source
// by a binary search in cu_seqlens_padded), so no atomics are needed, every output element is
// written exactly once, and results are deterministic.
#include "mrl_internal.h"

namespace {

constexpr int kBlock = 256;
constexpr int kScanBlock = 1024;

__device__ __forceinline__ int64_t load_index(const void* p, int dtype, int64_t i) {
    return dtype == MRL_I32 ? (int64_t) reinterpret_cast<const int32_t*>(p)[i]
                            : reinterpret_cast<const int64_t*>(p)[i];
}

// mask element != 0 counted as its integer value (torch's sum(dtype=int32) adds the values)
__device__ __forceinline__ int32_t mask_value(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case MRL_I64: return (int32_t) reinterpret_cast<const int64_t*>(p)[i];
        case MRL_I32: return reinterpret_cast<const int32_t*>(p)[i];
        case MRL_U8: return (int32_t) reinterpret_cast<const uint8_t*>(p)[i];
        default: return (int32_t) reinterpret_cast<const float*>(p)[i];
    }
}

// Row sums of the attention mask: one workgroup per sequence.
__global__ __launch_bounds__(kBlock) void mask_row_sum_kernel(const void* __restrict__ mask, int dtype,
                                                              int64_t width, int32_t* __restrict__ seqlens) {
    __shared__ int32_t part[kBlock / 64];
    const int64_t i = blockIdx.x;
    int32_t acc = 0;
    for (int64_t j = threadIdx.x; j < width; j += kBlock) acc += mask_value(mask, dtype, i * width + j);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        int32_t s = 0;
        for (int w = 0; w < kBlock / 64; ++w) s += part[w];
        seqlens[i] = s;
    }
}

// Inclusive scan of the aligned lengths by ONE workgroup, chunk by chunk; int32 wrap-around
// arithmetic like an int32 tensor assignment.
__global__ __launch_bounds__(kScanBlock) void cu_seqlens_kernel(const int32_t* __restrict__ seqlens,
                                                                int64_t batch, int32_t align,
                                                                int32_t* __restrict__ cu,
                                                                int64_t* __restrict__ total) {
    __shared__ uint32_t wave_sum[kScanBlock / 64];
    __shared__ uint32_t carry_s;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        carry_s = 0;
        cu[0] = 0;
    }
    __syncthreads();
    for (int64_t base = 0; base < batch; base += kScanBlock) {
        const int64_t i = base + tid;
        uint32_t v = 0;
        if (i < batch) {
            const int32_t len = seqlens[i];
            // python's % takes the sign of the divisor: (align - len % align) % align
            int32_t rem = len % align;
            if (rem < 0) rem += align;
            const int32_t pad = (align - rem) % align;
            v = (uint32_t)(len + pad);
        }
        uint32_t x = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(x, off, 64);
            if (lane >= off) x += o;
        }
        if (lane == 63) wave_sum[wave] = x;
        __syncthreads();
        uint32_t prefix = carry_s;
        for (int w = 0; w < wave; ++w) prefix += wave_sum[w];
        if (i < batch) cu[i + 1] = (int32_t)(prefix + x);
        __syncthreads();
        if (tid == kScanBlock - 1) carry_s = prefix + x;
        __syncthreads();
    }
    if (tid == 0 && total != nullptr) *total = (int64_t)(int32_t)carry_s;
}

// Largest i in [0, batch) with cu[i] <= t.  cu is non-decreasing, so for 0 <= t < cu[batch] this
// is the one sequence whose padded range covers t (cu[i] <= t < cu[i+1]); sequences of padded
// length zero are never returned.
__device__ __forceinline__ int find_sequence(const int32_t* __restrict__ cu, int batch, int64_t t) {
    int lo = 0, hi = batch;  // invariant: cu[lo] <= t, answer in [lo, hi)
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)cu[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void pack_rows_kernel(const T* __restrict__ src, T* __restrict__ dst,
                                                           const T* __restrict__ src2, T* __restrict__ dst2,
                                                           int batch, int64_t width,
                                                           const int32_t* __restrict__ seqlens,
                                                           const int32_t* __restrict__ cu, int64_t total,
                                                           int32_t* __restrict__ pos) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total) return;
    T a = 0, b = 0;
    int32_t p = 0;
    if (batch > 0 && t < (int64_t)cu[batch]) {
        const int i = find_sequence(cu, batch, t);
        const int64_t j = t - (int64_t)cu[i];
        p = (int32_t)j;
        if (j < (int64_t)seqlens[i] && j < width) {
            a = src[(int64_t)i * width + j];
            if (src2) b = src2[(int64_t)i * width + j];
        }
    }
    dst[t] = a;
    if (dst2) dst2[t] = b;
    if (pos) pos[t] = p;
}

// (start, n) of the window that postprocess_packed_seqs copies for sequence i
__device__ __forceinline__ void unpad_window(const int32_t* __restrict__ seqlens, const int32_t* __restrict__ cu,
                                             const void* __restrict__ prompt, int prompt_dtype, int i,
                                             int64_t& start, int64_t& n) {
    start = (int64_t)cu[i];
    n = (int64_t)seqlens[i];
    if (prompt != nullptr) {
        const int64_t skip = load_index(prompt, prompt_dtype, i) - 1;
        if (skip < n) {
            n -= skip + 1;
            start += skip;
        }
    }
}

// out[i, j, :] for one (i, j) per thread-group of `inner` elements; T is the element's storage type.
template <typename T>
__global__ __launch_bounds__(kBlock) void unpad_gather_kernel(const T* __restrict__ packed, int64_t total,
                                                              int64_t inner, const int32_t* __restrict__ seqlens,
                                                              const int32_t* __restrict__ cu,
                                                              const void* __restrict__ prompt, int prompt_dtype,
                                                              int64_t seq_len, int64_t n_out, T* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_out) return;
    const int64_t c = e % inner;
    const int64_t ij = e / inner;
    const int64_t j = ij % seq_len;
    const int i = (int)(ij / seq_len);
    int64_t start, n;
    unpad_window(seqlens, cu, prompt, prompt_dtype, i, start, n);
    T v = 0;
    const int64_t t = start + j;
    if (j < n && t >= 0 && t < total) v = packed[t * inner + c];
    out[e] = v;
}

__global__ __launch_bounds__(kBlock) void pad_scatter_kernel(const float* __restrict__ g_out, int batch,
                                                             int64_t seq_len, const int32_t* __restrict__ seqlens,
                                                             const int32_t* __restrict__ cu,
                                                             const void* __restrict__ prompt, int prompt_dtype,
                                                             int64_t total, float* __restrict__ g_packed) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total) return;
    float g = 0.f;
    if (batch > 0 && t < (int64_t)cu[batch]) {
        // windows of different sequences never overlap (each lies inside its own cu range as long as
        // prompt_length >= 1), so the covering sequence is the only candidate
        const int i = find_sequence(cu, batch, t);
        int64_t start, n;
        unpad_window(seqlens, cu, prompt, prompt_dtype, i, start, n);
        const int64_t j = t - start;
        if (j >= 0 && j < n && j < seq_len) g = g_out[(int64_t)i * seq_len + j];
    }
    g_packed[t] = g;
}

__device__ __forceinline__ void clamped_window(const void* __restrict__ window, int dtype, int64_t i,
                                               int64_t width, int64_t& lo, int64_t& hi) {
    lo = load_index(window, dtype, 2 * i);
    hi = load_index(window, dtype, 2 * i + 1);
    lo = lo < 0 ? 0 : (lo > width ? width : lo);
    hi = hi < 0 ? 0 : (hi > width ? width : hi);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void window_gather_kernel(const T* __restrict__ src, int64_t width,
                                                               int64_t inner, const void* __restrict__ window,
                                                               int window_dtype, int64_t out_len, T pad,
                                                               int64_t n_out, T* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_out) return;
    const int64_t c = e % inner;
    const int64_t ij = e / inner;
    const int64_t j = ij % out_len;
    const int64_t i = ij / out_len;
    int64_t lo, hi;
    clamped_window(window, window_dtype, i, width, lo, hi);
    T v = pad;
    if (j < hi - lo) v = src[(i * width + lo + j) * inner + c];
    out[e] = v;
}

__global__ __launch_bounds__(kBlock) void window_scatter_kernel(const float* __restrict__ g_out, int64_t width,
                                                                const void* __restrict__ window, int window_dtype,
                                                                int64_t out_len, int64_t n_src,
                                                                float* __restrict__ g_src) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_src) return;
    const int64_t s = e % width;
    const int64_t i = e / width;
    int64_t lo, hi;
    clamped_window(window, window_dtype, i, width, lo, hi);
    const int64_t j = s - lo;
    float g = 0.f;
    if (j >= 0 && s < hi && j < out_len) g = g_out[i * out_len + j];
    g_src[e] = g;
}

__global__ __launch_bounds__(kBlock) void generate_mask_kernel(const void* __restrict__ lengths, int dtype,
                                                               int64_t width, int64_t n_out,
                                                               int64_t* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_out) return;
    const int64_t j = e % width;
    const int64_t i = e / width;
    out[e] = (j < load_index(lengths, dtype, i)) ? 1 : 0;
}


// ----------------------------------------------------------------------------- ragged <-> padded
// Exclusive scan of clamped row lengths plus their maximum, by one workgroup:
//   cu[0] = 0, cu[i+1] = cu[i] + len_i;  info[0] = cu[batch];  info[1] = max_i len_i rounded up to `multiple`.
// With width > 0, len_i follows truncate_rows: clamped to [0, width]; with left_pad a zero index keeps the
// whole row (python's x[-0:]); and, if `rows` is given, 0 where index_i == 0 and rows[i, 0] == -1.
template <typename T>
__global__ __launch_bounds__(kScanBlock) void ragged_layout_kernel(const void* __restrict__ lengths, int ldtype,
                                                                   int64_t batch, int64_t multiple,
                                                                   const T* __restrict__ rows, int64_t width,
                                                                   int left_pad, int32_t* __restrict__ eff_len,
                                                                   int32_t* __restrict__ cu, int64_t* __restrict__ info) {
    __shared__ uint32_t wave_sum[kScanBlock / 64];
    __shared__ int32_t wave_max[kScanBlock / 64];
    __shared__ uint32_t carry_s;
    __shared__ int32_t max_s;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        carry_s = 0;
        max_s = 0;
        cu[0] = 0;
    }
    __syncthreads();
    for (int64_t base = 0; base < batch; base += kScanBlock) {
        const int64_t i = base + tid;
        int32_t len = 0;
        if (i < batch) {
            int64_t n = load_index(lengths, ldtype, i);
            if (width > 0) {
                if (rows != nullptr && n == 0 && rows[i * width] == (T)-1) n = 0;
                else if (left_pad && n == 0) n = width;
                if (n > width) n = width;
            }
            if (n < 0) n = 0;
            len = (int32_t)n;
            if (eff_len) eff_len[i] = len;
        }
        uint32_t x = (uint32_t)len;
        int32_t mx = len;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(x, off, 64);
            if (lane >= off) x += o;
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mx = max(mx, __shfl_xor(mx, off, 64));
        if (lane == 63) wave_sum[wave] = x;
        if (lane == 0) wave_max[wave] = mx;
        __syncthreads();
        uint32_t prefix = carry_s;
        for (int w = 0; w < wave; ++w) prefix += wave_sum[w];
        if (i < batch) cu[i + 1] = (int32_t)(prefix + x);
        __syncthreads();
        if (tid == kScanBlock - 1) carry_s = prefix + x;
        if (tid == 0) {
            int32_t m = max_s;
            for (int w = 0; w < kScanBlock / 64; ++w) m = max(m, wave_max[w]);
            max_s = m;
        }
        __syncthreads();
    }
    if (tid == 0) {
        info[0] = (int64_t)(int32_t)carry_s;
        int64_t m = max_s;
        if (multiple > 1) m = (m + multiple - 1) / multiple * multiple;
        info[1] = m;
    }
}

// out[i, d, j] = flat[d, cu[i] + j] for j < len_i, pad elsewhere (unpack_pad_experience)
template <typename T>
__global__ __launch_bounds__(kBlock) void ragged_to_padded_kernel(const T* __restrict__ flat, int64_t first_dim,
                                                                  int64_t flat_stride, const int32_t* __restrict__ cu,
                                                                  int64_t width, T pad, int64_t n_out,
                                                                  T* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_out) return;
    const int64_t j = e % width;
    const int64_t d = (e / width) % first_dim;
    const int64_t i = e / (width * first_dim);
    const int64_t lo = cu[i], n = (int64_t)cu[i + 1] - lo;
    out[e] = j < n ? flat[d * flat_stride + lo + j] : pad;
}

// flat[cu[i] + j] = padded[i, j] (or padded[i, width - len_i + j] when the rows are left-padded)
template <typename T>
__global__ __launch_bounds__(kBlock) void padded_to_ragged_kernel(const T* __restrict__ padded, int batch,
                                                                  int64_t width, const int32_t* __restrict__ cu,
                                                                  int left_pad, int64_t total, T* __restrict__ flat) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total) return;
    const int i = find_sequence(cu, batch, t);
    const int64_t j = t - cu[i];
    const int64_t n = (int64_t)cu[i + 1] - cu[i];
    flat[t] = padded[(int64_t)i * width + (left_pad ? width - n + j : j)];
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + kBlock - 1) / kBlock); }

int check_elems(const char* fn, int64_t n) {
    MRL_REQUIRE(n >= 0, MRL_ERR_INVALID_ARG, "%s: negative element count", fn);
    MRL_REQUIRE((n + kBlock - 1) / kBlock <= 0x7fffffffLL, MRL_ERR_UNSUPPORTED, "%s: %lld elements exceed the grid limit",
                fn, (long long)n);
    return MRL_OK;
}

// first[i] = smallest j with rows[i, j] == value, or width if there is none; `extra` is added to a
// found index (clamped to width).  One wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void first_match_kernel(const T* __restrict__ rows, int64_t batch, int64_t width,
                                                          T value, int extra, int32_t* __restrict__ first) {
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= batch) return;
    const int lane = threadIdx.x & 63;
    const T* row = rows + i * width;
    int64_t best = width;
    for (int64_t j0 = 0; j0 < width && best == width; j0 += 64) {       // `best` is uniform after the reduction
        const int64_t j = j0 + lane;
        int64_t mine = (j < width && row[j] == value) ? j : width;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const int64_t o = __shfl_xor(mine, off, 64);
            mine = o < mine ? o : mine;
        }
        best = mine;
    }
    if (lane == 0) {
        int64_t n = best < width ? best + extra : width;
        first[i] = (int32_t)(n < width ? n : width);
    }
}

}  // namespace

extern "C" int mrl_pack_index_build(const void* attention_mask, int mask_dtype, int64_t batch, int64_t width,
                                    int64_t align, int32_t* seqlens, int32_t* cu_seqlens_padded, int64_t* total,
                                    void* stream) {
    const char* fn = "mrl_pack_index_build";
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20), MRL_ERR_INVALID_ARG, "%s: batch=%lld out of [0, 2^20]", fn,
                (long long)batch);
    MRL_REQUIRE(align >= 1 && align <= (1 << 20), MRL_ERR_INVALID_ARG, "%s: align=%lld out of [1, 2^20]", fn,
                (long long)align);
    MRL_REQUIRE(cu_seqlens_padded != nullptr, MRL_ERR_INVALID_ARG, "%s: cu_seqlens_padded is NULL", fn);
    MRL_REQUIRE(batch == 0 || seqlens != nullptr, MRL_ERR_INVALID_ARG, "%s: seqlens is NULL", fn);
    MRL_REQUIRE(mrl::aligned(seqlens, 4) && mrl::aligned(cu_seqlens_padded, 4) && mrl::aligned(total, 8),
                MRL_ERR_MISALIGNED, "%s: misaligned integer buffer", fn);
    hipStream_t s = mrl::as_stream(stream);
    if (attention_mask != nullptr && batch > 0) {
        const int mb = mrl::mask_dtype_bytes(mask_dtype);
        MRL_REQUIRE(mb != 0, MRL_ERR_UNSUPPORTED, "%s: mask dtype %d (want F32, I32, I64 or U8)", fn, mask_dtype);
        MRL_REQUIRE(width >= 0, MRL_ERR_INVALID_ARG, "%s: width=%lld", fn, (long long)width);
        MRL_REQUIRE(mrl::aligned(attention_mask, mb), MRL_ERR_MISALIGNED, "%s: mask misaligned", fn);
        hipLaunchKernelGGL(mask_row_sum_kernel, dim3((unsigned)batch), dim3(kBlock), 0, s, attention_mask,
                           mask_dtype, width, seqlens);
        int rc = mrl::check_launch(fn);
        if (rc != MRL_OK) return rc;
    }
    hipLaunchKernelGGL(cu_seqlens_kernel, dim3(1), dim3(kScanBlock), 0, s, (const int32_t*)seqlens, batch,
                       (int32_t)align, cu_seqlens_padded, total);
    return mrl::check_launch(fn);
}

extern "C" int mrl_pack_rows(const void* src, void* dst, const void* src2, void* dst2, int elem_bytes,
                             int64_t batch, int64_t width, const int32_t* seqlens,
                             const int32_t* cu_seqlens_padded, int64_t total, int32_t* position_ids,
                             void* stream) {
    const char* fn = "mrl_pack_rows";
    MRL_REQUIRE(elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED, "%s: elem_bytes=%d (want 4 or 8)", fn,
                elem_bytes);
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20) && width >= 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld",
                fn, (long long)batch, (long long)width);
    int rc = check_elems(fn, total);
    if (rc != MRL_OK) return rc;
    if (total == 0) return MRL_OK;
    MRL_REQUIRE(dst != nullptr && cu_seqlens_padded != nullptr, MRL_ERR_INVALID_ARG, "%s: NULL dst or cu", fn);
    MRL_REQUIRE(batch == 0 || (src != nullptr && seqlens != nullptr), MRL_ERR_INVALID_ARG, "%s: NULL src or seqlens",
                fn);
    MRL_REQUIRE((src2 == nullptr) == (dst2 == nullptr), MRL_ERR_INVALID_ARG, "%s: src2 and dst2 go together", fn);
    MRL_REQUIRE(mrl::aligned(src, elem_bytes) && mrl::aligned(dst, elem_bytes) && mrl::aligned(src2, elem_bytes) &&
                    mrl::aligned(dst2, elem_bytes) && mrl::aligned(position_ids, 4),
                MRL_ERR_MISALIGNED, "%s: misaligned buffer", fn);
    hipStream_t s = mrl::as_stream(stream);
    if (elem_bytes == 4) {
        hipLaunchKernelGGL(pack_rows_kernel<int32_t>, dim3(blocks_for(total)), dim3(kBlock), 0, s,
                           (const int32_t*)src, (int32_t*)dst, (const int32_t*)src2, (int32_t*)dst2, (int)batch,
                           width, seqlens, cu_seqlens_padded, total, position_ids);
    } else {
        hipLaunchKernelGGL(pack_rows_kernel<int64_t>, dim3(blocks_for(total)), dim3(kBlock), 0, s,
                           (const int64_t*)src, (int64_t*)dst, (const int64_t*)src2, (int64_t*)dst2, (int)batch,
                           width, seqlens, cu_seqlens_padded, total, position_ids);
    }
    return mrl::check_launch(fn);
}

extern "C" int mrl_unpad_gather(const void* packed, int elem_bytes, int64_t total, int64_t inner,
                                const int32_t* seqlens, const int32_t* cu_seqlens_padded,
                                const void* prompt_length, int prompt_dtype, int64_t batch, int64_t seq_len,
                                void* out, void* stream) {
    const char* fn = "mrl_unpad_gather";
    MRL_REQUIRE(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED,
                "%s: elem_bytes=%d (want 2, 4 or 8)", fn, elem_bytes);
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20) && seq_len >= 0 && inner >= 1 && total >= 0, MRL_ERR_INVALID_ARG,
                "%s: batch=%lld seq_len=%lld inner=%lld total=%lld", fn, (long long)batch, (long long)seq_len,
                (long long)inner, (long long)total);
    MRL_REQUIRE(prompt_length == nullptr || mrl::int_dtype_bytes(prompt_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: prompt_length dtype %d (want I32 or I64)", fn, prompt_dtype);
    const int64_t n_out = batch * seq_len * inner;
    int rc = check_elems(fn, n_out);
    if (rc != MRL_OK) return rc;
    if (n_out == 0) return MRL_OK;
    MRL_REQUIRE(out && seqlens && cu_seqlens_padded && (packed || total == 0), MRL_ERR_INVALID_ARG,
                "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(packed, elem_bytes) && mrl::aligned(out, elem_bytes), MRL_ERR_MISALIGNED,
                "%s: misaligned buffer", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid(blocks_for(n_out)), block(kBlock);
#define MRL_UNPAD(T)                                                                                             \
    hipLaunchKernelGGL(unpad_gather_kernel<T>, grid, block, 0, s, (const T*)packed, total, inner, seqlens,        \
                       cu_seqlens_padded, prompt_length, prompt_dtype, seq_len, n_out, (T*)out)
    if (elem_bytes == 2) MRL_UNPAD(uint16_t);
    else if (elem_bytes == 4) MRL_UNPAD(uint32_t);
    else MRL_UNPAD(uint64_t);
#undef MRL_UNPAD
    return mrl::check_launch(fn);
}

extern "C" int mrl_pad_scatter(const float* g_out, int64_t batch, int64_t seq_len, const int32_t* seqlens,
                               const int32_t* cu_seqlens_padded, const void* prompt_length, int prompt_dtype,
                               int64_t total, float* g_packed, void* stream) {
    const char* fn = "mrl_pad_scatter";
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20) && seq_len >= 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld seq_len=%lld",
                fn, (long long)batch, (long long)seq_len);
    MRL_REQUIRE(prompt_length == nullptr || mrl::int_dtype_bytes(prompt_dtype) != 0, MRL_ERR_UNSUPPORTED,
                "%s: prompt_length dtype %d (want I32 or I64)", fn, prompt_dtype);
    int rc = check_elems(fn, total);
    if (rc != MRL_OK) return rc;
    if (total == 0) return MRL_OK;
    MRL_REQUIRE(g_packed && cu_seqlens_padded && (batch == 0 || (g_out && seqlens)), MRL_ERR_INVALID_ARG,
                "%s: NULL pointer", fn);
    hipLaunchKernelGGL(pad_scatter_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, mrl::as_stream(stream), g_out,
                       (int)batch, seq_len, seqlens, cu_seqlens_padded, prompt_length, prompt_dtype, total, g_packed);
    return mrl::check_launch(fn);
}

extern "C" int mrl_window_gather(const void* src, int elem_bytes, int64_t batch, int64_t width, int64_t inner,
                                 const void* window, int window_dtype, int64_t out_len, uint64_t pad_bits,
                                 void* out, void* stream) {
    const char* fn = "mrl_window_gather";
    MRL_REQUIRE(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED,
                "%s: elem_bytes=%d (want 2, 4 or 8)", fn, elem_bytes);
    MRL_REQUIRE(batch >= 0 && width >= 0 && inner >= 1 && out_len >= 0, MRL_ERR_INVALID_ARG,
                "%s: batch=%lld width=%lld inner=%lld out_len=%lld", fn, (long long)batch, (long long)width,
                (long long)inner, (long long)out_len);
    MRL_REQUIRE(mrl::int_dtype_bytes(window_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: window dtype %d (want I32 or I64)",
                fn, window_dtype);
    const int64_t n_out = batch * out_len * inner;
    int rc = check_elems(fn, n_out);
    if (rc != MRL_OK) return rc;
    if (n_out == 0) return MRL_OK;
    MRL_REQUIRE(out && window && (src || width == 0), MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(src, elem_bytes) && mrl::aligned(out, elem_bytes), MRL_ERR_MISALIGNED,
                "%s: misaligned buffer", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid(blocks_for(n_out)), block(kBlock);
#define MRL_WIN(T)                                                                                          \
    hipLaunchKernelGGL(window_gather_kernel<T>, grid, block, 0, s, (const T*)src, width, inner, window,       \
                       window_dtype, out_len, (T)pad_bits, n_out, (T*)out)
    if (elem_bytes == 2) MRL_WIN(uint16_t);
    else if (elem_bytes == 4) MRL_WIN(uint32_t);
    else MRL_WIN(uint64_t);
#undef MRL_WIN
    return mrl::check_launch(fn);
}

extern "C" int mrl_window_scatter(const float* g_out, int64_t batch, int64_t width, const void* window,
                                  int window_dtype, int64_t out_len, float* g_src, void* stream) {
    const char* fn = "mrl_window_scatter";
    MRL_REQUIRE(batch >= 0 && width >= 0 && out_len >= 0, MRL_ERR_INVALID_ARG, "%s: negative size", fn);
    MRL_REQUIRE(mrl::int_dtype_bytes(window_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: window dtype %d (want I32 or I64)",
                fn, window_dtype);
    const int64_t n_src = batch * width;
    int rc = check_elems(fn, n_src);
    if (rc != MRL_OK) return rc;
    if (n_src == 0) return MRL_OK;
    MRL_REQUIRE(g_src && window && (g_out || out_len == 0), MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    hipLaunchKernelGGL(window_scatter_kernel, dim3(blocks_for(n_src)), dim3(kBlock), 0, mrl::as_stream(stream),
                       g_out, width, window, window_dtype, out_len, n_src, g_src);
    return mrl::check_launch(fn);
}

extern "C" int mrl_generate_mask(const void* lengths, int lengths_dtype, int64_t batch, int64_t width,
                                 int64_t* out, void* stream) {
    const char* fn = "mrl_generate_mask";
    MRL_REQUIRE(batch >= 0 && width >= 0, MRL_ERR_INVALID_ARG, "%s: negative size", fn);
    MRL_REQUIRE(mrl::int_dtype_bytes(lengths_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: lengths dtype %d (want I32 or I64)",
                fn, lengths_dtype);
    const int64_t n_out = batch * width;
    int rc = check_elems(fn, n_out);
    if (rc != MRL_OK) return rc;
    if (n_out == 0) return MRL_OK;
    MRL_REQUIRE(lengths && out, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    MRL_REQUIRE(mrl::aligned(out, 8), MRL_ERR_MISALIGNED, "%s: out misaligned", fn);
    hipLaunchKernelGGL(generate_mask_kernel, dim3(blocks_for(n_out)), dim3(kBlock), 0, mrl::as_stream(stream),
                       lengths, lengths_dtype, width, n_out, out);
    return mrl::check_launch(fn);
}

extern "C" int mrl_ragged_layout(const void* lengths, int lengths_dtype, int64_t batch, int64_t multiple,
                                 const void* rows, int elem_bytes, int64_t width, int left_pad, int32_t* eff_len,
                                 int32_t* cu, int64_t* info, void* stream) {
    const char* fn = "mrl_ragged_layout";
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20), MRL_ERR_INVALID_ARG, "%s: batch=%lld out of [0, 2^20]", fn,
                (long long)batch);
    MRL_REQUIRE(multiple >= 1, MRL_ERR_INVALID_ARG, "%s: multiple=%lld", fn, (long long)multiple);
    MRL_REQUIRE(mrl::int_dtype_bytes(lengths_dtype) != 0, MRL_ERR_UNSUPPORTED, "%s: lengths dtype %d (want I32 or I64)",
                fn, lengths_dtype);
    MRL_REQUIRE(cu != nullptr && info != nullptr && (batch == 0 || lengths != nullptr), MRL_ERR_INVALID_ARG,
                "%s: NULL pointer", fn);
    MRL_REQUIRE(width >= 0, MRL_ERR_INVALID_ARG, "%s: width=%lld", fn, (long long)width);
    MRL_REQUIRE(rows == nullptr || ((elem_bytes == 4 || elem_bytes == 8) && width >= 1), MRL_ERR_UNSUPPORTED,
                "%s: rows need 4- or 8-byte elements and width >= 1", fn);
    hipStream_t s = mrl::as_stream(stream);
    if (rows != nullptr && elem_bytes == 8) {
        hipLaunchKernelGGL(ragged_layout_kernel<int64_t>, dim3(1), dim3(kScanBlock), 0, s, lengths, lengths_dtype, batch,
                           multiple, (const int64_t*)rows, width, left_pad, eff_len, cu, info);
    } else {
        hipLaunchKernelGGL(ragged_layout_kernel<int32_t>, dim3(1), dim3(kScanBlock), 0, s, lengths, lengths_dtype, batch,
                           multiple, (const int32_t*)rows, width, left_pad, eff_len, cu, info);
    }
    return mrl::check_launch(fn);
}

extern "C" int mrl_ragged_to_padded(const void* flat, int elem_bytes, int64_t first_dim, int64_t flat_stride,
                                    const int32_t* cu, int64_t batch, int64_t width, uint64_t pad_bits, void* out,
                                    void* stream) {
    const char* fn = "mrl_ragged_to_padded";
    MRL_REQUIRE(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED,
                "%s: elem_bytes=%d (want 2, 4 or 8)", fn, elem_bytes);
    MRL_REQUIRE(batch >= 0 && width >= 0 && first_dim >= 1 && flat_stride >= 0, MRL_ERR_INVALID_ARG,
                "%s: batch=%lld width=%lld first_dim=%lld", fn, (long long)batch, (long long)width,
                (long long)first_dim);
    const int64_t n_out = batch * first_dim * width;
    int rc = check_elems(fn, n_out);
    if (rc != MRL_OK) return rc;
    if (n_out == 0) return MRL_OK;
    MRL_REQUIRE(out && cu && (flat || flat_stride == 0), MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid(blocks_for(n_out)), block(kBlock);
#define MRL_R2P(T)                                                                                             \
    hipLaunchKernelGGL(ragged_to_padded_kernel<T>, grid, block, 0, s, (const T*)flat, first_dim, flat_stride, cu, \
                       width, (T)pad_bits, n_out, (T*)out)
    if (elem_bytes == 2) MRL_R2P(uint16_t);
    else if (elem_bytes == 4) MRL_R2P(uint32_t);
    else MRL_R2P(uint64_t);
#undef MRL_R2P
    return mrl::check_launch(fn);
}

extern "C" int mrl_padded_to_ragged(const void* padded, int elem_bytes, int64_t batch, int64_t width,
                                    const int32_t* cu, int left_pad, int64_t total, void* flat, void* stream) {
    const char* fn = "mrl_padded_to_ragged";
    MRL_REQUIRE(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED,
                "%s: elem_bytes=%d (want 2, 4 or 8)", fn, elem_bytes);
    MRL_REQUIRE(batch >= 0 && batch <= (1LL << 20) && width >= 0, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn,
                (long long)batch, (long long)width);
    int rc = check_elems(fn, total);
    if (rc != MRL_OK) return rc;
    if (total == 0) return MRL_OK;
    MRL_REQUIRE(padded && cu && flat && batch > 0, MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    hipStream_t s = mrl::as_stream(stream);
    const dim3 grid(blocks_for(total)), block(kBlock);
#define MRL_P2R(T)                                                                                              \
    hipLaunchKernelGGL(padded_to_ragged_kernel<T>, grid, block, 0, s, (const T*)padded, (int)batch, width, cu, left_pad, \
                       total, (T*)flat)
    if (elem_bytes == 2) MRL_P2R(uint16_t);
    else if (elem_bytes == 4) MRL_P2R(uint32_t);
    else MRL_P2R(uint64_t);
#undef MRL_P2R
    return mrl::check_launch(fn);
}

extern "C" int mrl_first_match(const void* rows, int elem_bytes, int64_t batch, int64_t width, int64_t value, int extra,
                               int32_t* first, void* stream) {
    const char* fn = "mrl_first_match";
    MRL_REQUIRE(batch >= 0 && width >= 0 && width <= 0x7fffffffLL, MRL_ERR_INVALID_ARG, "%s: batch=%lld width=%lld", fn,
                (long long)batch, (long long)width);
    MRL_REQUIRE(elem_bytes == 4 || elem_bytes == 8, MRL_ERR_UNSUPPORTED, "%s: elem_bytes=%d (want 4 or 8)", fn, elem_bytes);
    MRL_REQUIRE(extra == 0 || extra == 1, MRL_ERR_INVALID_ARG, "%s: extra=%d", fn, extra);
    if (batch == 0) return MRL_OK;
    MRL_REQUIRE(first != nullptr && (rows != nullptr || width == 0), MRL_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    const dim3 grid((unsigned)((batch + 3) / 4)), block(256);
    hipStream_t s = mrl::as_stream(stream);
    if (elem_bytes == 8)
        hipLaunchKernelGGL(first_match_kernel<int64_t>, grid, block, 0, s, (const int64_t*)rows, batch, width, value, extra,
                           first);
    else
        hipLaunchKernelGGL(first_match_kernel<int32_t>, grid, block, 0, s, (const int32_t*)rows, batch, width,
                           (int32_t)value, extra, first);
    return mrl::check_launch(fn);
}
