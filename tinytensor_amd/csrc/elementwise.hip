// elementwise.hip — strided view -> dense copy (the `identity` op behind Tensor::contiguous()/clone(),
// tinytensor/tensor/tensor.cpp:583-596, CPU form tinytensor/tensor/backend/cpu/unary.cpp:26-58 with the
// index map of tinytensor/tensor/backend/common/util.h:18-34).  The GEMM kernels never need it (they
// read views in place); it exists for the callers around them (reshape of a non-dense view, conv's
// grad_output) and moves raw bytes, so one kernel per element size serves every dtype.
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace ttamd {
namespace {

constexpr int kMaxDims = 8;
struct ViewDesc {
    int64_t shape[kMaxDims];
    int64_t stride[kMaxDims];
    int ndim;
};

template <typename W>
__global__ void __launch_bounds__(256) contiguous_kernel(const W *__restrict__ src, W *__restrict__ dst, ViewDesc v,
                                                        int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step) {
        int64_t rank = i, flat = 0;
        for (int d = v.ndim - 1; d >= 0; --d) {
            flat += (rank % v.shape[d]) * v.stride[d];
            rank /= v.shape[d];
        }
        dst[i] = src[flat];
    }
}

// Dense view: a plain copy, 16 bytes per lane.
typedef uint32_t copy16_t __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) copy16_kernel(const copy16_t *__restrict__ src, copy16_t *__restrict__ dst, int64_t nvec) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step)
        dst[i] = __builtin_nontemporal_load(src + i);  // read once
}

// Transposing copy for a view whose unit-stride dimension `fast` is not the last one (a permuted tensor): 64 x 64
// tiles over (fast, last) go through LDS so that both the reads (along `fast`) and the writes (along the last
// dimension) are coalesced.  The remaining dimensions are folded into the tile index.
struct TransposeDesc {
    ViewDesc outer;              // the dimensions other than `fast` and the last, with the source strides
    int64_t outer_dst[kMaxDims];  // their strides in the dense result
    int64_t rows, cols;          // extent of `fast` and of the last dimension
    int64_t src_col_stride;      // source stride of the last dimension (the `fast` stride is 1)
    int64_t dst_row_stride;      // dense stride of `fast` in the result (the last dimension's is 1)
    int tiles_r, tiles_c;
};

template <typename W>
__global__ void __launch_bounds__(256) transpose_copy_kernel(const W *__restrict__ src, W *__restrict__ dst, TransposeDesc t) {
    __shared__ W tile[64][65];
    int64_t id = blockIdx.x;
    const int tc = static_cast<int>(id % t.tiles_c);
    id /= t.tiles_c;
    const int tr = static_cast<int>(id % t.tiles_r);
    int64_t rank = id / t.tiles_r, s_off = 0, d_off = 0;
    for (int d = t.outer.ndim - 1; d >= 0; --d) {
        const int64_t i = rank % t.outer.shape[d];
        rank /= t.outer.shape[d];
        s_off += i * t.outer.stride[d];
        d_off += i * t.outer_dst[d];
    }
    const int64_t r0 = static_cast<int64_t>(tr) * 64, c0 = static_cast<int64_t>(tc) * 64;
    const int lane = threadIdx.x % 64, group = threadIdx.x / 64;
    const W *sp = src + s_off + (r0 + lane) + (c0 + group) * t.src_col_stride;
    W *dp = dst + d_off + (r0 + group) * t.dst_row_stride + (c0 + lane);
    if (r0 + 64 <= t.rows && c0 + 64 <= t.cols) {  // interior tile: 16 independent loads per lane, no bounds tests
        W v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = __builtin_nontemporal_load(sp + 4 * i * t.src_col_stride);  // read once
#pragma unroll
        for (int i = 0; i < 16; ++i) tile[group + 4 * i][lane] = v[i];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 16; ++i) dp[4 * i * t.dst_row_stride] = tile[lane][group + 4 * i];
        return;
    }
    // read: lanes run along `fast` (unit source stride)
    for (int c = group; c < 64; c += 4)
        if (r0 + lane < t.rows && c0 + c < t.cols) tile[c][lane] = sp[(c - group) * t.src_col_stride];
    __syncthreads();
    // write: lanes run along the last dimension (unit result stride)
    for (int r = group; r < 64; r += 4)
        if (r0 + r < t.rows && c0 + lane < t.cols) dp[(r - group) * t.dst_row_stride] = tile[lane][r];
}

template <typename W>
ttamd_status launch_contiguous(const void *src, void *dst, const ViewDesc &v, int64_t numel, hipStream_t stream) {
    // dense: plain copy
    bool dense = true;
    {
        int64_t expect = 1;
        for (int d = v.ndim - 1; d >= 0; --d) {
            if (v.shape[d] != 1 && v.stride[d] != expect) dense = false;
            expect *= v.shape[d];
        }
    }
    if (dense) {
        const int64_t bytes = numel * static_cast<int64_t>(sizeof(W));
        int64_t done = 0;
        if (reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 && bytes >= 16) {
            const int64_t nvec = bytes / 16;
            int64_t blocks = (nvec + 255) / 256;  // one vector per lane; the loop only runs again beyond 2^22 workgroups
            if (blocks > (1 << 22)) blocks = 1 << 22;
            copy16_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(static_cast<const copy16_t *>(src), static_cast<copy16_t *>(dst), nvec);
            done = nvec * 16 / static_cast<int64_t>(sizeof(W));
        }
        if (done < numel) {
            ViewDesc flat{};
            flat.ndim = 1;
            flat.shape[0] = numel - done;
            flat.stride[0] = 1;
            contiguous_kernel<W><<<dim3(1), dim3(256), 0, stream>>>(static_cast<const W *>(src) + done, static_cast<W *>(dst) + done, flat, numel - done);
        }
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    }
    // permuted: the last dimension is strided and another one has unit stride
    const int last = v.ndim - 1;
    int fast = -1;
    if (v.ndim >= 2 && v.stride[last] != 1 && v.shape[last] >= 16)
        for (int d = 0; d < last; ++d)
            if (v.stride[d] == 1 && v.shape[d] >= 16) fast = d;
    if (fast >= 0) {
        TransposeDesc t{};
        int64_t dense_stride[kMaxDims];
        int64_t expect = 1;
        for (int d = last; d >= 0; --d) {
            dense_stride[d] = expect;
            expect *= v.shape[d];
        }
        int64_t outer_count = 1;
        for (int d = 0; d < last; ++d) {
            if (d == fast) continue;
            t.outer.shape[t.outer.ndim] = v.shape[d];
            t.outer.stride[t.outer.ndim] = v.stride[d];
            t.outer_dst[t.outer.ndim] = dense_stride[d];
            ++t.outer.ndim;
            outer_count *= v.shape[d];
        }
        t.rows = v.shape[fast];
        t.cols = v.shape[last];
        t.src_col_stride = v.stride[last];
        t.dst_row_stride = dense_stride[fast];
        const int64_t tiles_r = (t.rows + 63) / 64, tiles_c = (t.cols + 63) / 64;
        const int64_t blocks = tiles_r * tiles_c * outer_count;
        if (tiles_r <= 0x7fffffff && tiles_c <= 0x7fffffff && blocks <= 0x7fffffff) {
            t.tiles_r = static_cast<int>(tiles_r);
            t.tiles_c = static_cast<int>(tiles_c);
            transpose_copy_kernel<W><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(static_cast<const W *>(src), static_cast<W *>(dst), t);
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        }
    }
    int64_t blocks = (numel + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    contiguous_kernel<W><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(static_cast<const W *>(src),
                                                                                       static_cast<W *>(dst), v, numel);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}


// ---------------------------------------------------------------------------------------------
// Elementwise set that an MLP training step needs around its GEMMs (tinytensor/tensor/backend_base.h:
// add/sub/mul/div/pow/maximum/minimum, lt/le/gt/ge/eq/ne, relu & friends, where, sum, full).  Operands are
// strided views of ONE shape (the frontend has already broadcast with expand(), include/tt/tensor.h:600);
// results are dense.  Functors follow tinytensor/tensor/backend/common/kernel/binary.hpp:20-140.

__device__ __forceinline__ int64_t flat_of(int64_t rank, const ViewDesc &v) {
    int64_t flat = 0;
    for (int d = v.ndim - 1; d >= 0; --d) {
        flat += (rank % v.shape[d]) * v.stride[d];
        rank /= v.shape[d];
    }
    return flat;
}

enum { BIN_ADD = 0, BIN_SUB, BIN_MUL, BIN_DIV, BIN_POW, BIN_MAXIMUM, BIN_MINIMUM, BIN_LT, BIN_LE, BIN_GT, BIN_GE, BIN_EQ, BIN_NE, BIN_COUNT };
enum { UN_RELU = 0, UN_NEGATE, UN_ABS, UN_SQRT, UN_EXP, UN_LOG, UN_SIGMOID, UN_TANH, UN_COUNT };

template <typename T>
__device__ __forceinline__ T pow_of(T a, T b) {
    if constexpr (std::is_floating_point_v<T>) {
        if (b == T(2)) return a * a;  // exact square, as a correctly rounded pow would give
        return pow(a, b);
    } else {
        // integer power by squaring with wrap-around; negative exponents follow std::pow's real result truncated
        using U = std::make_unsigned_t<T>;
        if (b < T(0)) return a == T(1) ? T(1) : (a == T(-1) ? ((b & 1) ? T(-1) : T(1)) : T(0));
        U base = static_cast<U>(a), r = 1;
        U e = static_cast<U>(b);
        while (e) {
            if (e & 1) r *= base;
            base *= base;
            e >>= 1;
        }
        return static_cast<T>(r);
    }
}

template <typename T, int OP>
__device__ __forceinline__ auto binary_apply(T a, T b) {
    if constexpr (OP == BIN_ADD) return static_cast<T>(a + b);
    else if constexpr (OP == BIN_SUB) return static_cast<T>(a - b);
    else if constexpr (OP == BIN_MUL) return static_cast<T>(a * b);
    else if constexpr (OP == BIN_DIV) {
        if constexpr (std::is_integral_v<T>) return static_cast<T>(b == T(0) ? T(0) : a / b);  // no trap on the device
        else return static_cast<T>(a / b);
    }
    else if constexpr (OP == BIN_POW) return pow_of<T>(a, b);
    else if constexpr (OP == BIN_MAXIMUM) return (a > b) ? a : b;
    else if constexpr (OP == BIN_MINIMUM) return (a < b) ? a : b;
    else if constexpr (OP == BIN_LT) return static_cast<uint8_t>(a < b);
    else if constexpr (OP == BIN_LE) return static_cast<uint8_t>(a <= b);
    else if constexpr (OP == BIN_GT) return static_cast<uint8_t>(a > b);
    else if constexpr (OP == BIN_GE) return static_cast<uint8_t>(a >= b);
    else if constexpr (OP == BIN_EQ) return static_cast<uint8_t>(a == b);
    else return static_cast<uint8_t>(a != b);
}

template <typename T, int OP, bool DENSE>
__global__ void __launch_bounds__(256) binary_kernel(const T *__restrict__ a, ViewDesc va, const T *__restrict__ b, ViewDesc vb,
                                                    void *__restrict__ out, int64_t numel) {
    using R = decltype(binary_apply<T, OP>(T(0), T(0)));
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step) {
        const T x = DENSE ? a[i] : a[flat_of(i, va)];
        const T y = DENSE ? b[i] : b[flat_of(i, vb)];
        static_cast<R *>(out)[i] = binary_apply<T, OP>(x, y);
    }
}

template <typename T, int OP>
__device__ __forceinline__ T unary_apply(T x) {
    if constexpr (OP == UN_RELU) return x > T(0) ? x : T(0);
    else if constexpr (OP == UN_NEGATE) return static_cast<T>(T(0) - x);
    else if constexpr (OP == UN_ABS) {
        if constexpr (std::is_unsigned_v<T>) return x;
        else return x < T(0) ? static_cast<T>(T(0) - x) : x;
    } else if constexpr (std::is_floating_point_v<T>) {
        if constexpr (OP == UN_SQRT) return sqrt(x);
        else if constexpr (OP == UN_EXP) return exp(x);
        else if constexpr (OP == UN_LOG) return log(x);
        else if constexpr (OP == UN_SIGMOID) return T(1) / (T(1) + exp(-x));
        else return tanh(x);
    } else {
        return x;
    }
}

template <typename T, int OP, bool DENSE>
__global__ void __launch_bounds__(256) unary_kernel(const T *__restrict__ a, ViewDesc va, T *__restrict__ out, int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step)
        out[i] = unary_apply<T, OP>(DENSE ? a[i] : a[flat_of(i, va)]);
}

// Dense streaming forms: every lane moves one 16-byte vector of each T-typed operand per step (N = 16 / sizeof(T)
// elements; a result of another width is written as one N-element vector too), so a wavefront requests 1 KiB per
// load instruction.  Used when all operands are dense and 16-byte aligned; the last numel % N elements go through
// the element-wise kernels.
template <typename T, int N>
using vec_t = T __attribute__((ext_vector_type(N)));

// Load of data that the kernel reads exactly once: the non-temporal hint keeps a long stream from displacing what the
// caches hold (measured on an 805 MB add: 155 -> 120 us; a 4 MiB operand that is already cached still hits).
template <typename V>
__device__ __forceinline__ V stream_load(const V *p) {
    return __builtin_nontemporal_load(p);
}

// SA / SB: the operand is one element broadcast over the shape (every stride 0: `x < 0`, `g * lr`), read once per lane.
template <typename T, int OP, bool SA = false, bool SB = false>
__global__ void __launch_bounds__(256) binary_vec_kernel(const T *__restrict__ a, const T *__restrict__ b, void *__restrict__ out, int64_t nvec) {
    constexpr int N = 16 / sizeof(T);
    using R = decltype(binary_apply<T, OP>(T(0), T(0)));
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    vec_t<T, N> x, y;
    if constexpr (SA) x = a[0];
    if constexpr (SB) y = b[0];
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step) {
        if constexpr (!SA) x = stream_load(reinterpret_cast<const vec_t<T, N> *>(a) + i);
        if constexpr (!SB) y = stream_load(reinterpret_cast<const vec_t<T, N> *>(b) + i);
        vec_t<R, N> r;
#pragma unroll
        for (int j = 0; j < N; ++j) r[j] = binary_apply<T, OP>(x[j], y[j]);
        static_cast<vec_t<R, N> *>(out)[i] = r;
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(256) unary_vec_kernel(const T *__restrict__ a, T *__restrict__ out, int64_t nvec) {
    constexpr int N = 16 / sizeof(T);
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step) {
        const vec_t<T, N> x = stream_load(reinterpret_cast<const vec_t<T, N> *>(a) + i);
        vec_t<T, N> r;
#pragma unroll
        for (int j = 0; j < N; ++j) r[j] = unary_apply<T, OP>(x[j]);
        reinterpret_cast<vec_t<T, N> *>(out)[i] = r;
    }
}

template <typename T, bool SA = false, bool SB = false>
__global__ void __launch_bounds__(256) where_vec_kernel(const uint8_t *__restrict__ c, const T *__restrict__ a, const T *__restrict__ b,
                                                       T *__restrict__ out, int64_t nvec) {
    constexpr int N = 16 / sizeof(T);
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    vec_t<T, N> x, y;
    if constexpr (SA) x = a[0];
    if constexpr (SB) y = b[0];
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step) {
        const vec_t<uint8_t, N> m = stream_load(reinterpret_cast<const vec_t<uint8_t, N> *>(c) + i);
        if constexpr (!SA) x = stream_load(reinterpret_cast<const vec_t<T, N> *>(a) + i);
        if constexpr (!SB) y = stream_load(reinterpret_cast<const vec_t<T, N> *>(b) + i);
        vec_t<T, N> r;
#pragma unroll
        for (int j = 0; j < N; ++j) r[j] = m[j] ? x[j] : y[j];
        reinterpret_cast<vec_t<T, N> *>(out)[i] = r;
    }
}

template <typename T>
__global__ void __launch_bounds__(256) where_kernel(const uint8_t *__restrict__ c, ViewDesc vc, const T *__restrict__ a, ViewDesc va,
                                                   const T *__restrict__ b, ViewDesc vb, T *__restrict__ out, int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step)
        out[i] = c[flat_of(i, vc)] ? a[flat_of(i, va)] : b[flat_of(i, vb)];
}

template <typename T>
__global__ void __launch_bounds__(256) full_kernel(T *__restrict__ out, T value, int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step) out[i] = value;
}

// Sums read elements of type T and accumulate in A: A = T for the float types; every integer type (and bool) is summed
// into int64, which is also the result's type (common/reduce.h:56-61: "sum reductions on low width int types get cast to
// larger width to circumvent overflows"; cpu/reduce.cpp:38-54 allocates the result as that type).
//
// sum over one dimension: one lane per output element walks the reduced dimension in index order, which is
// the order of the reference's reduce_dim_kernel (cpu/kernel/reduce.hpp:15-32).  `outer` = view without `dim`.
template <typename T, typename A>
__global__ void __launch_bounds__(256) sum_dim_kernel(const T *__restrict__ a, ViewDesc outer, int64_t dim_len, int64_t dim_stride,
                                                     A *__restrict__ out, int64_t n_out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n_out) return;
    const T *p = a + flat_of(i, outer);
    A acc = A(0);
    int64_t j = 0;
    for (; j + 8 <= dim_len; j += 8) {  // eight loads in flight, added in index order
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[(j + u) * dim_stride];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = static_cast<A>(acc + static_cast<A>(v[u]));
    }
    for (; j < dim_len; ++j) acc = static_cast<A>(acc + static_cast<A>(p[j * dim_stride]));
    out[i] = acc;
}

// Few outputs and a long reduced dimension (a bias gradient: [1024,1024] summed over the batch has 1024 outputs) leave
// the one-lane-per-output kernel with a handful of workgroups.  Two parallel forms, both with a fixed summation order:
//  * cols: 64 consecutive outputs x 4 row lanes per workgroup, the reduced dimension cut into slices (grid.y);
//    partial sums per slice go to scratch and a second sum_dim_kernel adds them in slice order;
//  * rows (the reduced dimension has unit stride): one wavefront per output, lanes stride the dimension and combine
//    with a shuffle tree.
template <typename T, typename A>
__global__ void __launch_bounds__(256) sum_dim_cols_kernel(const T *__restrict__ a, ViewDesc outer, int64_t dim_len, int64_t dim_stride,
                                                          A *__restrict__ partial, int64_t n_out, int64_t rows_per_slice) {
    __shared__ A red[4][64];
    const int ol = threadIdx.x % 64, rl = threadIdx.x / 64;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * 64 + ol;
    const int64_t r0 = static_cast<int64_t>(blockIdx.y) * rows_per_slice;
    const int64_t r1 = r0 + rows_per_slice < dim_len ? r0 + rows_per_slice : dim_len;
    A acc = A(0);
    if (o < n_out) {
        const T *p = a + flat_of(o, outer);
        for (int64_t r = r0 + rl; r < r1; r += 4) acc = static_cast<A>(acc + static_cast<A>(p[r * dim_stride]));
    }
    red[rl][ol] = acc;
    __syncthreads();
    if (rl == 0 && o < n_out)
        partial[static_cast<int64_t>(blockIdx.y) * n_out + o] =
            static_cast<A>(static_cast<A>(red[0][ol] + red[1][ol]) + static_cast<A>(red[2][ol] + red[3][ol]));
}

template <typename T, typename A>
__global__ void __launch_bounds__(256) sum_dim_rows_kernel(const T *__restrict__ a, ViewDesc outer, int64_t dim_len, A *__restrict__ out,
                                                          int64_t n_out) {
    __shared__ A red[4][64];
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * 4 + w;
    A acc = A(0);
    if (o < n_out) {
        const T *p = a + flat_of(o, outer);
        for (int64_t j = lane; j < dim_len; j += 64) acc = static_cast<A>(acc + static_cast<A>(p[j]));
    }
    red[w][lane] = acc;
    __syncthreads();
    for (int h = 32; h > 0; h >>= 1) {
        if (lane < h) red[w][lane] = static_cast<A>(red[w][lane] + red[w][lane + h]);
        __syncthreads();
    }
    if (lane == 0 && o < n_out) out[o] = red[w][0];
}

// sum of everything: per-workgroup partial sums (stage 1) then one workgroup adds the partials (stage 2).
template <typename T, typename A>
__global__ void __launch_bounds__(256) sum_all_kernel(const T *__restrict__ a, ViewDesc v, bool dense, int64_t numel, A *__restrict__ out) {
    __shared__ A red[256];
    A acc = A(0);
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    int64_t first = 0;  // elements [0, first) are covered by 16-byte loads
    if (dense && reinterpret_cast<uintptr_t>(a) % 16 == 0) {
        constexpr int N = 16 / sizeof(T);
        const int64_t nvec = numel / N;
        for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step) {
            const vec_t<T, N> x = stream_load(reinterpret_cast<const vec_t<T, N> *>(a) + i);
#pragma unroll
            for (int j = 0; j < N; ++j) acc = static_cast<A>(acc + static_cast<A>(x[j]));
        }
        first = nvec * N;
    }
    for (int64_t i = first + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step)
        acc = static_cast<A>(acc + static_cast<A>(dense ? a[i] : a[flat_of(i, v)]));
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (static_cast<int>(threadIdx.x) < s) red[threadIdx.x] = static_cast<A>(red[threadIdx.x] + red[threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = red[0];
}

// Seeded draws (tinytensor/tensor/random.cpp:36-43, backend/common/kernel/distribution.hpp:92-99, 232-246):
// element i owns a generator whose state is the i-th output of the master generator; the states are produced on
// the host and uploaded, exactly as the reference's GPU backend does (cuda/distribution.cu:32-99).
__device__ __forceinline__ uint64_t xorshift64(uint64_t &x) {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return x;
}
__device__ __forceinline__ float unit_sample(uint64_t &st, float) {
    return __builtin_bit_cast(float, (static_cast<uint32_t>(xorshift64(st)) >> 9) | 0x3F800000u) - 1.0f;
}
__device__ __forceinline__ double unit_sample(uint64_t &st, double) {
    return __builtin_bit_cast(double, (xorshift64(st) >> 12) | 0x3FF0000000000000ull) - 1.0;
}
// Element i of the view (row-major rank over its shape) takes state i and is written at the view's address of that
// rank, as the in-place kernel of the CPU backend does (cpu/kernel/distribution.hpp:28-32 with common/util.h:18-34).
template <typename T>
__global__ void __launch_bounds__(256) uniform_real_kernel(const uint64_t *__restrict__ states, T low, T high, T *__restrict__ out, ViewDesc v,
                                                          bool dense, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t st = states[i];
    const T r = unit_sample(st, T(0));
    out[dense ? i : flat_of(i, v)] = fma(r, high - low, low);  // r * (high - low) + low, contracted as the fma flavour of the host build does
}
template <typename T>
__global__ void __launch_bounds__(256) normal_kernel(const uint64_t *__restrict__ states, T mu, T stddev, T *__restrict__ out, ViewDesc v,
                                                    bool dense, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t st = states[i];
    const T u1 = unit_sample(st, T(0));
    const T u2 = unit_sample(st, T(0));
    const T r = sqrt(T(-2) * log1p(-u1));
    const T theta = T(2) * T(3.14159265358979323846) * u2;
    out[dense ? i : flat_of(i, v)] = stddev * (r * sin(theta)) + mu;
}

// The same draws with a parameter pair per element (the tensor forms of BackendBase::uniform_real / normal,
// backend_base.h:83-103): element i reads its parameters at rank i of the parameter views, which is what the CPU
// backend's params[i] on the parameters made contiguous reads (cpu/distribution.cpp:42-47, cpu/kernel/distribution.hpp:28-32).
template <typename T, int DIST>
__global__ void __launch_bounds__(256) random_params_kernel(const uint64_t *__restrict__ states, const T *__restrict__ p0, ViewDesc v0,
                                                           const T *__restrict__ p1, ViewDesc v1, T *__restrict__ out, ViewDesc v, bool dense,
                                                           int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t st = states[i];
    const T a = p0[flat_of(i, v0)];
    const T b = p1[flat_of(i, v1)];
    T value;
    if (DIST == 0) {
        const T r = unit_sample(st, T(0));
        value = fma(r, b - a, a);
    } else {
        const T u1 = unit_sample(st, T(0));
        const T u2 = unit_sample(st, T(0));
        const T r = sqrt(T(-2) * log1p(-u1));
        const T theta = T(2) * T(3.14159265358979323846) * u2;
        value = b * (r * sin(theta)) + a;
    }
    out[dense ? i : flat_of(i, v)] = value;
}

// to(dtype): out[i] = static_cast<R>(view[i]) (tinytensor/tensor/backend/cpu/cast.cpp:27-34; bool keeps C++'s
// "non-zero is true").
template <typename T, typename R>
__global__ void __launch_bounds__(256) cast_kernel(const T *__restrict__ a, ViewDesc va, bool dense, R *__restrict__ out, int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step) {
        const T x = dense ? a[i] : a[flat_of(i, va)];
        out[i] = static_cast<R>(x);
    }
}

template <typename T, typename R>
__global__ void __launch_bounds__(256) cast_vec_kernel(const T *__restrict__ a, R *__restrict__ out, int64_t nvec) {
    // 16 bytes of the wider side per lane: a widening cast then stores one vector per lane, so a wave's store covers
    // contiguous memory (with 16 bytes of the input per lane a lane wrote two vectors 32 bytes apart from its
    // neighbour's, every store instruction touching half of each line).
    constexpr int N = 16 / (sizeof(T) > sizeof(R) ? sizeof(T) : sizeof(R));
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += step) {
        const vec_t<T, N> x = stream_load(reinterpret_cast<const vec_t<T, N> *>(a) + i);
        R r[N];
#pragma unroll
        for (int j = 0; j < N; ++j) r[j] = static_cast<R>(x[j]);
#pragma unroll
        for (int j = 0; j < N; ++j) out[i * N + j] = r[j];  // consecutive stores of one lane merge into vector stores
    }
}

// assign: lhs_view[i] = rhs_view[i] over one shape (tinytensor/tensor/backend/cpu/kernel/assign.hpp:15-21).
// Moves raw bytes, so one kernel per element size serves every dtype.
template <typename W>
__global__ void __launch_bounds__(256) assign_kernel(W *__restrict__ dst, ViewDesc vd, const W *__restrict__ src, ViewDesc vs, int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step)
        dst[flat_of(i, vd)] = src[flat_of(i, vs)];
}

// Vector kernels: one 16-byte vector per lane (a full grid measured 10 % faster than 8192 workgroups looping); the
// grid-stride loop only runs again beyond 2^22 workgroups.
inline unsigned grid_for_vec(int64_t nvec) {
    int64_t blocks = (nvec + 255) / 256;
    if (blocks > (1 << 22)) blocks = 1 << 22;
    return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

inline unsigned grid_for(int64_t numel) {
    int64_t blocks = (numel + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

inline bool is_dense(const ViewDesc &v) {
    int64_t expect = 1;
    for (int d = v.ndim - 1; d >= 0; --d) {
        if (v.shape[d] != 1 && v.stride[d] != expect) return false;
        expect *= v.shape[d];
    }
    return true;
}

ttamd_status make_view(const char *who, int ndim, const int64_t *shape, const int64_t *stride, ViewDesc *v, int64_t *numel) {
    if (ndim < 0 || ndim > kMaxDims || (ndim > 0 && (!shape || !stride))) {
        set_error("%s: ndim must be in [0,%d] with non-NULL shape/stride", who, kMaxDims);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *v = ViewDesc{};
    v->ndim = ndim;
    int64_t n = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0 || stride[d] < 0) {
            set_error("%s: negative extent or stride in dimension %d", who, d);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        v->shape[d] = shape[d];
        v->stride[d] = stride[d];
        n *= shape[d];
    }
    if (numel) *numel = n;
    return TTAMD_OK;
}

inline bool aligned16(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// One element broadcast over the whole shape (more than one element, every extent > 1 has stride 0).
inline bool is_broadcast_scalar(const ViewDesc &v) {
    bool any = false;
    for (int d = 0; d < v.ndim; ++d) {
        if (v.shape[d] == 1) continue;
        if (v.stride[d] != 0) return false;
        any = true;
    }
    return any;
}

template <typename T, int OP>
ttamd_status launch_binary_op(const void *a, const ViewDesc &va, const void *b, const ViewDesc &vb, void *out, int64_t numel, hipStream_t st) {
    const bool sa = is_broadcast_scalar(va), sb = is_broadcast_scalar(vb);
    if ((sa != sb) && (sa ? is_dense(vb) : is_dense(va))) {  // tensor (op) scalar: the vector kernel with one operand splat
        using R = std::conditional_t<(OP >= BIN_LT), uint8_t, T>;
        constexpr int N = 16 / sizeof(T);
        const T *pa = static_cast<const T *>(a), *pb = static_cast<const T *>(b);
        int64_t done = 0;
        if (aligned16(sa ? b : a) && aligned16(out) && numel >= N) {
            const int64_t nvec = numel / N;
            if (sa) binary_vec_kernel<T, OP, true, false><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(pa, pb, out, nvec);
            else binary_vec_kernel<T, OP, false, true><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(pa, pb, out, nvec);
            done = nvec * N;
        }
        if (done < numel) {
            ViewDesc ta{}, tb{};
            ta.ndim = tb.ndim = 1;
            ta.shape[0] = tb.shape[0] = numel - done;
            ta.stride[0] = sa ? 0 : 1;
            tb.stride[0] = sb ? 0 : 1;
            binary_kernel<T, OP, false><<<dim3(grid_for(numel - done)), dim3(256), 0, st>>>(pa + (sa ? 0 : done), ta, pb + (sb ? 0 : done), tb,
                                                                                        static_cast<R *>(out) + done, numel - done);
        }
    } else if (is_dense(va) && is_dense(vb)) {
        using R = std::conditional_t<(OP >= BIN_LT), uint8_t, T>;  // comparisons yield bool bytes
        constexpr int N = 16 / sizeof(T);
        int64_t done = 0;
        if (aligned16(a) && aligned16(b) && aligned16(out) && numel >= N) {
            const int64_t nvec = numel / N;
            binary_vec_kernel<T, OP><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(static_cast<const T *>(a), static_cast<const T *>(b), out, nvec);
            done = nvec * N;
        }
        if (done < numel)
            binary_kernel<T, OP, true><<<dim3(1), dim3(256), 0, st>>>(static_cast<const T *>(a) + done, va, static_cast<const T *>(b) + done, vb,
                                                                     static_cast<R *>(out) + done, numel - done);
    } else
        binary_kernel<T, OP, false><<<dim3(grid_for(numel)), dim3(256), 0, st>>>(static_cast<const T *>(a), va, static_cast<const T *>(b), vb, out, numel);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T, int OP = 0>
ttamd_status dispatch_binary(int op, const void *a, const ViewDesc &va, const void *b, const ViewDesc &vb, void *out, int64_t numel, hipStream_t st) {
    if constexpr (OP < BIN_COUNT) {
        if (op == OP) return launch_binary_op<T, OP>(a, va, b, vb, out, numel, st);
        return dispatch_binary<T, OP + 1>(op, a, va, b, vb, out, numel, st);
    } else {
        set_error("binary: unknown op code %d", op);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
}

template <typename T, int OP = 0>
ttamd_status dispatch_unary(int op, const void *a, const ViewDesc &va, void *out, int64_t numel, hipStream_t st) {
    if constexpr (OP < UN_COUNT) {
        if (op == OP) {
            if (is_dense(va)) {
                constexpr int N = 16 / sizeof(T);
                int64_t done = 0;
                if (aligned16(a) && aligned16(out) && numel >= N) {
                    const int64_t nvec = numel / N;
                    unary_vec_kernel<T, OP><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(static_cast<const T *>(a), static_cast<T *>(out), nvec);
                    done = nvec * N;
                }
                if (done < numel)
                    unary_kernel<T, OP, true><<<dim3(1), dim3(256), 0, st>>>(static_cast<const T *>(a) + done, va, static_cast<T *>(out) + done, numel - done);
            } else unary_kernel<T, OP, false><<<dim3(grid_for(numel)), dim3(256), 0, st>>>(static_cast<const T *>(a), va, static_cast<T *>(out), numel);
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        }
        return dispatch_unary<T, OP + 1>(op, a, va, out, numel, st);
    } else {
        set_error("unary: unknown op code %d", op);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
}

template <typename T>
ttamd_status sum_typed(int device, const void *a, const ViewDesc &v, int64_t numel, int dim, void *out, hipStream_t st) {
    using A = std::conditional_t<std::is_floating_point_v<T>, T, int64_t>;  // accumulator and result type
    const T *src = static_cast<const T *>(a);
    if (dim < 0) {
        const unsigned blocks = numel > (1 << 22) ? 2048 : (numel > 256 * 64 ? 256 : 1);
        if (blocks == 1) {
            sum_all_kernel<T, A><<<dim3(1), dim3(256), 0, st>>>(src, v, is_dense(v), numel, static_cast<A *>(out));
        } else {
            void *ws = nullptr;
            if (ttamd_status s = stream_scratch(device, st, blocks * sizeof(A), &ws)) return s;
            sum_all_kernel<T, A><<<dim3(blocks), dim3(256), 0, st>>>(src, v, is_dense(v), numel, static_cast<A *>(ws));
            ViewDesc pv{};
            pv.ndim = 1;
            pv.shape[0] = blocks;
            pv.stride[0] = 1;
            sum_all_kernel<A, A><<<dim3(1), dim3(256), 0, st>>>(static_cast<const A *>(ws), pv, true, blocks, static_cast<A *>(out));
        }
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    }
    ViewDesc outer{};
    for (int d = 0; d < v.ndim; ++d) {
        if (d == dim) continue;
        outer.shape[outer.ndim] = v.shape[d];
        outer.stride[outer.ndim] = v.stride[d];
        ++outer.ndim;
    }
    const int64_t n_out = v.shape[dim] ? numel / v.shape[dim] : 0;
    if (n_out == 0) return TTAMD_OK;
    const int64_t dim_len = v.shape[dim], dim_stride = v.stride[dim];
    if (n_out < 32768 && dim_len >= 128) {
        if (dim_stride == 1) {
            sum_dim_rows_kernel<T, A><<<dim3(static_cast<unsigned>((n_out + 3) / 4)), dim3(256), 0, st>>>(src, outer, dim_len, static_cast<A *>(out), n_out);
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        }
        const int64_t col_blocks = (n_out + 63) / 64;
        int64_t slices = 1024 / col_blocks;
        if (slices > dim_len / 32) slices = dim_len / 32;  // at least 32 rows per slice
        if (slices > 256) slices = 256;
        if (slices >= 2) {
            const int64_t rows_per_slice = (dim_len + slices - 1) / slices;
            slices = (dim_len + rows_per_slice - 1) / rows_per_slice;
            void *ws = nullptr;
            if (ttamd_status s = stream_scratch(device, st, static_cast<size_t>(slices) * n_out * sizeof(A), &ws)) return s;
            sum_dim_cols_kernel<T, A><<<dim3(static_cast<unsigned>(col_blocks), static_cast<unsigned>(slices)), dim3(256), 0, st>>>(
                src, outer, dim_len, dim_stride, static_cast<A *>(ws), n_out, rows_per_slice);
            ViewDesc flat{};
            flat.ndim = 1;
            flat.shape[0] = n_out;
            flat.stride[0] = 1;
            sum_dim_kernel<A, A><<<dim3(static_cast<unsigned>((n_out + 255) / 256)), dim3(256), 0, st>>>(static_cast<const A *>(ws), flat, slices, n_out,
                                                                                                       static_cast<A *>(out), n_out);
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        }
    }
    sum_dim_kernel<T, A><<<dim3(static_cast<unsigned>((n_out + 255) / 256)), dim3(256), 0, st>>>(src, outer, v.shape[dim], v.stride[dim],
                                                                                                 static_cast<A *>(out), n_out);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

// bool is stored as one byte holding 0 or 1
struct BoolByte {
    uint8_t v;
    __host__ __device__ BoolByte() : v(0) {}
    template <typename X>
    __host__ __device__ explicit BoolByte(X x) : v(x != X(0) ? 1 : 0) {}
};

template <typename T, typename R>
ttamd_status launch_cast(const void *a, const ViewDesc &va, void *out, int64_t numel, hipStream_t st) {
    constexpr int N = 16 / (sizeof(T) > sizeof(R) ? sizeof(T) : sizeof(R));  // (cast_vec_kernel's vector length)
    const bool dense = is_dense(va);
    int64_t done = 0;
    if (dense && aligned16(a) && aligned16(out) && numel >= N) {
        const int64_t nvec = numel / N;
        cast_vec_kernel<T, R><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(static_cast<const T *>(a), static_cast<R *>(out), nvec);
        done = nvec * N;
    }
    if (done < numel)
        cast_kernel<T, R><<<dim3(grid_for(numel - done)), dim3(256), 0, st>>>(static_cast<const T *>(a) + (dense ? done : 0), va, dense,
                                                                             static_cast<R *>(out) + done, numel - done);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T>
ttamd_status cast_from(ttamd_dtype to, const void *a, const ViewDesc &va, void *out, int64_t numel, hipStream_t st) {
    switch (to) {
    case TTAMD_BOOL: return launch_cast<T, BoolByte>(a, va, out, numel, st);
    case TTAMD_U8: return launch_cast<T, uint8_t>(a, va, out, numel, st);
    case TTAMD_I16: return launch_cast<T, int16_t>(a, va, out, numel, st);
    case TTAMD_I32: return launch_cast<T, int32_t>(a, va, out, numel, st);
    case TTAMD_I64: return launch_cast<T, int64_t>(a, va, out, numel, st);
    case TTAMD_F32: return launch_cast<T, float>(a, va, out, numel, st);
    case TTAMD_F64: return launch_cast<T, double>(a, va, out, numel, st);
    default: break;
    }
    set_error("cast: unknown target dtype code %d", static_cast<int>(to));
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

#define TTAMD_DISPATCH_DTYPE(dtype, CALL)                      \
    switch (dtype) {                                           \
    case TTAMD_U8: { using T_ = uint8_t; return CALL; }        \
    case TTAMD_I16: { using T_ = int16_t; return CALL; }       \
    case TTAMD_I32: { using T_ = int32_t; return CALL; }       \
    case TTAMD_I64: { using T_ = int64_t; return CALL; }       \
    case TTAMD_F32: { using T_ = float; return CALL; }         \
    case TTAMD_F64: { using T_ = double; return CALL; }        \
    default: break;                                            \
    }

// nn::mse_loss with mean reduction (nn/loss.cpp:69-72: pow(input - target, 2).mean(), the mean being
// (x / numel).sum(), autograd/reduce_ops.cpp:195-200) together with its backward (grad_output / numel from the mean,
// times 2 * (input - target) from pow: autograd/reduce_ops.cpp:201-205, binary_ops.cpp:153-159) and, for narrow
// matrices, the column sums of that gradient (the bias gradient of the Linear layer that produced `input`).
// Lane layout: CP column lanes (a power of two >= cols, at most 64) by THREADS / CP row lanes; a lane walks its column
// down the rows in steps of (row lanes * blocks), U rows to a batch whose loads are all issued before the first is
// used (a small matrix is one memory round trip away, not one per row).  Sums are folded over the row lanes in a fixed
// tree, per-block partials ([blocks][cols + 1]: column sums, then the loss) are added by block index: deterministic.
// THREADS = 1024 with U = 16 is the form for a matrix that a single workgroup takes in one batch: no partials, no
// finishing kernel.
template <typename T, int CP, int THREADS, int U>
__global__ void __launch_bounds__(THREADS) mse_loss_kernel(const T *__restrict__ y, const T *__restrict__ t, int64_t rows, int cols,
                                                          T inv_n, T *__restrict__ grad, T *__restrict__ partial,
                                                          T *__restrict__ loss, T *__restrict__ colsum) {
    constexpr int RL = THREADS / CP;
    __shared__ T red[RL][CP + 1];
    __shared__ T red_loss[THREADS];
    const int cl = threadIdx.x % CP, rl = threadIdx.x / CP;
    const T scale = inv_n * T(2);  // (1 / numel) * 2, the factor the reference's backward forms
    T csum = T(0), lsum = T(0);
    if (cl < cols) {
        const int64_t step = static_cast<int64_t>(gridDim.x) * RL;
        for (int64_t r0 = static_cast<int64_t>(blockIdx.x) * RL + rl; r0 < rows; r0 += step * U) {
            T yv[U], tv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t r = r0 + u * step;
                const int64_t i = (r < rows ? r : rows - 1) * cols + cl;  // no branch around a load: they all go out together
                yv[u] = y[i];
                tv[u] = t[i];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t r = r0 + u * step;
                const T d = r < rows ? yv[u] - tv[u] : T(0);
                // the reference divides each term by numel ((x / numel).sum(), reduce_ops.cpp:199); the product with 1 / numel
                // can differ from that quotient in the last bit, and the sum's order is this kernel's own anyway (a division
                // per term measured 0.9 us on this one-workgroup kernel, 6.1 -> 7.0 us)
                lsum += d * d * inv_n;
                const T g = scale * d;
                if (grad && r < rows) grad[r * cols + cl] = g;
                csum += g;
            }
        }
    }
    red[rl][cl] = csum;
    red_loss[threadIdx.x] = lsum;
    __syncthreads();
    for (int h = RL / 2; h > 0; h >>= 1) {
        if (rl < h) red[rl][cl] += red[rl + h][cl];
        __syncthreads();
    }
    for (int h = THREADS / 2; h > 0; h >>= 1) {
        if (static_cast<int>(threadIdx.x) < h) red_loss[threadIdx.x] += red_loss[threadIdx.x + h];
        __syncthreads();
    }
    if (gridDim.x == 1) {  // a single workgroup holds the final sums: no partials, no finishing kernel
        if (rl == 0 && cl < cols && colsum) colsum[cl] = red[0][cl];
        if (threadIdx.x == 0) loss[0] = red_loss[0];
        return;
    }
    T *p = partial + static_cast<int64_t>(blockIdx.x) * (cols + 1);
    if (rl == 0 && cl < cols) p[cl] = red[0][cl];
    if (threadIdx.x == 0) p[cols] = red_loss[0];
}

// out[j] = sum over blocks b (ascending) of partial[b][j], j < cols + 1; column sums to colsum (may be null), the
// last entry to loss.
template <typename T>
__global__ void __launch_bounds__(256) mse_loss_finish_kernel(const T *__restrict__ partial, int blocks, int cols, T *__restrict__ loss,
                                                             T *__restrict__ colsum) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j > cols) return;
    T v = T(0);
    for (int b = 0; b < blocks; ++b) v += partial[static_cast<int64_t>(b) * (cols + 1) + j];
    if (j == cols) loss[0] = v;
    else if (colsum) colsum[j] = v;
}

template <typename T>
ttamd_status launch_mse_loss(int device, int64_t rows, int64_t cols, const void *y, const void *t, void *loss, void *grad, void *colsum,
                             hipStream_t st) {
    // wide matrices (no column sums there): one flat column of rows * cols elements
    if (cols > 64) {
        rows *= cols;
        cols = 1;
    }
    int cp = 1;
    while (cp < cols) cp *= 2;
    const bool small = rows * cp <= 1024 * 16;  // one workgroup of 1024 lanes, at most 16 rows to a lane: a single batch
    const int rl = 256 / cp;
    int64_t blocks = (rows + static_cast<int64_t>(rl) * 8 - 1) / (static_cast<int64_t>(rl) * 8);  // about 8 rows per lane
    if (blocks > 1024) blocks = 1024;
    if (blocks < 1 || small) blocks = 1;
    void *ws = nullptr;
    if (blocks > 1)
        if (ttamd_status s = stream_scratch(device, st, static_cast<size_t>(blocks) * (cols + 1) * sizeof(T), &ws)) return s;
    const T inv_n = T(1) / static_cast<T>(rows * cols);
    const T *yp = static_cast<const T *>(y), *tp = static_cast<const T *>(t);
    T *gp = static_cast<T *>(grad), *pp = static_cast<T *>(ws), *lp = static_cast<T *>(loss), *cs = static_cast<T *>(colsum);
    const dim3 grid(static_cast<unsigned>(blocks));
    const int c = static_cast<int>(cols);
#define TTAMD_MSE_CASE(CP)                                                                                        \
    case CP:                                                                                                      \
        if (small) mse_loss_kernel<T, CP, 1024, 16><<<grid, dim3(1024), 0, st>>>(yp, tp, rows, c, inv_n, gp, pp, lp, cs); \
        else mse_loss_kernel<T, CP, 256, 8><<<grid, dim3(256), 0, st>>>(yp, tp, rows, c, inv_n, gp, pp, lp, cs);   \
        break;
    switch (cp) {
        TTAMD_MSE_CASE(1)
        TTAMD_MSE_CASE(2)
        TTAMD_MSE_CASE(4)
        TTAMD_MSE_CASE(8)
        TTAMD_MSE_CASE(16)
        TTAMD_MSE_CASE(32)
    default:
        if (small) mse_loss_kernel<T, 64, 1024, 16><<<grid, dim3(1024), 0, st>>>(yp, tp, rows, c, inv_n, gp, pp, lp, cs);
        else mse_loss_kernel<T, 64, 256, 8><<<grid, dim3(256), 0, st>>>(yp, tp, rows, c, inv_n, gp, pp, lp, cs);
        break;
    }
#undef TTAMD_MSE_CASE
    if (blocks > 1) mse_loss_finish_kernel<T><<<dim3(1), dim3(256), 0, st>>>(pp, static_cast<int>(blocks), c, lp, cs);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" ttamd_status ttamd_contiguous(int device, ttamd_dtype dtype, int ndim, const int64_t *shape,
                                         const int64_t *stride, const void *data, int64_t offset, void *out,
                                         void *stream) {
    const size_t esz = dtype_size(dtype);
    if (esz == 0 || dtype < TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("contiguous: unknown dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (ndim < 0 || ndim > kMaxDims || (ndim > 0 && (!shape || !stride)) || offset < 0) {
        set_error("contiguous: ndim must be in [0,%d] with non-NULL shape/stride and offset >= 0", kMaxDims);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ViewDesc v{};
    v.ndim = ndim;
    int64_t numel = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0 || stride[d] < 0) {
            set_error("contiguous: negative extent or stride in dimension %d", d);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        v.shape[d] = shape[d];
        v.stride[d] = stride[d];
        numel *= shape[d];
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!data || !out) {
        set_error("contiguous: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const char *src = static_cast<const char *>(data) + offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (esz) {
    case 1: return launch_contiguous<uint8_t>(src, out, v, numel, st);
    case 2: return launch_contiguous<uint16_t>(src, out, v, numel, st);
    case 4: return launch_contiguous<uint32_t>(src, out, v, numel, st);
    default: return launch_contiguous<uint64_t>(src, out, v, numel, st);
    }
}

extern "C" {

ttamd_status ttamd_binary(int device, ttamd_dtype dtype, int op, int ndim, const int64_t *shape, const void *lhs, int64_t lhs_offset,
                          const int64_t *lhs_stride, const void *rhs, int64_t rhs_offset, const int64_t *rhs_stride, void *out,
                          void *stream) {
    ViewDesc va, vb;
    int64_t numel = 0;
    if (ttamd_status s = make_view("binary", ndim, shape, lhs_stride, &va, &numel)) return s;
    if (ttamd_status s = make_view("binary", ndim, shape, rhs_stride, &vb, nullptr)) return s;
    const size_t esz = dtype_size(dtype);
    if (dtype <= TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("binary: unsupported dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (lhs_offset < 0 || rhs_offset < 0) {
        set_error("binary: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!lhs || !rhs || !out) {
        set_error("binary: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *a = static_cast<const char *>(lhs) + lhs_offset * static_cast<int64_t>(esz);
    const void *b = static_cast<const char *>(rhs) + rhs_offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    TTAMD_DISPATCH_DTYPE(dtype, (dispatch_binary<T_>(op, a, va, b, vb, out, numel, st)))
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_unary(int device, ttamd_dtype dtype, int op, int ndim, const int64_t *shape, const void *src, int64_t offset,
                         const int64_t *stride, void *out, void *stream) {
    ViewDesc va;
    int64_t numel = 0;
    if (ttamd_status s = make_view("unary", ndim, shape, stride, &va, &numel)) return s;
    const size_t esz = dtype_size(dtype);
    if (dtype <= TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("unary: unsupported dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (op >= UN_SQRT && op < UN_COUNT && dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("unary: op %d needs a floating point dtype", op);
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (offset < 0) {
        set_error("unary: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!src || !out) {
        set_error("unary: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *a = static_cast<const char *>(src) + offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    TTAMD_DISPATCH_DTYPE(dtype, (dispatch_unary<T_>(op, a, va, out, numel, st)))
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_cast(int device, ttamd_dtype from, ttamd_dtype to, int ndim, const int64_t *shape, const void *src,
                        int64_t offset, const int64_t *stride, void *out, void *stream) {
    ViewDesc va;
    int64_t numel = 0;
    if (ttamd_status s = make_view("cast", ndim, shape, stride, &va, &numel)) return s;
    if (from < TTAMD_BOOL || from > TTAMD_F64 || to < TTAMD_BOOL || to > TTAMD_F64) {
        set_error("cast: unknown dtype code %d -> %d", static_cast<int>(from), static_cast<int>(to));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (offset < 0) {
        set_error("cast: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!src || !out) {
        set_error("cast: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *a = static_cast<const char *>(src) + offset * static_cast<int64_t>(dtype_size(from));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (from == TTAMD_BOOL) return cast_from<uint8_t>(to, a, va, out, numel, st);  // stored as 0 / 1
    TTAMD_DISPATCH_DTYPE(from, (cast_from<T_>(to, a, va, out, numel, st)))
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_assign(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, void *dst, int64_t dst_offset,
                          const int64_t *dst_stride, const void *src, int64_t src_offset, const int64_t *src_stride, void *stream) {
    ViewDesc vd, vs;
    int64_t numel = 0;
    if (ttamd_status s = make_view("assign", ndim, shape, dst_stride, &vd, &numel)) return s;
    if (ttamd_status s = make_view("assign", ndim, shape, src_stride, &vs, nullptr)) return s;
    const size_t esz = dtype_size(dtype);
    if (dtype < TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("assign: unknown dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (dst_offset < 0 || src_offset < 0) {
        set_error("assign: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!dst || !src) {
        set_error("assign: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    char *d = static_cast<char *>(dst) + dst_offset * static_cast<int64_t>(esz);
    const char *a = static_cast<const char *>(src) + src_offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto go = [&](auto tag) -> ttamd_status {
        using W = decltype(tag);
        assign_kernel<W><<<dim3(grid_for(numel)), dim3(256), 0, st>>>(reinterpret_cast<W *>(d), vd, reinterpret_cast<const W *>(a), vs, numel);
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    };
    switch (esz) {
    case 1: return go(uint8_t{});
    case 2: return go(uint16_t{});
    case 4: return go(uint32_t{});
    default: return go(uint64_t{});
    }
}

ttamd_status ttamd_where(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, const void *cond, int64_t cond_offset,
                         const int64_t *cond_stride, const void *lhs, int64_t lhs_offset, const int64_t *lhs_stride, const void *rhs,
                         int64_t rhs_offset, const int64_t *rhs_stride, void *out, void *stream) {
    ViewDesc vc, va, vb;
    int64_t numel = 0;
    if (ttamd_status s = make_view("where", ndim, shape, cond_stride, &vc, &numel)) return s;
    if (ttamd_status s = make_view("where", ndim, shape, lhs_stride, &va, nullptr)) return s;
    if (ttamd_status s = make_view("where", ndim, shape, rhs_stride, &vb, nullptr)) return s;
    const size_t esz = dtype_size(dtype);
    if (dtype <= TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("where: unsupported dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (cond_offset < 0 || lhs_offset < 0 || rhs_offset < 0) {
        set_error("where: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!cond || !lhs || !rhs || !out) {
        set_error("where: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const uint8_t *c = static_cast<const uint8_t *>(cond) + cond_offset;
    const void *a = static_cast<const char *>(lhs) + lhs_offset * static_cast<int64_t>(esz);
    const void *b = static_cast<const char *>(rhs) + rhs_offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto run = [&](auto tag) -> ttamd_status {
        using T = decltype(tag);
        constexpr int N = 16 / sizeof(T);
        int64_t done = 0;
        const bool sa = is_broadcast_scalar(va), sb = is_broadcast_scalar(vb);
        if ((sa || sb) && is_dense(vc) && (sa || is_dense(va)) && (sb || is_dense(vb))) {  // scalar branch values: splat in the vector kernel
            const T *pa = static_cast<const T *>(a), *pb = static_cast<const T *>(b);
            if (aligned16(c) && (sa || aligned16(a)) && (sb || aligned16(b)) && aligned16(out) && numel >= N) {
                const int64_t nvec = numel / N;
                const dim3 grid(grid_for_vec(nvec)), block(256);
                if (sa && sb) where_vec_kernel<T, true, true><<<grid, block, 0, st>>>(c, pa, pb, static_cast<T *>(out), nvec);
                else if (sa) where_vec_kernel<T, true, false><<<grid, block, 0, st>>>(c, pa, pb, static_cast<T *>(out), nvec);
                else where_vec_kernel<T, false, true><<<grid, block, 0, st>>>(c, pa, pb, static_cast<T *>(out), nvec);
                done = nvec * N;
            }
            if (done < numel) {
                ViewDesc tc{}, ta{}, tb{};
                tc.ndim = ta.ndim = tb.ndim = 1;
                tc.shape[0] = ta.shape[0] = tb.shape[0] = numel - done;
                tc.stride[0] = 1;
                ta.stride[0] = sa ? 0 : 1;
                tb.stride[0] = sb ? 0 : 1;
                where_kernel<T><<<dim3(grid_for(numel - done)), dim3(256), 0, st>>>(c + done, tc, pa + (sa ? 0 : done), ta, pb + (sb ? 0 : done), tb,
                                                                                  static_cast<T *>(out) + done, numel - done);
            }
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        }
        const bool dense = is_dense(vc) && is_dense(va) && is_dense(vb);
        if (dense && aligned16(c) && aligned16(a) && aligned16(b) && aligned16(out) && numel >= N) {
            const int64_t nvec = numel / N;
            where_vec_kernel<T><<<dim3(grid_for_vec(nvec)), dim3(256), 0, st>>>(c, static_cast<const T *>(a), static_cast<const T *>(b),
                                                                          static_cast<T *>(out), nvec);
            done = nvec * N;
        }
        if (done < numel) {
            const int64_t skip = dense ? done : 0;  // a dense tail continues behind the vectors
            where_kernel<T><<<dim3(grid_for(numel - done)), dim3(256), 0, st>>>(c + skip, vc, static_cast<const T *>(a) + skip, va,
                                                                              static_cast<const T *>(b) + skip, vb,
                                                                              static_cast<T *>(out) + done, numel - done);
        }
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    };
    TTAMD_DISPATCH_DTYPE(dtype, run(T_{}))
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_sum(int device, ttamd_dtype dtype, int ndim, const int64_t *shape, const void *src, int64_t offset,
                       const int64_t *stride, int dim, void *out, void *stream) {
    ViewDesc va;
    int64_t numel = 0;
    if (ttamd_status s = make_view("sum", ndim, shape, stride, &va, &numel)) return s;
    const size_t esz = dtype_size(dtype);
    if (dtype < TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("sum: unsupported dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (dim >= ndim || offset < 0) {
        set_error("sum: dim %d out of range for %d dimensions, or negative offset", dim, ndim);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (!out || (numel > 0 && !src)) {
        set_error("sum: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *a = static_cast<const char *>(src) + offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TTAMD_BOOL) return sum_typed<uint8_t>(device, a, va, numel, dim, out, st);  // one byte holding 0 or 1
    TTAMD_DISPATCH_DTYPE(dtype, (sum_typed<T_>(device, a, va, numel, dim, out, st)))
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_full(int device, ttamd_dtype dtype, const void *value, int64_t numel, void *out, void *stream) {
    const size_t esz = dtype_size(dtype);
    if (dtype < TTAMD_BOOL || dtype > TTAMD_F64 || esz == 0) {
        set_error("full: unsupported dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (!value || numel < 0) {
        set_error("full: NULL value or negative count");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!out) {
        set_error("full: out is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    auto run = [&](auto tag) -> ttamd_status {
        using W = decltype(tag);
        W v;
        memcpy(&v, value, sizeof(W));
        full_kernel<W><<<dim3(grid_for(numel)), dim3(256), 0, st>>>(static_cast<W *>(out), v, numel);
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    };
    switch (esz) {
    case 1: return run(uint8_t{});
    case 2: return run(uint16_t{});
    case 4: return run(uint32_t{});
    default: return run(uint64_t{});
    }
}


// dist: 0 = uniform_real(low = p0, high = p1), 1 = normal(mu = p0, std = p1).  `states`: one generator state per element
// of the view, in the view's row-major order, produced on the host (cpu/distribution.cpp:31-38 draws them from the
// caller's Generator one by one; the reference's GPU backend uploads them the same way, cuda/distribution.cu:32-99).
namespace {
// Parameters of a draw: one pair of values for the whole tensor, or a pair of views read per element
struct DrawParams {
    double p0 = 0.0, p1 = 0.0;
    const void *d0 = nullptr, *d1 = nullptr;  // per-element parameter data (at the views' offsets) when both are set
    ViewDesc v0{}, v1{};
};

ttamd_status random_fill_impl(int device, ttamd_dtype dtype, int dist, const DrawParams &par, const uint64_t *states, const ViewDesc &v,
                              int64_t numel, void *data, int64_t offset, void *stream);
}  // namespace

ttamd_status ttamd_random_fill_states(int device, ttamd_dtype dtype, int dist, double p0, double p1, const uint64_t *states, int ndim,
                                      const int64_t *shape, const int64_t *stride, void *data, int64_t offset, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("random_fill: floating point dtypes only");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (offset < 0 || (dist != 0 && dist != 1) || (dist == 0 && !(p0 < p1))) {
        set_error("random_fill: invalid arguments (Expected low < high for uniform_real)");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ViewDesc v;
    int64_t numel = 0;
    if (ttamd_status s = make_view("random_fill", ndim, shape, stride, &v, &numel)) return s;
    DrawParams par;
    par.p0 = p0;
    par.p1 = p1;
    return random_fill_impl(device, dtype, dist, par, states, v, numel, data, offset, stream);
}

// The draws with a parameter pair per element: p0 / p1 are views over the same shape as the result (element offsets and
// strides, stride 0 for an expanded parameter), read on the device.  uniform_real expects low < high in every element,
// which the reference only asserts (common/kernel/distribution.hpp:95); it is not checked here.
ttamd_status ttamd_random_fill_states_params(int device, ttamd_dtype dtype, int dist, const void *p0, int64_t p0_offset,
                                             const int64_t *p0_stride, const void *p1, int64_t p1_offset, const int64_t *p1_stride,
                                             const uint64_t *states, int ndim, const int64_t *shape, const int64_t *stride, void *data,
                                             int64_t offset, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("random_fill: floating point dtypes only");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (offset < 0 || p0_offset < 0 || p1_offset < 0 || (dist != 0 && dist != 1)) {
        set_error("random_fill: invalid arguments (negative offset or unknown distribution)");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ViewDesc v;
    DrawParams par;
    int64_t numel = 0;
    if (ttamd_status s = make_view("random_fill", ndim, shape, stride, &v, &numel)) return s;
    if (ttamd_status s = make_view("random_fill", ndim, shape, p0_stride, &par.v0, nullptr)) return s;
    if (ttamd_status s = make_view("random_fill", ndim, shape, p1_stride, &par.v1, nullptr)) return s;
    if (numel > 0 && (!p0 || !p1)) {
        set_error("random_fill: NULL parameter pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const int64_t es = static_cast<int64_t>(dtype_size(dtype));
    par.d0 = static_cast<const char *>(p0) + p0_offset * es;
    par.d1 = static_cast<const char *>(p1) + p1_offset * es;
    return random_fill_impl(device, dtype, dist, par, states, v, numel, data, offset, stream);
}

namespace {
ttamd_status random_fill_impl(int device, ttamd_dtype dtype, int dist, const DrawParams &par, const uint64_t *states, const ViewDesc &v,
                              int64_t numel, void *data, int64_t offset, void *stream) {
    const double p0 = par.p0, p1 = par.p1;
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!data || !states) {
        set_error("random_fill: NULL data or states pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const bool dense = is_dense(v);
    void *out = static_cast<char *>(data) + offset * static_cast<int64_t>(dtype_size(dtype));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t state_bytes = static_cast<size_t>(numel) * sizeof(uint64_t);
    // staging: pinned host copy (the caller's array may be pageable and may go away when this call returns) and a
    // device copy; both are released once the stream has consumed them
    uint64_t *host_states = nullptr;
    TTAMD_HIP_CHECK(hipHostMalloc(reinterpret_cast<void **>(&host_states), state_bytes, hipHostMallocDefault));
    memcpy(host_states, states, state_bytes);
    void *dev_states = nullptr;
    hipError_t e = hipMalloc(&dev_states, state_bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipHostFree(host_states);
        set_error("random_fill: unable to allocate %lld generator states", static_cast<long long>(numel));
        return TTAMD_ERR_OUT_OF_MEMORY;
    }
    ttamd_status rc = TTAMD_OK;
    auto fail = [&](hipError_t err, const char *what) {
        set_error("%s failed: %s", what, hipGetErrorString(err));
        rc = TTAMD_ERR_LAUNCH;
    };
    if ((e = hipMemcpyAsync(dev_states, host_states, state_bytes, hipMemcpyHostToDevice, st)) != hipSuccess) fail(e, "hipMemcpyAsync");
    if (rc == TTAMD_OK) {
        const unsigned blocks = static_cast<unsigned>((numel + 255) / 256);
        const uint64_t *sp = static_cast<const uint64_t *>(dev_states);
        if (par.d0 && par.d1) {
            auto launch = [&]<typename T>(T) {
                const T *a = static_cast<const T *>(par.d0), *b = static_cast<const T *>(par.d1);
                if (dist == 0) random_params_kernel<T, 0><<<dim3(blocks), dim3(256), 0, st>>>(sp, a, par.v0, b, par.v1, static_cast<T *>(out), v, dense, numel);
                else random_params_kernel<T, 1><<<dim3(blocks), dim3(256), 0, st>>>(sp, a, par.v0, b, par.v1, static_cast<T *>(out), v, dense, numel);
            };
            if (dtype == TTAMD_F32) launch(float{});
            else launch(double{});
        } else if (dtype == TTAMD_F32) {
            if (dist == 0) uniform_real_kernel<float><<<dim3(blocks), dim3(256), 0, st>>>(sp, static_cast<float>(p0), static_cast<float>(p1), static_cast<float *>(out), v, dense, numel);
            else normal_kernel<float><<<dim3(blocks), dim3(256), 0, st>>>(sp, static_cast<float>(p0), static_cast<float>(p1), static_cast<float *>(out), v, dense, numel);
        } else {
            if (dist == 0) uniform_real_kernel<double><<<dim3(blocks), dim3(256), 0, st>>>(sp, p0, p1, static_cast<double *>(out), v, dense, numel);
            else normal_kernel<double><<<dim3(blocks), dim3(256), 0, st>>>(sp, p0, p1, static_cast<double *>(out), v, dense, numel);
        }
        if ((e = hipGetLastError()) != hipSuccess) fail(e, "kernel launch");
    }
    if ((e = hipStreamSynchronize(st)) != hipSuccess && rc == TTAMD_OK) fail(e, "hipStreamSynchronize");
    (void)hipFree(dev_states);
    (void)hipHostFree(host_states);
    return rc;
}
}  // namespace

// The same with the states drawn here: *master_state is the caller's master generator state (Generator::state, xorshift64
// with shifts 13, 7, 17: tensor/random.cpp:36-43); it advances by one output per element of the view.
ttamd_status ttamd_random_fill_view(int device, ttamd_dtype dtype, int dist, double p0, double p1, uint64_t *master_state, int ndim,
                                    const int64_t *shape, const int64_t *stride, void *data, int64_t offset, void *stream) {
    if (!master_state) {
        set_error("random_fill: master_state is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ViewDesc v;
    int64_t numel = 0;
    if (ttamd_status s = make_view("random_fill", ndim, shape, stride, &v, &numel)) return s;
    uint64_t *states = static_cast<uint64_t *>(malloc(static_cast<size_t>(numel > 0 ? numel : 1) * sizeof(uint64_t)));
    if (!states) {
        set_error("random_fill: unable to allocate %lld generator states on the host", static_cast<long long>(numel));
        return TTAMD_ERR_OUT_OF_MEMORY;
    }
    uint64_t x = *master_state;
    for (int64_t i = 0; i < numel; ++i) {
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        states[i] = x;
    }
    const ttamd_status rc = ttamd_random_fill_states(device, dtype, dist, p0, p1, states, ndim, shape, stride, data, offset, stream);
    free(states);
    if (rc == TTAMD_OK) *master_state = x;
    return rc;
}

// The dense case of ttamd_random_fill_view: `out` is a dense tensor of numel elements.
ttamd_status ttamd_random_fill(int device, ttamd_dtype dtype, int dist, double p0, double p1, uint64_t *master_state, int64_t numel,
                               void *out, void *stream) {
    if (numel < 0) {
        set_error("random_fill: negative element count");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const int64_t shape[1] = {numel}, stride[1] = {1};
    return ttamd_random_fill_view(device, dtype, dist, p0, p1, master_state, 1, shape, stride, out, 0, stream);
}

ttamd_status ttamd_mse_loss(int device, ttamd_dtype dtype, int64_t rows, int64_t cols, const void *input, const void *target,
                            void *loss_out, void *grad_input_out, void *grad_colsum_out, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("mse_loss: floating point dtypes only");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (rows < 0 || cols < 0 || rows * cols > 0x7fffffffLL) {
        set_error("mse_loss: invalid shape [%lld, %lld]", static_cast<long long>(rows), static_cast<long long>(cols));
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (grad_colsum_out && cols > 64) {
        set_error("mse_loss: the fused column sums serve at most 64 columns (given %lld); sum the gradient with ttamd_sum",
                  static_cast<long long>(cols));
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (!loss_out || (rows * cols > 0 && (!input || !target))) {
        set_error("mse_loss: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TTAMD_F32) return launch_mse_loss<float>(device, rows, cols, input, target, loss_out, grad_input_out, grad_colsum_out, st);
    return launch_mse_loss<double>(device, rows, cols, input, target, loss_out, grad_input_out, grad_colsum_out, st);
}

}  // extern "C"
