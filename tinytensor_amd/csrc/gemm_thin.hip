// gemm_thin.hip — products with at most 16 output columns (the 10-class head of an MLP: y = h . W of nn::Linear,
// tinytensor/nn/linear.cpp, and its weight gradient h^T . dy from TensorBatchedMatmul::backward,
// tinytensor/autograd/binary_ops.cpp:173-179), f32 and f64.
//
// The 64 x 64 tiles of the general kernels would spend three quarters of their MFMA work and of their B traffic on
// padding columns, and having too few tiles they split the reduction over workgroups and add the parts in a second
// kernel.  Here one workgroup owns 16 rows of C with all their columns and the whole reduction: its 16 waves share
// out k in interleaved chunks, every wave runs 16x16x4 MFMAs on operands it loads straight from memory into
// registers (each element of A is read exactly once by the whole grid, B is small and comes from L2), and the waves'
// 16 x 16 partial results are added through LDS in wave order.  One launch, one memory round trip per chunk.
//
// The second kernel here is for a reduction of at most 16 (dz = (dy . W^T) * mask with 10 classes: the product that
// carries the gradient back through the head): four MFMA steps make a 16 x 16 tile, so the kernel is a stream of
// tiles bounded by the mask it reads and the result it writes.  A workgroup owns a strip of 16 columns and up to 1024
// rows of it; B's 16 x 16 corner stays in registers, every wave issues the loads of all its tiles before the first
// MFMA, and a workgroup that owns all the rows of its strip finishes the bias gradient's column sums by itself.
//
// MFMA operand lanes (both dtypes): lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16] of a 16 x 4 by 4 x 16
// step.  Which k a step's four slices stand for is free as long as A and B agree, so a lane that loads a 16-byte
// vector of its row uses the vector's elements in consecutive steps.
#include "common.h"

namespace ttamd {
namespace {

typedef float thin_f32x4 __attribute__((ext_vector_type(4)));
typedef double thin_f64x4 __attribute__((ext_vector_type(4)));
typedef double thin_f64x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct ThinMma;
template <>
struct ThinMma<float> {
    static constexpr int VEC = 4;  // elements in 16 bytes
    using acc_t = thin_f32x4;
    using vec_t = thin_f32x4;
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    // accumulator element e of lane l is C[acc_row(e, l)][l % 16]
    static __device__ __forceinline__ int acc_row(int e, int lane) { return 4 * (lane / 16) + e; }
};
template <>
struct ThinMma<double> {
    static constexpr int VEC = 2;
    using acc_t = thin_f64x4;
    using vec_t = thin_f64x2;
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int acc_row(int e, int lane) { return 4 * e + lane / 16; }
};

// The loaded value is needed here, whatever is done with it afterwards.  Without this the compiler turns "load a
// stand-in, then select zero" into a branch around the load and waits for each such load by itself; with it, a run of
// loads followed by a run of keep() calls is a run of loads in flight together.
template <typename V>
__device__ __forceinline__ void keep(V &v) {
    asm volatile("" : "+v"(v));
}

constexpr int kThinWaves = 16;
constexpr int kThinMinK = 64;  // below this most waves would have nothing to do
constexpr int kSmallMinK = 128;
constexpr int64_t kSmallMaxBlocks = 512;
constexpr int64_t kThinKMinOutput = 64 * 64;  // smaller outputs of a short reduction: a single tile of the general kernels

// VECA: A's rows are contiguous in k, 16-byte aligned, and K is a whole number of 16-byte vectors.
template <typename T, bool VECA>
__global__ void __launch_bounds__(64 * kThinWaves) gemm_thin_kernel(GemmArgs g) {
    using MI = ThinMma<T>;
    using acc_t = typename MI::acc_t;
    constexpr int VEC = VECA ? MI::VEC : 1;
    constexpr int KC = 16 * MI::VEC;    // k per wave and iteration (64 f32, 32 f64)
    constexpr int NJ = KC / (4 * VEC);  // loads of A per lane and iteration
    __shared__ T red[kThinWaves][256];
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, q = lane / 16;
    const int batch = blockIdx.z, m0 = blockIdx.x * 16, n0 = blockIdx.y * 16;
    // Rows beyond M and columns beyond N read a valid element (row M-1, column N-1): a row's garbage stays in that
    // row, which is not stored; the columns' B values are zeroed.  Beyond K both operands are zeroed.
    const int row = m0 + li < g.M ? m0 + li : g.M - 1;
    const int col = n0 + li < g.N ? n0 + li : g.N - 1;
    const bool col_ok = n0 + li < g.N;
    const T *__restrict__ A = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(row) * g.a_sm;
    const T *__restrict__ B = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(col) * g.b_sn;
    acc_t acc0 = {}, acc1 = {};
    for (int64_t kb = static_cast<int64_t>(wave) * KC; kb < g.K; kb += kThinWaves * KC) {
        T a[NJ][VEC], b[NJ][VEC];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {  // every load of the chunk goes out before the first is used
            const int64_t k = kb + (j * 4 + q) * VEC;
            const bool ok = k < g.K;
            const int64_t kc = ok ? k : 0;  // (no branch around a load: an address that is always valid instead)
            if constexpr (VEC > 1) {
                const typename MI::vec_t v = *reinterpret_cast<const typename MI::vec_t *>(A + kc);
#pragma unroll
                for (int s = 0; s < VEC; ++s) a[j][s] = ok ? v[s] : T(0);
            } else {
                const T v = A[kc * g.a_sk];
                a[j][0] = ok ? v : T(0);
            }
#pragma unroll
            for (int s = 0; s < VEC; ++s) {
                const T v = B[(kc + s) * g.b_sk];
                b[j][s] = ok && col_ok ? v : T(0);
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int s = 0; s < VEC; ++s) {  // two accumulators: half the length of the dependent MFMA chain
                if ((j * VEC + s) & 1) acc1 = MI::mma(a[j][s], b[j][s], acc1);
                else acc0 = MI::mma(a[j][s], b[j][s], acc0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][e * 64 + lane] = acc0[e] + acc1[e];
    __syncthreads();
    if (tid >= 256) return;
    T v = T(0);
#pragma unroll
    for (int w = 0; w < kThinWaves; ++w) v += red[w][tid];  // wave order: deterministic
    const int e = tid / 64, l = tid % 64;
    const int m = m0 + MI::acc_row(e, l), n = n0 + l % 16;
    if (m >= g.M || n >= g.N) return;
    // The store's steps in the order of the general kernels: bias, ReLU-backward mask, ReLU, accumulate, second output.
    const int64_t idx = (static_cast<int64_t>(batch) * g.M + m) * g.N + n;
    const T *bias = static_cast<const T *>(g.bias);
    if (g.bias_mode == 1) v += bias[n];
    if (g.bias_mode == 2) v += bias[m];
    if (g.zmask && static_cast<const T *>(g.zmask)[idx] < T(0)) v = v * T(0);  // the reference multiplies by 0: an infinite or NaN value under the mask stays NaN
    if (g.relu) v = v > T(0) ? v : T(0);
    T *C = static_cast<T *>(g.C);
    if (g.accumulate) v += C[idx];
    C[idx] = v;
    if (g.relu_out) static_cast<T *>(g.relu_out)[idx] = v > T(0) ? v : T(0);
}

// ---------------------------------------------------------------------------------------------------------------
// K <= 16.  Where a lane's four accumulator elements sit in the 16 x 16 tile decides how it stores them:
//   f32, computed as the transposed tile (B's slice as the first operand): row l % 16, columns 4 * (l / 16) + e --
//        four consecutive columns, one 16-byte store when the row length allows;
//   f64: rows 4 * e + l / 16, column l % 16 -- 16 lanes write 128 contiguous bytes of a row.
template <typename T>
struct ThinTile;
template <>
struct ThinTile<float> {
    static constexpr bool kTransposed = true;
    static __device__ __forceinline__ int row(int e, int lane) { return lane % 16; }
    static __device__ __forceinline__ int col(int e, int lane) { return 4 * (lane / 16) + e; }
};
template <>
struct ThinTile<double> {
    static constexpr bool kTransposed = false;
    static __device__ __forceinline__ int row(int e, int lane) { return 4 * e + lane / 16; }
    static __device__ __forceinline__ int col(int e, int lane) { return lane % 16; }
};

// TPW tiles per wave; a workgroup's 16 waves take the 16 * TPW row tiles of its block in turn (tile = u * 16 + wave,
// rotated by the strip's number).
// colsum_dst: [batch][gridDim.y][N] -- the launcher passes the final array when gridDim.y == 1.
template <typename T, int TPW>
__global__ void __launch_bounds__(64 * kThinWaves) gemm_thin_k_kernel(GemmArgs g, T *__restrict__ colsum_dst, int vec_rows) {
    using MI = ThinMma<T>;
    using TL = ThinTile<T>;
    using acc_t = typename MI::acc_t;
    __shared__ T red[kThinWaves][16];
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, q = lane / 16;
    const int n0 = blockIdx.x * 16, batch = blockIdx.z;
    const int m_block = blockIdx.y * (256 * TPW);
    // Neighbouring strips start at different row tiles: rows are a multiple of the memory channels' interleave apart
    // when N is a power of two, and strips that walked the rows in step would all queue at the same channels.
    const int rot = blockIdx.x % (kThinWaves * TPW);
    const T *__restrict__ A = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb;
    const T *__restrict__ B = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb;
    const T *__restrict__ Z = g.zmask ? static_cast<const T *>(g.zmask) + static_cast<int64_t>(batch) * g.M * g.N : nullptr;
    T *__restrict__ C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    T *__restrict__ R = g.relu_out ? static_cast<T *>(g.relu_out) + static_cast<int64_t>(batch) * g.M * g.N : nullptr;
    // Step s of a tile multiplies slice k = 4 s + q.  Beyond K, M or N the loads read a valid stand-in element and the
    // value is zeroed (beyond K on both sides, so that no stand-in infinity meets a zero).
    // Every load of the wave's tiles goes out before the first value is looked at.
    T bop[4], aop[TPW][4], zv[TPW][4];
    acc_t zvec[TPW];
    const bool vec = TL::kTransposed && vec_rows;  // (then N is a multiple of 4: a lane's four columns are in range together)
    {
        const int n = n0 + li < g.N ? n0 + li : g.N - 1;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int k = 4 * s + q;
            bop[s] = B[static_cast<int64_t>(k < g.K ? k : 0) * g.b_sk + static_cast<int64_t>(n) * g.b_sn];
        }
    }
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int m0 = m_block + ((u * kThinWaves + wave + rot) % (kThinWaves * TPW)) * 16;
        const int m = m0 + li < g.M ? m0 + li : g.M - 1;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int k = 4 * s + q;
            aop[u][s] = A[static_cast<int64_t>(m) * g.a_sm + static_cast<int64_t>(k < g.K ? k : 0) * g.a_sk];
        }
    }
    if (Z && vec) {  // workgroup-uniform
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
            const int m0 = m_block + ((u * kThinWaves + wave + rot) % (kThinWaves * TPW)) * 16;
            const int zr = m0 + TL::row(0, lane) < g.M ? m0 + TL::row(0, lane) : g.M - 1;
            const int zc = n0 + TL::col(0, lane) < g.N ? n0 + TL::col(0, lane) : 0;
            zvec[u] = *reinterpret_cast<const acc_t *>(Z + static_cast<int64_t>(zr) * g.N + zc);
        }
#pragma unroll
        for (int u = 0; u < TPW; ++u) keep(zvec[u]);
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
#pragma unroll
            for (int e = 0; e < 4; ++e) zv[u][e] = zvec[u][e];
        }
    } else if (Z) {
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
            const int m0 = m_block + ((u * kThinWaves + wave + rot) % (kThinWaves * TPW)) * 16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = m0 + TL::row(e, lane) < g.M ? m0 + TL::row(e, lane) : g.M - 1;
                const int c = n0 + TL::col(e, lane) < g.N ? n0 + TL::col(e, lane) : g.N - 1;
                zv[u][e] = Z[static_cast<int64_t>(r) * g.N + c];
            }
        }
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
#pragma unroll
            for (int e = 0; e < 4; ++e) keep(zv[u][e]);
        }
    } else {
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
#pragma unroll
            for (int e = 0; e < 4; ++e) zv[u][e] = T(0);
        }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        keep(bop[s]);
        bop[s] = 4 * s + q < g.K && n0 + li < g.N ? bop[s] : T(0);
    }
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            keep(aop[u][s]);
            aop[u][s] = 4 * s + q < g.K ? aop[u][s] : T(0);
        }
    }
    const T *bias = static_cast<const T *>(g.bias);
    T csum[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int m0 = m_block + ((u * kThinWaves + wave + rot) % (kThinWaves * TPW)) * 16;
        acc_t acc = {};
#pragma unroll
        for (int s = 0; s < 4; ++s) acc = TL::kTransposed ? MI::mma(bop[s], aop[u][s], acc) : MI::mma(aop[u][s], bop[s], acc);
        T out[4];
        bool in[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // bias, ReLU-backward mask, ReLU, accumulate: the order of the general kernels
            const int m = m0 + TL::row(e, lane), n = n0 + TL::col(e, lane);
            in[e] = m < g.M && n < g.N;
            T v = acc[e];
            if (g.bias_mode == 1 && in[e]) v += bias[n];
            if (g.bias_mode == 2 && in[e]) v += bias[m];
            if (zv[u][e] < T(0)) v = v * T(0);  // the reference multiplies by 0: an infinite or NaN value under the mask stays NaN
            if (g.relu) v = v > T(0) ? v : T(0);
            if (g.accumulate && in[e]) v += C[static_cast<int64_t>(m) * g.N + n];
            out[e] = v;
            csum[e] += in[e] ? v : T(0);
        }
        if (TL::kTransposed && vec_rows) {
            if (in[0]) {  // a lane's four columns are in range together
                const int64_t idx = static_cast<int64_t>(m0 + TL::row(0, lane)) * g.N + n0 + TL::col(0, lane);
                acc_t o, r;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o[e] = out[e];
                    r[e] = out[e] > T(0) ? out[e] : T(0);
                }
                *reinterpret_cast<acc_t *>(C + idx) = o;
                if (R) *reinterpret_cast<acc_t *>(R + idx) = r;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (!in[e]) continue;
                const int64_t idx = static_cast<int64_t>(m0 + TL::row(e, lane)) * g.N + n0 + TL::col(e, lane);
                C[idx] = out[e];
                if (R) R[idx] = out[e] > T(0) ? out[e] : T(0);
            }
        }
    }
    if (!colsum_dst) return;  // workgroup-uniform
    // Column sums of the block's rows: over a wave's lanes first, then over the waves in wave order.
    if (TL::kTransposed) {  // lanes of one q hold 16 rows of columns 4 q + e
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int d = 1; d < 16; d *= 2) csum[e] += __shfl_xor(csum[e], d, 64);
        }
        if (li == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][4 * q + e] = csum[e];
        }
    } else {  // a lane holds four rows of column l % 16; the other twelve are in the lanes 16, 32, 48 further on
        T v = (csum[0] + csum[1]) + (csum[2] + csum[3]);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (lane < 16) red[wave][lane] = v;
    }
    __syncthreads();
    if (tid < 16 && n0 + tid < g.N) {
        T v = T(0);
#pragma unroll
        for (int w = 0; w < kThinWaves; ++w) v += red[w][tid];
        colsum_dst[(static_cast<int64_t>(batch) * gridDim.y + blockIdx.y) * g.N + n0 + tid] = v;
    }
}

template <typename T>
ttamd_status launch_thin_k_typed(ttamd_dtype dt, const GemmArgs &g, int device, hipStream_t stream, bool fixed_scratch) {
    const int strips = (g.N + 15) / 16;
    // With column sums: 1024 rows to a workgroup, so that up to 1024 rows finish their sums inside the kernel and longer
    // matrices leave few partial rows; fewer rows when the matrix is shorter.  Without: 256 rows, the most workgroups
    // (measured at 1024 x 10 x 1024: 6.3 us against 8.9).
    int tpw = g.colsum_out ? 4 : 1;
    while (tpw > 1 && g.M <= 256 * (tpw / 2)) tpw /= 2;
    const int row_blocks = (g.M + 256 * tpw - 1) / (256 * tpw);
    if (row_blocks > 65535 || g.batch > 65535) {
        set_error("batched_matmul: %d row blocks by %d batch items exceed the grid limit", row_blocks, g.batch);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    T *colsum_dst = static_cast<T *>(g.colsum_out);
    if (g.colsum_out && row_blocks > 1) {  // partial rows now, colsum_reduce adds them
        void *ws = nullptr;
        const size_t bytes = static_cast<size_t>(g.batch) * row_blocks * g.N * sizeof(T);
        if (ttamd_status st = gemm_scratch(device, stream, bytes, fixed_scratch, &ws)) return st;
        colsum_dst = static_cast<T *>(ws);
    }
    auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const int vec_rows = g.N % 4 == 0 && aligned(g.C) && aligned(g.zmask) && aligned(g.relu_out) ? 1 : 0;
    const dim3 grid(static_cast<unsigned>(strips), static_cast<unsigned>(row_blocks), static_cast<unsigned>(g.batch)), block(64 * kThinWaves);
    if (tpw == 4) gemm_thin_k_kernel<T, 4><<<grid, block, 0, stream>>>(g, colsum_dst, vec_rows);
    else if (tpw == 2) gemm_thin_k_kernel<T, 2><<<grid, block, 0, stream>>>(g, colsum_dst, vec_rows);
    else gemm_thin_k_kernel<T, 1><<<grid, block, 0, stream>>>(g, colsum_dst, vec_rows);
    TTAMD_HIP_CHECK(hipGetLastError());
    if (g.colsum_out && row_blocks > 1) return launch_colsum_reduce(dt, colsum_dst, row_blocks, g.N, g.batch, g.colsum_out, stream);
    return TTAMD_OK;
}

template <typename T>
ttamd_status launch_thin_typed(const GemmArgs &g, hipStream_t stream, const char **variant, bool variant_only, const char *name_vec,
                               const char *name_any) {
    constexpr int VEC = ThinMma<T>::VEC;
    const bool vec = g.a_sk == 1 && g.K % VEC == 0 && g.a_sm % VEC == 0 && g.a_sb % VEC == 0 &&
                     (variant_only || reinterpret_cast<uintptr_t>(g.A) % 16 == 0);
    *variant = vec ? name_vec : name_any;
    if (variant_only) return TTAMD_OK;
    const dim3 grid(static_cast<unsigned>((g.M + 15) / 16), static_cast<unsigned>((g.N + 15) / 16), static_cast<unsigned>(g.batch));
    const dim3 block(64 * kThinWaves);
    if (vec) gemm_thin_kernel<T, true><<<grid, block, 0, stream>>>(g);
    else gemm_thin_kernel<T, false><<<grid, block, 0, stream>>>(g);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// The head of an MLP in two launches: y = x . W + b of a Linear layer with at most 16 outputs (nn/linear.cpp:42-50),
// nn::mse_loss(y, t) with mean reduction (nn/loss.cpp:69-72) and the backward of both -- dy = (1 / numel) * 2 * (y - t)
// (autograd/reduce_ops.cpp:201-205, binary_ops.cpp:153-159), dx = (dy . W^T) * where(relu_input < 0, 0, 1)
// (binary_ops.cpp:173-179, unary_ops.cpp:568-573), dW = x^T . dy, db = dy summed over the rows.  As four separate
// launches (the two kernels above, the short-reduction product of the general kernels and mse_loss) each step is a
// launch and a memory round trip long, 5 - 6 us, for a few MFLOP.  Here the first kernel is gemm_thin_kernel with the
// loss's element-wise steps in its store (y, dy, and per block of 16 rows the parts of the loss and of db), and the
// second runs gemm_thin_k_kernel's strips of 16 columns of dx and, in workgroups of their own beside them, the same
// strips of dW (each a sum over all the rows; beyond 1024 rows in stretches that a third small kernel adds up), and
// one workgroup that adds up the first kernel's parts of db and of the loss.  All sums in fixed orders.
struct HeadArgs {
    const float *x, *w, *bias, *t, *z;  // x [R,K], w [K,N], bias [N] or null, t [R,N], z [R,K] or null; all dense
    float *y, *dy, *dx, *dw, *db, *loss;  // y, dy [R,N], dx [R,K], dw [K,N], db [N] or null, loss [1]
    float *part_b, *part_l;             // [row blocks][16], [row blocks]
    // dy once more for the second kernel's 16-byte loads, per block of 16 rows and zero beyond R and N:
    // dy_rows[block][r][j] and dy_cols[block][j][r]
    float *dy_rows, *dy_cols;
    float *part_w;  // [stretches of 1024 rows][strips of 16 k][16 x 16]: the stretches' tiles of dW (more than one stretch)
    int R, K, N;
    float inv_n;  // 1 / (R * N)
};

// y = x . W + b for a block of 16 rows (gemm_thin_kernel<float, true>), then d = y - t, dy = ((1 / numel) * 2) * d, and the
// block's sums of d * d / numel and of dy's columns.
__global__ void __launch_bounds__(64 * kThinWaves) linear_mse_head_forward_kernel(HeadArgs a) {
    using MI = ThinMma<float>;
    using acc_t = MI::acc_t;
    __shared__ float red[kThinWaves][256];
    __shared__ float dyt[16][17];
    __shared__ float lterm[256];
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, q = lane / 16;
    const int m0 = blockIdx.x * 16;
    const int row = m0 + li < a.R ? m0 + li : a.R - 1;
    const int col = li < a.N ? li : a.N - 1;
    const bool col_ok = li < a.N;
    const float *__restrict__ A = a.x + static_cast<int64_t>(row) * a.K;
    const float *__restrict__ B = a.w + col;
    acc_t acc0 = {}, acc1 = {};
    for (int kb = wave * 64; kb < a.K; kb += kThinWaves * 64) {
        float av[4][4], bv[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // every load of the chunk goes out before the first is used
            const int k = kb + (j * 4 + q) * 4;
            const bool ok = k < a.K;
            const int kc = ok ? k : 0;
            const thin_f32x4 v = *reinterpret_cast<const thin_f32x4 *>(A + kc);
#pragma unroll
            for (int s = 0; s < 4; ++s) av[j][s] = ok ? v[s] : 0.f;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float b = B[static_cast<int64_t>(kc + s) * a.N];
                bv[j][s] = ok && col_ok ? b : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if ((j * 4 + s) & 1) acc1 = MI::mma(av[j][s], bv[j][s], acc1);
                else acc0 = MI::mma(av[j][s], bv[j][s], acc0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][e * 64 + lane] = acc0[e] + acc1[e];
    __syncthreads();
    if (tid < 256) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kThinWaves; ++w) v += red[w][tid];  // wave order: deterministic (and gemm_thin_kernel's order)
        const int e = tid / 64, l = tid % 64;
        const int ml = MI::acc_row(e, l), n = l % 16, m = m0 + ml;
        float g = 0.f, term = 0.f;
        if (m < a.R && n < a.N) {
            const int64_t idx = static_cast<int64_t>(m) * a.N + n;
            if (a.bias) v += a.bias[n];
            const float d = v - a.t[idx];
            g = (a.inv_n * 2.0f) * d;
            term = d * d * a.inv_n;
            a.y[idx] = v;
            a.dy[idx] = g;
        }
        dyt[ml][n] = g;
        lterm[tid] = term;
    }
    __syncthreads();
    if (tid < 256) {
        const int64_t o = static_cast<int64_t>(blockIdx.x) * 256 + tid;
        a.dy_rows[o] = dyt[tid / 16][tid % 16];
        a.dy_cols[o] = dyt[tid % 16][tid / 16];
    }
    if (wave == 0) {
        float s = (lterm[lane] + lterm[lane + 64]) + (lterm[lane + 128] + lterm[lane + 192]);
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) s += __shfl_down(s, d, 64);
        if (lane == 0) a.part_l[blockIdx.x] = s;
    } else if (wave == 1 && lane < 16) {
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) s += dyt[r][lane];
        a.part_b[blockIdx.x * 16 + lane] = s;
    }
}

constexpr int kHeadTiles = 4;  // 16-row tiles per wave of the second kernel

// db's columns and the loss from the first kernel's parts, by one workgroup of 256: column c (16 = the loss) is summed by
// 15 lanes, lane p over the blocks p, p + 15, ... in ascending order, and their sums are added in the order of p: a fixed
// order.  The parts pass through LDS, 240 blocks at a time, so that their loads are in flight together.
__device__ __forceinline__ void head_sums(const HeadArgs &a, int row_blocks) {
    constexpr int kChunk = 240, kLanes = 15;  // 17 * 15 = 255 threads at work
    __shared__ float buf[kChunk * 17];
    __shared__ float part[17 * kLanes];
    const int tid = threadIdx.x, c = tid / kLanes, p = tid % kLanes;
    float acc = 0.f;
    for (int b0 = 0; b0 < row_blocks; b0 += kChunk) {
        const int nb = row_blocks - b0 < kChunk ? row_blocks - b0 : kChunk;
        for (int e = tid; e < nb * 17; e += 64 * 4) {
            const int b = b0 + e / 17, col = e % 17;
            buf[e] = col < 16 ? a.part_b[b * 16 + col] : a.part_l[b];
        }
        __syncthreads();
        if (c < 17)
            for (int b = p; b < nb; b += kLanes) acc += buf[b * 17 + c];
        __syncthreads();
    }
    if (c < 17) part[c * kLanes + p] = acc;
    __syncthreads();
    if (tid < 17) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kLanes; ++i) s += part[tid * kLanes + i];
        if (tid == 16) a.loss[0] = s;
        else if (a.db && tid < a.N) a.db[tid] = s;
    }
}

// The second kernel: workgroups of four waves in two roles, told apart by blockIdx.y.  Both products as transposed
// tiles, and with the reduced index of a step's slice q numbered 4 q + s (s the step), so that a lane's four values of
// dy are one 16-byte load.
//   blockIdx.y >= stretches: columns k0 .. k0 + 15 of dx = (dy . W^T) * mask for a chunk of 256 rows, four 16-row tiles per
//     wave.  dx^T = W . dy^T: first operand W[k0 + li][j], second dy[r = li][j], j = 4 q + s: the lane holds
//     dx[m0 + li][k0 + 4 q + e], four consecutive columns -- the mask's 16-byte load, the result's 16-byte store.
//   blockIdx.y < stretches: rows k0 .. k0 + 15 of dW = x^T . dy over a stretch of 1024 rows, sixteen tiles per wave.
//     dW^T = dy^T . x: first operand dy[r][j = li], second x[r][k0 + li], r = 4 q + s: the lane holds
//     dW[k0 + li][4 q + e]; the four waves' tiles are added through LDS in wave order.  With one stretch that is dW's
//     tile; with more, part_w[stretch][strip] receives it and the finishing kernel adds the stretches in order.
// One workgroup beside the strips' adds up the first kernel's parts of db and of the loss.
constexpr int kHeadWaves = 4;
constexpr int kHeadChunkRows = kHeadWaves * kHeadTiles * 16;  // 256
constexpr int kHeadStretchRows = 4 * kHeadChunkRows;           // 1024
__global__ void __launch_bounds__(64 * kHeadWaves) linear_mse_head_backward_kernel(HeadArgs a, int row_blocks, int chunks, int stretches) {
    using MI = ThinMma<float>;
    using acc_t = MI::acc_t;
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, q = lane / 16;
    const int strips = gridDim.x - 1;
    if (static_cast<int>(blockIdx.x) == strips) {  // (uniform: no barrier is left waiting)
        if (blockIdx.y == 0) head_sums(a, row_blocks);
        return;
    }
    const int k0 = blockIdx.x * 16;
    const bool k_ok = k0 + li < a.K;  // this lane's row of W / column of x
    const int kr = k_ok ? k0 + li : 0;
    // Neighbouring strips start at different row tiles (tile u of this wave: u * 4 + wave, rotated by the strip's number):
    // rows are a multiple of the memory channels' interleave apart when K is a power of two, and strips that walked the
    // rows in step would all queue at the same channels.
    const int rot = blockIdx.x % (kHeadWaves * kHeadTiles);
    if (static_cast<int>(blockIdx.y) >= stretches) {  // (the longer-running role is launched first)
        const bool kv_ok = k0 + 4 * q < a.K;  // this lane's four columns of dx (K is a multiple of 4: in range together)
        const int kz = kv_ok ? k0 + 4 * q : 0;
        const int base = (blockIdx.y - stretches) * kHeadChunkRows;
        float wf[4];
        thin_f32x4 dyb[kHeadTiles], zv[kHeadTiles];
#pragma unroll
        for (int s = 0; s < 4; ++s) {  // every load of the wave goes out before the first is used
            const int j = 4 * q + s;
            wf[s] = a.w[static_cast<int64_t>(kr) * a.N + (j < a.N ? j : 0)];
        }
#pragma unroll
        for (int u = 0; u < kHeadTiles; ++u) {
            const int m0 = base + ((u * kHeadWaves + wave + rot) % (kHeadWaves * kHeadTiles)) * 16;
            const int blk = m0 / 16 < row_blocks ? m0 / 16 : row_blocks - 1;
            const int rl = m0 + li < a.R ? m0 + li : a.R - 1;
            dyb[u] = *reinterpret_cast<const thin_f32x4 *>(a.dy_rows + static_cast<int64_t>(blk) * 256 + li * 16 + 4 * q);
            zv[u] = a.z ? *reinterpret_cast<const thin_f32x4 *>(a.z + static_cast<int64_t>(rl) * a.K + kz) : thin_f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            keep(wf[s]);
            wf[s] = k_ok && 4 * q + s < a.N ? wf[s] : 0.f;  // (dy's copies are zero beyond R and N: no stand-in value meets a zero)
        }
#pragma unroll
        for (int u = 0; u < kHeadTiles; ++u) {
            keep(dyb[u]);
            keep(zv[u]);
        }
#pragma unroll
        for (int u = 0; u < kHeadTiles; ++u) {
            const int m0 = base + ((u * kHeadWaves + wave + rot) % (kHeadWaves * kHeadTiles)) * 16;
            if (m0 >= a.R) continue;  // wave-uniform (every lane of the wave takes part in an MFMA)
            acc_t dxa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) dxa = MI::mma(wf[s], dyb[u][s], dxa);
            thin_f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = zv[u][e] < 0.f ? dxa[e] * 0.f : dxa[e];  // a product, as the reference's mask is
            if (m0 + li < a.R && kv_ok) *reinterpret_cast<thin_f32x4 *>(a.dx + static_cast<int64_t>(m0 + li) * a.K + k0 + 4 * q) = o;
        }
        return;
    }
    __shared__ float red[kHeadWaves][256];
    const int stretch = blockIdx.y;
    const int first = stretch * kHeadStretchRows;
    const int end = first + kHeadStretchRows < a.R ? first + kHeadStretchRows : a.R;
    constexpr int kTiles = kHeadTiles;  // per wave and pass (256 rows): their loads are in flight together
    const int rot_w = blockIdx.x % (kHeadWaves * kTiles);
    acc_t wacc0 = {0.f, 0.f, 0.f, 0.f}, wacc1 = {0.f, 0.f, 0.f, 0.f};
    for (int base = first; base < end; base += kHeadWaves * kTiles * 16) {
        thin_f32x4 dya[kTiles];
        float xf[kTiles][4];
#pragma unroll
        for (int u = 0; u < kTiles; ++u) {
            const int m0 = base + ((u * kHeadWaves + wave + rot_w) % (kHeadWaves * kTiles)) * 16;
            const int blk = m0 / 16 < row_blocks ? m0 / 16 : row_blocks - 1;
            dya[u] = *reinterpret_cast<const thin_f32x4 *>(a.dy_cols + static_cast<int64_t>(blk) * 256 + li * 16 + 4 * q);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int r = m0 + 4 * q + s;
                xf[u][s] = a.x[static_cast<int64_t>(r < a.R ? r : a.R - 1) * a.K + kr];
            }
        }
#pragma unroll
        for (int u = 0; u < kTiles; ++u) {
#pragma unroll
            for (int s = 0; s < 4; ++s) keep(xf[u][s]);
            keep(dya[u]);
        }
#pragma unroll
        for (int u = 0; u < kTiles; ++u) {
            const int m0 = base + ((u * kHeadWaves + wave + rot_w) % (kHeadWaves * kTiles)) * 16;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                // beyond R the stand-in row of x is zeroed, and beyond K its stand-in column: dy's zeros there meet zeros
                const float xv = m0 + 4 * q + s < a.R && k_ok ? xf[u][s] : 0.f;
                const float dv = m0 < a.R ? dya[u][s] : 0.f;  // (a tile beyond R: the stand-in block's dy is not this tile's)
                if (s & 1) wacc1 = MI::mma(dv, xv, wacc1);
                else wacc0 = MI::mma(dv, xv, wacc0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][e * 64 + lane] = wacc0[e] + wacc1[e];
    __syncthreads();
    // element tid of the tile: e = tid / 64, lane l = tid % 64: dW[k0 + l % 16][4 (l / 16) + e]
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < kHeadWaves; ++w) v += red[w][tid];  // wave order: deterministic
    const int k = k0 + tid % 16, j = 4 * ((tid % 64) / 16) + tid / 64;
    if (stretches > 1) a.part_w[(static_cast<int64_t>(stretch) * strips + blockIdx.x) * 256 + tid] = v;
    else if (k < a.K && j < a.N) a.dw[static_cast<int64_t>(k) * a.N + j] = v;
}

// dW's 16 x 16 tiles from the stretches' tiles, added in the order of the stretches.
__global__ void __launch_bounds__(256) linear_mse_head_finish_kernel(HeadArgs a, int strips, int stretches) {
    const int tid = threadIdx.x;
    const float *tiles = a.part_w + static_cast<int64_t>(blockIdx.x) * 256 + tid;
    float sum = 0.f;
    int c = 0;
    for (; c + 8 <= stretches; c += 8) {  // eight loads in flight, added in order
        float t[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = tiles[static_cast<int64_t>(c + i) * strips * 256];
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += t[i];
    }
    for (; c < stretches; ++c) sum += tiles[static_cast<int64_t>(c) * strips * 256];
    const int k = blockIdx.x * 16 + tid % 16, j = 4 * ((tid % 64) / 16) + tid / 64;
    if (k < a.K && j < a.N) a.dw[static_cast<int64_t>(k) * a.N + j] = sum;
}

constexpr int64_t kHeadMaxRows = 16384;  // (16 stretches of 1024 rows)
constexpr int64_t kHeadMaxElements = int64_t(1) << 26;  // of the input (the stretches' tiles of dW take a 64th of that); larger
                                                        // layers fill the chip with the separate products

}  // namespace

// The launcher of the two kernels above; *handled = false (and nothing launched) when the operands rule them out.
ttamd_status launch_linear_mse_head(int device, int64_t rows, int64_t in_features, int64_t out_features, const void *input,
                                    const void *weight, const void *bias, const void *target, const void *relu_input, void *output,
                                    void *loss_out, void *grad_output_out, void *grad_input_out, void *grad_weight_out,
                                    void *grad_bias_out, hipStream_t stream, bool *handled) {
    *handled = false;
    auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (rows < 1 || rows > kHeadMaxRows || in_features < 16 || in_features % 4 != 0 || in_features > (1 << 20) || out_features < 1 ||
        out_features > 16 || rows * in_features > kHeadMaxElements)
        return TTAMD_OK;
    if (!aligned(input) || !aligned(relu_input) || !aligned(grad_input_out)) return TTAMD_OK;
    HeadArgs a{};
    a.x = static_cast<const float *>(input);
    a.w = static_cast<const float *>(weight);
    a.bias = static_cast<const float *>(bias);
    a.t = static_cast<const float *>(target);
    a.z = static_cast<const float *>(relu_input);
    a.y = static_cast<float *>(output);
    a.dy = static_cast<float *>(grad_output_out);
    a.dx = static_cast<float *>(grad_input_out);
    a.dw = static_cast<float *>(grad_weight_out);
    a.db = static_cast<float *>(grad_bias_out);
    a.loss = static_cast<float *>(loss_out);
    a.R = static_cast<int>(rows);
    a.K = static_cast<int>(in_features);
    a.N = static_cast<int>(out_features);
    a.inv_n = 1.0f / static_cast<float>(rows * out_features);
    const int row_blocks = static_cast<int>((rows + 15) / 16);
    const int strips = (a.K + 15) / 16, chunks = (a.R + kHeadChunkRows - 1) / kHeadChunkRows;
    const int stretches = (a.R + kHeadStretchRows - 1) / kHeadStretchRows;
    const size_t tile_floats = stretches > 1 ? static_cast<size_t>(stretches) * strips * 256 : 0;
    void *ws = nullptr;
    if (ttamd_status st = stream_scratch(device, stream, (static_cast<size_t>(row_blocks) * (512 + 17) + tile_floats) * sizeof(float), &ws))
        return st;
    a.dy_rows = static_cast<float *>(ws);
    a.dy_cols = a.dy_rows + static_cast<size_t>(row_blocks) * 256;
    a.part_w = a.dy_cols + static_cast<size_t>(row_blocks) * 256;
    a.part_b = a.part_w + tile_floats;
    a.part_l = a.part_b + static_cast<size_t>(row_blocks) * 16;
    *handled = true;
    linear_mse_head_forward_kernel<<<dim3(static_cast<unsigned>(row_blocks)), dim3(64 * kThinWaves), 0, stream>>>(a);
    TTAMD_HIP_CHECK(hipGetLastError());
    // (one column of workgroups more than strips: its first adds up db and the loss while the strips run)
    linear_mse_head_backward_kernel<<<dim3(static_cast<unsigned>(strips + 1), static_cast<unsigned>(chunks + stretches)), dim3(64 * kHeadWaves), 0,
                                      stream>>>(a, row_blocks, chunks, stretches);
    TTAMD_HIP_CHECK(hipGetLastError());
    if (stretches > 1) {
        linear_mse_head_finish_kernel<<<dim3(static_cast<unsigned>(strips)), dim3(256), 0, stream>>>(a, strips, stretches);
        TTAMD_HIP_CHECK(hipGetLastError());
    }
    return TTAMD_OK;
}

ttamd_status launch_gemm_thin(ttamd_dtype dt, const GemmArgs &g, int device, hipStream_t stream, const char **variant,
                              bool variant_only, bool *handled, bool fixed_scratch) {
    *handled = false;
    if ((dt == TTAMD_F32 || dt == TTAMD_F64) && g.K <= 16 && g.N >= 16 && static_cast<int64_t>(g.M) * g.N >= kThinKMinOutput &&
        g.batch <= 65535 && (g.M + 255) / 256 <= 65535) {  // (grid limits: anything beyond goes to the general kernels)
        *handled = true;
        *variant = dt == TTAMD_F32 ? "thin_f32_k16" : "thin_f64_k16";
        if (variant_only) return TTAMD_OK;
        return dt == TTAMD_F32 ? launch_thin_k_typed<float>(dt, g, device, stream, fixed_scratch)
                               : launch_thin_k_typed<double>(dt, g, device, stream, fixed_scratch);
    }
    if ((dt != TTAMD_F32 && dt != TTAMD_F64) || g.colsum_out || g.batch > 65535) return TTAMD_OK;
    const int64_t blocks = static_cast<int64_t>((g.M + 15) / 16) * ((g.N + 15) / 16) * g.batch;
    // A wave's share of k is a chain of memory round trips, one per chunk: beyond four chunks per wave (two when A's
    // rows cannot be read as vectors) the tiles with their reduction split over workgroups are faster again
    // (measured at 1024 x K x 10, f32: 12.2 against 14.9 us at K = 4096, 23.7 against 21.5 at K = 8192).
    const int vec_len = dt == TTAMD_F32 ? 4 : 2;
    const bool rows_vec = g.a_sk == 1 && g.K % vec_len == 0 && g.a_sm % vec_len == 0 && g.a_sb % vec_len == 0;
    const int max_k = (rows_vec ? 4 : 2) * kThinWaves * 16 * vec_len;
    const bool thin = g.N <= 16 && g.K >= kThinMinK && g.K <= max_k;
    // A small output with a long reduction: on 64 x 64 tiles it would have a few tiles, split k over workgroups and add
    // the parts in a second kernel.  As 16 x 16 blocks it fills the chip in one round of workgroups (two fit a CU).
    const bool small = g.N > 16 && g.K >= kSmallMinK && g.K <= max_k && blocks <= kSmallMaxBlocks;
    if (!thin && !small) return TTAMD_OK;
    *handled = true;
    if (dt == TTAMD_F32)
        return thin ? launch_thin_typed<float>(g, stream, variant, variant_only, "thin_f32_16rows_vec4", "thin_f32_16rows")
                    : launch_thin_typed<float>(g, stream, variant, variant_only, "small_f32_16x16_vec4", "small_f32_16x16");
    return thin ? launch_thin_typed<double>(g, stream, variant, variant_only, "thin_f64_16rows_vec2", "thin_f64_16rows")
                : launch_thin_typed<double>(g, stream, variant, variant_only, "small_f64_16x16_vec2", "small_f64_16x16");
}

}  // namespace ttamd
