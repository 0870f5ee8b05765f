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

constexpr int kThinWaves = 16;
constexpr int kThinMinK = 64;  // below this most waves would have nothing to do

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
    const int batch = blockIdx.y, m0 = blockIdx.x * 16;
    // Rows beyond M and columns beyond N read a valid element (row M-1, column N-1): a row's garbage stays in that
    // row, which is not stored; the columns' B values are zeroed.  Beyond K both operands are zeroed.
    const int row = m0 + li < g.M ? m0 + li : g.M - 1;
    const int col = li < g.N ? li : g.N - 1;
    const bool col_ok = li < g.N;
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
    const int m = m0 + MI::acc_row(e, l), n = l % 16;
    if (m >= g.M || n >= g.N) return;
    // The store's steps in the order of the general kernels: bias, ReLU-backward mask, ReLU, accumulate, second output.
    const int64_t idx = (static_cast<int64_t>(batch) * g.M + m) * g.N + n;
    const T *bias = static_cast<const T *>(g.bias);
    if (g.bias_mode == 1) v += bias[n];
    if (g.bias_mode == 2) v += bias[m];
    if (g.zmask && static_cast<const T *>(g.zmask)[idx] < T(0)) v = T(0);
    if (g.relu) v = v > T(0) ? v : T(0);
    T *C = static_cast<T *>(g.C);
    if (g.accumulate) v += C[idx];
    C[idx] = v;
    if (g.relu_out) static_cast<T *>(g.relu_out)[idx] = v > T(0) ? v : T(0);
}

template <typename T>
ttamd_status launch_thin_typed(const GemmArgs &g, hipStream_t stream, const char **variant, bool variant_only, const char *name_vec,
                               const char *name_any) {
    constexpr int VEC = ThinMma<T>::VEC;
    const bool vec = g.a_sk == 1 && g.K % VEC == 0 && g.a_sm % VEC == 0 && g.a_sb % VEC == 0 &&
                     (variant_only || reinterpret_cast<uintptr_t>(g.A) % 16 == 0);
    *variant = vec ? name_vec : name_any;
    if (variant_only) return TTAMD_OK;
    const dim3 grid(static_cast<unsigned>((g.M + 15) / 16), static_cast<unsigned>(g.batch)), block(64 * kThinWaves);
    if (vec) gemm_thin_kernel<T, true><<<grid, block, 0, stream>>>(g);
    else gemm_thin_kernel<T, false><<<grid, block, 0, stream>>>(g);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace

ttamd_status launch_gemm_thin(ttamd_dtype dt, const GemmArgs &g, hipStream_t stream, const char **variant, bool variant_only,
                              bool *handled) {
    *handled = false;
    if ((dt != TTAMD_F32 && dt != TTAMD_F64) || g.N > 16 || g.K < kThinMinK || g.colsum_out || g.batch > 65535) return TTAMD_OK;
    *handled = true;
    if (dt == TTAMD_F32) return launch_thin_typed<float>(g, stream, variant, variant_only, "thin_f32_16rows_vec4", "thin_f32_16rows");
    return launch_thin_typed<double>(g, stream, variant, variant_only, "thin_f64_16rows_vec2", "thin_f64_16rows");
}

}  // namespace ttamd
