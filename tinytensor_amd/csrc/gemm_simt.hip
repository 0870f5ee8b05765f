// gemm_simt.hip — LDS-tiled vector-ALU GEMM for arbitrary strided views, all six dtypes.
//
// Role: (1) the integer dtypes (u8,i16,i32,i64), which have no MFMA form with wrap-around
// results; tinytensor's CPU kernel computes them lane-wise modulo 2^n
// (tinytensor/tensor/backend/cpu/kernel/simd.h:120-127), so accumulation here is done in
// unsigned 32/64-bit registers and truncated, which is the same value modulo 2^n.
// (2) the small-shape path for f32/f64: products too thin to fill one MFMA tile
// (skinny N = 10 outputs of an MLP head, K = 10 outer-product-like updates).
// (3) operands whose extent does not fit 32-bit buffer addressing.
//
// A workgroup of 256 lanes owns a TILE_M x TILE_N block of C; each lane a 4 x 4 (or 4 x 1)
// register block.  Operand tiles are gathered through 64-bit strided addresses with bounds
// predicates (zero fill) and staged in LDS k-major so the inner product reads are
// conflict-free broadcasts/rows.
#include "common.h"

namespace ttamd {
namespace {

template <typename T>
struct AccOf { using type = T; };
template <>
struct AccOf<uint8_t> { using type = uint32_t; };
template <>
struct AccOf<int16_t> { using type = uint32_t; };
template <>
struct AccOf<int32_t> { using type = uint32_t; };
template <>
struct AccOf<int64_t> { using type = uint64_t; };

template <typename T>
__device__ __forceinline__ T relu_of(T v) {
    return v > T(0) ? v : T(0);
}
template <>
__device__ __forceinline__ uint8_t relu_of<uint8_t>(uint8_t v) {
    return v;
}

// TILE_M x TILE_N x 16 tile, 256 lanes, lane block RM x RN with RM = TILE_M/16, RN = TILE_N/16.
template <typename T, int TILE_M, int TILE_N>
__global__ void __launch_bounds__(256) gemm_simt_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    using Acc = typename AccOf<T>::type;
    constexpr int BK = 16;
    constexpr int RM = TILE_M / 16;
    constexpr int RN = TILE_N / 16;
    __shared__ Acc As[BK][TILE_M + 1];
    __shared__ Acc Bs[BK][TILE_N + 1];

    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int batch = blockIdx.y;
    const int tm = tile / tiles_n;
    const int tn = tile % tiles_n;
    const int m0 = tm * TILE_M;
    const int n0 = tn * TILE_N;

    const T *__restrict__ A = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb;
    const T *__restrict__ B = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb;

    // Lane order inside a tile follows the operand's smaller stride, for coalescing.
    const bool a_k_fast = g.a_sk <= g.a_sm;
    const bool b_n_fast = g.b_sn <= g.b_sk;

    const int tx = tid % 16;  // column group
    const int ty = tid / 16;  // row group

    Acc acc[RM][RN];
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < RN; ++j) acc[i][j] = Acc(0);

    for (int k0 = 0; k0 < g.K; k0 += BK) {
        // A tile: TILE_M x BK elements
#pragma unroll
        for (int e = tid; e < TILE_M * BK; e += 256) {
            int mm, kk;
            if (a_k_fast) {
                kk = e % BK;
                mm = e / BK;
            } else {
                mm = e % TILE_M;
                kk = e / TILE_M;
            }
            const int m = m0 + mm, k = k0 + kk;
            Acc v = Acc(0);
            if (m < g.M && k < g.K) v = static_cast<Acc>(A[static_cast<int64_t>(m) * g.a_sm + static_cast<int64_t>(k) * g.a_sk]);
            As[kk][mm] = v;
        }
#pragma unroll
        for (int e = tid; e < TILE_N * BK; e += 256) {
            int nn, kk;
            if (b_n_fast) {
                nn = e % TILE_N;
                kk = e / TILE_N;
            } else {
                kk = e % BK;
                nn = e / BK;
            }
            const int n = n0 + nn, k = k0 + kk;
            Acc v = Acc(0);
            if (n < g.N && k < g.K) v = static_cast<Acc>(B[static_cast<int64_t>(k) * g.b_sk + static_cast<int64_t>(n) * g.b_sn]);
            Bs[kk][nn] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            Acc a[RM], b[RN];
#pragma unroll
            for (int i = 0; i < RM; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < RN; ++j) b[j] = Bs[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < RN; ++j) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }

    T *__restrict__ C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    const T *bias = static_cast<const T *>(g.bias);
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        const int m = m0 + ty + 16 * i;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < RN; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n >= g.N) continue;
            T v = static_cast<T>(acc[i][j]);
            if (g.bias_mode == 1) v = static_cast<T>(v + bias[n]);
            if (g.bias_mode == 2) v = static_cast<T>(v + bias[m]);
            const int64_t idx = static_cast<int64_t>(m) * g.N + n;
            if (g.zmask && static_cast<const T *>(g.zmask)[static_cast<int64_t>(batch) * g.M * g.N + idx] < T(0)) v = static_cast<T>(v * T(0));  // the reference multiplies by 0: an infinite or NaN value under the mask stays NaN
            if (g.relu) v = relu_of<T>(v);
            if (g.accumulate) v = static_cast<T>(v + C[idx]);
            C[idx] = v;
            if (g.relu_out) static_cast<T *>(g.relu_out)[static_cast<int64_t>(batch) * g.M * g.N + idx] = relu_of<T>(v);
        }
    }
}

template <typename T>
ttamd_status launch_typed(const GemmArgs &g, hipStream_t stream, const char **variant, bool variant_only,
                          const char *name_wide, const char *name_thin) {
    // Thin outputs (N <= 16 columns, e.g. the 10-wide MLP head) use a 128 x 16 tile so that lanes are
    // not wasted on padding columns; everything else a 64 x 64 tile.
    const bool thin = g.N <= 16;
    *variant = thin ? name_thin : name_wide;
    if (variant_only) return TTAMD_OK;
    if (thin) {
        const int tiles_m = (g.M + 127) / 128, tiles_n = (g.N + 15) / 16;
        gemm_simt_kernel<T, 128, 16><<<dim3(tiles_m * tiles_n, g.batch), dim3(256), 0, stream>>>(g, tiles_m, tiles_n);
    } else {
        const int tiles_m = (g.M + 63) / 64, tiles_n = (g.N + 63) / 64;
        gemm_simt_kernel<T, 64, 64><<<dim3(tiles_m * tiles_n, g.batch), dim3(256), 0, stream>>>(g, tiles_m, tiles_n);
    }
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace

ttamd_status launch_gemm_simt(ttamd_dtype dt, const GemmArgs &g, hipStream_t stream, const char **variant,
                              bool variant_only) {
    if (g.batch > 65535) {
        set_error("batched_matmul: batch %d exceeds the grid limit of the vector-ALU kernel", g.batch);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    switch (dt) {
    case TTAMD_U8: return launch_typed<uint8_t>(g, stream, variant, variant_only, "simt_u8_64x64", "simt_u8_128x16");
    case TTAMD_I16: return launch_typed<int16_t>(g, stream, variant, variant_only, "simt_i16_64x64", "simt_i16_128x16");
    case TTAMD_I32: return launch_typed<int32_t>(g, stream, variant, variant_only, "simt_i32_64x64", "simt_i32_128x16");
    case TTAMD_I64: return launch_typed<int64_t>(g, stream, variant, variant_only, "simt_i64_64x64", "simt_i64_128x16");
    case TTAMD_F32: return launch_typed<float>(g, stream, variant, variant_only, "simt_f32_64x64", "simt_f32_128x16");
    case TTAMD_F64: return launch_typed<double>(g, stream, variant, variant_only, "simt_f64_64x64", "simt_f64_128x16");
    default: break;
    }
    set_error("matmul does not support dtype code %d", static_cast<int>(dt));
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

}  // namespace ttamd
