// gemm_mfma.hip — fp32 / fp64 matrix-core GEMM for gfx950 (MI355X), reading strided views in place.
//
// Computes C[b] = A[b] . B[b] (C dense row-major) for the operands that
// BackendBase::batched_matmul receives (tinytensor/tensor/backend_base.h:130): any 3-D view whose
// row or column stride is 1 is streamed with 16-byte buffer loads; anything else is gathered
// element-wise by the same kernel structure.  No contiguous copy is made, unlike
// tinytensor/tensor/backend/cpu/matmul.cpp:37-38 and cuda/matmul.cu:40-41.
// The tile engine (LDS double buffering, MFMA loop, layouts) lives in mfma_core.h; this file adds the
// kernel entry, the workgroup -> tile mapping and the host-side operand classification.
#include "mfma_core.h"

namespace ttamd {
namespace {

using namespace mfma;

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC>
__global__ void __launch_bounds__(kThreads, 2) gemm_mfma_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC>;
    using Engine = TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);

    const int tid = threadIdx.x;
    int batch, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, gridDim.x), tiles_m, tiles_n, batch, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // Operand bases at the tile's first row / column; the stagers size their buffer extents from there.
    const T *a_base = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(m0) * g.a_sm;
    const T *b_base = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(n0) * g.b_sn;
    StA sa;
    StB sb;
    sa.init(a_base, tid, g.M - m0, g.a_sm, g.a_sk, g.K);
    sb.init(b_base, tid, g.N - n0, g.b_sn, g.b_sk, g.K);

    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, g.K, !sa.edge && !sb.edge && g.K % BK == 0);

    T *C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    store_tile_dense<T>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate);
}

// ---------------------------------------------------------------------------------------------
// Host side: operand classification and variant table.

struct OperandClass {
    bool kc;   // LDS/global vectors run along k
    int vec;   // elements per load (1 = element-wise gather)
};

// s_row: stride of the m (or n) index, s_k: stride of the k index, s_b: batch stride (elements).
template <typename T>
OperandClass classify(const void *ptr, int64_t s_row, int64_t s_k, int64_t s_b, int batch) {
    constexpr int VK = Mfma<T>::VK;
    const bool ptr_ok = reinterpret_cast<uintptr_t>(ptr) % 16 == 0;
    const bool batch_ok = batch == 1 || s_b % VK == 0;
    if (s_k == 1 && ptr_ok && batch_ok && s_row % VK == 0) return {true, VK};
    if (s_row == 1 && ptr_ok && batch_ok && s_k % VK == 0) return {false, VK};
    return {s_k <= s_row, 1};
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC>
ttamd_status launch_variant(const GemmArgs &g, hipStream_t stream) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC>;
    constexpr size_t lds_bytes = TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>::kLdsBytes;
    auto kernel = gemm_mfma_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC>;
    static bool configured = false;  // raising the dynamic LDS limit is per kernel, once
    if (!configured && lds_bytes > 48 * 1024) {
        TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        configured = true;
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.batch;
    if (blocks > 0x7fffffff) {
        set_error("batched_matmul: %lld workgroups exceed the grid limit", static_cast<long long>(blocks));
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(kThreads), lds_bytes, stream>>>(g, tiles_m, tiles_n);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, int VEC>
ttamd_status launch_layouts(const GemmArgs &g, bool a_kc, bool b_kc, hipStream_t stream) {
    if (a_kc && b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, true, VEC, true, VEC>(g, stream);
    if (a_kc && !b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, true, VEC, false, VEC>(g, stream);
    if (!a_kc && b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, false, VEC, true, VEC>(g, stream);
    return launch_variant<T, BM, BN, BK, WGM, WGN, false, VEC, false, VEC>(g, stream);
}

template <typename T>
struct TileShapes;
template <>
struct TileShapes<float> {
    static constexpr int LBM = 128, LBN = 128, LBK = 32;  // large: 4 waves of 64 x 64
    static constexpr int SBM = 64, SBN = 64, SBK = 32;    // small: 4 waves of 32 x 32
    static constexpr const char *prefix = "mfma_f32";
};
template <>
struct TileShapes<double> {
    static constexpr int LBM = 128, LBN = 128, LBK = 16;  // 4 waves of 64 x 64 (4 x 4 blocks of 16 x 16)
    static constexpr int SBM = 64, SBN = 64, SBK = 16;    // 4 waves of 32 x 32
    static constexpr const char *prefix = "mfma_f64";
};

template <typename T>
ttamd_status launch_mfma_typed(const GemmArgs &g, hipStream_t stream, const char **variant, bool variant_only,
                               bool *handled) {
    using TS = TileShapes<T>;
    constexpr int VK = Mfma<T>::VK;
    *handled = false;
    // Very thin outputs leave a 64-wide MFMA tile almost empty: those go to the vector-ALU kernel.
    if (g.M <= 16 || g.N <= 16) return TTAMD_OK;

    OperandClass ca = classify<T>(g.A, g.a_sm, g.a_sk, g.a_sb, g.batch);
    OperandClass cb = classify<T>(g.B, g.b_sn, g.b_sk, g.b_sb, g.batch);
    const bool vec = ca.vec > 1 && cb.vec > 1;

    const int64_t tiles_large = static_cast<int64_t>((g.M + TS::LBM - 1) / TS::LBM) * ((g.N + TS::LBN - 1) / TS::LBN) * g.batch;
    const bool large = vec && tiles_large >= 192;
    const int bm = large ? TS::LBM : TS::SBM;

    // 32-bit buffer addressing: the bytes reachable from a tile's first row must stay below 2^31.
    const int64_t a_reach = (static_cast<int64_t>(bm - 1) * g.a_sm + static_cast<int64_t>(g.K - 1) * g.a_sk + VK) * sizeof(T);
    const int64_t b_reach = (static_cast<int64_t>(bm - 1) * g.b_sn + static_cast<int64_t>(g.K - 1) * g.b_sk + VK) * sizeof(T);
    if (a_reach >= 0x7fffffffLL || b_reach >= 0x7fffffffLL) return TTAMD_OK;

    static thread_local char name[96];
    snprintf(name, sizeof(name), "%s_%s_a%s%d_b%s%d", TS::prefix, large ? "128x128" : "64x64", ca.kc ? "kc" : "mc",
             vec ? VK : 1, cb.kc ? "kc" : "mc", vec ? VK : 1);
    *variant = name;
    *handled = true;
    if (variant_only) return TTAMD_OK;

    if (large) return launch_layouts<T, TS::LBM, TS::LBN, TS::LBK, 2, 2, VK>(g, ca.kc, cb.kc, stream);
    if (vec) return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, VK>(g, ca.kc, cb.kc, stream);
    return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, 1>(g, ca.kc, cb.kc, stream);
}

}  // namespace

ttamd_status launch_gemm_mfma(ttamd_dtype dt, const GemmArgs &g, hipStream_t stream, const char **variant,
                              bool variant_only, bool *handled) {
    *handled = false;
    if (dt == TTAMD_F32) return launch_mfma_typed<float>(g, stream, variant, variant_only, handled);
    if (dt == TTAMD_F64) return launch_mfma_typed<double>(g, stream, variant, variant_only, handled);
    return TTAMD_OK;
}

}  // namespace ttamd
