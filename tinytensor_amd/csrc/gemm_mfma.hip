// gemm_mfma.hip — fp32 / fp64 matrix-core GEMM for gfx950 (MI355X), reading strided views in place.
//
// Computes C[b] = A[b] . B[b] (C dense row-major) for the operands that
// BackendBase::batched_matmul receives (tinytensor/tensor/backend_base.h:130): any 3-D view whose
// row or column stride is 1 is streamed with 16-byte buffer loads; anything else is gathered
// element-wise by the same kernel structure.  No contiguous copy is made, unlike
// tinytensor/tensor/backend/cpu/matmul.cpp:37-38 and cuda/matmul.cu:40-41.
//
// Structure (one workgroup = 4 wavefronts of 64 lanes):
//   * a BM x BN tile of C per workgroup, BK-deep operand tiles double-buffered in LDS: the global
//     loads of tile t+1 are issued before the MFMA work of tile t and written to the other LDS
//     buffer afterwards, one barrier per tile;
//   * fp32: v_mfma_f32_32x32x2_f32, fp64: v_mfma_f64_16x16x4_f64; accumulators stay in registers
//     for the whole K loop;
//   * LDS layout follows the operand's memory layout so that no transposition happens on the
//     way in: "KC" (k contiguous, rows padded by one 16-byte vector so 16-byte fragment reads of
//     8 consecutive rows land in distinct banks) or "MC" (row/column index contiguous);
//     fragment reads pair k indices so that both operands agree whatever their layouts;
//   * buffer loads carry the operand's exact byte extent, so a lane that is out of the tile
//     reads zero instead of touching memory (offset with bit 31 set), plus component masks for
//     the contiguous dimension's tail;
//   * workgroup ids are remapped so that each XCD (8 per chip, one L2 each) owns a compact
//     block of neighbouring C tiles.
#include "common.h"

namespace ttamd {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kChunk = 8;            // k extent of one fragment read (both dtypes)
constexpr uint32_t kOob = 0x80000000u;  // byte offset that is out of range for every buffer used here

// ---------------------------------------------------------------------------------------------
// MFMA instruction traits.  A lane l holds A[i = l % MB][k = l / MB] and B[k = l / MB][j = l % MB].
template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
    static constexpr int MB = 32;   // block is MB x MB
    static constexpr int KG = 2;    // lane groups along k
    static constexpr int VK = 4;    // elements in 16 bytes
    static constexpr int NACC = 16;
    using acc_t = f32x16;
    using vec_t = f32x4;
    using pair_t = f32x2;
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // accumulator element e of lane l is C[acc_row(e,l)][l % MB]
    static __device__ __forceinline__ int acc_row(int e, int lane) { return (e / 4) * 8 + (lane / 32) * 4 + (e % 4); }
};

template <>
struct Mfma<double> {
    static constexpr int MB = 16;
    static constexpr int KG = 4;
    static constexpr int VK = 2;
    static constexpr int NACC = 4;
    using acc_t = f64x4;
    using vec_t = f64x2;
    using pair_t = f64x2;
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int acc_row(int e, int lane) { return 4 * e + lane / 16; }
};

// ---------------------------------------------------------------------------------------------
// Typed buffer loads of 1 element or of one 16-byte vector.
template <typename T, int VEC>
struct Vec;
template <>
struct Vec<float, 1> {
    using type = float;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
    }
};
template <>
struct Vec<float, 4> {
    using type = f32x4;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
    }
};
template <>
struct Vec<double, 1> {
    using type = double;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    }
};
template <>
struct Vec<double, 2> {
    using type = f64x2;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(f64x2, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
    }
};

template <typename T, int VEC>
__device__ __forceinline__ void zero_component(typename Vec<T, VEC>::type &v, int j) {
    if constexpr (VEC == 1) {
        v = T(0);
    } else {
        v[j] = T(0);
    }
}

// ---------------------------------------------------------------------------------------------
// Global -> register -> LDS staging of one operand tile (ROWS along m or n, BK along k).
//   KC: LDS element (r, k) at r * LD + k, vectors run along k (operand's k stride is 1 when VEC > 1)
//   MC: LDS element (r, k) at k * LD + r, vectors run along r (operand's row stride is 1 when VEC > 1)
template <typename T, int ROWS, int BK, bool KC, int VEC>
struct Stager {
    using V = typename Vec<T, VEC>::type;
    static constexpr int PAD = Mfma<T>::VK;  // one 16-byte vector
    static constexpr int LD = KC ? (BK + PAD) : (ROWS + PAD);
    static constexpr int LDS_ELEMS = KC ? ROWS * LD : BK * LD;
    static constexpr int VPL = (KC ? BK : ROWS) / VEC;  // vectors per LDS line
    static constexpr int NV = ROWS * BK / VEC;
    static constexpr int P = NV / kThreads;
    static_assert(NV % kThreads == 0, "tile must split evenly over the workgroup");

    V reg[P];
    uint32_t voff[P];
    int nval[P];  // MC only: valid components of the vector along the row dimension

    // line/column coordinates of pass p for this lane
    static __device__ __forceinline__ int line_of(int p, int tid) { return (p * kThreads + tid) / VPL; }
    static __device__ __forceinline__ int col_of(int p, int tid) { return ((p * kThreads + tid) % VPL) * VEC; }

    // rows_left = number of valid rows from the tile's first row; strides in bytes.
    __device__ __forceinline__ void init(int tid, int rows_left, uint32_t s_row_b, uint32_t s_k_b) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int line = line_of(p, tid), col = col_of(p, tid);
            if constexpr (KC) {
                const bool ok = line < rows_left;
                voff[p] = ok ? (line * s_row_b + col * s_k_b) : kOob;
                nval[p] = VEC;
            } else {
                int nv = rows_left - col;
                nv = nv < 0 ? 0 : (nv > VEC ? VEC : nv);
                nval[p] = nv;
                voff[p] = nv > 0 ? (col * s_row_b + line * s_k_b) : kOob;
            }
        }
    }

    // Loads the next tile.  k_left = K - kt*BK; `edge` = tile overlaps the row bound (MC masks needed).
    // MASK = false is the steady state (full k tile, interior rows): loads only, no selects.
    template <bool MASK>
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t rsrc, int tid, int k_left, bool edge,
                                         uint32_t k_step_b) {
        const bool k_tail = k_left < BK;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            V v = Vec<T, VEC>::load(rsrc, voff[p]);
            voff[p] += k_step_b;
            if constexpr (!MASK) {
                reg[p] = v;
                continue;
            }
            if constexpr (KC) {
                if (k_tail) {
                    const int col = col_of(p, tid);
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (col + j >= k_left) zero_component<T, VEC>(v, j);
                }
            } else {
                if (k_tail) {
                    if (line_of(p, tid) >= k_left) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) zero_component<T, VEC>(v, j);
                    }
                }
                if (VEC > 1 && edge) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (j >= nval[p]) zero_component<T, VEC>(v, j);
                }
            }
            reg[p] = v;
        }
    }

    __device__ __forceinline__ void store(T *lds, int tid) const {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int line = line_of(p, tid), col = col_of(p, tid);
            *reinterpret_cast<V *>(&lds[line * LD + col]) = reg[p];
        }
    }
};

// ---------------------------------------------------------------------------------------------
// LDS -> MFMA operand fragments for NB blocks of one wave, one chunk of 8 k.
// Step j of a chunk multiplies k = chunk*8 + VK*kg + j, kg = lane / MB, for both operands.
template <typename T, int LD, bool KC, int NB>
struct Fragment {
    using M = Mfma<T>;
    static constexpr bool PAIRED = (!KC) && (NB % 2 == 0);
    T v[NB][M::VK];

    // w0 = first tile-local row of this wave.
    __device__ __forceinline__ void read(const T *lds, int w0, int chunk, int lane) {
        const int i = lane % M::MB, kg = lane / M::MB;
        const int kb = chunk * kChunk + M::VK * kg;
        if constexpr (KC) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const typename M::vec_t t = *reinterpret_cast<const typename M::vec_t *>(&lds[(w0 + b * M::MB + i) * LD + kb]);
#pragma unroll
                for (int j = 0; j < M::VK; ++j) v[b][j] = t[j];
            }
        } else if constexpr (PAIRED) {
#pragma unroll
            for (int j = 0; j < M::VK; ++j)
#pragma unroll
                for (int pr = 0; pr < NB / 2; ++pr) {
                    const typename M::pair_t t =
                        *reinterpret_cast<const typename M::pair_t *>(&lds[(kb + j) * LD + w0 + pr * 2 * M::MB + 2 * i]);
                    v[2 * pr][j] = t[0];
                    v[2 * pr + 1][j] = t[1];
                }
        } else {
#pragma unroll
            for (int j = 0; j < M::VK; ++j)
#pragma unroll
                for (int b = 0; b < NB; ++b) v[b][j] = lds[(kb + j) * LD + w0 + b * M::MB + i];
        }
    }

    // tile-local row (or column) that block b, in-block index i stands for
    static __device__ __forceinline__ int index_of(int w0, int b, int i) {
        if constexpr (PAIRED) {
            return w0 + (b / 2) * 2 * M::MB + 2 * i + (b % 2);
        } else {
            return w0 + b * M::MB + i;
        }
    }
};

// Each XCD receives every 8th workgroup id; give it a contiguous range of logical ids instead.
__device__ __forceinline__ int remap_xcd(int pid, int total) {
    constexpr int XCDS = 8;
    const int q = total / XCDS, r = total % XCDS;
    const int xcd = pid % XCDS, idx = pid / XCDS;
    return xcd * q + (xcd < r ? xcd : r) + idx;
}

// ---------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC>
__global__ void __launch_bounds__(kThreads, 2) gemm_mfma_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    using M = Mfma<T>;
    static_assert(WGM * WGN == kWaves, "4 waves per workgroup");
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int NBM = WM / M::MB, NBN = WN / M::MB;
    static_assert(WM % M::MB == 0 && WN % M::MB == 0 && BK % kChunk == 0, "tile shape");
    using StA = Stager<T, BM, BK, A_KC, A_VEC>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC>;
    using FrA = Fragment<T, StA::LD, A_KC, NBM>;
    using FrB = Fragment<T, StB::LD, B_KC, NBN>;

    // LDS: [A buf 0][A buf 1][B buf 0][B buf 1]; addressed as offsets from the one shared base so that
    // every access stays a DS instruction (no generic-pointer loads, which would also wait on vmcnt).
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);
    constexpr int kBOff = 2 * StA::LDS_ELEMS;

    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = tid / 64;
    const int wm0 = (wave / WGN) * WM;
    const int wn0 = (wave % WGN) * WN;

    // workgroup -> (batch, tile row, tile column)
    const int tiles = tiles_m * tiles_n;
    int pid = remap_xcd(blockIdx.x, gridDim.x);
    const int batch = pid / tiles;
    pid -= batch * tiles;
    constexpr int GROUP = 8;
    const int group_sz = GROUP * tiles_n;
    const int first_m = (pid / group_sz) * GROUP;
    const int gm = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int tm = first_m + (pid % group_sz) % gm;
    const int tn = (pid % group_sz) / gm;
    const int m0 = tm * BM, n0 = tn * BN;

    // Buffer resources based at the tile's first row/column, sized to the operand's true extent.
    const T *a_base = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(m0) * g.a_sm;
    const T *b_base = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(n0) * g.b_sn;
    const int a_rows = g.M - m0, b_rows = g.N - n0;
    const int64_t a_ext = (static_cast<int64_t>(a_rows - 1) * g.a_sm + static_cast<int64_t>(g.K - 1) * g.a_sk + 1) * sizeof(T);
    const int64_t b_ext = (static_cast<int64_t>(b_rows - 1) * g.b_sn + static_cast<int64_t>(g.K - 1) * g.b_sk + 1) * sizeof(T);
    // With 16-byte loads the extent is rounded up to the vector size: the base is 16-byte aligned, so
    // the last vector stays inside the allocation's final 16-byte block and its tail is masked anyway.
    constexpr int64_t a_round = A_VEC > 1 ? 15 : 0, b_round = B_VEC > 1 ? 15 : 0;
    const int64_t a_ext_r = (a_ext + a_round) & ~a_round, b_ext_r = (b_ext + b_round) & ~b_round;
    const int a_rec = a_ext_r > 0x7fffffff ? 0x7fffffff : static_cast<int>(a_ext_r);
    const int b_rec = b_ext_r > 0x7fffffff ? 0x7fffffff : static_cast<int>(b_ext_r);
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(a_base), 0, a_rec, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(b_base), 0, b_rec, 0x00020000);

    const uint32_t a_sm_b = static_cast<uint32_t>(g.a_sm * sizeof(T)), a_sk_b = static_cast<uint32_t>(g.a_sk * sizeof(T));
    const uint32_t b_sn_b = static_cast<uint32_t>(g.b_sn * sizeof(T)), b_sk_b = static_cast<uint32_t>(g.b_sk * sizeof(T));
    const bool a_edge = a_rows < BM, b_edge = b_rows < BN;

    StA sa;
    StB sb;
    sa.init(tid, a_rows, a_sm_b, a_sk_b);
    sb.init(tid, b_rows, b_sn_b, b_sk_b);

    typename M::acc_t acc[NBM][NBN];
#pragma unroll
    for (int i = 0; i < NBM; ++i)
#pragma unroll
        for (int j = 0; j < NBN; ++j)
#pragma unroll
            for (int e = 0; e < M::NACC; ++e) acc[i][j][e] = T(0);

    const int KT = (g.K + BK - 1) / BK;
    sa.template load<true>(a_rsrc, tid, g.K, a_edge, a_sk_b * BK);
    sb.template load<true>(b_rsrc, tid, g.K, b_edge, b_sk_b * BK);
    sa.store(smem, tid);
    sb.store(smem + kBOff, tid);
    __syncthreads();

    auto compute = [&](int buf) {
        const T *la = smem + buf * StA::LDS_ELEMS;
        const T *lb = smem + kBOff + buf * StB::LDS_ELEMS;
#pragma unroll
        for (int c = 0; c < BK / kChunk; ++c) {
            FrA fa;
            FrB fb;
            fa.read(la, wm0, c, lane);
            fb.read(lb, wn0, c, lane);
#pragma unroll
            for (int j = 0; j < M::VK; ++j)
#pragma unroll
                for (int bm = 0; bm < NBM; ++bm)
#pragma unroll
                    for (int bn = 0; bn < NBN; ++bn) acc[bm][bn] = M::mma(fa.v[bm][j], fb.v[bn][j], acc[bm][bn]);
        }
    };

    // Tiles 0 .. KT-2: prefetch tile kt+1 into registers, multiply tile kt out of LDS, then park the
    // prefetched tile in the other LDS buffer.  The last tile is multiplied after the loop, so the loop
    // body has no conditionals.  MASK = false is the steady state (interior workgroup, K a multiple of BK).
    auto pipeline = [&]<bool MASK>() {
        for (int kt = 0; kt + 1 < KT; ++kt) {
            const int cur = kt & 1;
            const int k_left = g.K - (kt + 1) * BK;
            sa.template load<MASK>(a_rsrc, tid, k_left, a_edge, a_sk_b * BK);
            sb.template load<MASK>(b_rsrc, tid, k_left, b_edge, b_sk_b * BK);
            compute(cur);
            sa.store(smem + (cur ^ 1) * StA::LDS_ELEMS, tid);
            sb.store(smem + kBOff + (cur ^ 1) * StB::LDS_ELEMS, tid);
            __syncthreads();
        }
    };
    if (!a_edge && !b_edge && g.K % BK == 0) {
        pipeline.template operator()<false>();
    } else {
        pipeline.template operator()<true>();
    }
    if (KT > 0) compute((KT - 1) & 1);

    // Epilogue: registers -> C (dense row-major), optional bias / ReLU / accumulate.
    T *__restrict__ C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    const T *__restrict__ bias = static_cast<const T *>(g.bias);
    const int jcol = lane % M::MB;
    auto finish = [&](T v, int m, int n, int64_t idx) {
        if (g.bias_mode == 1) v += bias[n];
        if (g.bias_mode == 2) v += bias[m];
        if (g.relu) v = v > T(0) ? v : T(0);
        if (g.accumulate) v += C[idx];
        return v;
    };
    if constexpr (FrB::PAIRED) {
        // Blocks 2p and 2p+1 of an MC-layout B operand hold columns n and n+1 of the same lane: store them
        // together so that a wave writes whole contiguous row segments.
        const bool can_pair = (g.N % 2 == 0) && (reinterpret_cast<uintptr_t>(C) % (2 * sizeof(T)) == 0);
#pragma unroll
        for (int pr = 0; pr < NBN / 2; ++pr) {
            const int n = n0 + FrB::index_of(wn0, 2 * pr, jcol);  // even column; n + 1 belongs to block 2p+1
#pragma unroll
            for (int bm = 0; bm < NBM; ++bm) {
#pragma unroll
                for (int e = 0; e < M::NACC; ++e) {
                    const int m = m0 + FrA::index_of(wm0, bm, M::acc_row(e, lane));
                    if (m >= g.M) continue;
                    const int64_t idx = static_cast<int64_t>(m) * g.N + n;
                    if (can_pair && n + 1 < g.N) {
                        typename M::pair_t out;
                        out[0] = finish(acc[bm][2 * pr][e], m, n, idx);
                        out[1] = finish(acc[bm][2 * pr + 1][e], m, n + 1, idx + 1);
                        *reinterpret_cast<typename M::pair_t *>(&C[idx]) = out;
                    } else {
                        if (n < g.N) C[idx] = finish(acc[bm][2 * pr][e], m, n, idx);
                        if (n + 1 < g.N) C[idx + 1] = finish(acc[bm][2 * pr + 1][e], m, n + 1, idx + 1);
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int bn = 0; bn < NBN; ++bn) {
            const int n = n0 + FrB::index_of(wn0, bn, jcol);
            if (n >= g.N) continue;
#pragma unroll
            for (int bm = 0; bm < NBM; ++bm) {
#pragma unroll
                for (int e = 0; e < M::NACC; ++e) {
                    const int m = m0 + FrA::index_of(wm0, bm, M::acc_row(e, lane));
                    if (m >= g.M) continue;
                    const int64_t idx = static_cast<int64_t>(m) * g.N + n;
                    C[idx] = finish(acc[bm][bn][e], m, n, idx);
                }
            }
        }
    }
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
    constexpr size_t lds_bytes = 2 * (StA::LDS_ELEMS + StB::LDS_ELEMS) * sizeof(T);
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
