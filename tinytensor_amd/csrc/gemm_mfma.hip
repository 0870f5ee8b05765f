// gemm_mfma.hip — fp32 / fp64 matrix-core GEMM for gfx950 (MI355X), reading strided views in place.
//
// Computes C[b] = A[b] . B[b] (C dense row-major) for the operands that
// BackendBase::batched_matmul receives (tinytensor/tensor/backend_base.h:130): any 3-D view whose
// row or column stride is 1 is streamed with 16-byte buffer loads; anything else is gathered
// element-wise by the same kernel structure.  No contiguous copy is made, unlike
// tinytensor/tensor/backend/cpu/matmul.cpp:37-38 and cuda/matmul.cu:40-41.
// The tile engine (LDS double buffering, MFMA loop, layouts) lives in mfma_core.h; this file adds the
// kernel entry, the workgroup -> tile mapping and the host-side operand classification.
#include <atomic>
#include "mfma_core.h"

#include <algorithm>
#include <cmath>

#include <mutex>

namespace ttamd {
namespace {

using namespace mfma;

// Partial tiles of split-k launches made through ttamd_batched_matmul_noalloc: a fixed array in the code object
// instead of the growing per-stream buffer, so that the call never allocates.  Every GPU that loads the library holds
// its own copy (kFixedScratchBytes of its memory, until the process ends) at its own address; the name below is only
// the host-side handle of the symbol, the device address comes from hipGetSymbolAddress, once per device.
constexpr size_t kFixedScratchBytes = size_t(8) << 20;
static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];

ttamd_status fixed_scratch_address(int device, void **out) {
    static std::mutex mu;
    static void *address[kMaxDevices] = {};
    if (device < 0 || device >= kMaxDevices) {
        set_error("batched_matmul_noalloc: device id %d beyond the %d devices the fixed scratch serves", device, kMaxDevices);
        return TTAMD_ERR_INVALID_DEVICE;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!address[device]) {  // the caller has made `device` current (use_device)
        void *p = nullptr;
        TTAMD_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) {
            set_error("batched_matmul_noalloc: the scratch symbol has no address on device %d", device);
            return TTAMD_ERR_LAUNCH;
        }
        address[device] = p;
    }
    *out = address[device];
    return TTAMD_OK;
}

// ksplit > 1: the reduction is cut into `ksplit` ranges of `k_chunk` (a multiple of BK); workgroup column z =
// batch * ksplit + split writes the raw partial tile to `partial[z]` and splitk_reduce_kernel finishes the job.
// PF = tiles kept in flight in registers: 1 for the big tiles (a k tile's MFMA work outlasts a global load there,
// and registers are scarce), 2 or 4 for the 64 x 64 tile, whose 16 MFMAs per k tile (~0.43 us) are shorter than a
// load from L2 under traffic: with one tile in flight a lone workgroup on a CU (1024^3 is 256 tiles) waited for
// memory in every step.  Measured at depth 4: 1024 x 784 x 1024 26.2 -> 22.1 us, 1024 x 4096 x 1024 87 -> 78 us; the
// host picks the depth per launch (launch_mfma_typed).
// EPI: which epilogues the kernel carries.  kEpiAny tests the epilogue flags at run time and supports split k (the
// 64 x 64 tile).  The big tiles are compiled three times, kEpiLean (plain store only), kEpiFull (bias / ReLU /
// accumulate) and kEpiExt (those plus second output, mask and column sums), and never split k: with several store
// walks in one kernel the register allocator spills accumulators ahead of the branch for the sake of the heaviest
// walk, and the plain store pays for it.
constexpr int kEpiAny = 0, kEpiLean = 1, kEpiFull = 2, kEpiExt = 3;
// kEpiLean for a problem of whole k tiles and whole vectors along m and n (K a multiple of BK; M, N multiples of the
// vector length of an operand that is contiguous along them): no masked loop in the kernel, whose
// registers otherwise cost the plain kernel of the biggest tiles 228 bytes of scratch per lane.
constexpr int kEpiLeanWhole = 4;

// The store's extensions for one workgroup: pointers moved to the batch, partial column sums to this tile row's rows.
template <typename T>
__device__ __forceinline__ EpilogueExt<T> make_ext(const GemmArgs &g, int batch, int tm, int wgm) {
    const int64_t mn = static_cast<int64_t>(g.M) * g.N;
    EpilogueExt<T> e;
    e.relu_out = g.relu_out ? static_cast<T *>(g.relu_out) + batch * mn : nullptr;
    e.zmask = g.zmask ? static_cast<const T *>(g.zmask) + batch * mn : nullptr;
    e.colsum = g.colsum_partial ? static_cast<T *>(g.colsum_partial) + static_cast<int64_t>(batch) * g.colsum_rows * g.N : nullptr;
    e.colsum_row0 = tm * wgm;
    return e;
}
__host__ __device__ inline bool ext_store(const GemmArgs &g) { return g.relu_out || g.zmask || g.colsum_out; }
__host__ __device__ inline bool plain_store(const GemmArgs &g) {
    return g.bias_mode == 0 && !g.relu && !g.accumulate && !ext_store(g);
}
template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC, int PF, int EPI>
__global__ void __launch_bounds__(kThreads, (BM * BN * sizeof(T) > 256 * 128 * 4 || (sizeof(T) == 8 && BM * BN >= 128 * 128)) ? 1 : 2)  // 256 x 256 (fp64 128 x 128 and up): one workgroup per CU, accumulators in AGPRs
gemm_mfma_kernel(GemmArgs g, int tiles_m, int tiles_n, int ksplit, int k_chunk, T *partial) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC, PF>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC, PF>;
    using Engine = TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);

    const int tid = threadIdx.x;
    int z, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, gridDim.x), tiles_m, tiles_n, z, tm, tn);
    const int batch = z / ksplit, split = z - batch * ksplit;
    const int k0 = split * k_chunk;
    const int Kc = (g.K - k0) < k_chunk ? (g.K - k0) : k_chunk;
    const int m0 = tm * BM, n0 = tn * BN;

    // Operand bases at the tile's first row / column and first k; the stagers size their buffer extents from there.
    const T *a_base = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(m0) * g.a_sm +
                      static_cast<int64_t>(k0) * g.a_sk;
    const T *b_base = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(n0) * g.b_sn +
                      static_cast<int64_t>(k0) * g.b_sk;
    StA sa;
    StB sb;
    sa.init(a_base, tid, g.M - m0, g.a_sm, g.a_sk, Kc);
    sb.init(b_base, tid, g.N - n0, g.b_sn, g.b_sk, Kc);

    Engine eng;
    eng.init(tid);
    eng.template run<EPI == kEpiLeanWhole>(sa, sb, smem, Kc, !sa.row_mask && !sb.row_mask);

    T *C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    if constexpr (EPI == kEpiLean || EPI == kEpiLeanWhole) {
        store_tile_dense<T, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
    } else if constexpr (EPI == kEpiFull) {
        store_tile_dense<T, false>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate);
    } else if constexpr (EPI == kEpiExt) {
        store_tile_dense<T, false, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate,
                                         make_ext<T>(g, batch, tm, WGM));
    } else if (ksplit == 1) {
        if (plain_store(g))  // the common case gets a store loop free of epilogue work
            store_tile_dense<T, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
        else if (!ext_store(g))
            store_tile_dense<T, false>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate);
        else
            store_tile_dense<T, false, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate,
                                             make_ext<T>(g, batch, tm, WGM));
    } else {
        store_tile_dense<T, true>(eng, partial + static_cast<int64_t>(z) * g.M * g.N, g.M, g.N, m0, n0,
                                  static_cast<const T *>(nullptr), 0, 0, 0);
    }
}

// Two halves of the reduction in one workgroup of 512 lanes: lanes 0-255 multiply k in [0, K/2), lanes 256-511 k in
// [K/2, K), each half with its own LDS buffers and the same tile and lane layout; the upper half then parks its
// accumulators in LDS and the lower half adds them and stores.  For launches with at most one workgroup per CU: a
// SIMD then holds two waves instead of one, and each covers the other's waits (memory, LDS, barrier).  Both halves
// run the same number of k tiles (the host only launches this when ceil(k_half / BK) == ceil((K - k_half) / BK)), so
// they pass the engine's barriers in step; a half whose length is not a whole number of tiles takes the masked loop,
// which has the same barriers.  The sum is (first half) + (second half), each accumulated in k order: deterministic.
// BSUM (B with its columns contiguous, 16-byte vectors): the workgroups of the first row of tiles also add up the
// vectors of B that they stage -- every element of B's column panel passes through their registers once -- and write
// g.rhs_colsum[batch][n] = sum over k of B[k][n]: the bias gradient of a Linear layer when this product is its weight
// gradient x^T . dy (nn/linear.cpp:45-48: the bias is an expanded view, its gradient sums the batch dimension).  Order:
// a lane adds its k rows in k order, the 16 lanes of a column are added in lane order, lower half + upper half.
template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC, int PF, bool BSUM = false>
__global__ void __launch_bounds__(2 * kThreads, 1)
gemm_mfma_dual_kernel(GemmArgs g, int tiles_m, int tiles_n, int k_half) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC, PF>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC, PF, BSUM>;
    using Engine = TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>;
    constexpr size_t kExchangeBytes = Engine::kAccPerLane * kThreads * sizeof(T);
    constexpr size_t kSumBytes = BSUM ? 2 * StB::kSumParts * BN * sizeof(T) : 0;
    static_assert(kExchangeBytes + kSumBytes <= 2 * Engine::kLdsBytes, "the parked accumulators (and operand sums) fit the two halves' buffers");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    // The half is the same for every lane of a wave.  Said through readfirstlane so that the compiler keeps it, and the
    // half's length, k tile count and every loop condition and mask decision derived from it, in scalar registers
    // (left as a function of threadIdx.x they are per-lane values: compares on the vector ALU, loops and branches by
    // execution mask).
    const int half = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / kThreads));
    const int tid = threadIdx.x % kThreads;
    T *const smem = reinterpret_cast<T *>(smem_raw + half * Engine::kLdsBytes);
    int batch, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, gridDim.x), tiles_m, tiles_n, batch, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN, k0 = half * k_half;
    const int Kc = half == 0 ? k_half : g.K - k_half;
    const T *a_base = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(m0) * g.a_sm +
                      static_cast<int64_t>(k0) * g.a_sk;
    const T *b_base = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(n0) * g.b_sn +
                      static_cast<int64_t>(k0) * g.b_sk;
    StA sa;
    StB sb;
    sa.init(a_base, tid, g.M - m0, g.a_sm, g.a_sk, Kc);
    sb.init(b_base, tid, g.N - n0, g.b_sn, g.b_sk, Kc);
    if constexpr (BSUM) sb.start_sums(tm == 0);
    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, Kc, !sa.row_mask && !sb.row_mask);
    __syncthreads();  // every wave is done with its tiles: the lower half's buffers become the exchange area
    T *const exchange = reinterpret_cast<T *>(smem_raw);
    T *const sums = reinterpret_cast<T *>(smem_raw + kExchangeBytes);  // [half][part][BN]
    if (half == 1) eng.park_acc(exchange, tid);
    if constexpr (BSUM) {
        if (tm == 0)
            *reinterpret_cast<typename StB::V *>(&sums[(half * StB::kSumParts + sb.sum_part()) * BN + sb.sum_row0()]) = sb.sum;
    }
    __syncthreads();
    if (half == 1) return;
    eng.add_parked_acc(exchange, tid);
    if constexpr (BSUM) {
        if (tm == 0 && tid < BN && n0 + tid < g.N) {
            T lower = T(0), upper = T(0);
#pragma unroll
            for (int r = 0; r < StB::kSumParts; ++r) {
                lower += sums[r * BN + tid];
                upper += sums[(StB::kSumParts + r) * BN + tid];
            }
            static_cast<T *>(g.rhs_colsum)[static_cast<int64_t>(batch) * g.N + n0 + tid] = lower + upper;
        }
    }
    T *C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    if (plain_store(g))
        store_tile_dense<T, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
    else if (!ext_store(g))
        store_tile_dense<T, false>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate);
    else
        store_tile_dense<T, false, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate,
                                         make_ext<T>(g, batch, tm, WGM));
}

// C[b][i] = epilogue(sum over s of partial[b * ksplit + s][i]).  G lanes share an element: lane g adds the splits g,
// g + G, ... in ascending order, eight loads in flight at a time, and the G sums are added in a fixed tree -- the same
// order on every run (deterministic).  G = 1 is the plain ascending sum; G = 4 gives a small output with many splits
// four times the lanes and a quarter of the dependent rounds (256 x 9216 x 128 in 64 splits: 9.3 -> 4.8 us).
// Lanes of one g are consecutive elements: a wave reads 64 / G contiguous elements per split.
template <typename T, int G>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(GemmArgs g, const T *__restrict__ partial, int ksplit) {
    const int64_t mn = static_cast<int64_t>(g.M) * g.N;
    constexpr int PER_WAVE = 64 / G;
    const int lane = threadIdx.x % 64, part = lane / PER_WAVE;
    const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / 64;
    const int64_t want = wave * PER_WAVE + lane % PER_WAVE;
    const bool live = want < mn;
    const int64_t i = live ? want : mn - 1;  // (every lane takes part in the shuffles below)
    const int batch = blockIdx.y;
    const T *p = partial + static_cast<int64_t>(batch) * ksplit * mn + i;
    T v = T(0);
    int s = part;
    for (; s + 7 * G < ksplit; s += 8 * G) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = p[static_cast<int64_t>(s + u * G) * mn];
#pragma unroll
        for (int u = 0; u < 8; ++u) v += x[u];
    }
    for (; s < ksplit; s += G) v += p[static_cast<int64_t>(s) * mn];
#pragma unroll
    for (int d = PER_WAVE; d < 64; d *= 2) v += __shfl_xor(v, d, 64);
    if (!live || part != 0) return;
    const T *bias = static_cast<const T *>(g.bias);
    if (g.bias_mode == 1) v += bias[i % g.N];
    if (g.bias_mode == 2) v += bias[i / g.N];
    if (g.zmask && static_cast<const T *>(g.zmask)[static_cast<int64_t>(batch) * mn + i] < T(0)) v = v * T(0);  // the reference multiplies by 0: an infinite or NaN value under the mask stays NaN
    if (g.relu) v = v > T(0) ? v : T(0);
    T *C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * mn;
    if (g.accumulate) v += C[i];
    C[i] = v;
    if (g.relu_out) static_cast<T *>(g.relu_out)[static_cast<int64_t>(batch) * mn + i] = v > T(0) ? v : T(0);
}

// colsum[b][n] = sum over r of partial[b][r][n], r ascending (deterministic).
template <typename T>
__global__ void __launch_bounds__(256) colsum_reduce_kernel(const T *__restrict__ partial, int rows, int N, T *__restrict__ out) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const T *p = partial + static_cast<int64_t>(blockIdx.y) * rows * N + n;
    T v = T(0);
    int r = 0;
    for (; r + 8 <= rows; r += 8) {  // eight loads in flight, added in row order
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = p[static_cast<int64_t>(r + u) * N];
#pragma unroll
        for (int u = 0; u < 8; ++u) v += x[u];
    }
    for (; r < rows; ++r) v += p[static_cast<int64_t>(r) * N];
    out[static_cast<int64_t>(blockIdx.y) * N + n] = v;
}

// Scratch of a launch: the library's fixed array (calls that must not allocate) or the stream's growing buffer.
ttamd_status launch_scratch(int device, hipStream_t stream, size_t bytes, bool fixed, void **out);

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

template <typename T>
struct TileShapes;
template <>
struct TileShapes<float> {
    static constexpr bool kHasXL = true;
    static constexpr int YBM = 256, YBN = 256, YBK = 16;  // largest: 4 waves of 128 x 128 (4 x 4 MFMA blocks), one workgroup per CU
    static constexpr int XBM = 256, XBN = 128, XBK = 16;  // extra large: 4 waves of 128 x 64 (4 x 2 MFMA blocks)
    static constexpr int MBM = 192, MBN = 192, MBK = 16;  // 4 waves of 96 x 96 (3 x 3 blocks), one workgroup per CU: for outputs
                                                          // that 256 x 256 tiles cut into an awkward number (3072^2 = 256 of these)
    static constexpr int LBM = 128, LBN = 128, LBK = 16;  // large: 4 waves of 64 x 64
    static constexpr int SBM = 64, SBN = 64, SBK = 32;    // small: 4 waves of 32 x 32
    static constexpr int SPF = 2, SPF_DEEP = 4;            // k tiles in flight in registers (16-byte operands only)
    static constexpr const char *prefix = "mfma_f32";
};
template <>
struct TileShapes<double> {
    static constexpr bool kHasXL = true;
    static constexpr int YBM = 256, YBN = 128, YBK = 16;  // (no larger tile: 128 x 64 per wave already fills 256 accumulator registers)
    static constexpr int XBM = 256, XBN = 128, XBK = 16;  // 4 waves of 128 x 64 (8 x 4 blocks of 16 x 16), one workgroup per CU
    static constexpr int LBM = 128, LBN = 128, LBK = 16;  // 4 waves of 64 x 64 (4 x 4 blocks of 16 x 16)
    static constexpr int SBM = 64, SBN = 64, SBK = 16;    // 4 waves of 32 x 32
    static constexpr int SPF = 2, SPF_DEEP = 4;
    static constexpr const char *prefix = "mfma_f64";
};

struct SplitPlan {
    int ksplit = 1;
    int k_chunk = 0;
    bool fixed_scratch = false;  // partial tiles go to the library's fixed array (the call must not allocate)
};

ttamd_status launch_scratch(int device, hipStream_t stream, size_t bytes, bool fixed, void **out) {
    if (!fixed) return stream_scratch(device, stream, bytes, out);
    if (bytes > kFixedScratchBytes) {
        set_error("batched_matmul_noalloc: this product needs %zu bytes of partial results (a split reduction's tiles or "
                  "the column sums' rows); the fixed scratch holds %zu (use ttamd_batched_matmul)", bytes, kFixedScratchBytes);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    // Every stream of a GPU shares the one array.  The last stream that used it is remembered; a call on another stream
    // is only let through once the whole device has been synchronised since that use (ttamd_device_synchronize), because
    // two products in flight at once would overwrite each other's partial results without any error.
    {
        struct LastUse {
            bool used = false;
            hipStream_t stream = nullptr;
            uint64_t syncs_started = 0;
        };
        static std::mutex mu;
        static LastUse last[kMaxDevices];
        if (device < 0 || device >= kMaxDevices) {
            set_error("batched_matmul_noalloc: device id %d beyond the %d devices the fixed scratch serves", device, kMaxDevices);
            return TTAMD_ERR_INVALID_DEVICE;
        }
        std::lock_guard<std::mutex> lock(mu);
        LastUse &u = last[device];
        if (u.used && u.stream != stream && device_sync_completed(device) <= u.syncs_started) {
            set_error("batched_matmul_noalloc: the fixed scratch of device %d was last used on another stream and the device has "
                      "not been synchronised since (ttamd_device_synchronize); products in flight on two streams would "
                      "overwrite each other's partial results", device);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        u.used = true;
        u.stream = stream;
        u.syncs_started = device_sync_started(device);
    }
    return fixed_scratch_address(device, out);
}

// Column sums: `rows` partial rows per batch item go to scratch, finish_colsum adds them up after the GEMM.
template <typename T>
ttamd_status prepare_colsum(GemmArgs &g, int rows, int device, hipStream_t stream, bool fixed) {
    if (!g.colsum_out) return TTAMD_OK;
    void *ws = nullptr;
    const size_t bytes = static_cast<size_t>(g.batch) * rows * g.N * sizeof(T);
    if (ttamd_status st = launch_scratch(device, stream, bytes, fixed, &ws)) return st;
    g.colsum_partial = ws;
    g.colsum_rows = rows;
    return TTAMD_OK;
}
template <typename T>
ttamd_status finish_colsum(const GemmArgs &g, hipStream_t stream) {
    if (!g.colsum_out) return TTAMD_OK;
    colsum_reduce_kernel<T><<<dim3(static_cast<unsigned>((g.N + 63) / 64), g.batch), dim3(64), 0, stream>>>(
        static_cast<const T *>(g.colsum_partial), g.colsum_rows, g.N, static_cast<T *>(g.colsum_out));
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC, int PF>
ttamd_status launch_variant(const GemmArgs &g, const SplitPlan &sp, int device, hipStream_t stream) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC, PF>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC, PF>;
    constexpr size_t lds_bytes = TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>::kLdsBytes;
    constexpr bool kTwoKernels = BM * BN >= 128 * 128;
    const bool lean = plain_store(g);
    if (kTwoKernels && sp.ksplit != 1) {
        set_error("batched_matmul: internal error, split k planned for a %d x %d tile", BM, BN);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    constexpr int kEpiA = kTwoKernels ? kEpiLean : kEpiAny, kEpiB = kTwoKernels ? kEpiFull : kEpiAny,
                  kEpiC = kTwoKernels ? kEpiExt : kEpiAny;
    // the biggest tiles (one workgroup per CU, every register taken) have a kernel for problems of whole tiles
    // (fp32 256 x 256 only: the fp64 256 x 128 kernel has no scratch with its masked loop and 460 bytes without)
    constexpr bool kHasWhole = sizeof(T) == 4 && BM * BN >= 256 * 256 && A_VEC > 1 && B_VEC > 1;
    constexpr int kEpiD = kHasWhole ? kEpiLeanWhole : kEpiA;
    // (rows and columns outside the matrix need no masked loop: their loads carry out-of-range offsets either way; what
    // needs it is a k tile that reaches past K, or a 16-byte vector along m or n that straddles the matrix's edge)
    const bool whole = kHasWhole && lean && sp.ksplit == 1 && g.K % BK == 0 && g.K > 0 && (A_KC || g.M % A_VEC == 0) && (B_KC || g.N % B_VEC == 0);
    const int which = whole ? 3 : (lean ? 0 : (ext_store(g) ? 2 : 1));
    auto kernel = which == 0   ? gemm_mfma_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC, PF, kEpiA>
                  : which == 1 ? gemm_mfma_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC, PF, kEpiB>
                  : which == 2 ? gemm_mfma_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC, PF, kEpiC>
                               : gemm_mfma_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC, PF, kEpiD>;
    static std::atomic<bool> configured[kMaxDevices][4] = {};  // raising the dynamic LDS limit: once per kernel and device (host threads may race here: setting the attribute twice is harmless, a torn flag would not be)
    const int slot = device >= 0 && device < kMaxDevices ? device : 0;
    if ((!configured[slot][which].load(std::memory_order_acquire) || slot != device) && lds_bytes > 48 * 1024) {
        TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        configured[slot][which].store(true, std::memory_order_release);
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.batch * sp.ksplit;
    if (blocks > 0x7fffffff) {
        set_error("batched_matmul: %lld workgroups exceed the grid limit", static_cast<long long>(blocks));
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    T *partial = nullptr;
    GemmArgs ga = g;
    if (sp.ksplit > 1) {  // (never together with column sums: the planner does not split then)
        void *ws = nullptr;
        const size_t bytes = static_cast<size_t>(sp.ksplit) * g.batch * g.M * g.N * sizeof(T);
        if (ttamd_status st = launch_scratch(device, stream, bytes, sp.fixed_scratch, &ws)) return st;
        partial = static_cast<T *>(ws);
    } else if (ttamd_status st = prepare_colsum<T>(ga, tiles_m * WGM, device, stream, sp.fixed_scratch)) {
        return st;
    }
    kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(kThreads), lds_bytes, stream>>>(ga, tiles_m, tiles_n, sp.ksplit,
                                                                                      sp.ksplit > 1 ? sp.k_chunk : g.K, partial);
    TTAMD_HIP_CHECK(hipGetLastError());
    if (sp.ksplit > 1) {
        const int64_t mn = static_cast<int64_t>(g.M) * g.N;
        if (sp.ksplit >= 16 && mn * g.batch <= (1 << 20))  // few elements, many splits: four lanes to an element
            splitk_reduce_kernel<T, 4><<<dim3(static_cast<unsigned>((mn + 63) / 64), g.batch), dim3(256), 0, stream>>>(g, partial, sp.ksplit);
        else
            splitk_reduce_kernel<T, 1><<<dim3(static_cast<unsigned>((mn + 255) / 256), g.batch), dim3(256), 0, stream>>>(g, partial, sp.ksplit);
        TTAMD_HIP_CHECK(hipGetLastError());
    }
    return finish_colsum<T>(ga, stream);
}

// First k of the upper half of a two-half launch: half of K rounded up to a whole 16-byte vector, so that the upper
// half's operands keep their alignment.
template <typename T>
int dual_k_half(int K) {
    constexpr int VK = Mfma<T>::VK;
    return ((K + 1) / 2 + VK - 1) / VK * VK;
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KC, int A_VEC, bool B_KC, int B_VEC, int PF, bool BSUM = false>
ttamd_status launch_dual_variant(const GemmArgs &g, int device, hipStream_t stream, bool fixed_scratch) {
    using StA = Stager<T, BM, BK, A_KC, A_VEC, PF>;
    using StB = Stager<T, BN, BK, B_KC, B_VEC, PF, BSUM>;
    constexpr size_t lds_bytes = 2 * TileEngine<T, BM, BN, BK, WGM, WGN, StA, StB>::kLdsBytes;
    auto kernel = gemm_mfma_dual_kernel<T, BM, BN, BK, WGM, WGN, A_KC, A_VEC, B_KC, B_VEC, PF, BSUM>;
    static std::atomic<bool> configured[kMaxDevices] = {};  // once per kernel and device
    const int slot = device >= 0 && device < kMaxDevices ? device : 0;
    if (!configured[slot].load(std::memory_order_acquire) || slot != device) {
        TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            static_cast<int>(lds_bytes)));
        configured[slot].store(true, std::memory_order_release);
    }
    const int k_half = dual_k_half<T>(g.K);
    if (k_half <= 0 || (k_half + BK - 1) / BK != (g.K - k_half + BK - 1) / BK) {  // the halves share the engine's barriers
        set_error("batched_matmul: internal error, two-half kernel planned for K = %d", g.K);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.batch;
    GemmArgs ga = g;
    if (ttamd_status st = prepare_colsum<T>(ga, tiles_m * WGM, device, stream, fixed_scratch)) return st;
    kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(2 * kThreads), lds_bytes, stream>>>(ga, tiles_m, tiles_n, k_half);
    TTAMD_HIP_CHECK(hipGetLastError());
    return finish_colsum<T>(ga, stream);
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, int VEC, int PF, bool BSUM_OK = false>
ttamd_status launch_dual_layouts(const GemmArgs &g, bool a_kc, bool b_kc, int device, hipStream_t stream, bool fixed_scratch) {
    if constexpr (BSUM_OK) {  // the sums of B in the same launch (the caller has checked that b_kc is false)
        if (g.rhs_colsum && !b_kc) {
            if (a_kc) return launch_dual_variant<T, BM, BN, BK, WGM, WGN, true, VEC, false, VEC, PF, true>(g, device, stream, fixed_scratch);
            return launch_dual_variant<T, BM, BN, BK, WGM, WGN, false, VEC, false, VEC, PF, true>(g, device, stream, fixed_scratch);
        }
    }
    if (a_kc && b_kc) return launch_dual_variant<T, BM, BN, BK, WGM, WGN, true, VEC, true, VEC, PF>(g, device, stream, fixed_scratch);
    if (a_kc && !b_kc) return launch_dual_variant<T, BM, BN, BK, WGM, WGN, true, VEC, false, VEC, PF>(g, device, stream, fixed_scratch);
    if (!a_kc && b_kc) return launch_dual_variant<T, BM, BN, BK, WGM, WGN, false, VEC, true, VEC, PF>(g, device, stream, fixed_scratch);
    return launch_dual_variant<T, BM, BN, BK, WGM, WGN, false, VEC, false, VEC, PF>(g, device, stream, fixed_scratch);
}

template <typename T, int BM, int BN, int BK, int WGM, int WGN, int A_VEC, int B_VEC, int PF = 1>
ttamd_status launch_layouts(const GemmArgs &g, bool a_kc, bool b_kc, const SplitPlan &sp, int device, hipStream_t stream) {
    if (a_kc && b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, true, A_VEC, true, B_VEC, PF>(g, sp, device, stream);
    if (a_kc && !b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, true, A_VEC, false, B_VEC, PF>(g, sp, device, stream);
    if (!a_kc && b_kc) return launch_variant<T, BM, BN, BK, WGM, WGN, false, A_VEC, true, B_VEC, PF>(g, sp, device, stream);
    return launch_variant<T, BM, BN, BK, WGM, WGN, false, A_VEC, false, B_VEC, PF>(g, sp, device, stream);
}

// Two independent products in one launch (fp32, the 64 x 64 tile, whole reductions): workgroups [0, blocks0) compute
// tiles of the first, the rest tiles of the second.  Each product alone would leave the chip a single workgroup per CU
// (a Linear layer's two gradients at batch 1024: 256 tiles each) and pay its launch, its first loads and its stores with
// nothing else running; together two workgroups share every CU and each covers the other's waits.  BSUM: the second
// product's first row of tiles also adds up the vectors of B that it stages (see gemm_mfma_dual_kernel).
template <typename T, bool A_KC, bool B_KC, int PF, bool BSUM>
__device__ __forceinline__ void small_tile_product(const GemmArgs &g, int tiles_m, int tiles_n, unsigned block, unsigned blocks, unsigned char *smem_raw) {
    using TS = TileShapes<T>;
    constexpr int BM = TS::SBM, BN = TS::SBN, BK = TS::SBK, VK = Mfma<T>::VK;
    using StA = Stager<T, BM, BK, A_KC, VK, PF>;
    using StB = Stager<T, BN, BK, B_KC, VK, PF, BSUM>;
    using Engine = TileEngine<T, BM, BN, BK, 2, 2, StA, StB>;
    static_assert(!BSUM || static_cast<size_t>(StB::kSumParts) * BN * sizeof(T) <= Engine::kLdsBytes, "the operand sums fit the tile buffers");
    T *const smem = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    int batch, tm, tn;
    decode_tile(remap_xcd(block, blocks), tiles_m, tiles_n, batch, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const T *a_base = static_cast<const T *>(g.A) + static_cast<int64_t>(batch) * g.a_sb + static_cast<int64_t>(m0) * g.a_sm;
    const T *b_base = static_cast<const T *>(g.B) + static_cast<int64_t>(batch) * g.b_sb + static_cast<int64_t>(n0) * g.b_sn;
    StA sa;
    StB sb;
    sa.init(a_base, tid, g.M - m0, g.a_sm, g.a_sk, g.K);
    sb.init(b_base, tid, g.N - n0, g.b_sn, g.b_sk, g.K);
    if constexpr (BSUM) sb.start_sums(tm == 0);
    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, g.K, !sa.row_mask && !sb.row_mask);
    if constexpr (BSUM) {
        if (tm == 0) {  // (workgroup-uniform) a lane's k rows were added in k order; the lanes of a column follow in lane order
            __syncthreads();  // every wave is done with the tile buffers
            *reinterpret_cast<typename StB::V *>(&smem[sb.sum_part() * BN + sb.sum_row0()]) = sb.sum;
            __syncthreads();
            if (tid < BN && n0 + tid < g.N) {
                T v = T(0);
#pragma unroll
                for (int r = 0; r < StB::kSumParts; ++r) v += smem[r * BN + tid];
                static_cast<T *>(g.rhs_colsum)[static_cast<int64_t>(batch) * g.N + n0 + tid] = v;
            }
        }
    }
    T *C = static_cast<T *>(g.C) + static_cast<int64_t>(batch) * g.M * g.N;
    if (plain_store(g))
        store_tile_dense<T, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
    else if (!ext_store(g))
        store_tile_dense<T, false>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate);
    else
        store_tile_dense<T, false, true>(eng, C, g.M, g.N, m0, n0, static_cast<const T *>(g.bias), g.bias_mode, g.relu, g.accumulate,
                                         make_ext<T>(g, batch, tm, 2));
}

template <typename T, bool A0_KC, bool B0_KC, bool A1_KC, bool B1_KC, int PF, bool BSUM1>
__global__ void __launch_bounds__(kThreads, 2)  // (two workgroups per CU: at most 256 registers per lane)
gemm_mfma_pair_kernel(GemmArgs g0, int tiles_m0, int tiles_n0, GemmArgs g1, int tiles_m1, int tiles_n1, unsigned blocks0) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    if (blockIdx.x < blocks0)
        small_tile_product<T, A0_KC, B0_KC, PF, false>(g0, tiles_m0, tiles_n0, blockIdx.x, blocks0, smem_raw);
    else
        small_tile_product<T, A1_KC, B1_KC, PF, BSUM1>(g1, tiles_m1, tiles_n1, blockIdx.x - blocks0, gridDim.x - blocks0, smem_raw);
}

// Launches the two products as one grid when each is a dense fp32 product that would take the small tile with one
// workgroup per CU at most: first operand pair (k contiguous, k contiguous), second (m contiguous, n contiguous) -- the
// layouts of TensorBatchedMatmul::backward's two products on dense operands (autograd/binary_ops.cpp:173-179:
// dA = dC . B^T, dB = A^T . dC).  *handled = false: nothing was launched.
ttamd_status launch_pair_f32(const GemmArgs &g0, const GemmArgs &g1, int device, hipStream_t stream, bool *handled) {
    using T = float;
    using TS = TileShapes<T>;
    constexpr int VK = Mfma<T>::VK, PF = TS::SPF_DEEP;
    auto tiles_of = [](const GemmArgs &g) {
        return static_cast<int64_t>((g.M + TS::SBM - 1) / TS::SBM) * ((g.N + TS::SBN - 1) / TS::SBN) * g.batch;
    };
    auto fits = [&](const GemmArgs &g, bool kc) {
        if (g.M < 256 || g.N < 256 || g.K < 16 * TS::SBK || g.batch < 1 || g.colsum_out) return false;
        const OperandClass ca = classify<T>(g.A, g.a_sm, g.a_sk, g.a_sb, g.batch);
        const OperandClass cb = classify<T>(g.B, g.b_sn, g.b_sk, g.b_sb, g.batch);
        if (ca.vec != VK || cb.vec != VK || ca.kc != kc || cb.kc != kc) return false;
        // 32-bit byte offsets inside a tile's operand panels and output rows
        const int64_t a_reach = (static_cast<int64_t>(TS::SBM - 1) * g.a_sm + static_cast<int64_t>(g.K - 1) * g.a_sk + VK) * sizeof(T);
        const int64_t b_reach = (static_cast<int64_t>(TS::SBN - 1) * g.b_sn + static_cast<int64_t>(g.K - 1) * g.b_sk + VK) * sizeof(T);
        const int64_t c_reach = static_cast<int64_t>(TS::SBM) * g.N * static_cast<int64_t>(sizeof(T));
        if (a_reach >= 0x7fffffffLL || b_reach >= 0x7fffffffLL || c_reach >= 0x7fffffffLL) return false;
        const int64_t tiles = tiles_of(g);
        return tiles >= 128 && tiles <= 256;
    };
    *handled = false;
    static const bool enabled = std::getenv("TTAMD_MATMUL_PAIR") == nullptr || std::atoi(std::getenv("TTAMD_MATMUL_PAIR")) != 0;
    if (!enabled || !fits(g0, true) || !fits(g1, false)) return TTAMD_OK;
    const bool bsum = g1.rhs_colsum != nullptr;
    using StK = Stager<T, TS::SBM, TS::SBK, true, VK, PF>;
    using StM = Stager<T, TS::SBM, TS::SBK, false, VK, PF>;
    constexpr size_t lds0 = TileEngine<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, StK, StK>::kLdsBytes;
    constexpr size_t lds1 = TileEngine<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, StM, StM>::kLdsBytes;
    constexpr size_t lds_bytes = lds0 > lds1 ? lds0 : lds1;
    static_assert(lds_bytes <= 48 * 1024, "within the default dynamic LDS limit");
    const unsigned blocks0 = static_cast<unsigned>(tiles_of(g0)), blocks1 = static_cast<unsigned>(tiles_of(g1));
    const int tm0 = (g0.M + TS::SBM - 1) / TS::SBM, tn0 = (g0.N + TS::SBN - 1) / TS::SBN;
    const int tm1 = (g1.M + TS::SBM - 1) / TS::SBM, tn1 = (g1.N + TS::SBN - 1) / TS::SBN;
    if (bsum)
        gemm_mfma_pair_kernel<T, true, true, false, false, PF, true><<<dim3(blocks0 + blocks1), dim3(kThreads), lds_bytes, stream>>>(g0, tm0, tn0, g1, tm1, tn1, blocks0);
    else
        gemm_mfma_pair_kernel<T, true, true, false, false, PF, false><<<dim3(blocks0 + blocks1), dim3(kThreads), lds_bytes, stream>>>(g0, tm0, tn0, g1, tm1, tn1, blocks0);
    TTAMD_HIP_CHECK(hipGetLastError());
    if (bsum && g1.rhs_colsum_done) *g1.rhs_colsum_done = true;
    *handled = true;
    return TTAMD_OK;
}

// Split the reduction when the output has too few tiles to fill 256 CUs and K is long enough to share out.
// Every split gets a whole number of BK tiles; at most 64 splits and 32 MiB of partial tiles.
template <typename T>
SplitPlan plan_split(const GemmArgs &g, int bm, int bn, int bk) {
    SplitPlan sp;
    sp.k_chunk = g.K;
    const int64_t tiles = static_cast<int64_t>((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * g.batch;
    const int k_tiles = (g.K + bk - 1) / bk;
    if (tiles >= 128 || k_tiles < 4 || g.batch > 65535 || g.colsum_out) return sp;  // (column sums come from whole tiles)
    int want = static_cast<int>((256 + tiles - 1) / tiles);
    const int max_by_k = k_tiles / 2;  // at least two k tiles per split
    if (want > max_by_k) want = max_by_k;
    if (want > 64) want = 64;
    const int64_t bytes_per_split = static_cast<int64_t>(g.batch) * g.M * g.N * static_cast<int64_t>(sizeof(T));
    const int64_t cap = (32LL << 20) / (bytes_per_split > 0 ? bytes_per_split : 1);
    if (want > cap) want = static_cast<int>(cap);
    if (want < 2) return sp;
    const int chunk_tiles = (k_tiles + want - 1) / want;
    sp.k_chunk = chunk_tiles * bk;
    sp.ksplit = (g.K + sp.k_chunk - 1) / sp.k_chunk;
    if (sp.ksplit < 2) {
        sp.ksplit = 1;
        sp.k_chunk = g.K;
    }
    return sp;
}

template <typename T>
ttamd_status launch_mfma_typed(const GemmArgs &g, int device, hipStream_t stream, const char **variant, bool variant_only,
                               bool *handled, bool fixed_scratch) {
    using TS = TileShapes<T>;
    constexpr int VK = Mfma<T>::VK;
    *handled = false;

    OperandClass ca = classify<T>(g.A, g.a_sm, g.a_sk, g.a_sb, g.batch);
    OperandClass cb = classify<T>(g.B, g.b_sn, g.b_sk, g.b_sb, g.batch);
    const bool vec = ca.vec > 1 && cb.vec > 1;

    // Tile choice by a small cost model fitted to measurements on MI355X (256 CUs): a configuration keeps `per_cu`
    // workgroups resident per CU and sustains `rate` flop/s when every slot is busy; workgroups are dealt to the
    // CUs round-robin, so a partial last round costs a whole round as soon as any CU holds a full complement,
    // and a fraction of it when the CUs are thinly populated (a workgroup alone on a CU runs faster).
    const double scale = sizeof(T) == 4 ? 1.0 : 0.5;
    auto estimate = [&](int bm_, int bn_, int per_cu, double rate, double thin = 0.12) {
        const double tiles = static_cast<double>((g.M + bm_ - 1) / bm_) * ((g.N + bn_ - 1) / bn_) * g.batch;
        const double slots = 256.0 * per_cu;
        const double rounds = std::floor(tiles / slots), frac = tiles / slots - rounds;
        double last = 0.0;
        if (frac > 0.0) {
            const double fill = std::ceil(frac * per_cu - 1e-9) / per_cu;  // busiest CU's share of its slots
            last = fill >= 1.0 ? 1.0 : thin + (1.0 - thin) * fill;
        }
        const double round_time = 2.0 * bm_ * bn_ * static_cast<double>(g.K) * slots / (rate * scale);
        return (rounds + last) * round_time;
    };
    // The small tile sustains 139 TFLOP/s once several rounds overlap each other's first loads and stores (5120^3:
    // 1.92 ms in 6.25 rounds); a launch pays for that ramp once, about 6 % of a round (2048^3 in exactly one round:
    // 130 us, 132 TFLOP/s).
    const double t_small = estimate(TS::SBM, TS::SBN, 4, 139e12) +
                           0.06 * 2.0 * TS::SBM * TS::SBN * static_cast<double>(g.K) * 1024.0 / (139e12 * scale);
    constexpr bool f32 = sizeof(T) == 4;  // the fp64 big tiles run one workgroup per CU (accumulators in AGPRs)
    const double t_large = vec ? estimate(TS::LBM, TS::LBN, f32 ? 2 : 1, f32 ? 150e12 : 148e12, 0.08) : 1e300;
    const double t_xl = (TS::kHasXL && vec) ? estimate(TS::XBM, TS::XBN, f32 ? 2 : 1, f32 ? 149e12 : 152e12) : 1e300;
    const double t_xxl = (TS::kHasXL && vec && sizeof(T) == 4) ? estimate(TS::YBM, TS::YBN, 1, 151e12) : 1e300;
    double t_mid = 1e300;
    if constexpr (sizeof(T) == 4)  // whole tiles only: its ragged edge tiles run at two thirds of the rate (5120^3: 2.9 ms against 2.0)
        if (vec && g.M % TS::MBM == 0 && g.N % TS::MBN == 0) t_mid = estimate(TS::MBM, TS::MBN, 1, 149e12);
    const double t_best = std::min(std::min(std::min(t_xxl, t_xl), std::min(t_large, t_small)), t_mid);
    const bool xxl = t_xxl <= t_best;
    const bool xl = !xxl && t_xl <= t_best;
    const bool mid = !xxl && !xl && t_mid <= t_best;
    const bool large = !xxl && !xl && !mid && t_large <= t_best;
    const int bm = (xxl || xl) ? TS::XBM : (mid ? 192 : (large ? TS::LBM : TS::SBM));
    // 32-bit buffer addressing: the bytes reachable from a tile's first row must stay below 2^31.
    const int64_t a_reach = (static_cast<int64_t>(bm - 1) * g.a_sm + static_cast<int64_t>(g.K - 1) * g.a_sk + VK) * sizeof(T);
    const int64_t b_reach = (static_cast<int64_t>(bm - 1) * g.b_sn + static_cast<int64_t>(g.K - 1) * g.b_sk + VK) * sizeof(T);
    const int64_t c_reach = static_cast<int64_t>(g.M < bm ? g.M : bm) * g.N * static_cast<int64_t>(sizeof(T));
    if (a_reach >= 0x7fffffffLL || b_reach >= 0x7fffffffLL || c_reach >= 0x7fffffffLL) return TTAMD_OK;

    SplitPlan sp = (xxl || xl || mid || large) ? SplitPlan{1, g.K} : plan_split<T>(g, TS::SBM, TS::SBN, TS::SBK);
    sp.fixed_scratch = fixed_scratch;

    // Small tiles, at most one workgroup per CU and a long reduction: two halves of k in one workgroup of 8 waves.
    const int64_t small_wgs = static_cast<int64_t>((g.M + TS::SBM - 1) / TS::SBM) * ((g.N + TS::SBN - 1) / TS::SBN) * g.batch;
    const int k_half = dual_k_half<T>(g.K);
    const int half_tiles = (k_half + TS::SBK - 1) / TS::SBK;
    const bool dual = !(xxl || xl || mid || large) && vec && sp.ksplit == 1 && small_wgs <= 256 && half_tiles >= 8 &&
                      (g.K - k_half + TS::SBK - 1) / TS::SBK == half_tiles;

    // The 128 x 128 tile (fp32) with at most one workgroup per CU and a reduction of 2048 or more: the same two halves
    // (2048^3: 128.4 -> 126.5 us, 2048 x 4096 x 2048: 250.3 -> 244.6; shorter reductions lose: K = 784 53.8 -> 60.9).
    const int64_t large_wgs = static_cast<int64_t>((g.M + TS::LBM - 1) / TS::LBM) * ((g.N + TS::LBN - 1) / TS::LBN) * g.batch;
    const int large_half_tiles = (k_half + TS::LBK - 1) / TS::LBK;
    const bool dual_large = sizeof(T) == 4 && large && large_wgs <= 256 && large_half_tiles >= 64 &&
                            (g.K - k_half + TS::LBK - 1) / TS::LBK == large_half_tiles;

    static thread_local char name[112];
    char split_tag[24] = "";
    if (sp.ksplit > 1) snprintf(split_tag, sizeof(split_tag), "_splitk%d", sp.ksplit);
    if (dual || dual_large) snprintf(split_tag, sizeof(split_tag), "_halves");
    snprintf(name, sizeof(name), "%s_%s_a%s%d_b%s%d%s", TS::prefix, xxl ? "256x256" : (xl ? "256x128" : (mid ? "192x192" : (large ? "128x128" : "64x64"))), ca.kc ? "kc" : "mc",
             ca.vec, cb.kc ? "kc" : "mc", cb.vec, split_tag);
    *variant = name;
    *handled = true;
    if (variant_only) return TTAMD_OK;

    // The large tile exists for 16-byte operands only; the small tile for every mix of 16-byte and element-wise.
    if constexpr (TS::kHasXL) {
        if (xxl) return launch_layouts<T, TS::YBM, TS::YBN, TS::YBK, 2, 2, VK, VK>(g, ca.kc, cb.kc, sp, device, stream);
        if (xl) return launch_layouts<T, TS::XBM, TS::XBN, TS::XBK, 2, 2, VK, VK>(g, ca.kc, cb.kc, sp, device, stream);
    }
    if constexpr (sizeof(T) == 4)
        if (mid) return launch_layouts<T, TS::MBM, TS::MBN, TS::MBK, 2, 2, VK, VK>(g, ca.kc, cb.kc, sp, device, stream);
    if constexpr (sizeof(T) == 4)
        if (dual_large) return launch_dual_layouts<T, TS::LBM, TS::LBN, TS::LBK, 2, 2, VK, 1>(g, ca.kc, cb.kc, device, stream, fixed_scratch);
    if (large) return launch_layouts<T, TS::LBM, TS::LBN, TS::LBK, 2, 2, VK, VK>(g, ca.kc, cb.kc, sp, device, stream);
    if (dual) {
        if (g.rhs_colsum && !cb.kc && g.rhs_colsum_done) *g.rhs_colsum_done = true;  // (the kernel's first row of tiles adds B up)
        return launch_dual_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, VK, TS::SPF_DEEP, true>(g, ca.kc, cb.kc, device, stream, fixed_scratch);
    }
    if (ca.vec > 1 && cb.vec > 1) {
        // Register prefetch depth of the small tile: 4 k tiles in flight when a CU holds at most two workgroups and the
        // reduction is long (a lone workgroup otherwise waits for memory in every step), else 2, whose smaller register
        // footprint keeps more workgroups resident (832 tiles with K = 288: 26.5 us against 31.2 us at depth 4).
        const int64_t wgs = static_cast<int64_t>((g.M + TS::SBM - 1) / TS::SBM) * ((g.N + TS::SBN - 1) / TS::SBN) * g.batch * sp.ksplit;
        const int k_tiles = ((sp.ksplit > 1 ? sp.k_chunk : g.K) + TS::SBK - 1) / TS::SBK;
        if (k_tiles >= 16 && wgs <= 512)
            return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, VK, VK, TS::SPF_DEEP>(g, ca.kc, cb.kc, sp, device, stream);
        return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, VK, VK, TS::SPF>(g, ca.kc, cb.kc, sp, device, stream);
    }
    if (ca.vec > 1) return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, VK, 1>(g, ca.kc, cb.kc, sp, device, stream);
    if (cb.vec > 1) return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, 1, VK>(g, ca.kc, cb.kc, sp, device, stream);
    return launch_layouts<T, TS::SBM, TS::SBN, TS::SBK, 2, 2, 1, 1>(g, ca.kc, cb.kc, sp, device, stream);
}

}  // namespace

ttamd_status gemm_scratch(int device, hipStream_t stream, size_t bytes, bool fixed, void **out) {
    return launch_scratch(device, stream, bytes, fixed, out);
}

ttamd_status launch_colsum_reduce(ttamd_dtype dt, const void *partial, int rows, int N, int batch, void *out, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((N + 63) / 64), static_cast<unsigned>(batch));
    if (dt == TTAMD_F32)
        colsum_reduce_kernel<float><<<grid, dim3(64), 0, stream>>>(static_cast<const float *>(partial), rows, N, static_cast<float *>(out));
    else
        colsum_reduce_kernel<double><<<grid, dim3(64), 0, stream>>>(static_cast<const double *>(partial), rows, N, static_cast<double *>(out));
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

ttamd_status launch_gemm_pair(ttamd_dtype dt, const GemmArgs &g0, const GemmArgs &g1, int device, hipStream_t stream, bool *handled) {
    *handled = false;
    if (dt == TTAMD_F32) return launch_pair_f32(g0, g1, device, stream, handled);
    return TTAMD_OK;
}

ttamd_status launch_gemm_mfma(ttamd_dtype dt, const GemmArgs &g, int device, hipStream_t stream, const char **variant,
                              bool variant_only, bool *handled, bool fixed_scratch) {
    *handled = false;
    if (dt == TTAMD_F32) return launch_mfma_typed<float>(g, device, stream, variant, variant_only, handled, fixed_scratch);
    if (dt == TTAMD_F64) return launch_mfma_typed<double>(g, device, stream, variant, variant_only, handled, fixed_scratch);
    return TTAMD_OK;
}

}  // namespace ttamd
