// mfma_core.h — device-side building blocks of the matrix-core kernels (gfx950 only).
//
// One workgroup = 4 wavefronts of 64 lanes computing a BM x BN tile of C = A . B:
//   * operand tiles (BM x BK, BN x BK) are staged global -> registers -> LDS by a "stager" per operand;
//     two LDS buffers per operand, the loads of tile t+1 are issued before the MFMA work of tile t and
//     parked in the other buffer afterwards, one barrier per tile;
//   * fp32: v_mfma_f32_32x32x2_f32, fp64: v_mfma_f64_16x16x4_f64; accumulators stay in registers;
//   * LDS layout follows the operand's memory layout, so nothing is transposed on the way in:
//       KC  element (r, k) at r * LD + k   (k contiguous; rows padded by one 16-byte vector so that 16-byte
//                                           fragment reads of consecutive rows land in distinct banks)
//       MC  element (r, k) at k * LD + r   (row/column index contiguous)
//     fragment reads pair k indices so that both operands agree whatever their layouts;
//   * all global reads are buffer loads that carry the operand's byte extent: a lane that is out of the tile
//     uses an offset with bit 31 set and receives zero instead of touching memory.
//
// A stager is any type with
//     static constexpr bool kKC; static constexpr int LD, LDS_ELEMS;
//     static constexpr int kPF;                                  // register slots = tiles kept in flight
//     template <bool MASK, int SLOT> void load(int k_left);      // fetch the next BK-deep tile into slot SLOT
//     template <int SLOT> void store(T *lds) const;              // write that slot to an LDS buffer
// Stager<> below reads a strided matrix view; conv.hip adds gather stagers (implicit im2col).
#ifndef TTAMD_CSRC_MFMA_CORE_H_
#define TTAMD_CSRC_MFMA_CORE_H_

#include "common.h"

namespace ttamd {
namespace mfma {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kChunk = 8;               // k extent of one fragment read (both dtypes)
constexpr uint32_t kOob = 0x80000000u;  // byte offset that is out of range for every buffer used here

// ---------------------------------------------------------------------------------------------
// MFMA instruction traits.  A lane l holds A[i = l % MB][k = l / MB] and B[k = l / MB][j = l % MB].
template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
    static constexpr int MB = 32;  // block is MB x MB
    static constexpr int VK = 4;   // elements in 16 bytes = k steps per chunk
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
    // per-lane offset plus a wave-uniform one (the scalar offset operand of the load)
    static __device__ __forceinline__ type load_at(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t uniform_off) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, uniform_off, 0));
    }
};
template <>
struct Vec<float, 2> {  // 8-byte gathers of the conv stagers for rows of 2n (but not 4n) elements
    using type = float __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    }
};
template <>
struct Vec<float, 4> {
    using type = f32x4;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
    }
    static __device__ __forceinline__ type load_at(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t uniform_off) {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, uniform_off, 0));
    }
};
template <>
struct Vec<double, 1> {
    using type = double;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    }
    static __device__ __forceinline__ type load_at(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t uniform_off) {
        return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, off, uniform_off, 0));
    }
};
template <>
struct Vec<double, 2> {
    using type = f64x2;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(f64x2, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
    }
    static __device__ __forceinline__ type load_at(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t uniform_off) {
        return __builtin_bit_cast(f64x2, __builtin_amdgcn_raw_buffer_load_b128(r, off, uniform_off, 0));
    }
};

// Typed buffer stores of one element or of a pair of neighbouring elements.
using u32x2 = uint32_t __attribute__((ext_vector_type(2)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void buffer_store(__amdgpu_buffer_rsrc_t r, uint32_t off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, off, 0, 0);
}
__device__ __forceinline__ void buffer_store(__amdgpu_buffer_rsrc_t r, uint32_t off, double v) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), r, off, 0, 0);
}
__device__ __forceinline__ void buffer_store(__amdgpu_buffer_rsrc_t r, uint32_t off, f32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), r, off, 0, 0);
}
__device__ __forceinline__ void buffer_store(__amdgpu_buffer_rsrc_t r, uint32_t off, f64x2 v) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, off, 0, 0);
}

template <typename T, int VEC>
__device__ __forceinline__ void zero_component(typename Vec<T, VEC>::type &v, int j) {
    if constexpr (VEC == 1) {
        v = T(0);
    } else {
        v[j] = T(0);
    }
}

// Raw buffer descriptor over [base, base + bytes), bytes clamped to 2^31 - 1 (offsets >= 2^31 are the
// out-of-range marker).  Base and size are the same for every lane of a workgroup; they are passed through
// readfirstlane so that the descriptor provably lives in scalar registers (otherwise each buffer load is
// wrapped in a waterfall loop, which also fences the instruction scheduler).
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const T *base, int64_t bytes) {
    int rec = bytes > 0x7fffffff ? 0x7fffffff : (bytes < 0 ? 0 : static_cast<int>(bytes));
    const uint64_t addr = reinterpret_cast<uint64_t>(base);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32));
    rec = __builtin_amdgcn_readfirstlane(rec);
    T *uniform_base = reinterpret_cast<T *>((static_cast<uint64_t>(hi) << 32) | lo);
    return __builtin_amdgcn_make_buffer_rsrc(uniform_base, 0, rec, 0x00020000);
}

// LDS geometry shared by every stager of a given layout.
template <typename T, int ROWS, int BK, bool KC>
struct TileLayout {
    static constexpr bool kKC = KC;
    static constexpr int PAD = Mfma<T>::VK;  // one 16-byte vector
    static constexpr int LD = KC ? (BK + PAD) : (ROWS + PAD);
    static constexpr int LDS_ELEMS = KC ? ROWS * LD : BK * LD;
};

// ---------------------------------------------------------------------------------------------
// Stager for a strided matrix view (ROWS along m or n, BK along k).  Vectors of VEC elements run along k
// for KC (operand's k stride is 1 when VEC > 1) and along the row index for MC (row stride 1 when VEC > 1).
// PF register slots hold PF tiles in flight (prefetch distance PF).
// SUM (MC with whole vectors only): every vector that is parked in LDS is also added to `sum` when `sum_on` is set -- a
// lane's vectors all hold the same VEC rows of the operand (columns of B), so after the reduction `sum` is this
// lane's share of the operand's sums over k, masked elements counting as zero.
template <typename T, int ROWS, int BK, bool KC, int VEC, int PF = 1, bool SUM = false>
struct Stager : TileLayout<T, ROWS, BK, KC> {
    using L = TileLayout<T, ROWS, BK, KC>;
    using V = typename Vec<T, VEC>::type;
    static constexpr int kPF = PF;
    static constexpr int VPL = (KC ? BK : ROWS) / VEC;  // vectors per LDS line
    static constexpr int NV = ROWS * BK / VEC;
    static constexpr int P = NV / kThreads;
    static_assert(NV % kThreads == 0, "tile must split evenly over the workgroup");

    static_assert(!SUM || (!KC && VEC > 1 && kThreads % VPL == 0), "sums: vectors along the rows, the same rows in every pass of a lane");
    V reg[PF][P];
    mutable V sum;        // SUM only
    bool sum_on = false;  // SUM only, workgroup-uniform
    uint32_t voff[P];
    int nval[P];  // MC only: valid components of the vector along the row dimension
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t k_step_b;
    uint32_t k_off;  // wave-uniform part of the walk along k (see load)
    int tid;
    bool edge;
    bool row_mask;  // some vector of this tile holds rows both inside and outside the matrix: loads must mask

    // line/column coordinates of pass p for this lane
    static __device__ __forceinline__ int line_of(int p, int tid) { return (p * kThreads + tid) / VPL; }
    static __device__ __forceinline__ int col_of(int p, int tid) { return ((p * kThreads + tid) % VPL) * VEC; }

    // base: element (row 0 of this tile, k = 0); rows_left: valid rows from there; strides in elements;
    // K: full reduction length (sizes the buffer extent).
    __device__ __forceinline__ void init(const T *base, int tid_, int rows_left, int64_t s_row, int64_t s_k, int K) {
        tid = tid_;
        edge = rows_left < ROWS;
        // KC vectors run along k and element-wise loads fetch one row: a row outside the matrix costs only its offset
        // (out of range, the load returns 0).  MC vectors hold VEC consecutive rows.
        row_mask = !KC && VEC > 1 && edge && rows_left % VEC != 0;
        int64_t ext = (static_cast<int64_t>(rows_left - 1) * s_row + static_cast<int64_t>(K - 1) * s_k + 1) * sizeof(T);
        // With 16-byte loads the extent is rounded up to the vector size: the base is 16-byte aligned, so the
        // last vector stays inside the allocation's final 16-byte block and its tail is masked anyway.
        if (VEC > 1) ext = (ext + 15) & ~static_cast<int64_t>(15);
        rsrc = make_rsrc(base, ext);
        const uint32_t s_row_b = static_cast<uint32_t>(s_row * sizeof(T)), s_k_b = static_cast<uint32_t>(s_k * sizeof(T));
        k_step_b = s_k_b * BK;
        k_off = 0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int line = line_of(p, tid), col = col_of(p, tid);
            if constexpr (KC) {
                voff[p] = line < rows_left ? (line * s_row_b + col * s_k_b) : kOob;
                nval[p] = VEC;
            } else {
                int nv = rows_left - col;
                nv = nv < 0 ? 0 : (nv > VEC ? VEC : nv);
                nval[p] = nv;
                voff[p] = nv > 0 ? (col * s_row_b + line * s_k_b) : kOob;
            }
        }
    }

    // Fetches the next tile into register slot SLOT; k_left = K - (first k of that tile).  MASK = false is
    // the steady state (full k tile, interior rows): loads only, no selects.
    // UNIFORM_K: the step along k is kept in a scalar register and handed to the load as its scalar offset, so the
    // walk costs one scalar add per tile instead of a vector add per load.  The hardware does not range-check the
    // scalar offset: only for loads whose tile lies inside K (rows outside the matrix still have their out-of-range
    // per-lane offset and load zeros).  The two forms may be mixed: the address is always voff + k_off.
    template <bool MASK, int SLOT = 0, bool UNIFORM_K = false>
    __device__ __forceinline__ void load(int k_left) {
        static_assert(!(MASK && UNIFORM_K), "a masked load relies on the range check of its whole offset");
        // A vector that lies wholly beyond K (or wholly in rows outside the matrix: init) is requested at the
        // out-of-range offset and comes back as zeros.  Only a vector that straddles the edge needs a select on the
        // loaded data, and a select makes the wave wait for its load on the spot, a full memory round trip per load
        // with nothing else in flight: that is left to the layouts that can have such vectors (a k extent that is
        // not a multiple of the vector, rows_left not a multiple of it), under a workgroup-uniform condition.
        const bool k_straddle = KC && VEC > 1 && k_left > 0 && k_left < BK && k_left % VEC != 0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            V v;
            if constexpr (UNIFORM_K) {
                v = Vec<T, VEC>::load_at(rsrc, voff[p], k_off);
            } else {
                uint32_t off = voff[p] + k_off;
                if constexpr (MASK) {
                    if ((KC ? col_of(p, tid) : line_of(p, tid)) >= k_left) off = kOob;
                }
                v = Vec<T, VEC>::load(rsrc, off);
                voff[p] += k_step_b;
            }
            if constexpr (MASK && VEC > 1) {
                if constexpr (KC) {
                    if (k_straddle) {
                        const int col = col_of(p, tid);
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (col + j >= k_left) zero_component<T, VEC>(v, j);
                    }
                } else {
                    if (row_mask) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (j >= nval[p]) zero_component<T, VEC>(v, j);
                    }
                }
            }
            reg[SLOT][p] = v;
        }
        if constexpr (UNIFORM_K) k_off += k_step_b;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int line = line_of(p, tid), col = col_of(p, tid);
            *reinterpret_cast<V *>(&lds[line * L::LD + col]) = reg[SLOT][p];
        }
        if constexpr (SUM) {
            if (sum_on) {  // (every tile is parked exactly once: tile 0 by the prologue, tile kt + 1 by step kt)
#pragma unroll
                for (int p = 0; p < P; ++p) sum += reg[SLOT][p];
            }
        }
    }
    // SUM: start the sums (before the first tile is parked).
    __device__ __forceinline__ void start_sums(bool on) {
        sum_on = on;
#pragma unroll
        for (int j = 0; j < VEC; ++j) sum[j] = T(0);
    }
    // SUM: the rows this lane's sums belong to (tile-local, VEC consecutive ones) and which of the kThreads / VPL
    // lanes with the same rows this one is.
    __device__ __forceinline__ int sum_row0() const { return col_of(0, tid); }
    __device__ __forceinline__ int sum_part() const { return tid / VPL; }
    static constexpr int kSumParts = SUM ? kThreads / VPL : 1;
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

// Logical workgroup id -> (batch, tile row, tile column); tiles are walked in groups of 8 tile rows so that
// the workgroups resident on one XCD share operand panels through its L2.
__device__ __forceinline__ void decode_tile(int pid, int tiles_m, int tiles_n, int &batch, int &tm, int &tn) {
    // (All values are workgroup-uniform; an integer division is some forty scalar instructions in a kernel's first
    // microsecond, so the common cases -- one batch item, a full group of eight tile rows -- go without.)
    const int tiles = tiles_m * tiles_n;
    batch = pid < tiles ? 0 : pid / tiles;
    pid -= batch * tiles;
    constexpr int GROUP = 8;
    const int group_sz = GROUP * tiles_n;
    const int group = pid < group_sz ? 0 : pid / group_sz;
    const int first_m = group * GROUP;
    const int in_group = pid - group * group_sz;
    const int gm = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    if (gm == GROUP) {
        tm = first_m + in_group % GROUP;
        tn = in_group / GROUP;
    } else {
        tm = first_m + in_group % gm;
        tn = in_group / gm;
    }
}

// ---------------------------------------------------------------------------------------------
// The tile engine: software pipeline + MFMA loop + register -> memory walk of the finished tile.
template <typename T, int BM, int BN, int BK, int WGM, int WGN, class StA, class StB>
struct TileEngine {
    using M = Mfma<T>;
    static_assert(WGM * WGN == kWaves, "4 waves per workgroup");
    static constexpr int kBM = BM, kBN = BN;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int NBM = WM / M::MB, NBN = WN / M::MB;
    static_assert(WM % M::MB == 0 && WN % M::MB == 0 && BK % kChunk == 0, "tile shape");
    using FrA = Fragment<T, StA::LD, StA::kKC, NBM>;
    using FrB = Fragment<T, StB::LD, StB::kKC, NBN>;
    // LDS: [A buf 0][A buf 1][B buf 0][B buf 1]; addressed as offsets from the one shared base so that every
    // access stays a DS instruction (generic-pointer loads would also wait on the global-load counter).
    static constexpr int kBOff = 2 * StA::LDS_ELEMS;
    static constexpr size_t kLdsBytes = 2 * (StA::LDS_ELEMS + StB::LDS_ELEMS) * sizeof(T);

    typename M::acc_t acc[NBM][NBN];
    // Two schedules of the main loop, chosen by the number of MFMA blocks a wave owns:
    //  * pipelined (two chunks per k tile and at least 4 fp32 / 16 fp64 blocks: 128 x 128, 256 x 128, 256 x 256) - see
    //    step_pipe();
    //  * rotated (at most 4 blocks: 64 x 64 tiles, conv tiles) - see step_rot().
    static constexpr bool kPipe = BK / kChunk == 2 && NBM * NBN >= (sizeof(T) == 4 ? 4 : 16);
    static constexpr bool kRotate = !kPipe && NBM * NBN <= 4;
    FrA last_a;  // fragments of the previous tile's last chunk, multiplied after the barrier
    FrB last_b;
    int lane, wm0, wn0;

    __device__ __forceinline__ void init(int tid) {
        lane = tid % 64;
        const int wave = tid / 64;
        wm0 = (wave / WGN) * WM;
        wn0 = (wave % WGN) * WN;
#pragma unroll
        for (int i = 0; i < NBM; ++i)
#pragma unroll
            for (int j = 0; j < NBN; ++j)
#pragma unroll
                for (int e = 0; e < M::NACC; ++e) acc[i][j][e] = T(0);
    }

    // ---- rotated schedule (tiles with at most 4 MFMA blocks per wave) ----
    __device__ __forceinline__ void read_frags(const T *smem, int buf, int chunk, FrA &fa, FrB &fb) const {
        fa.read(smem + buf * StA::LDS_ELEMS, wm0, chunk, lane);
        fb.read(smem + kBOff + buf * StB::LDS_ELEMS, wn0, chunk, lane);
    }
    __device__ __forceinline__ void mma_chunk(const FrA &fa, const FrB &fb) {
#pragma unroll
        for (int j = 0; j < M::VK; ++j)
#pragma unroll
            for (int bm = 0; bm < NBM; ++bm)
#pragma unroll
                for (int bn = 0; bn < NBN; ++bn) acc[bm][bn] = M::mma(fa.v[bm][j], fb.v[bn][j], acc[bm][bn]);
    }
    // One pipeline step for tile kt.  The loop is rotated so that the barrier sits between reading the last chunk's
    // fragments and multiplying them:
    //   on entry the barrier that published tile kt has just been passed and (PENDING) the fragments of the
    //   previous tile's last chunk wait in registers (last_a, last_b);
    //   1. request chunk 0 of tile kt from LDS and (LOAD) tile kt + PF from memory into slot kt % PF, and multiply
    //      the pending chunk: its MFMAs cover the LDS latency of the request, which is otherwise exposed after every
    //      barrier when a SIMD has few waves to run; in the unmasked loop the first of them is issued ahead of the
    //      requests;
    //   2. for c = 0 .. NC-2: request chunk c + 1 of tile kt from LDS (the last chunk's fragments go to (last_a,
    //      last_b)), then multiply chunk c;
    //   3. the last multiplied chunk also parks tile kt + 1 (slot (kt + 1) % PF) in the other LDS buffer, its stores
    //      slotted between the MFMAs;
    //   4. barrier.
    // The other LDS buffer was last read in part 2 of the previous step (before its barrier), so it may be
    // overwritten here; tile kt's buffer is only read.
    template <int S, bool LOAD, bool MASK, bool PENDING>
    __device__ __forceinline__ void step_rot(StA &sa, StB &sb, T *smem, int K, int kt) {
        constexpr int PF = StA::kPF;
        constexpr int NC = BK / kChunk;
        static_assert(NC >= 2, "a k tile holds at least two chunks");
        constexpr int kChunkMfmas = M::VK * NBM * NBN;  // MFMAs of one chunk
        constexpr int kStores = StA::P + StB::P;        // LDS store instructions (and global loads) of one tile, per lane
        constexpr int kAllReads = 64;                   // "every LDS read of the region" for a scheduling group
        const int cur = kt & 1;
        // Fragments are double-buffered in registers: chunk c + 1 is requested from LDS before chunk c is multiplied,
        // so a read has a chunk's MFMAs to arrive in (requested just in time it stalls the wave for the LDS latency,
        // several times per step).
        FrA fa[2];
        FrB fb[2];
        constexpr bool kMfmaFirst = PENDING && !MASK && LOAD && kChunkMfmas >= 2;
        // (s_setprio is a fixed point for the instruction scheduler: where the requests are to be moved behind the
        // first MFMA it has to come before them)
        if constexpr (kMfmaFirst) __builtin_amdgcn_s_setprio(3);
        read_frags(smem, cur, 0, fa[0], fb[0]);
        if constexpr (LOAD) {
            const int k_left = K - (kt + PF) * BK;
            sa.template load<MASK, S>(k_left);
            sb.template load<MASK, S>(k_left);
        }
        if constexpr (kMfmaFirst) {
            // The pending chunk's operands are in registers: its first MFMA goes out right after the barrier and the
            // requests follow in its shadow (LDS reads first, they are needed first), instead of the matrix pipe
            // idling while every wave of the workgroup issues its requests at the same moment.
            mma_chunk(last_a, last_b);
            constexpr int kGaps = kChunkMfmas - 1;
            constexpr int kPerGap = (kStores + kGaps - 1) / kGaps;
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);          // MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, kAllReads, 0);  // DS read
#pragma unroll
            for (int i = 0; i < kGaps; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x020, kPerGap, 0);  // VMEM read
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
            __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the MFMA work
            __builtin_amdgcn_s_setprio(3);      // multiply ahead of the other waves' address arithmetic (+1 % at 2048^3)
            if constexpr (PENDING) mma_chunk(last_a, last_b);
        }
#pragma unroll
        for (int c = 0; c < NC - 1; ++c) {
            // Request chunk c + 1 (the tile's last chunk goes to the registers that wait across the barrier), then
            // multiply chunk c; the last multiplied chunk also parks tile kt + 1 in the other LDS buffer, its stores
            // slotted between the MFMAs.
            if (c + 1 < NC - 1) read_frags(smem, cur, c + 1, fa[(c + 1) & 1], fb[(c + 1) & 1]);
            else read_frags(smem, cur, NC - 1, last_a, last_b);
            if (c == NC - 2) {
                sa.template store<(S + 1) % PF>(smem + (cur ^ 1) * StA::LDS_ELEMS);
                // Keep A's stores ahead of B's, the order in which their loads were issued: each store then waits only
                // for the loads up to its own instead of for all of them.
                asm volatile("" ::: "memory");
                sb.template store<(S + 1) % PF>(smem + kBOff + (cur ^ 1) * StB::LDS_ELEMS);
            }
            mma_chunk(fa[c & 1], fb[c & 1]);
            __builtin_amdgcn_sched_group_barrier(0x100, kAllReads, 0);
            if (c == NC - 2) {
                if constexpr (kChunkMfmas >= 2 * kStores) {
#pragma unroll
                    for (int i = 0; i < kStores; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, kChunkMfmas / kStores > 2 ? 2 : 1, 0);  // MFMA
                        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                                  // DS write
                    }
                }
            } else {
                __builtin_amdgcn_sched_group_barrier(0x008, kChunkMfmas, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
    }

    template <bool LOAD, bool MASK, bool PENDING, int S = 0>
    __device__ __forceinline__ void step_any_rot(StA &sa, StB &sb, T *smem, int K, int kt, int slot) {
        if constexpr (S < StA::kPF) {
            if (slot == S) step_rot<S, LOAD, MASK, PENDING>(sa, sb, smem, K, kt);
            else step_any_rot<LOAD, MASK, PENDING, S + 1>(sa, sb, smem, K, kt, slot);
        }
    }

    // PF consecutive steps starting at a tile index kt with kt % PF == 1: slots 1, 2, .., PF - 1, 0.
    template <bool MASK, int I>
    __device__ __forceinline__ void step_group(StA &sa, StB &sb, T *smem, int K, int kt) {
        if constexpr (I < StA::kPF) {
            step_rot<(1 + I) % StA::kPF, true, MASK, true>(sa, sb, smem, K, kt + I);
            step_group<MASK, I + 1>(sa, sb, smem, K, kt);
        }
    }
    // Up to PF steps from kt (kt % PF == 1) while kt + I < steps, same slot sequence as step_group; the step that
    // requests tile `first_partial` (the one k tile that reaches past K) takes the masked body, the others the
    // unmasked one.  first_partial < 0: every step masked.
    template <int I>
    __device__ __forceinline__ void step_group_tail(StA &sa, StB &sb, T *smem, int K, int kt, int steps, int first_partial) {
        if constexpr (I < StA::kPF) {
            if (kt + I < steps) {
                if (first_partial < 0 || kt + I + StA::kPF == first_partial) step_rot<(1 + I) % StA::kPF, true, true, true>(sa, sb, smem, K, kt + I);
                else step_rot<(1 + I) % StA::kPF, true, false, true>(sa, sb, smem, K, kt + I);
                step_group_tail<I + 1>(sa, sb, smem, K, kt, steps, first_partial);
            }
        }
    }

    __device__ __forceinline__ void run_rot(StA &sa, StB &sb, T *smem, int K, bool rows_ok) {
        constexpr int PF = StA::kPF;
        constexpr int NC = BK / kChunk;
        const int KT = (K + BK - 1) / BK;
        // Prologue: tiles 0 .. PF-1 are requested together, so that the first requests of a workgroup (the slowest
        // it makes: nothing of its operands is in a cache yet) overlap instead of queueing behind tile 0's round
        // trip; tile 0 then goes straight to LDS.
        sa.template load<true, 0>(K);
        sb.template load<true, 0>(K);
        prefetch_rest<1>(sa, sb, K, KT);
        sa.template store<0>(smem);
        sb.template store<0>(smem + kBOff);
        __syncthreads();
        // Tiles 0 .. KT-2; the first step has no pending chunk.  While kt + PF < KT a step also issues loads; the
        // remaining steps only drain the slots.
        // `rows_ok` (workgroup-uniform): no load of this workgroup needs a row mask, so only a k tile that reaches
        // past K needs masks.  That can only be the last tile, KT - 1, which is requested by step KT - 1 - PF: that
        // one step takes the masked body, every other one the unmasked body (straight-line loads slotted between the
        // MFMAs; requests past the end of K come back as zeros or unused data and are never parked).
        const int first_partial = (K % BK == 0) ? (KT + 2 * PF) : (KT - 1);  // first tile whose load needs a k mask
        if constexpr (PF > 1) {
            // Register slots are static inside a group of PF steps, so the compiler's wait counters know exactly
            // which loads a store depends on (a run-time slot switch merges the counters at every branch and
            // each store then waits for all loads in flight, the newest included).  Every step requests tile
            // kt + PF.
            const int steps = KT - 1;
            if (steps > 0) {
                if (rows_ok && PF != first_partial) step_rot<0, true, false, false>(sa, sb, smem, K, 0);
                else step_rot<0, true, true, false>(sa, sb, smem, K, 0);
                int kt = 1;
                if (rows_ok) {
                    for (; kt + PF <= steps && kt + 2 * PF - 1 < first_partial; kt += PF) step_group<false, 0>(sa, sb, smem, K, kt);
                    for (; kt + PF <= steps; kt += PF) step_group_tail<0>(sa, sb, smem, K, kt, steps, first_partial);
                    step_group_tail<0>(sa, sb, smem, K, kt, steps, first_partial);
                } else {
                    for (; kt + PF <= steps; kt += PF) step_group<true, 0>(sa, sb, smem, K, kt);
                    step_group_tail<0>(sa, sb, smem, K, kt, steps, -PF);  // (every step masked)
                }
            }
        } else {
            auto pipeline = [&]<bool MASK>() {
                int kt = 0, slot = 0;
                auto advance = [&] {
                    ++kt;
                    slot = slot + 1 == PF ? 0 : slot + 1;
                };
                if (KT > 1) {
                    if (PF < KT) step_any_rot<true, MASK, false>(sa, sb, smem, K, kt, slot);
                    else step_any_rot<false, MASK, false>(sa, sb, smem, K, kt, slot);
                    advance();
                }
                for (; kt + PF < KT; advance()) step_any_rot<true, MASK, true>(sa, sb, smem, K, kt, slot);
                for (; kt + 1 < KT; advance()) step_any_rot<false, MASK, true>(sa, sb, smem, K, kt, slot);
            };
            if (rows_ok && K % BK == 0) {
                pipeline.template operator()<false>();
            } else {
                pipeline.template operator()<true>();
            }
        }
        // Last tile: nothing left to request or park.
        if (KT > 0) {
            const int cur = (KT - 1) & 1;
            FrA f0a;
            FrB f0b;
            read_frags(smem, cur, 0, f0a, f0b);
            if (KT > 1) mma_chunk(last_a, last_b);
            // Only the chunks that hold some k below K: the rest of a partial tile is zeros (K = 392 = 12 tiles + 8
            // spends one chunk on its last tile instead of four).
            const int chunks = (K - (KT - 1) * BK + kChunk - 1) / kChunk;
            mma_chunk(f0a, f0b);
#pragma unroll
            for (int c = 1; c < NC; ++c) {
                if (c < chunks) {  // workgroup-uniform
                    FrA fa;
                    FrB fb;
                    read_frags(smem, cur, c, fa, fb);
                    mma_chunk(fa, fb);
                }
            }
        }
    }

    // ---- pipelined schedule (fp32 tiles with 8 or 16 MFMA blocks per wave, two chunks per k tile) ----
    // With one or two waves per SIMD nothing else hides a wave's own requests, so every load, LDS read and LDS
    // store of a step is slotted between MFMAs (sched_group_barrier), fragments are double-buffered in registers
    // and the barrier sits in the middle of chunk 1:
    //   chunk 0 (fragments f0, read after the previous barrier): its MFMAs carry the global loads of tile kt + 1
    //     and the LDS reads of chunk 1 (f1);
    //   chunk 1, first half: its MFMAs carry the LDS stores of tile kt + 1 into the other buffer, finishing a
    //     quarter of the half early so that the stores have landed when the barrier comes;
    //   barrier;
    //   chunk 1, second half: its MFMAs carry the LDS reads of chunk 0 of tile kt + 1 (the next f0).
    // 4096^3 fp32: 140 -> 145 (256 x 128, two workgroups per CU) / 147 TFLOP/s (256 x 256, one per CU).
    __device__ __forceinline__ void mma_half(const FrA &fa, const FrB &fb, int j0) {
#pragma unroll
        for (int j = j0; j < j0 + M::VK / 2; ++j)
#pragma unroll
            for (int bm = 0; bm < NBM; ++bm)
#pragma unroll
                for (int bn = 0; bn < NBN; ++bn) acc[bm][bn] = M::mma(fa.v[bm][j], fb.v[bn][j], acc[bm][bn]);
    }

    // CUR = kt & 1, the LDS buffer that holds tile kt: a template parameter in the unmasked loop, so that every LDS
    // address of the step is a per-lane base (the same in every step) plus an immediate offset; -1 = taken from kt at
    // run time (the masked loop, whose selects need the registers that two unrolled steps would take).
    template <bool MASK, int CUR = -1>
    __device__ __forceinline__ void step_pipe(StA &sa, StB &sb, T *smem, int K, int kt, FrA &f0a, FrB &f0b) {
        constexpr int kHalf = (M::VK / 2) * NBM * NBN;  // MFMAs of half a chunk
        constexpr int kLoads = StA::P + StB::P;         // global loads (and LDS stores) of one tile, per lane
        constexpr int kReads = NBM + NBN;               // LDS read instructions of one chunk's fragments
        const int cur = CUR >= 0 ? CUR : (kt & 1);
        FrA f1a;
        FrB f1b;
        const int k_left = K - (kt + 1) * BK;
        sa.template load<MASK, 0, !MASK>(k_left);  // (the unmasked loop only requests tiles inside K)
        sb.template load<MASK, 0, !MASK>(k_left);
        read_frags(smem, cur, 1, f1a, f1b);
        mma_half(f0a, f0b, 0);
        mma_half(f0a, f0b, M::VK / 2);
        {
            constexpr int per = 2 * kHalf / (kLoads + kReads) > 0 ? 2 * kHalf / (kLoads + kReads) : 1;
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, per, 0);  // MFMA
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);    // VMEM read
            }
#pragma unroll
            for (int i = 0; i < kReads; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, per, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // DS read
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        mma_half(f1a, f1b, 0);
        sa.template store<0>(smem + (cur ^ 1) * StA::LDS_ELEMS);
        sb.template store<0>(smem + kBOff + (cur ^ 1) * StB::LDS_ELEMS);
        {
            constexpr int per = (kHalf - kHalf / 4) / kLoads > 0 ? (kHalf - kHalf / 4) / kLoads : 1;
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, per, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);    // DS write
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        read_frags(smem, cur ^ 1, 0, f0a, f0b);
        mma_half(f1a, f1b, M::VK / 2);
        {
            constexpr int per = kHalf / kReads > 0 ? kHalf / kReads : 1;
#pragma unroll
            for (int i = 0; i < kReads; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, per, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // WHOLE: the caller promises at compile time what `unmasked` says at run time (and that K > 0), so the masked loop
    // and its registers are not part of the kernel at all.
    template <bool WHOLE>
    __device__ __forceinline__ void run_pipe(StA &sa, StB &sb, T *smem, int K, bool unmasked) {
        static_assert(StA::kPF == 1 && BK / kChunk == 2, "the pipelined schedule is written for two chunks per k tile");
        const int KT = (K + BK - 1) / BK;
        sa.template load<!WHOLE, 0>(K);
        sb.template load<!WHOLE, 0>(K);
        sa.template store<0>(smem);
        sb.template store<0>(smem + kBOff);
        __syncthreads();
        if (KT > 0) {
            FrA f0a;
            FrB f0b;
            read_frags(smem, 0, 0, f0a, f0b);
            int kt = 0;  // two steps to a round: the buffers alternate at compile time
            if (WHOLE || unmasked) {
                for (; kt + 2 < KT; kt += 2) {
                    step_pipe<false, 0>(sa, sb, smem, K, kt, f0a, f0b);
                    step_pipe<false, 1>(sa, sb, smem, K, kt + 1, f0a, f0b);
                }
                if (kt + 1 < KT) step_pipe<false, 0>(sa, sb, smem, K, kt, f0a, f0b);
            } else {
                for (; kt + 1 < KT; ++kt) step_pipe<true>(sa, sb, smem, K, kt, f0a, f0b);
            }
            const int cur = (KT - 1) & 1;
            FrA f1a;
            FrB f1b;
            read_frags(smem, cur, 1, f1a, f1b);
            mma_chunk(f0a, f0b);
            mma_chunk(f1a, f1b);
        }
    }

    // K: reduction length.  `rows_ok`: workgroup-uniform promise that every row of both operand tiles is inside
    // the matrix (a k tile that reaches past K is dealt with here).
    // WHOLE (pipelined schedule only): rows_ok and K % BK == 0 hold for every workgroup of the launch.
    template <bool WHOLE = false>
    __device__ __forceinline__ void run(StA &sa, StB &sb, T *smem, int K, bool rows_ok) {
        static_assert(StA::kPF == StB::kPF, "both operands use the same prefetch distance");
        static_assert(kPipe || kRotate, "no schedule for this tile shape");
        static_assert(!WHOLE || kPipe, "only the pipelined schedule has a form without masks");
        if constexpr (kPipe) run_pipe<WHOLE>(sa, sb, smem, K, rows_ok && K % BK == 0);
        else run_rot(sa, sb, smem, K, rows_ok);
    }

    // The accumulators of this lane as NBM * NBN * NACC values at lds[i * kThreads + tid]: lets two engines with the
    // same tile and lane layout (two halves of one reduction) add their results.
    static constexpr int kAccPerLane = NBM * NBN * M::NACC;
    __device__ __forceinline__ void park_acc(T *lds, int tid) const {
#pragma unroll
        for (int bm = 0; bm < NBM; ++bm)
#pragma unroll
            for (int bn = 0; bn < NBN; ++bn)
#pragma unroll
                for (int e = 0; e < M::NACC; ++e) lds[((bm * NBN + bn) * M::NACC + e) * kThreads + tid] = acc[bm][bn][e];
    }
    __device__ __forceinline__ void add_parked_acc(const T *lds, int tid) {
#pragma unroll
        for (int bm = 0; bm < NBM; ++bm)
#pragma unroll
            for (int bn = 0; bn < NBN; ++bn)
#pragma unroll
                for (int e = 0; e < M::NACC; ++e) acc[bm][bn][e] += lds[((bm * NBN + bn) * M::NACC + e) * kThreads + tid];
    }

    template <int S>
    __device__ __forceinline__ void prefetch_rest(StA &sa, StB &sb, int K, int KT) {
        if constexpr (S < StA::kPF) {
            // (unconditional: a tile beyond K is requested at out-of-range offsets and costs next to nothing, and
            // without a branch the wait counters of the stores that follow are exact)
            sa.template load<true, S>(K - S * BK);
            sb.template load<true, S>(K - S * BK);
            prefetch_rest<S + 1>(sa, sb, K, KT);
        }
    }

    // Walks the finished tile.  `one(m, n, v, bn)` receives a single element at tile-local (m, n);
    // `two(m, n, v0, v1, bn)` receives columns n and n + 1 of the same row (only called when B is MC/paired and
    // `pairs_ok`); both are expected to do their own bounds checks against the matrix size.  bn (a compile-time
    // constant after unrolling) numbers the lane's columns: a lane meets NBN distinct columns, column slot bn for
    // `one`, slots bn and bn + 1 for `two`.
    // FENCE keeps the scheduler from hoisting the work of later blocks over the stores of earlier ones (an epilogue
    // that loads per element would otherwise hold a whole tile's loads in flight and spill).
    //
    // The callbacks are templates over a phase and also receive e, the element's number inside its MFMA block (a
    // compile-time constant after unrolling).  PHASED = false: one call per element, phase 2 (everything).  PHASED =
    // true: a block's elements are walked twice, phase 0 (requests: the callback keeps what it loads in arrays indexed
    // by e) and then phase 1 (arithmetic and stores).  A store followed by a load through another descriptor cannot be
    // reordered by the compiler (they might alias), so a walk that loads and stores element by element is a chain of
    // memory round trips, one per element; in two phases a block's loads are in flight together.
    template <bool FENCE = false, bool PHASED = false, class One, class Two>
    __device__ __forceinline__ void for_each(bool pairs_ok, One one, Two two) {
        const int jcol = lane % M::MB;
        auto singles = [&]() {
#pragma unroll
            for (int bn = 0; bn < NBN; ++bn) {
                const int n = FrB::index_of(wn0, bn, jcol);
#pragma unroll
                for (int bm = 0; bm < NBM; ++bm) {
                    if constexpr (PHASED) {
#pragma unroll
                        for (int e = 0; e < M::NACC; ++e)
                            one.template operator()<0>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][bn][e], bn, e);
#pragma unroll
                        for (int e = 0; e < M::NACC; ++e)
                            one.template operator()<1>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][bn][e], bn, e);
                    } else {
#pragma unroll
                        for (int e = 0; e < M::NACC; ++e)
                            one.template operator()<2>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][bn][e], bn, e);
                    }
                    if constexpr (FENCE) __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if constexpr (FrB::PAIRED) {
            if (pairs_ok) {
#pragma unroll
                for (int pr = 0; pr < NBN / 2; ++pr) {
                    const int n = FrB::index_of(wn0, 2 * pr, jcol);  // even column; n + 1 belongs to block 2p+1
#pragma unroll
                    for (int bm = 0; bm < NBM; ++bm) {
                        if constexpr (PHASED) {
#pragma unroll
                            for (int e = 0; e < M::NACC; ++e)
                                two.template operator()<0>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][2 * pr][e],
                                                           acc[bm][2 * pr + 1][e], 2 * pr, e);
#pragma unroll
                            for (int e = 0; e < M::NACC; ++e)
                                two.template operator()<1>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][2 * pr][e],
                                                           acc[bm][2 * pr + 1][e], 2 * pr, e);
                        } else {
#pragma unroll
                            for (int e = 0; e < M::NACC; ++e)
                                two.template operator()<2>(FrA::index_of(wm0, bm, M::acc_row(e, lane)), n, acc[bm][2 * pr][e],
                                                           acc[bm][2 * pr + 1][e], 2 * pr, e);
                        }
                        if constexpr (FENCE) __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else {
                singles();
            }
        } else {
            singles();
        }
    }
};

// What the store of a tile can do beyond bias / ReLU / accumulate; every pointer may be null.  All three serve the
// callers either side of a Linear layer's GEMMs in a training step:
//   relu_out   dense like C: C keeps the value before the ReLU (what autograd saves as the ReLU's input,
//              autograd/unary_ops.cpp:562-567) and relu_out receives max(value, 0) -- Linear + ReLU in one launch;
//   zmask      dense like C: the value is replaced by 0 where zmask < 0 -- TensorRelu::backward's
//              grad_output * where(input < 0, 0, 1) (autograd/unary_ops.cpp:568-573) applied by the GEMM that
//              computes grad_output;
//   colsum     [rows of partial sums][N]: row (colsum_row0 + the wave's row index in the workgroup) receives the sums
//              over this wave's rows of what is stored to C, per column -- the bias gradient's sum over the batch
//              (nn/linear.cpp:45-48: the bias is an expanded view, its gradient sums the broadcast dimension); a
//              second kernel adds the partial rows in order.
template <typename T>
struct EpilogueExt {
    T *relu_out = nullptr;
    const T *zmask = nullptr;
    T *colsum = nullptr;
    int colsum_row0 = 0;
};

// Dense row-major store of a finished tile with the optional bias / ReLU / accumulate epilogue.
// C points at the matrix (already offset to the batch), M x N its size, (m0, n0) the tile origin.
//
// The tile is written through a buffer descriptor that starts at C[m0][n0] and ends with the last row of the matrix
// that the tile touches; an element outside the matrix gets the out-of-range offset and the hardware drops its
// store.  One straight-line path serves interior and edge tiles and an element costs one 32-bit offset.  The host
// only sends matrices here whose rows under one tile span less than 2^31 bytes (min(BM, M) * N * sizeof(T)).
// LEAN: no bias, ReLU, accumulation or extensions (those arguments are then ignored).  EXT: the walk also serves
// `ext` (a separate instantiation, because its extra loads, second store and column sums cost the big tiles registers
// that the plain bias / ReLU / accumulate walk should not pay for).
template <typename T, bool LEAN, bool EXT = false, class Engine>
__device__ __forceinline__ void store_tile_dense(Engine &eng, T *__restrict__ C, int M_, int N_, int m0, int n0,
                                                 const T *__restrict__ bias, int bias_mode, int relu, int accumulate,
                                                 const EpilogueExt<T> &ext = EpilogueExt<T>{}) {
    using pair_t = typename Mfma<T>::pair_t;
    using MI = Mfma<T>;
    constexpr uint32_t kOob = 0x80000000u;
    const int rows = M_ - m0 < Engine::kBM ? M_ - m0 : Engine::kBM;
    const int cols = N_ - n0;
    const int64_t tile_bytes = (static_cast<int64_t>(rows) * N_ - n0) * static_cast<int64_t>(sizeof(T));
    const int64_t tile_first = static_cast<int64_t>(m0) * N_ + n0;
    const __amdgpu_buffer_rsrc_t out = make_rsrc(C + tile_first, tile_bytes);
    // The epilogue options are uniform run-time flags.  Branching on them per element would put hundreds of branches
    // into the unrolled walk, so they are folded into data instead: a bias that is absent, a C that is not
    // accumulated into and a mask that is not asked for are read through descriptors of zero length, whose loads
    // return 0 without touching memory, and a second output that is not asked for is written through one, whose
    // stores the hardware drops.
    constexpr int64_t kSz = sizeof(T);
    const __amdgpu_buffer_rsrc_t bias_n = make_rsrc(bias, bias_mode == 1 ? N_ * kSz : 0);
    const __amdgpu_buffer_rsrc_t bias_m = make_rsrc(bias, bias_mode == 2 ? M_ * kSz : 0);
    const __amdgpu_buffer_rsrc_t prev = make_rsrc(C + tile_first, accumulate ? tile_bytes : 0);
    static_assert(!(LEAN && EXT), "the lean walk has no extensions");
    const __amdgpu_buffer_rsrc_t zmask = make_rsrc(ext.zmask ? ext.zmask + tile_first : ext.zmask, (EXT && ext.zmask) ? tile_bytes : 0);
    const __amdgpu_buffer_rsrc_t second =
        make_rsrc(ext.relu_out ? ext.relu_out + tile_first : ext.relu_out, (EXT && ext.relu_out) ? tile_bytes : 0);
    auto offset_of = [&](int ml, int nl) {
        return (ml < rows && nl < cols) ? static_cast<uint32_t>(ml * N_ + nl) * static_cast<uint32_t>(sizeof(T)) : kOob;
    };
    T csum[Engine::NBN];  // sums of what this lane stores, per column slot
#pragma unroll
    for (int i = 0; i < Engine::NBN; ++i) csum[i] = T(0);
    auto positive = [](T v) { return v > T(0) ? v : T(0); };
    // pairs: n is even and N is even, so n + 1 < N whenever n < N and a wave writes whole row segments
    const bool pairs_ok = (N_ % 2 == 0) && (reinterpret_cast<uintptr_t>(C) % (2 * sizeof(T)) == 0) &&
                          (!EXT || (reinterpret_cast<uintptr_t>(ext.relu_out) % (2 * sizeof(T)) == 0 &&
                                    reinterpret_cast<uintptr_t>(ext.zmask) % (2 * sizeof(T)) == 0));
    // What the walk loads for the elements of one MFMA block (see for_each: phase 0 requests, phase 1 uses).  Two phases
    // for tiles with up to 64 accumulators per lane; the big tiles have no registers to spare for a block's loads and
    // keep the element-by-element walk.
    constexpr bool kPhased = !LEAN && Engine::kAccPerLane <= 64;
    constexpr int NA = MI::NACC;
    uint32_t offs[NA];
    T l_bn[NA][2], l_bm[NA];
    pair_t l_z[NA], l_p[NA];
    constexpr uint32_t kSzU = static_cast<uint32_t>(sizeof(T));
    // W = 1: a single element (component 0 of the pairs); W = 2: columns n and n + 1.  The arithmetic per element, in
    // this order: + bias[n], + bias[m], mask, ReLU, + old value.
    auto element = [&]<int PHASE, int W>(int ml, int nl, const T (&in)[W], int slot, int e) {
        if constexpr (PHASE != 1) {
            offs[e] = offset_of(ml, nl);
            if constexpr (!LEAN) {
#pragma unroll
                for (int j = 0; j < W; ++j) l_bn[e][j] = Vec<T, 1>::load(bias_n, static_cast<uint32_t>(n0 + nl + j) * kSzU);
                l_bm[e] = Vec<T, 1>::load(bias_m, static_cast<uint32_t>(m0 + ml) * kSzU);
                if constexpr (W == 2) {
                    if constexpr (EXT) l_z[e] = Vec<T, 2>::load(zmask, offs[e]);  // (absent mask: zeros)
                    l_p[e] = Vec<T, 2>::load(prev, offs[e]);
                } else {
                    if constexpr (EXT) l_z[e][0] = Vec<T, 1>::load(zmask, offs[e]);
                    l_p[e][0] = Vec<T, 1>::load(prev, offs[e]);
                }
            }
        }
        if constexpr (PHASE != 0) {
            const uint32_t off = offs[e];
            T o[W];
#pragma unroll
            for (int j = 0; j < W; ++j) {
                T v = in[j];
                if constexpr (!LEAN) {
                    v += l_bn[e][j];
                    v += l_bm[e];
                    if constexpr (EXT) v = l_z[e][j] < T(0) ? v * T(0) : v;  // grad * where(input < 0, 0, 1): a product, so an infinite or NaN grad under the mask stays NaN
                    v = (v > T(0) || !relu) ? v : T(0);
                    v += l_p[e][j];
                    if constexpr (EXT) csum[slot + j] += off != kOob ? v : T(0);
                }
                o[j] = v;
            }
            if constexpr (W == 2) {
                pair_t ov, rv;
                ov[0] = o[0];
                ov[1] = o[1];
                buffer_store(out, off, ov);
                if constexpr (EXT) {
                    rv[0] = positive(o[0]);
                    rv[1] = positive(o[1]);
                    buffer_store(second, off, rv);
                }
            } else {
                buffer_store(out, off, o[0]);
                if constexpr (EXT) buffer_store(second, off, positive(o[0]));
            }
        }
    };
    eng.template for_each<!LEAN, kPhased>(
        pairs_ok,
        [&]<int PHASE>(int ml, int nl, T v, int slot, int e) {
            const T in[1] = {v};
            element.template operator()<PHASE, 1>(ml, nl, in, slot, e);
        },
        [&]<int PHASE>(int ml, int nl, T v0, T v1, int slot, int e) {
            const T in[2] = {v0, v1};
            element.template operator()<PHASE, 2>(ml, nl, in, slot, e);
        });
    if constexpr (EXT) {
        if (ext.colsum) {  // workgroup-uniform
            // Lanes l, l + MB, ... of a wave hold the same columns and different rows: fold them, then lanes 0 .. MB-1
            // write the wave's sums.  Column of slot s: the walk's own numbering (for_each).
            const int jcol = eng.lane % MI::MB;
            const bool paired = Engine::FrB::PAIRED && pairs_ok;
            T *row = ext.colsum + static_cast<int64_t>(ext.colsum_row0 + eng.wm0 / Engine::WM) * N_;
#pragma unroll
            for (int s = 0; s < Engine::NBN; ++s) {
                T v = csum[s];
#pragma unroll
                for (int d = MI::MB; d < 64; d *= 2) v += __shfl_xor(v, d, 64);
                int nl;
                if (paired) nl = Engine::FrB::index_of(eng.wn0, s & ~1, jcol) + (s & 1);
                else nl = Engine::FrB::index_of(eng.wn0, s, jcol);
                if (eng.lane < MI::MB && nl < cols) row[n0 + nl] = v;
            }
        }
    }
}

// A small second job that rides in a launch as workgroups appended to its grid: out[i] = sum over s < splits of
// partial[s * n + i] (a sum that an earlier launch on the stream left in parts, spared a launch of its own).  Workgroup r
// of the appended ones owns the 16-byte vectors 64 r .. 64 r + 63 of the result; each of its NW waves adds a contiguous
// share of the parts in increasing order, every load in flight together (parts beyond the share arrive as +0 from the
// buffer load, which changes no sum that started at +0), and the waves' sums are added through `lds` (NW * 64 vectors) in
// wave order: a fixed order.  n a multiple of the vector length, both pointers 16-byte aligned, splits * n * sizeof(T) < 2^31.
template <typename T, int NW>
__device__ __forceinline__ void add_up_parts(const T *partial, T *out, int n, int splits, int r, T *lds) {
    constexpr int VEC = 16 / sizeof(T);
    using V = typename Vec<T, VEC>::type;
    const int lane = threadIdx.x % 64;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int v = r * 64 + lane;
    const bool ok = VEC * v < n;
    const int per = (splits + NW - 1) / NW;
    const int s0 = w * per, s1 = s0 + per < splits ? s0 + per : splits;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(partial, static_cast<int64_t>(splits) * n * static_cast<int64_t>(sizeof(T)));
    const uint32_t voff = ok ? static_cast<uint32_t>(v) * 16u : kOob;
    V acc;
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = T(0);
#pragma unroll 1
    for (int s = s0; s < s1; s += 16) {
        V part[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            part[u] = Vec<T, VEC>::load_at(src, s + u < s1 ? voff : kOob, static_cast<uint32_t>(s + u) * static_cast<uint32_t>(n) * static_cast<uint32_t>(sizeof(T)));
#pragma unroll
        for (int u = 0; u < 16; ++u) acc += part[u];
    }
    *reinterpret_cast<V *>(lds + (w * 64 + lane) * VEC) = acc;
    __syncthreads();
    if (w == 0 && ok) {
        V sum = acc;
#pragma unroll
        for (int k = 1; k < NW; ++k) sum += *reinterpret_cast<const V *>(lds + (k * 64 + lane) * VEC);
        *reinterpret_cast<V *>(out + static_cast<int64_t>(VEC) * v) = sum;
    }
}

}  // namespace mfma
}  // namespace ttamd

#endif  // TTAMD_CSRC_MFMA_CORE_H_
