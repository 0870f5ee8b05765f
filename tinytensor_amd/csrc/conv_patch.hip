// conv_patch.hip — stride-1 fp32 convolution for layers whose whole weight matrix fits in LDS (gfx950).
//
// The implicit-GEMM kernels of conv.hip fetch every input element once per tap through the vector memory path and
// start a fresh workgroup (weights, prologue, epilogue) for every output tile.  With a short reduction (config
// "input [64,32,28,28], weight [64,32,3,3]": K = 288) those fixed costs and the address arithmetic of the gather
// dominate: on this chip every vector ALU instruction a SIMD issues takes about five cycles away from its MFMA pipe
// (a 32x32x2 fp32 MFMA occupies it for 64), whichever wave issues it, so the instructions per MFMA decide the rate.
// This kernel is built around that count:
//   * persistent workgroups, one per CU: the weight block [BM x K] is loaded into LDS once and stays there, a
//     workgroup then walks over its share of the (image, position tile) pairs;
//   * per tile the raw input rows under the tile (with the halo rows of the taps) are staged into LDS once --
//     16-byte loads along the rows, every element fetched once -- into a patch [R rows][pitch columns][C + 4]
//     with the channels innermost; its halo columns stay zero, rows above and below the image come back from the
//     buffer load as 0;
//   * the reduction runs tap by tap with the channels innermost (k' = tap * C + c), the order the weights are laid
//     out in LDS, so that four consecutive reduction indices are four consecutive floats on both sides: one 16-byte
//     LDS read of A and one of B feed four MFMAs, and a group of CC such chunks needs two address additions;
//     row pitches of 4 (2 n + 1) floats keep those reads free of bank conflicts;
//   * the next tile's rows are requested before the MFMA work of the current one and parked in the other patch
//     buffer after it: one barrier per tile.
// Same arithmetic as tinytensor/tensor/backend/cpu/conv.cpp:36-134 (im2col + GEMM per image) up to the order of
// the sum; exact on integer-valued data.  The same kernel computes the gradient with respect to the input
// (tinytensor/tensor/backend/cpu/conv.cpp:137-189 computes it as col2im of W^T dY): a convolution of dY with the
// taps reversed and the two channel axes of the weight exchanged, which only changes how the weights are laid out
// in LDS.  conv.hip takes this road when the geometry allows and keeps its own kernels for everything else.
#include <cstdlib>

#include "mfma_core.h"

namespace ttamd {
namespace {

using namespace mfma;

constexpr int kStageLoads = 64;   // most 16-byte loads per tile and lane, times the waves of the workgroup
constexpr int kWeightLoads = 80;  // likewise for the loads in flight while the weights are brought in
constexpr int kLdsBytes = 160 * 1024;  // per workgroup on gfx950
constexpr int kPairs = 4;        // (row, channel) pairs of the weight a lane moves together

__device__ __forceinline__ f32x4 lds_load4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }

// Issue order of one group: an LDS read after every second MFMA (2 CC reads, 4 CC MFMAs).  Left to itself the
// scheduler sinks each read down to the MFMA that consumes it, which exposes the LDS latency once per chunk.
template <int N, int I = 0>
__device__ __forceinline__ void interleave_reads() {
    if constexpr (I < N) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (I % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        interleave_reads<N, I + 1>();
    }
}

// Tail accumulators per lane of the twelve-wave form: a 4x4x1 MFMA covers 16 / (BM / 4) groups of four positions, and a
// tail is at most two groups (8 positions).
template <int WGM>
constexpr int tail_accumulators() {
    return WGM >= 2 ? 2 : 1;
}

// WGM x WGN waves of one 32 x 32 MFMA block each: output tile (32 WGM) channels x (32 WGN) positions.
// CC: chunks of 8 reduction indices (8 channels of one tap) that are read and multiplied as one straight-line group;
// C / 8 is a multiple of it.
// MAXS: staging slots (16-byte loads per lane and tile).
// KS: 1, or 2 sets of WGM x WGN waves that each take half of the reduction groups of the same tile (a second wave per
// SIMD where a wider tile's patch would not fit in LDS); the upper set hands its accumulators over through LDS.
template <int WGM, int WGN, int CC, int MAXS, int KS = 1>
__global__ void __launch_bounds__(64 * WGM * WGN * KS, 1) conv_patch_kernel(ConvPatchArgs a) {
    constexpr int NW = WGM * WGN * KS, NT = 64 * NW;  // 4 waves (one per SIMD), 8 or 12
    static_assert(NW == 4 || NW == 8 || NW == 12, "4, 8 or 12 waves");
    // Twelve waves: the tile is a.bne = 32 WGN + a.tail positions, the tail (4 or 8 positions that would leave a whole
    // 32-position block all but empty) computed with 4x4x1 MFMAs after the blocks -- see `tail` below.
    constexpr bool kTail = NW == 12;
    constexpr bool kStoreEarly = KS == 1;
    constexpr int NTA = tail_accumulators<WGM>();  // tail accumulators per lane: 8 positions at most
    static_assert(KS == 1 || KS == 2, "one or two halves of the reduction");
    constexpr int WVECS = kWeightLoads / NW;
    constexpr int BM = 32 * WGM, BN = 32 * WGN;
    const int bne = kTail ? a.bne : BN;  // positions per tile
    extern __shared__ __attribute__((aligned(16))) float smem_patch[];
    const int conv_blocks = static_cast<int>(gridDim.x) - a.red_blocks;
    if (static_cast<int>(blockIdx.x) >= conv_blocks) {  // an appended workgroup: the launch's second job
        const int r = static_cast<int>(blockIdx.x) - conv_blocks, first = a.red_blocks - a.red2_blocks;
        if (r < first) add_up_parts<float, NW>(a.red_partial, a.red_out, a.red_n, a.red_splits, r, smem_patch);
        else add_up_parts<float, NW>(a.red2_partial, a.red2_out, a.red2_n, a.red2_splits, r - first, smem_patch);
        return;
    }
    float *const A = smem_patch;                   // [BM][lda], k' = tap * C + c
    float *const patch = smem_patch + BM * a.lda;  // [1 or 2][R][pitch][cpad]
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int ks = wave / (WGM * WGN), wtile = wave % (WGM * WGN);
    const int wm = wtile / WGN, wn = wtile % WGN;
    const int li = lane % 32, kg = lane / 32;
    const int C = a.C, K = a.K, pitch = a.pitch, cpad = a.cpad;
    const int patch_elems = a.R * pitch * cpad;

    // which tiles: workgroup (m, gi) of `groups` per output-channel block walks j = gi, gi + groups, ...
    const int groups = conv_blocks / a.tiles_m;
    const int mblk = blockIdx.x % a.tiles_m, gi = blockIdx.x / a.tiles_m;
    const int m0 = mblk * BM;
    const int n_tiles = a.B * a.tiles_n;
    const int n_groups = K / (8 * CC);
    const float *const ap = A + (wm * 32 + li) * a.lda + 4 * kg;
    const int HoWo = a.Ho * a.Wo;
    // ---- staging geometry.  A wave moves one item per slot: 8 or 16 channels x one row x 64 / that many consecutive
    // 16-byte vectors of the row.  Which item is wave-uniform, so its memory offset rides in the load's scalar offset
    // and its LDS offset is one scalar addition; the lanes run over the channels first: 64 or 128 contiguous bytes
    // per channel on the memory side, and on the LDS side (channels innermost, 16 (2 n + 1) floats between the
    // vectors) every bank once.
    const int cl_mask = (1 << a.cl_shift) - 1;
    const int c_lo = lane & cl_mask, xv_lo = lane >> a.cl_shift;
    const uint32_t lane_goff = static_cast<uint32_t>((c_lo * a.xs_c + 4 * xv_lo) * 4);
    const int lane_lds = 4 * xv_lo * cpad + c_lo;
    const bool lane_in_last = xv_lo < a.last_vecs;  // in the last column block of a row only these lanes hold a vector
    // per lane and slot (registers): byte offset in the image, float offset in a patch buffer (-1: no vector), patch row
    uint32_t s_voff[MAXS];
    int s_lds[MAXS], s_row[MAXS];
#pragma unroll
    for (int i = 0; i < MAXS; ++i) {  // (slots beyond the last item: loads that fetch nothing, writes with no lane)
        const uint32_t item = static_cast<uint32_t>(i * NW + wave);
        uint32_t t, xv_hi, c_hi, r;
        a.d_xh.divmod(item, t, xv_hi);
        a.d_R.divmod(t, c_hi, r);
        const bool last = static_cast<int>(xv_hi) == a.xh - 1;
        const bool ok = item < static_cast<uint32_t>(a.n_items) && (!last || lane_in_last);
        const int xv0 = static_cast<int>(xv_hi) * (64 >> a.cl_shift);
        s_voff[i] = lane_goff + static_cast<uint32_t>(((static_cast<int32_t>(c_hi) << a.cl_shift) * a.xs_c + static_cast<int32_t>(r) * a.xs_h + 4 * xv0) * 4);
        s_lds[i] = ok ? lane_lds + (static_cast<int>(r) * pitch + a.P + 4 * xv0) * cpad + (static_cast<int>(c_hi) << a.cl_shift) : -1;
        s_row[i] = ok ? static_cast<int>(r) : -(1 << 28);  // never passes the row test
    }
    f32x4 staged[MAXS];
    auto request = [&](int b, int h_first) {  // rows of a tile of image b whose first output row is h_first: global -> registers
        const int y0 = h_first - a.P;
        // the descriptor starts at patch row 0 of this tile (which may lie above the image: such rows fail the test)
        const int64_t first = static_cast<int64_t>(b) * a.xs_b + static_cast<int64_t>(y0) * a.xs_h;
        const __amdgpu_buffer_rsrc_t xsrc = make_rsrc(a.x + first, a.image_bytes - static_cast<int64_t>(y0) * a.xs_h * 4);
#pragma unroll
        for (int i = 0; i < MAXS; ++i) {
            const bool ok = static_cast<unsigned>(y0 + s_row[i]) < static_cast<unsigned>(a.H);
            staged[i] = Vec<float, 4>::load(xsrc, ok ? s_voff[i] : kOob);
        }
    };
    auto park = [&](int buf) {  // registers -> patch buffer `buf`, channels innermost
        float *dst = patch + buf * patch_elems;
#pragma unroll
        for (int i = 0; i < MAXS; ++i) {
            if (s_lds[i] >= 0) {
                float *p = dst + s_lds[i];
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e * cpad] = staged[i][e];
            }
        }
    };
    // The tile walk: j = gi, gi + groups, ... as (image, position tile), advanced without divisions.
    int j = gi;
    uint32_t t_b, t_n;
    a.d_tiles_n.divmod(static_cast<uint32_t>(j), t_b, t_n);
    int tile_b = static_cast<int>(t_b), tile_n = static_cast<int>(t_n);
    int tile_h = static_cast<int>(a.d_Wo.div(static_cast<uint32_t>(tile_n * bne)));  // first output row of the tile
    uint32_t step_b, step_n;
    a.d_tiles_n.divmod(static_cast<uint32_t>(groups), step_b, step_n);
    if (j < n_tiles) request(tile_b, tile_h);  // on its way while the weights are brought in
    // bias of this lane's 16 accumulator rows
    const bool full_rows = m0 + BM <= a.O;
    float bias_v[16];
    {
        const __amdgpu_buffer_rsrc_t bsrc = make_rsrc(a.bias, a.bias ? static_cast<int64_t>(a.O) * 4 : 0);  // absent: loads 0
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            if (full_rows)  // the row part of the offset is wave-uniform
                bias_v[e] = Vec<float, 1>::load_at(bsrc, static_cast<uint32_t>(kg * 16), static_cast<uint32_t>(m0 + wm * 32 + (e / 4) * 8 + e % 4) * 4u);
            else
                bias_v[e] = Vec<float, 1>::load(bsrc, static_cast<uint32_t>(m0 + wm * 32 + Mfma<float>::acc_row(e, lane)) * 4u);
        }
    }

    // twelve waves: the bias of the tail element that this lane will add up and store (requested here, with the loads
    // above, so that its latency is not in front of the tail's store)
    float tail_bias = 0.f;
    if constexpr (kTail) {
        if (a.bias && tid < BM * a.tail) {
            const int o = m0 + static_cast<int>(a.d_tail.div(static_cast<uint32_t>(tid)));
            if (o < a.O) tail_bias = a.bias[o];
        }
    }

    // ---- once per workgroup: the weight block, into A in the order k' = tap * C + c.
    // 3 x 3 kernels: a lane takes (row, reduction channel) pairs, reads the pair's nine taps (consecutive floats in
    // memory in both weight layouts) straight from memory, every load of its pairs in flight together, and writes them
    // C floats apart; the lanes run along the axis in which pairs lie nine floats apart, so a load instruction covers
    // a contiguous stretch of the weight and a store instruction consecutive floats of A.
    // Other kernel sizes: the block is copied through the still unused patch area with 16-byte vectors, segment by
    // segment (one output row's [C][k k] in the forward layout), and moved from there to A, per pair k*k reads a float
    // apart and k*k writes C floats apart.
    if (a.k == 3) {
        const int step = a.w_flip ? -C : C;
        const __amdgpu_buffer_rsrc_t wsrc = make_rsrc(a.w, a.weight_bytes);
        const int n_pairs = a.n_seg * a.n_fast;
#pragma unroll 1
        for (int v = tid; v < n_pairs; v += kPairs * NT) {
            float *dst[kPairs];
            float taps[kPairs][9];
            bool have[kPairs];
#pragma unroll
            for (int i = 0; i < kPairs; ++i) {
                have[i] = v + i * NT < n_pairs;
                const uint32_t vv = static_cast<uint32_t>(v + i * NT);
                int row, red;
                if (a.w_rows_fast) {
                    // 16 rows x 4 reduction channels per wave: the loads cover four stretches of 16 x 9 floats, and the
                    // stores -- rows 4 (2 n + 1) floats apart, channels one float apart -- every bank once
                    const uint32_t t = vv >> 6;
                    row = static_cast<int>((t % (BM / 16)) * 16 + (vv & 15));
                    red = static_cast<int>((t / (BM / 16)) * 4 + ((vv >> 4) & 3));
                } else {
                    uint32_t slow, fast;
                    a.d_wfast.divmod(vv, slow, fast);
                    row = static_cast<int>(slow), red = static_cast<int>(fast);
                }
                // rows beyond the last output channel are requested out of range and arrive as zeros
                const uint32_t off = have[i] && m0 + row < a.O ? static_cast<uint32_t>((m0 + row) * a.w_row + red * a.w_red) * 4u : kOob;
                dst[i] = A + row * a.lda + red + (a.w_flip ? 8 * C : 0);
#pragma unroll
                for (int u = 0; u < 9; ++u) taps[i][u] = Vec<float, 1>::load(wsrc, off + 4u * u);
            }
#pragma unroll
            for (int i = 0; i < kPairs; ++i)
                if (have[i]) {
#pragma unroll
                    for (int u = 0; u < 9; ++u) dst[i][u * step] = taps[i][u];
                }
        }
    } else {
        const int k2 = a.k * a.k;
        const int seg_vecs = a.seg_len / 4;
        const int step = a.w_flip ? -C : C;
        f32x4 wv[WVECS];
        if (a.w_dense) {
            // consecutive segments are contiguous in memory: one linear copy with all loads in flight together; rows
            // beyond the last output channel lie behind the end of the descriptor and arrive as zeros
            const int rows_here = a.w_rows_fast ? a.n_seg : (a.O - m0 < BM ? a.O - m0 : BM);
            const __amdgpu_buffer_rsrc_t wsrc = make_rsrc(a.w + static_cast<int64_t>(m0) * a.w_row, static_cast<int64_t>(rows_here) * a.seg_len * 4);
#pragma unroll
            for (int i = 0; i < WVECS; ++i)
                if (i < a.n_wvec) wv[i] = Vec<float, 4>::load(wsrc, static_cast<uint32_t>(tid + i * NT) * 16u);
        }
        auto pair_of = [&](int v, int s0, const float *&src, float *&dst) {
            uint32_t slow, fast;
            a.d_wfast.divmod(static_cast<uint32_t>(v), slow, fast);
            const int row = a.w_rows_fast ? static_cast<int>(fast) : s0 + static_cast<int>(slow);
            const int red = a.w_rows_fast ? s0 + static_cast<int>(slow) : static_cast<int>(fast);
            src = patch + static_cast<int>(slow) * a.seg_len + static_cast<int>(fast) * k2;
            dst = A + row * a.lda + red + (a.w_flip ? (k2 - 1) * C : 0);
        };
#pragma unroll 1
        for (int s0 = 0; s0 < a.n_seg; s0 += a.segs_per_pass) {  // as many segments per pass as the patch area holds
            const int s1 = s0 + a.segs_per_pass < a.n_seg ? s0 + a.segs_per_pass : a.n_seg;
            const int v_lo = s0 * seg_vecs, v_hi = s1 * seg_vecs;
            if (s0 > 0) __syncthreads();  // the previous pass has been read out
            if (a.w_dense && a.w_pass_vecs > 0) {  // a pass is a whole number of the lanes' vectors: uniform tests
                const int i_lo = s0 / a.segs_per_pass * a.w_pass_vecs;
#pragma unroll
                for (int i = 0; i < WVECS; ++i)
                    if (i >= i_lo && i < i_lo + a.w_pass_vecs && i < a.n_wvec) *reinterpret_cast<f32x4 *>(patch + 4 * (tid + (i - i_lo) * NT)) = wv[i];
            } else if (a.w_dense) {
#pragma unroll
                for (int i = 0; i < WVECS; ++i) {
                    const int v = tid + i * NT;
                    if (i < a.n_wvec && v >= v_lo && v < v_hi) *reinterpret_cast<f32x4 *>(patch + 4 * (v - v_lo)) = wv[i];
                }
            } else {
                const __amdgpu_buffer_rsrc_t wsrc = make_rsrc(a.w, a.weight_bytes);
#pragma unroll 1
                for (int v0 = v_lo + tid; v0 < v_hi; v0 += 4 * NT) {
                    f32x4 part[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int v = v0 + i * NT;
                        uint32_t seg, x;
                        a.d_segv.divmod(static_cast<uint32_t>(v), seg, x);
                        const bool ok = v < v_hi && (a.w_rows_fast || m0 + static_cast<int>(seg) < a.O);
                        const int64_t first = a.w_rows_fast ? static_cast<int64_t>(m0) * a.w_row + static_cast<int64_t>(seg) * a.w_red
                                                            : static_cast<int64_t>(m0 + static_cast<int>(seg)) * a.w_row;
                        part[i] = Vec<float, 4>::load(wsrc, ok ? static_cast<uint32_t>((first + 4 * static_cast<int64_t>(x)) * 4) : kOob);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (v0 + i * NT < v_hi) *reinterpret_cast<f32x4 *>(patch + 4 * (v0 + i * NT - v_lo)) = part[i];
                }
            }
            __syncthreads();
            const int n_pairs = (s1 - s0) * a.n_fast;
#pragma unroll 1
            for (int v = tid; v < n_pairs; v += NT) {
                const float *src;
                float *dst;
                pair_of(v, s0, src, dst);
#pragma unroll 1
                for (int t = 0; t < k2; ++t) dst[t * step] = src[t];
            }
        }
    }
    __syncthreads();  // the weights have left the patch area
    // the halo columns of both patch buffers stay zero from here on; every other cell is rewritten for each tile
    {
        const int halo_cells = a.n_buf * a.R * 2 * a.P;  // (buffer, row, side, column)
#pragma unroll 1
        for (int v = tid; v < halo_cells * (cpad / 4); v += NT) {
            uint32_t cell, c4, br, sp, side, pc;
            a.d_cpad4.divmod(static_cast<uint32_t>(v), cell, c4);
            a.d_2P.divmod(cell, br, sp);
            a.d_P.divmod(sp, side, pc);
            const int x = side ? a.P + a.W + static_cast<int>(pc) : static_cast<int>(pc);
            *reinterpret_cast<f32x4 *>(patch + (static_cast<int>(br) * pitch + x) * cpad + 4 * static_cast<int>(c4)) = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    if (j < n_tiles) park(0);
    __syncthreads();

    // The reduction in groups of CC chunks: group g covers tap g / ngrp, channels (g % ngrp) * 8 CC ..., i.e. k' from
    // 8 CC g on.  The fragments of the next group are requested from LDS before the MFMAs of the current one (two
    // register sets, no copies), so a wave's own LDS latency hides behind its MFMA work: with one wave per SIMD
    // nothing else would hide it.
    for (int cur = 0; j < n_tiles; j += groups, cur ^= a.n_buf - 1) {
        const int jn = j + groups;
        const int b = tile_b, n0 = tile_n * bne, h_first = tile_h;
        if (jn < n_tiles) {  // the next tile's rows are in flight during this tile's MFMA work
            tile_n += static_cast<int>(step_n);
            tile_b += static_cast<int>(step_b);
            if (tile_n >= a.tiles_n) tile_n -= a.tiles_n, ++tile_b;
            tile_h = static_cast<int>(a.d_Wo.div(static_cast<uint32_t>(tile_n * bne)));
            request(tile_b, tile_h);
        }
        const int n = n0 + wn * 32 + li;
        uint32_t h, w;
        a.d_Wo.divmod(static_cast<uint32_t>(n < HoWo ? n : HoWo - 1), h, w);
        const float *const bp = patch + cur * patch_elems + ((static_cast<int>(h) - h_first) * pitch + static_cast<int>(w)) * cpad + 4 * kg;

        const bool wave_active = n0 + wn * 32 < HoWo;  // (the last tile of an image may leave whole waves without positions)
        f32x16 acc;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = 0.f;

        auto fetch = [&](int g, f32x4(&fa)[CC], f32x4(&fb)[CC]) {
            uint32_t tap, cg, p, q;
            a.d_ngrp.divmod(static_cast<uint32_t>(g), tap, cg);  // uniform: scalar unit
            a.d_k.divmod(tap, p, q);
            const float *const bq = bp + (static_cast<int>(p) * pitch + static_cast<int>(q)) * cpad + static_cast<int>(cg) * (8 * CC);
            const float *const aq = ap + 8 * CC * g;
#pragma unroll
            for (int i = 0; i < CC; ++i) {
                fa[i] = lds_load4(aq + 8 * i);
                fb[i] = lds_load4(bq + 8 * i);
            }
        };
        auto multiply = [&](const f32x4(&fa)[CC], const f32x4(&fb)[CC]) {
#pragma unroll
            for (int i = 0; i < CC; ++i)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][t], fb[i][t], acc, 0, 0, 0);
        };
        f32x4 fa0[CC], fa1[CC], fb0[CC], fb1[CC];
        const int g_end = KS == 1 ? n_groups : (ks + 1) * (n_groups / KS);  // this wave set's share of the groups
        int g = wave_active ? (KS == 1 ? 0 : ks * (n_groups / KS)) : g_end;
        if (wave_active) fetch(g, fa0, fb0);
        for (; g + 1 < g_end; g += 2) {
            fetch(g + 1, fa1, fb1);
            multiply(fa0, fb0);
            interleave_reads<4 * CC>();
            fetch(g + 2 < g_end ? g + 2 : g_end - 1, fa0, fb0);  // (past the end: a harmless repeat)
            multiply(fa1, fb1);
            interleave_reads<4 * CC>();
        }
        if (g < g_end) multiply(fa0, fb0);

        auto store_acc = [&]() {  // out[b][o][n] (+ bias[o]); positions outside the result are dropped by the buffer store
            if (!(wave_active && ks == 0)) return;
            float *ob = a.out + static_cast<int64_t>(b) * a.O * HoWo;
            const __amdgpu_buffer_rsrc_t osrc = make_rsrc(ob, static_cast<int64_t>(a.O) * HoWo * 4);
            if (full_rows) {
                // every row of the tile exists: the row part of the address is uniform per accumulator element and
                // rides in the instruction's scalar offset (which the range check does not see)
                const uint32_t voff = n < HoWo ? static_cast<uint32_t>(kg * 4 * HoWo + n) * 4u : kOob;
                const uint32_t row0 = static_cast<uint32_t>(m0 + wm * 32) * static_cast<uint32_t>(HoWo) * 4u;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t soff = row0 + static_cast<uint32_t>((e / 4) * 8 + e % 4) * static_cast<uint32_t>(HoWo) * 4u;
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, acc[e] + bias_v[e]), osrc, voff, soff, 0);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int o = m0 + wm * 32 + Mfma<float>::acc_row(e, lane);
                    const bool ok = o < a.O && n < HoWo;
                    buffer_store(osrc, ok ? static_cast<uint32_t>(o * HoWo + n) * 4u : kOob, acc[e] + bias_v[e]);
                }
            }
        };
        // One set of waves: a wave's block is complete here, and its store runs beside the other waves' multiplications
        // (behind the tile's barriers every wave of the workgroup would store at once, and with one tile per workgroup
        // every workgroup of the launch: 12.8 MB for [64,32,28,28] -> 64 channels, 2.7 us of nothing but stores;
        // forward 23.7 -> 23.1 us.  Descending priorities for the waves of a SIMD, to
        // make them finish one after the other, changed nothing: 23.05 us, the larger batches 0.5 - 1 % slower).
        if constexpr (kStoreEarly) store_acc();

        if constexpr (kTail) {
            // ---- the tile's last a.tail positions, n0 + BN ...: D[channel][position] in 4 x 4 blocks, sixteen to a
            // v_mfma_f32_4x4x1 -- lane l supplies A[block l / 4][row l % 4] and B[block l / 4][column l % 4] and receives
            // column l % 4 of its block, rows 0 .. 3.  A block is four channels by four positions: BM / 4 channel groups
            // times 16 / (BM / 4) position groups per instruction.  The waves share out the reduction groups; their
            // partial tails are added in wave order below.
            constexpr int NCG = BM / 4, PPM = 16 / NCG;
            f32x4 tacc[NTA];
#pragma unroll
            for (int u = 0; u < NTA; ++u) tacc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (a.tail > 0) {
                const int blk = lane / 4, ti = lane % 4;
                const int t_ch = 4 * (blk % NCG) + ti;
                const float *tb[NTA];
#pragma unroll
                for (int u = 0; u < NTA; ++u) {
                    const int pt = 4 * (u * PPM + blk / NCG) + ti;
                    int nt = n0 + BN + (pt < a.tail ? pt : 0);  // (beyond the tail: a column nobody reads)
                    nt = nt < HoWo ? nt : HoWo - 1;
                    uint32_t th, tw;
                    a.d_Wo.divmod(static_cast<uint32_t>(nt), th, tw);
                    tb[u] = patch + cur * patch_elems + ((static_cast<int>(th) - h_first) * pitch + static_cast<int>(tw)) * cpad;
                }
                const float *const ta = A + t_ch * a.lda;
                const int tg_lo = wave * n_groups / NW, tg_hi = (wave + 1) * n_groups / NW;
                const int n_tacc = (a.tail / 4 + PPM - 1) / PPM;
#pragma unroll 1
                for (int tg = tg_lo; tg < tg_hi; ++tg) {
                    uint32_t tap, cg, p, q;
                    a.d_ngrp.divmod(static_cast<uint32_t>(tg), tap, cg);
                    a.d_k.divmod(tap, p, q);
                    const int boff = (static_cast<int>(p) * pitch + static_cast<int>(q)) * cpad + static_cast<int>(cg) * (8 * CC);
#pragma unroll
                    for (int i = 0; i < 2 * CC; ++i) {
                        const f32x4 fa = lds_load4(ta + 8 * CC * tg + 4 * i);
#pragma unroll
                        for (int u = 0; u < NTA; ++u) {
                            if (u < n_tacc) {  // uniform
                                const f32x4 fb = lds_load4(tb[u] + boff + 4 * i);
#pragma unroll
                                for (int t = 0; t < 4; ++t) tacc[u] = __builtin_amdgcn_mfma_f32_4x4x1f32(fa[t], fb[t], tacc[u], 0, 0, 0);
                            }
                        }
                    }
                }
            }
            // The patch has been read: its memory takes the upper set's accumulators and the waves' tails.
            __syncthreads();
            float *const exch = patch + cur * patch_elems + wtile * 1024 + lane * 4;  // [wave][e / 4][lane][4]: consecutive lanes, consecutive vectors
            float *const tails = patch + cur * patch_elems + (KS == 2 ? WGM * WGN * 64 * 16 : 0);  // [NW][NTA][64 lanes][4]
            if (KS == 2 && ks == 1) {
#pragma unroll
                for (int e = 0; e < 16; e += 4) *reinterpret_cast<f32x4 *>(exch + e * 64) = f32x4{acc[e], acc[e + 1], acc[e + 2], acc[e + 3]};
            }
            if (a.tail > 0) {
#pragma unroll
                for (int u = 0; u < NTA; ++u) *reinterpret_cast<f32x4 *>(tails + ((wave * NTA + u) * 64 + lane) * 4) = tacc[u];
            }
            __syncthreads();
            if (KS == 2 && ks == 0) {  // (lower half of the groups) + (upper half): a fixed order
#pragma unroll
                for (int e = 0; e < 16; e += 4) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(exch + e * 64);
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[e + t] += v[t];
                }
            }
            if (tid < BM * a.tail) {  // one lane per element of the tail: the waves' parts in wave order, bias, store
                uint32_t ch, pt;
                a.d_tail.divmod(static_cast<uint32_t>(tid), ch, pt);
                const int pg = static_cast<int>(pt) / 4, j = static_cast<int>(pt) % 4;
                const int u = pg / PPM, src_lane = 4 * ((pg % PPM) * NCG + static_cast<int>(ch) / 4) + j;
                const float *src = tails + (u * 64 + src_lane) * 4 + static_cast<int>(ch) % 4;
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) v += src[w * NTA * 256];
                const int o = m0 + static_cast<int>(ch), nt = n0 + BN + static_cast<int>(pt);
                if (o < a.O && nt < HoWo) a.out[(static_cast<int64_t>(b) * a.O + o) * HoWo + nt] = v + tail_bias;
            }
            if (jn < n_tiles) __syncthreads();  // the next tile's rows overwrite what was just read
        } else if constexpr (KS == 2) {
            // the upper set's sums go to the lower set through LDS (behind the patch buffers), added as
            // (lower half of the groups) + (upper half): a fixed order
            float *const exch = patch + a.n_buf * patch_elems + wtile * 1024 + lane * 4;  // [wave][e / 4][lane][4]
            if (ks == 1) {
#pragma unroll
                for (int e = 0; e < 16; e += 4) *reinterpret_cast<f32x4 *>(exch + e * 64) = f32x4{acc[e], acc[e + 1], acc[e + 2], acc[e + 3]};
            }
            __syncthreads();  // (also: every wave has left the patch buffer)
            if (ks == 0) {
#pragma unroll
                for (int e = 0; e < 16; e += 4) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(exch + e * 64);
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[e + t] += v[t];
                }
            }
        } else {
            if (a.n_buf == 1) __syncthreads();  // one patch buffer: every wave has left it
        }
        if (jn < n_tiles) park(cur ^ (a.n_buf - 1));  // the loads were issued a whole tile ago

        if constexpr (!kStoreEarly) store_acc();
        __syncthreads();
    }
}

// Derived geometry for tiles of BM x BN computed by `waves` waves; false when this kernel does not apply.
// bne > 0 (twelve waves): the tile is bne = BN + tail positions, the tail of 4 or 8 computed apart; the exchange of the
// halves and the waves' tails pass through the patch buffer.
bool plan_patch(ConvPatchArgs &a, int BM, int BN, int waves, int n_buf, size_t *lds_bytes, int halves = 1, int bne = 0) {
    const int k = a.k, threads = 64 * waves;
    const int HoWo = a.Ho * a.Wo;
    a.bne = bne > 0 ? bne : BN;
    a.tail = a.bne - BN;
    a.d_tail = make_fastdiv(static_cast<uint32_t>(a.tail > 0 ? a.tail : 1));
    if (a.tail < 0 || a.tail > 8 || a.tail % 4 != 0) return false;
    BN = a.bne;  // the patch and the tile count follow the whole tile
    a.K = a.C * k * k;
    a.lda = a.K + 4;   // 4 (2 n + 1) floats: the 16-byte reads of 16 consecutive rows cover every bank once
    a.cpad = a.C + 4;  // likewise for 16 consecutive patch columns
    // rows of output positions under a tile (tiles of whole rows all start in column 0), plus the taps' halo rows
    a.R = (BN % a.Wo == 0 ? BN / a.Wo : (a.Wo - 1 + BN - 1) / a.Wo + 1) + (k - 1);
    a.pitch = a.W + 2 * a.P;  // columns -P .. W - 1 + P at index x + P
    a.vecs_per_row = a.W / 4;
    a.cl_shift = a.C % 16 == 0 ? 4 : 3;
    const int xl = 64 >> a.cl_shift;  // vectors of a row per staging item
    a.xh = (a.vecs_per_row + xl - 1) / xl;
    a.last_vecs = a.vecs_per_row - (a.xh - 1) * xl;
    a.n_items = (a.C >> a.cl_shift) * a.R * a.xh;
    a.stage_slots = (a.n_items + waves - 1) / waves;
    a.tiles_m = (a.O + BM - 1) / BM;
    a.tiles_n = (HoWo + BN - 1) / BN;
    const int64_t patch_elems = static_cast<int64_t>(a.R) * a.pitch * a.cpad;
    a.n_buf = n_buf;
    int64_t lds_floats = static_cast<int64_t>(BM) * a.lda + n_buf * patch_elems + (halves == 2 && bne == 0 ? waves / 2 * 64 * 16 : 0);
    if (bne > 0 && (halves == 2 ? waves / 2 * 64 * 16 : 0) + static_cast<int64_t>(waves) * 2 * 256 > patch_elems) return false;
    if (halves == 2 && (a.C % 32 != 0 || (static_cast<int64_t>(a.C) / 32 * k * k) % 2 != 0)) return false;  // an even number of 32-channel groups
    if (a.stage_slots > (waves == 12 ? 6 : kStageLoads / waves) || lds_floats * 4 > kLdsBytes) return false;
    if (static_cast<int64_t>(a.B) * a.tiles_n > 0x7fffffff || static_cast<int64_t>(a.O) * HoWo * 4 >= 0x7fffffff) return false;
    if (static_cast<int64_t>(a.C) * a.xs_c * 4 + static_cast<int64_t>(a.R) * a.xs_h * 4 >= 0x7fffffff) return false;
    if (static_cast<int64_t>(a.O + BM) * a.w_row * 4 + static_cast<int64_t>(a.C) * a.w_red * 4 >= 0x7fffffff) return false;
    // the weight block travels through the patch area in segments of 16-byte vectors
    a.n_fast = a.w_rows_fast ? BM : a.C;
    a.n_seg = a.w_rows_fast ? a.C : BM;
    a.seg_len = a.n_fast * k * k;
    if (a.seg_len % 4 != 0 || (a.w_rows_fast ? a.w_red : a.w_row) % 4 != 0) return false;  // 16-byte aligned segment starts
    // (the copy may run past the patch buffers into whatever LDS is left)
    const int64_t fit = (kLdsBytes / 4 - static_cast<int64_t>(BM) * a.lda) / a.seg_len;  // segments the area behind A holds
    if (fit < 1) return false;
    const int64_t passes = (a.n_seg + fit - 1) / fit;
    a.segs_per_pass = static_cast<int>((a.n_seg + passes - 1) / passes);
    if (static_cast<int64_t>(BM) * a.lda + static_cast<int64_t>(a.segs_per_pass) * a.seg_len > lds_floats)
        lds_floats = static_cast<int64_t>(BM) * a.lda + static_cast<int64_t>(a.segs_per_pass) * a.seg_len;
    const int seg_vecs = a.seg_len / 4;
    a.n_wvec = static_cast<int>((static_cast<int64_t>(a.n_seg) * seg_vecs + threads - 1) / threads);
    a.w_dense = (a.w_rows_fast ? a.w_red : a.w_row) == a.seg_len && a.n_wvec <= kWeightLoads / waves;
    a.w_pass_vecs = (a.segs_per_pass * seg_vecs) % threads == 0 ? a.segs_per_pass * seg_vecs / threads : 0;
    a.d_segv = make_fastdiv(static_cast<uint32_t>(seg_vecs));
    a.d_wfast = make_fastdiv(static_cast<uint32_t>(a.n_fast));
    a.d_xh = make_fastdiv(static_cast<uint32_t>(a.xh));
    a.d_R = make_fastdiv(static_cast<uint32_t>(a.R));
    a.d_cpad4 = make_fastdiv(static_cast<uint32_t>(a.cpad / 4));
    a.d_2P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? 2 * a.P : 1));
    a.d_P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? a.P : 1));
    a.d_Wo = make_fastdiv(static_cast<uint32_t>(a.Wo));
    a.d_tiles_n = make_fastdiv(static_cast<uint32_t>(a.tiles_n));
    a.d_k = make_fastdiv(static_cast<uint32_t>(k));
    *lds_bytes = static_cast<size_t>(lds_floats) * sizeof(float);
    return true;
}

template <int WGM, int WGN, int CC, int MAXS, int KS = 1>
ttamd_status launch_patch(ConvPatchArgs a, hipStream_t st, size_t lds) {
    const int64_t n_tiles = static_cast<int64_t>(a.B) * a.tiles_n;
    int64_t groups = 256 / a.tiles_m;
    if (groups < 1) groups = 1;
    if (groups > n_tiles) groups = n_tiles;
    a.d_ngrp = make_fastdiv(static_cast<uint32_t>(a.C / (8 * CC)));
    auto kernel = conv_patch_kernel<WGM, WGN, CC, MAXS, KS>;
    TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    a.red2_blocks = a.red2_splits > 0 ? (a.red2_n / 4 + 63) / 64 : 0;
    a.red_blocks = (a.red_splits > 0 ? (a.red_n / 4 + 63) / 64 : 0) + a.red2_blocks;
    if (lds < static_cast<size_t>(64 * WGM * WGN * KS) * 16) lds = static_cast<size_t>(64 * WGM * WGN * KS) * 16;  // (the second job's sums)
    kernel<<<dim3(static_cast<unsigned>(groups * a.tiles_m + a.red_blocks)), dim3(64 * WGM * WGN * KS), lds, st>>>(a);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <int WGM, int WGN, int KS = 1>
ttamd_status launch_patch_cc(const ConvPatchArgs &a, hipStream_t st, size_t lds) {
    constexpr int S1 = WGM * WGN * KS == 12 ? 6 : kStageLoads / (WGM * WGN * KS), S0 = S1 / 2;  // slot counts compiled for
    const bool few = a.stage_slots <= S0;
    if constexpr (KS == 2) {  // (only with 32-channel groups, of which each set takes half)
        // twelve waves have 168 registers each: groups of 16 channels (with groups of 32 the six staging slots of a
        // 64-channel patch spilled, and grad_input of [64,32,28,28] -> 64 channels took 34.3 us instead of 26.6)
        if constexpr (WGM * WGN * KS == 12) return few ? launch_patch<WGM, WGN, 2, S0, 2>(a, st, lds) : launch_patch<WGM, WGN, 2, S1, 2>(a, st, lds);
        return few ? launch_patch<WGM, WGN, 4, S0, 2>(a, st, lds) : launch_patch<WGM, WGN, 4, S1, 2>(a, st, lds);
    } else {
        if constexpr (WGM * WGN * KS == 12) {  // (C is a multiple of 32 here; more than three slots: groups of 16 channels, as above)
            return few ? launch_patch<WGM, WGN, 4, S0>(a, st, lds) : launch_patch<WGM, WGN, 2, S1>(a, st, lds);
        } else {
            if (a.C % 32 == 0) return few ? launch_patch<WGM, WGN, 4, S0>(a, st, lds) : launch_patch<WGM, WGN, 4, S1>(a, st, lds);
            return few ? launch_patch<WGM, WGN, 1, S0>(a, st, lds) : launch_patch<WGM, WGN, 1, S1>(a, st, lds);
        }
    }
}

}  // namespace

// Launches (unless `launch` is false: then only *variant is set) when the geometry fits this kernel: *variant is 0 when it does not, else 16 * waves + patch buffers.  Expects in `a`: the tensors and their
// strides, B C H W O k P Ho Wo, and the weight access (w_row, w_red, w_flip, w_rows_fast): tap t of (row, reduction
// channel) is at element  row * w_row + red * w_red + t  of the weight and is used as tap k*k - 1 - t when w_flip is
// set.  Eight waves (two per SIMD, which hide each other's staging and store latencies) where their larger patch
// fits in LDS, four otherwise; two patch buffers where they fit, one otherwise.
ttamd_status launch_conv_patch_f32(ConvPatchArgs a, hipStream_t st, int *variant, bool launch) {
    *variant = 0;
    const int k = a.k;
    if (a.B <= 0 || k < 1 || a.P >= k || a.C % 8 != 0 || a.W % 4 != 0) return TTAMD_OK;
    if (a.xs_h % 4 != 0 || a.xs_c % 4 != 0 || a.xs_b % 4 != 0 || reinterpret_cast<uintptr_t>(a.x) % 16 != 0) return TTAMD_OK;
    if (reinterpret_cast<uintptr_t>(a.w) % 16 != 0) return TTAMD_OK;
    if (a.Ho != a.H + 2 * a.P - k + 1 || a.Wo != a.W + 2 * a.P - k + 1 || a.Ho < 1 || a.Wo < 1) return TTAMD_OK;  // unit stride only
    const bool narrow = a.O <= 32;
    size_t lds = 0;
    // Twelve waves on a tile of 192 positions and a tail of 4 or 8 where that shares the tiles out better: cost = rounds of
    // the 256 workgroups times the MFMA blocks (whole reductions) a SIMD runs per tile.  [64,32,28,28] -> 64 channels: 448
    // tiles of 128 positions (the seventh of an image all but empty) are two rounds of 2 blocks per SIMD, 256 tiles of
    // 196 one round of 3.
    static const bool twelve_ok = std::getenv("TTAMD_CONV_PATCH_WAVES") == nullptr || std::atoi(std::getenv("TTAMD_CONV_PATCH_WAVES")) == 12;
    // 32 output channels: two sets of six waves on the halves of the reduction.
    if (twelve_ok && a.C % 32 == 0) {
        const int64_t HoWo = static_cast<int64_t>(a.Ho) * a.Wo;
        const int BM = narrow ? 32 : 64;
        const int64_t tiles_m = (a.O + BM - 1) / BM;
        const int64_t old_tiles = a.B * ((HoWo + 127) / 128) * tiles_m;
        const int64_t old_cost2 = ((old_tiles + 255) / 256) * (narrow ? 2 : 4);  // in half blocks per SIMD
        int best_bne = 0;
        int64_t best_cost2 = old_cost2;
        for (int64_t q = (HoWo + 199) / 200; q <= (HoWo + 191) / 192; ++q) {
            if (q < 1) continue;
            const int64_t pt = ((HoWo + q - 1) / q + 3) / 4 * 4;
            if (pt < 192 || pt > 200) continue;
            const int64_t cost2 = ((a.B * q * tiles_m + 255) / 256) * (narrow ? 3 : 6);
            if (cost2 < best_cost2) best_cost2 = cost2, best_bne = static_cast<int>(pt);
        }
        if (best_bne && plan_patch(a, BM, 192, 12, 1, &lds, narrow ? 2 : 1, best_bne)) {
            *variant = 12 * 16 + 1;
            if (!launch) return TTAMD_OK;
            return narrow ? launch_patch_cc<1, 6, 2>(a, st, lds) : launch_patch_cc<2, 6>(a, st, lds);
        }
    }
    static const bool wide_ok = std::getenv("TTAMD_CONV_PATCH_WAVES") == nullptr || std::atoi(std::getenv("TTAMD_CONV_PATCH_WAVES")) != 4;
    for (int n_buf = 2; n_buf >= 1; --n_buf) {  // one patch buffer (a second barrier per tile) when two do not fit
        if (wide_ok && plan_patch(a, narrow ? 32 : 64, narrow ? 256 : 128, 8, n_buf, &lds)) {
            *variant = 8 * 16 + n_buf;
            if (!launch) return TTAMD_OK;
            return narrow ? launch_patch_cc<1, 8>(a, st, lds) : launch_patch_cc<2, 4>(a, st, lds);
        }
        // the four-wave tile with a second set of waves on the other half of the reduction
        if (wide_ok && plan_patch(a, narrow ? 32 : 64, narrow ? 128 : 64, 8, n_buf, &lds, 2)) {
            *variant = 8 * 16 + n_buf;
            if (!launch) return TTAMD_OK;
            return narrow ? launch_patch_cc<1, 4, 2>(a, st, lds) : launch_patch_cc<2, 2, 2>(a, st, lds);
        }
        if (plan_patch(a, narrow ? 32 : 64, narrow ? 128 : 64, 4, n_buf, &lds)) {
            *variant = 4 * 16 + n_buf;
            if (!launch) return TTAMD_OK;
            return narrow ? launch_patch_cc<1, 4>(a, st, lds) : launch_patch_cc<2, 2>(a, st, lds);
        }
    }
    return TTAMD_OK;
}

}  // namespace ttamd
