// conv_wgrad_patch.hip — grad_weight of a stride-1 fp32 convolution with both operands staged in LDS (gfx950).
//
// grad_weight[o][c][p][q] = sum over images and output positions of grad_out[b][o][h][w] * x[b][c][h + p - P][w + q - P]
// (tinytensor/tensor/backend/cpu/conv.cpp:207-246 computes it per image as grad_out [O, HoWo] times im2col(x)^T and adds
// the images up).  As one GEMM the reduction runs over all B Ho Wo positions, M = O, N = C k k.  The implicit-GEMM
// kernel of conv.hip gathers the im2col operand through the vector memory path, every input element once per tap,
// with the tap decode in front of every load.  Here a workgroup takes a stage of whole output rows of one image:
//   * grad_out's rows of the stage go to LDS as [O][positions] and the input rows under them (with the taps' halo
//     rows, halo columns zero) as [C][rows][W + 2P], each element fetched once with 16-byte loads;
//   * four consecutive positions of a row are four consecutive floats on both sides, so a lane's A fragment for four
//     MFMAs is one 16-byte LDS read and its B fragment four 4-byte reads at  position + tap shift  -- no gather and no
//     decode; the 32 lanes of a B fragment are 32 channels, a plane pitch that is odd keeps them on distinct banks;
//   * the result tile [O x C k k] is cut into 32 x 32 blocks (32 output channels x 32 input channels of one tap); a
//     wave owns up to kMaxBlocks of them for one block of output channels, so its A fragment serves all its blocks;
//   * a workgroup adds up its stages in registers (fixed order) and writes one partial tile; the partial tiles are
//     summed in workgroup order by the caller (reduce_splits_kernel): deterministic, exact on integer-valued data.
#include "mfma_core.h"

namespace ttamd {
namespace {

using namespace mfma;

// Issue order of a chunk: the next chunk's 16-byte A read first, then a pair of 4-byte B reads behind every second
// MFMA of the current chunk.  Left to itself the scheduler sinks every read down to the MFMA that consumes it.
template <int N, int I = 0>
__device__ __forceinline__ void interleave_reads() {
    if constexpr (I == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    if constexpr (I < N) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (I % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // (the compiler pairs the 4-byte reads)
        interleave_reads<N, I + 1>();
    }
}

constexpr int kMaxBlocks = 5;        // 32 x 32 result blocks per wave (80 accumulator registers)
constexpr int kLdsBytes = 160 * 1024;
constexpr int kBatchA = 16, kBatchX = 16;  // most 16-byte loads per lane and stage: grad_out rows, input channels (O, C <= 64)

// NB: blocks per wave compiled for (the wave's actual count may be lower).
template <int NB>
__global__ void __launch_bounds__(kThreads, 1) conv_wgrad_patch_kernel(ConvWgradPatchArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem_wg[];
    // two stage buffers, each [O][pitch_a] grad_out rows + [C][plane] input rows (halo columns zero)
    const int buf_floats = a.O * a.pitch_a + a.C * a.plane;
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int li = lane % 32, kg = lane / 32;
    const int Wo = a.Wo, pitch = a.pitch, plane = a.plane, pitch_a = a.pitch_a;
    const int K = a.C * a.k * a.k;
    const int HoWo = a.Ho * Wo;

    // this wave's blocks: output-channel block ob, column blocks first .. first + nb - 1 (column block = tap * C/32 + cb)
    const int ob = wave / a.waves_per_ob;
    const int first = (wave % a.waves_per_ob) * a.blocks_per_wave;
    int nb = a.col_blocks - first;
    nb = nb < 0 ? 0 : (nb > a.blocks_per_wave ? a.blocks_per_wave : nb);
    int block_base[NB];  // float offset in a patch of (channel of this lane, tap) for position 0
    int block_col[NB];   // result column (c k k + tap) of the block's channel 0
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        uint32_t tap, cb, p, q;
        a.d_cblocks.divmod(static_cast<uint32_t>(first + (i < nb ? i : 0)), tap, cb);
        a.d_k.divmod(tap, p, q);
        block_base[i] = a.O * pitch_a + (static_cast<int>(cb) * 32 + li) * plane + static_cast<int>(p) * pitch + static_cast<int>(q);
        block_col[i] = static_cast<int>(cb) * 32 * a.k * a.k + static_cast<int>(tap);
    }
    f32x16 acc[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

    // halo columns of both patches: zero for the whole kernel (the staging below never writes them)
    for (int v = tid; v < 2 * a.C * a.R * 2 * a.P; v += kThreads) {
        uint32_t row, sp, side, pc, bc, r, bf, c;
        a.d_2P.divmod(static_cast<uint32_t>(v), row, sp);  // row = (buffer * C + c) * R + r
        a.d_P.divmod(sp, side, pc);
        a.d_R.divmod(row, bc, r);
        a.d_C.divmod(bc, bf, c);
        smem_wg[static_cast<int>(bf) * buf_floats + a.O * pitch_a + static_cast<int>(c) * plane + static_cast<int>(r) * pitch +
                (side ? a.P + a.W + static_cast<int>(pc) : static_cast<int>(pc))] = 0.f;
    }

    // The lane's part of the staging: vector `lane` of a grad_out row (an instruction of a wave loads one row); row
    // x_lane_r, vector x_lane_v of a channel's patch (an instruction loads a channel's R rows).  Which row or channel
    // is wave-uniform and rides in the load's scalar offset.
    const int a_vecs = pitch_a / 4;  // 16-byte vectors per staged grad_out row (behind the stage's positions: zeros)
    uint32_t xr, xv;
    a.d_vw.divmod(static_cast<uint32_t>(lane), xr, xv);
    const int x_lane_r = static_cast<int>(xr);
    const bool x_lane_ok = x_lane_r < a.R;
    const uint32_t x_lane_goff = static_cast<uint32_t>((x_lane_r * a.xs_h + 4 * static_cast<int>(xv)) * 4);
    const int x_lane_lds = a.O * pitch_a + x_lane_r * pitch + a.P + 4 * static_cast<int>(xv);

    // This workgroup's stages: units blockIdx.x, blockIdx.x + gridDim.x, ... (a unit: RS output rows of one image),
    // each cut into n_sub stages of RSS rows; stage t + 1 is loaded while stage t is multiplied.
    const int n_units = (a.n_units - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    const int n_t = n_units * a.n_sub;
    auto stage_at = [&](int t, int &b, int &r0, int &rows) {
        const int j = t / a.n_sub, sub = t - j * a.n_sub;  // (n_sub is 1 or 2)
        uint32_t bi, si;
        a.d_spi.divmod(static_cast<uint32_t>(static_cast<int>(blockIdx.x) + j * static_cast<int>(gridDim.x)), bi, si);
        const int ur0 = static_cast<int>(si) * a.RS;
        const int urows = a.Ho - ur0 < a.RS ? a.Ho - ur0 : a.RS;
        b = static_cast<int>(bi);
        r0 = ur0 + sub * a.RSS;
        rows = urows - sub * a.RSS;
        rows = rows < 0 ? 0 : (rows > a.RSS ? a.RSS : rows);
    };
    f32x4 da[kBatchA], dx[kBatchX];
    auto request = [&](int t) {  // global -> registers: all loads of a stage in flight together
        int b, r0, rows;
        stage_at(t, b, r0, rows);
        const int np = rows * Wo;
        const float *gbase = a.gout + (static_cast<int64_t>(b) * a.O) * HoWo + static_cast<int64_t>(r0) * Wo;
        const __amdgpu_buffer_rsrc_t gsrc = make_rsrc(gbase, (static_cast<int64_t>(a.O) * HoWo - static_cast<int64_t>(r0) * Wo) * 4);
        const int y0 = r0 - a.P;
        const int64_t first_x = static_cast<int64_t>(b) * a.xs_b + static_cast<int64_t>(y0) * a.xs_h;
        const __amdgpu_buffer_rsrc_t xsrc = make_rsrc(a.x + first_x, a.image_bytes - static_cast<int64_t>(y0) * a.xs_h * 4);
        const uint32_t a_voff = 4 * lane < np ? static_cast<uint32_t>(lane) * 16u : kOob;
        const uint32_t x_voff = x_lane_ok && static_cast<unsigned>(y0 + x_lane_r) < static_cast<unsigned>(a.H) ? x_lane_goff : kOob;
#pragma unroll
        for (int i = 0; i < kBatchA; ++i) {
            const int o = wave + i * kWaves;
            da[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(gsrc, o < a.O ? a_voff : kOob, static_cast<uint32_t>(o) * static_cast<uint32_t>(HoWo) * 4u, 0));
        }
#pragma unroll
        for (int i = 0; i < kBatchX; ++i) {
            const int c = wave + i * kWaves;
            dx[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(xsrc, c < a.C ? x_voff : kOob, static_cast<uint32_t>(c * a.xs_c * 4), 0));
        }
    };
    auto park = [&](int buf) {  // registers -> stage buffer `buf`
        float *base = smem_wg + buf * buf_floats;
        if (lane < a_vecs) {  // (vectors behind the stage's positions: the zeros the loads returned)
            float *dst = base + 4 * lane;
#pragma unroll
            for (int i = 0; i < kBatchA; ++i) {
                const int o = wave + i * kWaves;
                if (o < a.O) *reinterpret_cast<f32x4 *>(dst + o * pitch_a) = da[i];
            }
        }
        if (x_lane_ok) {
            float *dst = base + x_lane_lds;
#pragma unroll
            for (int i = 0; i < kBatchX; ++i) {
                const int c = wave + i * kWaves;
                if (c < a.C) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[c * plane + e] = dx[i][e];  // (the plane pitch is odd: no 16-byte alignment here)
                }
            }
        }
    };

    if (n_t > 0) {
        request(0);
        park(0);
    }
    __syncthreads();
    for (int t = 0; t < n_t; ++t) {
        const int cur = t & 1;
        if (t + 1 < n_t) request(t + 1);
        int b_, r0_, rows;
        stage_at(t, b_, r0_, rows);
        const int np = rows * Wo;  // positions of this stage (a multiple of 4)
        // ---- multiply: chunks of 8 positions; lane (li, kg) takes positions 8 ch + 4 kg .. + 3 of the chunk
        {
            const float *const stage = smem_wg + cur * buf_floats;
            const float *const ap = stage + (ob * 32 + li) * pitch_a + 4 * kg;
            const int chunks = (np + 7) / 8;
            const int last_off = (rows - 1) * pitch + Wo - 4;  // patch offset of the stage's last four positions
            int x = 4 * kg, off = 4 * kg, pos = 4 * kg;        // this lane's column, patch offset and position in the current chunk
            auto fetch = [&](int ch, f32x4 &fa, float(&fb)[NB][4]) {
                fa = *reinterpret_cast<const f32x4 *>(ap + 8 * ch);
                // behind the stage's last position grad_out holds zeros; the input is then read at a cell that belongs
                // to the sum anyway, so that a non-finite input value cannot reach a column it is not part of
                const int o = pos < np ? off : last_off;
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const float *bp = stage + block_base[i] + o;
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) fb[i][t4] = bp[t4];
                }
                // next chunk: 8 positions on, wrapping into the next row (Wo >= 8: at most one wrap)
                pos += 8;
                x += 8;
                const bool wrap = x >= Wo;
                x = wrap ? x - Wo : x;
                off += wrap ? 8 + pitch - Wo : 8;
            };
            auto multiply = [&](const f32x4 &fa, const float(&fb)[NB][4]) {
                // (a wave with fewer than NB blocks multiplies its first block again in the spare slots and drops the
                // result: the workgroup is as slow as its busiest wave either way, and the loop stays one basic block)
#pragma unroll
                for (int i = 0; i < NB; ++i)
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t4], fb[i][t4], acc[i], 0, 0, 0);
            };
            if (chunks > 0) {
                f32x4 fa0, fa1;
                float fb0[NB][4], fb1[NB][4];
                fetch(0, fa0, fb0);
                int ch = 0;
                for (; ch + 1 < chunks; ch += 2) {
                    fetch(ch + 1, fa1, fb1);
                    multiply(fa0, fb0);
                    interleave_reads<4 * NB>();
                    fetch(ch + 2 < chunks ? ch + 2 : chunks - 1, fa0, fb0);  // (past the end: fetched and not used)
                    multiply(fa1, fb1);
                    interleave_reads<4 * NB>();
                }
                if (ch < chunks) multiply(fa0, fb0);
            }
        }
        if (t + 1 < n_t) park(cur ^ 1);  // (the other buffer: last read before the previous barrier)
        __syncthreads();
    }

    // ---- partial tile of this workgroup, [O][C k k] as grad_weight is laid out: through LDS, so that the copy to
    // memory runs in whole rows
    float *const tile = smem_wg;  // [O][K + 4]
    const int tp = K + 4;
    const int k2 = a.k * a.k;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        if (i < nb) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                tile[(ob * 32 + Mfma<float>::acc_row(e, lane)) * tp + block_col[i] + li * k2] = acc[i][e];
        }
    }
    __syncthreads();
    float *const out = a.partial + static_cast<int64_t>(blockIdx.x) * a.O * K;
    for (int o = wave; o < a.O; o += kWaves)  // a row per wave and step, 64 vectors per instruction
        for (int x = lane; x < K / 4; x += 64)
            *reinterpret_cast<f32x4 *>(out + static_cast<int64_t>(o) * K + 4 * x) = *reinterpret_cast<const f32x4 *>(tile + o * tp + 4 * x);
}

// ---------------------------------------------------------------------------------------------------------------
// The same product for layers with more than 32 output channels, or whose column blocks do not share out evenly over
// four waves: a workgroup takes ONE block of 32 output channels (blockIdx.x % (O / 32)) and KS sets of four waves
// share out the positions of a stage -- set s multiplies chunks [s n / KS, (s + 1) n / KS) -- with the column blocks
// dealt to a set's waves one slot further round for every set: 9 blocks are 3 + 2 + 2 + 2 to the four waves of a set,
// and over four sets every SIMD gets 9 quarter blocks (with one set: 3 whole blocks against 2).  A workgroup's partial
// tile is [32][C k k], half of what the one-set kernel writes per workgroup at O = 64, and so is what the kernel that
// adds the partial tiles reads.  Every set leaves its accumulators in an LDS tile of its own; the copy to memory adds the
// sets' tiles in set order (deterministic).  One stage buffer: a stage is loaded, multiplied and then the next one loaded.
template <int NB, int KS>
__global__ void __launch_bounds__(256 * KS, 1) conv_wgrad_patch_sets_kernel(ConvWgradPatchArgs a) {
    constexpr int NW = 4 * KS, NT = 64 * NW;
    constexpr int MAXA = 16 / KS;  // most 16-byte loads of grad_out per lane and stage
    extern __shared__ __attribute__((aligned(16))) float smem_ws[];
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int set = wave / 4, ww = wave % 4;
    const int li = lane % 32, kg = lane / 32;
    const int Wo = a.Wo, pitch = a.pitch, plane = a.plane, pitch_a = a.pitch_a;
    const int K = a.C * a.k * a.k;
    const int HoWo = a.Ho * Wo;
    const int n_ob = a.O / 32;
    const int ob = static_cast<int>(blockIdx.x) % n_ob, gi = static_cast<int>(blockIdx.x) / n_ob, G = static_cast<int>(gridDim.x) / n_ob;
    float *const xs = smem_ws + 32 * pitch_a;  // [C][plane] behind the [32][pitch_a] rows of grad_out

    // this wave's column blocks: slot (ww + set * 4 / KS) % 4 of the four slots that the blocks are dealt to
    const int slot = (ww + set * (4 / KS)) & 3;
    const int per = a.col_blocks / 4, rem = a.col_blocks % 4;
    const int first = slot * per + (slot < rem ? slot : rem);
    const int nb = per + (slot < rem ? 1 : 0);
    int block_base[NB];  // float offset in the patch of (channel of this lane, tap) for position 0
    int block_col[NB];   // result column (c k k + tap) of the block's channel 0
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        uint32_t tap, cb, p, q;
        a.d_cblocks.divmod(static_cast<uint32_t>(first + (i < nb ? i : 0)), tap, cb);
        a.d_k.divmod(tap, p, q);
        block_base[i] = (static_cast<int>(cb) * 32 + li) * plane + static_cast<int>(p) * pitch + static_cast<int>(q);
        block_col[i] = static_cast<int>(cb) * 32 * a.k * a.k + static_cast<int>(tap);
    }
    f32x16 acc[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

    // halo columns of the patch: zero for the whole kernel (the staging never writes them)
    for (int v = tid; v < a.C * a.R * 2 * a.P; v += NT) {
        uint32_t row, sp, side, pc, c, r;
        a.d_2P.divmod(static_cast<uint32_t>(v), row, sp);  // row = c * R + r
        a.d_P.divmod(sp, side, pc);
        a.d_R.divmod(row, c, r);
        xs[static_cast<int>(c) * plane + static_cast<int>(r) * pitch + (side ? a.P + a.W + static_cast<int>(pc) : static_cast<int>(pc))] = 0.f;
    }

    // The lane's part of the staging.  grad_out: a wave takes rows wave, wave + NW, ... of the 32, a_instr instructions
    // of 64 vectors per row.  Input: channels wave, wave + NW, ..., x_instr instructions per channel's R rows; vector
    // lane + 64 j of a channel is row x_r[j], vector x_v[j] of that row.  Rows and channels are wave-uniform and ride
    // in the loads' scalar offsets.
    const int a_vecs = pitch_a / 4;
    const int a_rows = 32 / NW;                   // (NW is 8 or 16)
    const int x_chans = (a.C + NW - 1) / NW;
    int x_r[2], x_lds[2];
    uint32_t x_goff[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint32_t xr, xv;
        a.d_vw.divmod(static_cast<uint32_t>(lane + 64 * j), xr, xv);
        x_r[j] = static_cast<int>(xr) < a.R && j < a.x_instr ? static_cast<int>(xr) : -(1 << 28);  // never passes the row test
        x_goff[j] = static_cast<uint32_t>((static_cast<int>(xr) * a.xs_h + 4 * static_cast<int>(xv)) * 4);
        x_lds[j] = static_cast<int>(xr) * pitch + a.P + 4 * static_cast<int>(xv);
    }

    const int n_units = (a.n_units - gi + G - 1) / G;
    for (int t = 0; t < n_units; ++t) {
        uint32_t bi, si;
        a.d_spi.divmod(static_cast<uint32_t>(gi + t * G), bi, si);
        const int b = static_cast<int>(bi), r0 = static_cast<int>(si) * a.RS;
        const int rows = a.Ho - r0 < a.RS ? a.Ho - r0 : a.RS;
        const int np = rows * Wo;  // positions of this stage (a multiple of 4)
        // ---- stage: global -> registers (the loads of a batch in flight together) -> LDS.  A batch: grad_out's rows of
        // this wave and two of its input channels; further channels (more than 2 NW of them) in batches of two.
        {
            f32x4 da[MAXA], dx[4];
            const float *gbase = a.gout + (static_cast<int64_t>(b) * a.O + ob * 32) * HoWo + static_cast<int64_t>(r0) * Wo;
            const __amdgpu_buffer_rsrc_t gsrc = make_rsrc(gbase, (static_cast<int64_t>(32) * HoWo - static_cast<int64_t>(r0) * Wo) * 4);
            const int y0 = r0 - a.P;
            const int64_t first_x = static_cast<int64_t>(b) * a.xs_b + static_cast<int64_t>(y0) * a.xs_h;
            const __amdgpu_buffer_rsrc_t xsrc = make_rsrc(a.x + first_x, a.image_bytes - static_cast<int64_t>(y0) * a.xs_h * 4);
            auto load_x = [&](int c0) {  // channels wave + (c0 + i / 2) NW, instruction i % 2
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int ci = c0 + i / 2, j = i % 2;
                    const int c = wave + ci * NW;
                    const bool ok = ci < x_chans && c < a.C && static_cast<unsigned>(y0 + x_r[j]) < static_cast<unsigned>(a.H);
                    dx[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(xsrc, ok ? x_goff[j] : kOob, static_cast<uint32_t>(c * a.xs_c * 4), 0));
                }
            };
            auto park_x = [&](int c0) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int ci = c0 + i / 2, j = i % 2;
                    const int c = wave + ci * NW;
                    if (ci < x_chans && c < a.C && x_r[j] >= 0) {
                        float *dst = xs + c * plane + x_lds[j];
#pragma unroll
                        for (int e = 0; e < 4; ++e) dst[e] = dx[i][e];  // (the plane pitch is odd: no 16-byte alignment here)
                    }
                }
            };
#pragma unroll
            for (int i = 0; i < MAXA; ++i) {
                const int r = i / 2, j = i % 2;  // row wave + r NW, instruction j
                const int v = lane + 64 * j;
                const bool ok = r < a_rows && j < a.a_instr && 4 * v < np;
                da[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(gsrc, ok ? static_cast<uint32_t>(v) * 16u : kOob,
                                                                                       static_cast<uint32_t>(wave + r * NW) * static_cast<uint32_t>(HoWo) * 4u, 0));
            }
            load_x(0);
#pragma unroll
            for (int i = 0; i < MAXA; ++i) {
                const int r = i / 2, j = i % 2;
                const int v = lane + 64 * j;
                // (vectors behind the stage's positions, up to the end of its last chunk: the zeros the loads returned)
                if (r < a_rows && j < a.a_instr && v < a_vecs) *reinterpret_cast<f32x4 *>(smem_ws + (wave + r * NW) * pitch_a + 4 * v) = da[i];
            }
            park_x(0);
            for (int c0 = 2; c0 < x_chans; c0 += 2) {
                load_x(c0);
                park_x(c0);
            }
        }
        __syncthreads();
        // ---- multiply: chunks of 8 positions, this set's share of them; lane (li, kg) takes positions 8 ch + 4 kg .. + 3.
        // NBW: the wave's blocks, NB or one less (wave-uniform; a loop of its own for each, so that both stay one basic
        // block with the reads placed between the MFMAs).
        auto run = [&]<int NBW>() {
            const float *const ap = smem_ws + li * pitch_a + 4 * kg;
            const int chunks = (np + 7) / 8;
            const int c_lo = set * chunks / KS, n = (set + 1) * chunks / KS - c_lo;
            const int last_off = (rows - 1) * pitch + Wo - 4;  // patch offset of the stage's last four positions
            // Position, column and patch offset of the chunk's two groups of four positions (kg = 0, 1): the same for
            // all lanes of a group, so they are kept as wave-uniform values (scalar arithmetic) and a lane selects its
            // group's offset.  Wo and the positions are multiples of 4: a group never straddles a row.
            int pos_g[2], x_g[2], off_g[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                pos_g[h] = 8 * c_lo + 4 * h;
                const int row0 = static_cast<int>(a.d_Wo.div(static_cast<uint32_t>(pos_g[h])));
                x_g[h] = pos_g[h] - row0 * Wo;
                off_g[h] = row0 * pitch + x_g[h];
            }
            auto fetch = [&](int ch, f32x4 &fa, float(&fb)[NBW][4]) {
                fa = *reinterpret_cast<const f32x4 *>(ap + 8 * (c_lo + ch));
                // behind the stage's last position grad_out holds zeros; the input is then read at a cell that belongs
                // to the sum anyway, so that a non-finite input value cannot reach a column it is not part of
                const int o0 = pos_g[0] < np ? off_g[0] : last_off, o1 = pos_g[1] < np ? off_g[1] : last_off;
                const int o = kg ? o1 : o0;
#pragma unroll
                for (int i = 0; i < NBW; ++i) {
                    const float *bp = xs + block_base[i] + o;
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) fb[i][t4] = bp[t4];
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {  // the next chunk: 8 positions on, at most one wrap (Wo >= 8)
                    pos_g[h] += 8;
                    x_g[h] += 8;
                    const bool wrap = x_g[h] >= Wo;
                    x_g[h] = wrap ? x_g[h] - Wo : x_g[h];
                    off_g[h] += wrap ? 8 + pitch - Wo : 8;
                }
            };
            auto multiply = [&](const f32x4 &fa, const float(&fb)[NBW][4]) {
#pragma unroll
                for (int i = 0; i < NBW; ++i)
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t4], fb[i][t4], acc[i], 0, 0, 0);
            };
            if (n > 0) {
                f32x4 fa0, fa1;
                float fb0[NBW][4], fb1[NBW][4];
                fetch(0, fa0, fb0);
                int ch = 0;
                for (; ch + 1 < n; ch += 2) {
                    fetch(ch + 1, fa1, fb1);
                    multiply(fa0, fb0);
                    interleave_reads<4 * NBW>();
                    fetch(ch + 2 < n ? ch + 2 : n - 1, fa0, fb0);  // (past the end: fetched and not used)
                    multiply(fa1, fb1);
                    interleave_reads<4 * NBW>();
                }
                if (ch < n) multiply(fa0, fb0);
            }
        };
        if (nb == NB) run.template operator()<NB>();
        else if constexpr (NB > 1) run.template operator()<NB - 1>();
        __syncthreads();  // the stage has been read: the next one, or the tile below, may overwrite it
    }

    // ---- the workgroup's partial tile [32][C k k]: every set leaves its blocks in an LDS tile of its own, then whole
    // rows go to memory, the sets' tiles added in set order on the way
    const int tp = K + 4;
    const int k2 = a.k * a.k;
    float *const tile = smem_ws + set * 32 * tp;  // [KS][32][K + 4]
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        if (i < nb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) tile[Mfma<float>::acc_row(e, lane) * tp + block_col[i] + li * k2] = acc[i][e];
        }
    }
    __syncthreads();
    float *const out = a.partial + (static_cast<int64_t>(gi) * a.O + ob * 32) * K;
    for (int v = tid; v < 32 * (K / 4); v += NT) {  // consecutive lanes: consecutive vectors of a row
        uint32_t o, x;
        a.d_kvecs.divmod(static_cast<uint32_t>(v), o, x);
        const float *src = smem_ws + static_cast<int>(o) * tp + 4 * static_cast<int>(x);
        f32x4 sum = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
        for (int s = 1; s < KS; ++s) sum += *reinterpret_cast<const f32x4 *>(src + s * 32 * tp);
        *reinterpret_cast<f32x4 *>(out + static_cast<int64_t>(o) * K + 4 * static_cast<int>(x)) = sum;
    }
}

}  // namespace

// Whether (and how) this kernel serves a geometry: decided by the shape alone, so that the workspace query and the
// launch agree.  Rows per stage: as many as LDS holds, then the number of stages per image that gives the 256
// workgroups the shortest busiest one.
namespace {
// TTAMD_CONV_WGRAD_SETS=0 in the environment: never the kernel with sets of waves (for measurements).
bool wgrad_sets_enabled() {
    static const bool on = [] {
        const char *e = getenv("TTAMD_CONV_WGRAD_SETS");
        return !(e && e[0] == '0');
    }();
    return on;
}

// The plan of conv_wgrad_patch_sets_kernel, or use = false.
ConvWgradPatchPlan plan_sets(int B, int C, int H, int W, int O, int k, int P, int Ho, int Wo) {
    ConvWgradPatchPlan pl{};
    if (C % 32 != 0 || C > 64 || O % 32 != 0 || O / 32 > 256) return pl;
    const int n_ob = O / 32;
    const int col_blocks = k * k * (C / 32);
    const int nb = (col_blocks + 3) / 4;
    // Up to three blocks per wave (16 waves have 128 registers each).  Measured, backward pass of a whole layer with this
    // kernel against the other grad_weight kernels: [64,32,28,28] -> 32 channels 37.9 against 40.9 us, -> 64 channels
    // 57.1 against 60.8, [128,32,28,28] -> 64 95.7 against 106.4, [32,32,32,32] -> 96 74.3 against 81.7; with 64 input
    // channels (five blocks per wave, two sets) it was 1 - 1.5 % slower than the implicit-GEMM kernel on 56 x 56 and
    // 112 x 112 images, which therefore keeps those.
    if (nb > 3) return pl;
    const int sets = 4;
    const int pitch = W + 2 * P;
    const int64_t K = static_cast<int64_t>(C) * k * k;
    const int64_t tile = sets * 32 * (K + 4);  // a tile per set
    if (tile * 4 > kLdsBytes) return pl;
    // a stage of rs output rows: floats of the stage buffer, or 0 when two instructions per row / channel do not cover it
    auto stage_floats = [&](int rs, int *a_instr, int *x_instr) -> int64_t {
        const int64_t pitch_a = 4 * ((((static_cast<int64_t>(rs) * Wo + 7) / 8 * 8) / 4) | 1);  // whole chunks, 4 (2 n + 1) floats
        const int64_t x_vecs = static_cast<int64_t>(rs + k - 1) * (W / 4);
        if (pitch_a / 4 > 128 || x_vecs > 128) return 0;
        *a_instr = pitch_a / 4 > 64 ? 2 : 1;
        *x_instr = x_vecs > 64 ? 2 : 1;
        const int64_t plane = (static_cast<int64_t>(rs + k - 1) * pitch) | 1;
        return 32 * pitch_a + C * plane;
    };
    const int max_groups = 256 / n_ob > 0 ? 256 / n_ob : 1;  // groups of units; a group's units go to n_ob workgroups, one after the other
    int best_spi = 0;
    int64_t best_cost = 0;
    for (int spi = 1; spi <= Ho; ++spi) {
        const int rs = (Ho + spi - 1) / spi;
        if ((Ho + rs - 1) / rs != spi) continue;  // (the same rs as a smaller spi)
        int ai, xi;
        const int64_t sf = stage_floats(rs, &ai, &xi);
        if (sf == 0 || sf * 4 > kLdsBytes) continue;
        const int64_t units = static_cast<int64_t>(B) * spi;
        const int64_t groups = units < max_groups ? units : max_groups;
        const int64_t cost = ((units + groups - 1) / groups) * (static_cast<int64_t>(rs) * Wo + 112);  // positions, plus fixed costs per stage
        if (best_spi == 0 || cost < best_cost) best_spi = spi, best_cost = cost;
    }
    if (best_spi == 0) return pl;
    pl.SPI = best_spi;
    pl.RS = (Ho + best_spi - 1) / best_spi;
    pl.n_sub = 1;
    pl.RSS = pl.RS;
    const int64_t units = static_cast<int64_t>(B) * pl.SPI;
    if (units > 0x7fffffff) return pl;
    pl.n_units = static_cast<int>(units);
    pl.workgroups = units < max_groups ? pl.n_units : max_groups;
    const int64_t sf = stage_floats(pl.RS, &pl.a_instr, &pl.x_instr);
    pl.lds_bytes = static_cast<size_t>(sf > tile ? sf : tile) * 4;
    pl.blocks_per_wave = nb;
    pl.sets = sets;
    pl.use = true;
    return pl;
}
}  // namespace

ConvWgradPatchPlan plan_conv_wgrad_patch(int B, int C, int H, int W, int O, int k, int S, int P) {
    ConvWgradPatchPlan pl{};
    const int Ho = H + 2 * P - k + 1, Wo = W + 2 * P - k + 1;
    if (S != 1 || B <= 0 || k < 1 || P >= k || W % 4 != 0 || W > 256 || Ho < 1 || Wo < 8 || Wo % 4 != 0) return pl;
    if (wgrad_sets_enabled()) {
        const ConvWgradPatchPlan ps = plan_sets(B, C, H, W, O, k, P, Ho, Wo);
        if (ps.use) return ps;
    }
    // (Output-channel counts above 32: measured on a par with the implicit-GEMM kernel, whose 64-row tile is full there
    // -- 30.0 + 5.8 us against 31.1 + 4.7 us for [64,32,28,28] x [64,32,3,3] -- so that one keeps them.)
    if (S != 1 || B <= 0 || k < 1 || P >= k || C % 32 != 0 || O != 32 || W % 4 != 0 || W > 256 || Ho < 1 || Wo < 8 || Wo % 4 != 0) return pl;
    const int n_ob = O / 32;
    if (n_ob != 1 && n_ob != 2 && n_ob != 4) return pl;
    const int waves_per_ob = kWaves / n_ob;
    const int col_blocks = k * k * (C / 32);
    const int blocks_per_wave = (col_blocks + waves_per_ob - 1) / waves_per_ob;
    if (blocks_per_wave > kMaxBlocks) return pl;
    if (O > kWaves * kBatchA || C > kWaves * kBatchX) return pl;  // a wave stages O / 4 rows and C / 4 channels per stage
    const int pitch = W + 2 * P;
    const int64_t K = static_cast<int64_t>(C) * k * k;
    const int64_t tile = O * (K + 4);
    if (tile * 4 > kLdsBytes) return pl;
    // a stage of rss output rows: floats of one stage buffer, or 0 when a wave's load instructions do not cover it
    auto stage_floats = [&](int rss) -> int64_t {
        const int64_t pitch_a = 4 * ((((static_cast<int64_t>(rss) * Wo + 7) / 8 * 8) / 4) | 1);  // whole chunks, 4 (2 n + 1) floats
        if (pitch_a / 4 > 64 || rss + k - 1 > 64 / (W / 4)) return 0;  // one instruction per grad_out row / per channel
        const int64_t plane = (static_cast<int64_t>(rss + k - 1) * pitch) | 1;
        return O * pitch_a + C * plane;
    };
    // Units of rs = ceil(Ho / spi) rows, one or more per workgroup: the split that gives the busiest of the 256
    // workgroups the least to do.  A unit is one stage: cutting it into two double-buffered stages was measured and
    // gains nothing (the loads that arrive during the MFMA loop slow it by as much as the load phase they hide:
    // 94 against 74 cycles per MFMA), so n_sub stays 1; the kernel keeps the general form.
    int best_spi = 0;
    int64_t best_cost = 0;
    for (int spi = 1; spi <= Ho; ++spi) {
        const int rs = (Ho + spi - 1) / spi;
        if ((Ho + rs - 1) / rs != spi) continue;  // (the same rs as a smaller spi)
        const int n_sub = 1, rss = (rs + n_sub - 1) / n_sub;
        const int64_t sf = stage_floats(rss);
        if (sf == 0 || 2 * sf * 4 > kLdsBytes) continue;
        const int64_t units = static_cast<int64_t>(B) * spi;
        const int64_t cost = ((units + 255) / 256) * (static_cast<int64_t>(rs) * Wo + 48 * n_sub + 64);  // positions, plus fixed costs per stage and unit
        if (best_spi == 0 || cost < best_cost) best_spi = spi, best_cost = cost;
    }
    if (best_spi == 0) return pl;
    pl.SPI = best_spi;
    pl.RS = (Ho + best_spi - 1) / best_spi;
    pl.n_sub = 1;
    pl.RSS = (pl.RS + pl.n_sub - 1) / pl.n_sub;
    const int64_t units = static_cast<int64_t>(B) * pl.SPI;
    if (units > 0x7fffffff) return pl;
    pl.n_units = static_cast<int>(units);
    pl.workgroups = units < 256 ? pl.n_units : 256;
    const int64_t lds_floats = 2 * stage_floats(pl.RSS) > tile ? 2 * stage_floats(pl.RSS) : tile;
    pl.lds_bytes = static_cast<size_t>(lds_floats) * 4;
    pl.blocks_per_wave = blocks_per_wave;
    pl.use = true;
    return pl;
}

// Launches grad_weight's partial tiles ([workgroups][O][C k k] at a.partial); *handled = false when the operands'
// strides or alignment rule this kernel out (the caller then takes the implicit-GEMM kernel).
ttamd_status launch_conv_wgrad_patch_f32(ConvWgradPatchArgs a, const ConvWgradPatchPlan &pl, hipStream_t st, bool *handled) {
    *handled = false;
    if (!pl.use) return TTAMD_OK;
    if (a.xs_h % 4 != 0 || a.xs_c % 4 != 0 || a.xs_b % 4 != 0 || reinterpret_cast<uintptr_t>(a.x) % 16 != 0) return TTAMD_OK;
    if (reinterpret_cast<uintptr_t>(a.gout) % 16 != 0 || reinterpret_cast<uintptr_t>(a.partial) % 16 != 0) return TTAMD_OK;
    const int k = a.k;
    const int64_t HoWo = static_cast<int64_t>(a.Ho) * a.Wo;
    if (a.O * HoWo * 4 >= 0x7fffffff || static_cast<int64_t>(a.C) * a.xs_c * 4 + static_cast<int64_t>(a.H + 2 * k) * a.xs_h * 4 >= 0x7fffffff) return TTAMD_OK;
    a.RS = pl.RS;
    a.SPI = pl.SPI;
    a.RSS = pl.RSS;
    a.n_sub = pl.n_sub;
    a.n_units = pl.n_units;
    a.R = a.RSS + k - 1;
    a.pitch = a.W + 2 * a.P;
    a.plane = (a.R * a.pitch) | 1;
    a.pitch_a = 4 * ((((a.RSS * a.Wo + 7) / 8 * 8) / 4) | 1);
    a.waves_per_ob = kWaves / (a.O / 32);
    a.col_blocks = k * k * (a.C / 32);
    a.blocks_per_wave = pl.blocks_per_wave;
    a.d_cblocks = make_fastdiv(static_cast<uint32_t>(a.C / 32));
    a.d_k = make_fastdiv(static_cast<uint32_t>(k));
    a.d_2P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? 2 * a.P : 1));
    a.d_P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? a.P : 1));
    a.d_R = make_fastdiv(static_cast<uint32_t>(a.R));
    a.d_spi = make_fastdiv(static_cast<uint32_t>(a.SPI));
    a.d_C = make_fastdiv(static_cast<uint32_t>(a.C));
    a.d_vw = make_fastdiv(static_cast<uint32_t>(a.W / 4));
    a.d_Wo = make_fastdiv(static_cast<uint32_t>(a.Wo));
    a.d_kvecs = make_fastdiv(static_cast<uint32_t>(a.C * k * k / 4));
    a.a_instr = pl.a_instr;
    a.x_instr = pl.x_instr;
    if (pl.sets) {
        const int n_ob = a.O / 32;
        if (static_cast<int64_t>(32) * HoWo * 4 >= 0x7fffffff) return TTAMD_OK;
        auto go_sets = [&](auto kernel) -> ttamd_status {
            TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(pl.lds_bytes)));
            kernel<<<dim3(static_cast<unsigned>(pl.workgroups * n_ob)), dim3(256 * pl.sets), pl.lds_bytes, st>>>(a);
            TTAMD_HIP_CHECK(hipGetLastError());
            return TTAMD_OK;
        };
        if (pl.sets != 4 || pl.blocks_per_wave > 3) return TTAMD_OK;  // (nothing else is planned)
        *handled = true;
        switch (pl.blocks_per_wave) {
        case 1: return go_sets(conv_wgrad_patch_sets_kernel<1, 4>);
        case 2: return go_sets(conv_wgrad_patch_sets_kernel<2, 4>);
        default: return go_sets(conv_wgrad_patch_sets_kernel<3, 4>);
        }
    }
    auto go = [&](auto kernel) -> ttamd_status {
        TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(pl.lds_bytes)));
        kernel<<<dim3(static_cast<unsigned>(pl.workgroups)), dim3(kThreads), pl.lds_bytes, st>>>(a);
        TTAMD_HIP_CHECK(hipGetLastError());
        return TTAMD_OK;
    };
    *handled = true;
    switch (pl.blocks_per_wave) {
    case 1: return go(conv_wgrad_patch_kernel<1>);
    case 2: return go(conv_wgrad_patch_kernel<2>);
    case 3: return go(conv_wgrad_patch_kernel<3>);
    case 4: return go(conv_wgrad_patch_kernel<4>);
    default: return go(conv_wgrad_patch_kernel<5>);
    }
}

}  // namespace ttamd
