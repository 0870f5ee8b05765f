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
constexpr int kBatchA = 16, kBatchX = 8;  // 16-byte loads per lane and round of the staging: grad_out rows, input rows

// NB: blocks per wave compiled for (the wave's actual count may be lower).
template <int NB>
__global__ void __launch_bounds__(kThreads, 1) conv_wgrad_patch_kernel(ConvWgradPatchArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem_wg[];
    float *const gy = smem_wg;                      // [O][pitch_a]: grad_out rows of the stage
    float *const patch = smem_wg + a.O * a.pitch_a;  // [C][plane]: input rows of the stage, halo columns zero
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int li = lane % 32, kg = lane / 32;
    const int Wo = a.Wo, pitch = a.pitch, plane = a.plane, pitch_a = a.pitch_a;
    const int K = a.C * a.k * a.k;

    // this wave's blocks: output-channel block ob, column blocks first .. first + nb - 1 (column block = tap * C/32 + cb)
    const int ob = wave / a.waves_per_ob;
    const int first = (wave % a.waves_per_ob) * a.blocks_per_wave;
    int nb = a.col_blocks - first;
    nb = nb < 0 ? 0 : (nb > a.blocks_per_wave ? a.blocks_per_wave : nb);
    int block_base[NB];  // float offset in the patch of (channel of this lane, tap) for position 0
    int block_col[NB];   // first result column (c k k + tap) of the block's channel 0 ... see the store
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

    // halo columns of the patch: zero for the whole kernel (the staging below never writes them)
    for (int v = tid; v < a.C * a.R * 2 * a.P; v += kThreads) {
        uint32_t row, sp, side, pc;
        a.d_2P.divmod(static_cast<uint32_t>(v), row, sp);  // row = c * R + r
        a.d_P.divmod(sp, side, pc);
        uint32_t c, r;
        a.d_R.divmod(row, c, r);
        patch[static_cast<int>(c) * plane + static_cast<int>(r) * pitch + (side ? a.P + a.W + static_cast<int>(pc) : static_cast<int>(pc))] = 0.f;
    }

    // the lane's part of an input load: row x_lane_r of the item's row group, vector x_lane_v of that row
    uint32_t xr, xv;
    a.d_vw.divmod(static_cast<uint32_t>(lane), xr, xv);
    const int x_lane_r = static_cast<int>(xr);
    const bool x_lane_ok = x_lane_r < a.rows_per_load;
    const uint32_t x_lane_goff = static_cast<uint32_t>((x_lane_r * a.xs_h + 4 * static_cast<int>(xv)) * 4);
    const int x_lane_lds = x_lane_r * pitch + a.P + 4 * static_cast<int>(xv);
    const int a_vecs = pitch_a / 4;            // 16-byte vectors per staged grad_out row (the tail beyond the stage: zeros)
    const int HoWo = a.Ho * Wo;
    const float *const ap = gy + (ob * 32 + li) * pitch_a + 4 * kg;

    for (int s = blockIdx.x; s < a.n_stages; s += gridDim.x) {
        uint32_t b, si;
        a.d_spi.divmod(static_cast<uint32_t>(s), b, si);
        const int r0 = static_cast<int>(si) * a.RS;
        const int rows = a.Ho - r0 < a.RS ? a.Ho - r0 : a.RS;
        const int np = rows * Wo;  // positions of this stage (a multiple of 4)
        // ---- stage: grad_out rows [O][np] (zeros behind np), input rows r0 - P .. r0 - P + R - 1 of every channel
        {
            // Row-wise: an instruction of a wave loads 64 vectors of one grad_out row, or rows_per_load input rows of
            // one channel; which row or channel is wave-uniform and rides in the load's scalar offset, the lane's part
            // of the address is fixed for the whole kernel.  All loads of a round are issued before its first LDS
            // write, so a round costs one memory latency.
            const float *gbase = a.gout + (static_cast<int64_t>(b) * a.O) * HoWo + static_cast<int64_t>(r0) * Wo;
            const __amdgpu_buffer_rsrc_t gsrc = make_rsrc(gbase, (static_cast<int64_t>(a.O) * HoWo - static_cast<int64_t>(r0) * Wo) * 4);
            const int y0 = r0 - a.P;
            const int64_t first_x = static_cast<int64_t>(b) * a.xs_b + static_cast<int64_t>(y0) * a.xs_h;
            const __amdgpu_buffer_rsrc_t xsrc = make_rsrc(a.x + first_x, a.image_bytes - static_cast<int64_t>(y0) * a.xs_h * 4);
            // grad_out: wave w loads rows w, w + 4, ... (64 vectors of a row per instruction); input: channels w, w + 4,
            // ... (rows_per_load patch rows per instruction).  The usual stage is one round of each.
            const int a_groups = (a_vecs + 63) / 64, x_groups = (a.R + a.rows_per_load - 1) / a.rows_per_load;
            const int a_rounds = (a.O + kWaves * kBatchA - 1) / (kWaves * kBatchA) * a_groups;
            const int x_rounds = (a.C + kWaves * kBatchX - 1) / (kWaves * kBatchX) * x_groups;
            for (int round = 0; round < a_rounds || round < x_rounds; ++round) {
                f32x4 da[kBatchA], dx[kBatchX];
                const int vg = round % a_groups, o0 = wave + (round / a_groups) * (kWaves * kBatchA);
                const int rg = round % x_groups, c0 = wave + (round / x_groups) * (kWaves * kBatchX);
                const int ax = vg * 64 + lane;                              // this lane's vector of a grad_out row
                const int xr = x_lane_r + rg * a.rows_per_load;             // this lane's patch row
                const uint32_t a_voff = round < a_rounds && 4 * ax < np ? static_cast<uint32_t>(ax) * 16u : kOob;
                const bool x_in = round < x_rounds && x_lane_ok && xr < a.R;
                const uint32_t x_voff = x_in && static_cast<unsigned>(y0 + xr) < static_cast<unsigned>(a.H) ? x_lane_goff : kOob;
                const uint32_t x_soff = static_cast<uint32_t>(rg * a.rows_per_load * a.xs_h * 4);
#pragma unroll
                for (int i = 0; i < kBatchA; ++i) {
                    const int o = o0 + i * kWaves;
                    da[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(gsrc, o < a.O ? a_voff : kOob, static_cast<uint32_t>(o) * static_cast<uint32_t>(HoWo) * 4u, 0));
                }
#pragma unroll
                for (int i = 0; i < kBatchX; ++i) {
                    const int c = c0 + i * kWaves;
                    dx[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(xsrc, c < a.C ? x_voff : kOob, x_soff + static_cast<uint32_t>(c * a.xs_c * 4), 0));
                }
                if (round < a_rounds && ax < a_vecs) {  // (vectors behind np: the zeros the loads returned)
                    float *dst = gy + 4 * ax;
#pragma unroll
                    for (int i = 0; i < kBatchA; ++i) {
                        const int o = o0 + i * kWaves;
                        if (o < a.O) *reinterpret_cast<f32x4 *>(dst + o * pitch_a) = da[i];
                    }
                }
                if (x_in) {
                    float *dst = patch + rg * a.rows_per_load * pitch + x_lane_lds;
#pragma unroll
                    for (int i = 0; i < kBatchX; ++i) {
                        const int c = c0 + i * kWaves;
                        if (c < a.C) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) dst[c * plane + e] = dx[i][e];  // (the plane pitch is odd: no 16-byte alignment here)
                        }
                    }
                }
            }
        }
        __syncthreads();

        // ---- multiply: chunks of 8 positions; lane (li, kg) takes positions 8 ch + 4 kg .. + 3 of the chunk
        {
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
                    const float *bp = patch + block_base[i] + o;
#pragma unroll
                    for (int t = 0; t < 4; ++t) fb[i][t] = bp[t];
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
                    for (int t = 0; t < 4; ++t) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[t], fb[i][t], acc[i], 0, 0, 0);
            };
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
        __syncthreads();  // every wave has left the stage's buffers
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

}  // namespace

// Whether (and how) this kernel serves a geometry: decided by the shape alone, so that the workspace query and the
// launch agree.  Rows per stage: as many as LDS holds, then the number of stages per image that gives the 256
// workgroups the shortest busiest one.
ConvWgradPatchPlan plan_conv_wgrad_patch(int B, int C, int H, int W, int O, int k, int S, int P) {
    ConvWgradPatchPlan pl{};
    const int Ho = H + 2 * P - k + 1, Wo = W + 2 * P - k + 1;
    if (S != 1 || B <= 0 || k < 1 || P >= k || C % 32 != 0 || O % 32 != 0 || W % 4 != 0 || W > 256 || Ho < 1 || Wo < 8 || Wo % 4 != 0) return pl;
    const int n_ob = O / 32;
    if (n_ob != 1 && n_ob != 2 && n_ob != 4) return pl;
    const int waves_per_ob = kWaves / n_ob;
    const int col_blocks = k * k * (C / 32);
    const int blocks_per_wave = (col_blocks + waves_per_ob - 1) / waves_per_ob;
    if (blocks_per_wave > kMaxBlocks) return pl;
    const int pitch = W + 2 * P;
    const int64_t K = static_cast<int64_t>(C) * k * k;
    auto lds_floats = [&](int rs) {
        const int64_t pitch_a = 4 * ((((static_cast<int64_t>(rs) * Wo + 7) / 8 * 8) / 4) | 1);  // whole chunks, 4 (2 n + 1) floats
        const int64_t plane = (static_cast<int64_t>(rs + k - 1) * pitch) | 1;
        const int64_t stage = O * pitch_a + C * plane;
        const int64_t tile = O * (K + 4);
        return stage > tile ? stage : tile;
    };
    int rs_max = 0;
    for (int rs = 1; rs <= Ho; ++rs)
        if (lds_floats(rs) * 4 <= kLdsBytes) rs_max = rs;
    if (rs_max < 1 || static_cast<int64_t>(O) * (K + 4) * 4 > kLdsBytes) return pl;
    int best_spi = 0;
    int64_t best_cost = 0;
    for (int spi = (Ho + rs_max - 1) / rs_max; spi <= Ho; ++spi) {
        const int rs = (Ho + spi - 1) / spi;
        const int64_t stages = static_cast<int64_t>(B) * spi;
        const int64_t cost = ((stages + 255) / 256) * (rs * Wo + 64);  // positions of the busiest workgroup, plus a stage's fixed cost
        if (best_spi == 0 || cost < best_cost) best_spi = spi, best_cost = cost;
    }
    pl.RS = (Ho + best_spi - 1) / best_spi;
    pl.SPI = (Ho + pl.RS - 1) / pl.RS;
    const int64_t stages = static_cast<int64_t>(B) * pl.SPI;
    if (stages > 0x7fffffff) return pl;
    pl.n_stages = static_cast<int>(stages);
    pl.workgroups = stages < 256 ? pl.n_stages : 256;
    pl.lds_bytes = static_cast<size_t>(lds_floats(pl.RS)) * 4;
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
    a.n_stages = pl.n_stages;
    a.R = a.RS + k - 1;
    a.pitch = a.W + 2 * a.P;
    a.plane = (a.R * a.pitch) | 1;
    a.pitch_a = 4 * ((((a.RS * a.Wo + 7) / 8 * 8) / 4) | 1);
    a.waves_per_ob = kWaves / (a.O / 32);
    a.col_blocks = k * k * (a.C / 32);
    a.blocks_per_wave = pl.blocks_per_wave;
    a.d_cblocks = make_fastdiv(static_cast<uint32_t>(a.C / 32));
    a.d_k = make_fastdiv(static_cast<uint32_t>(k));
    a.d_2P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? 2 * a.P : 1));
    a.d_P = make_fastdiv(static_cast<uint32_t>(a.P > 0 ? a.P : 1));
    a.d_R = make_fastdiv(static_cast<uint32_t>(a.R));
    a.d_spi = make_fastdiv(static_cast<uint32_t>(a.SPI));
    a.rows_per_load = 64 / (a.W / 4);  // input rows one load instruction of a wave covers
    a.d_vw = make_fastdiv(static_cast<uint32_t>(a.W / 4));
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
