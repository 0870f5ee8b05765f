// common.h — internal declarations shared by the HIP sources of libttamd (gfx950 only).
#ifndef TTAMD_CSRC_COMMON_H_
#define TTAMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ttamd.h"

namespace ttamd {

// Thread-local text for ttamd_last_error_string().
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// Device ids the library's per-device tables are sized for; use_device refuses anything beyond.
constexpr int kMaxDevices = 64;

// Makes `device` current; TTAMD_ERR_INVALID_DEVICE when the id is out of range.
ttamd_status use_device(int device);

inline size_t dtype_size(ttamd_dtype dt) {
    switch (dt) {
    case TTAMD_BOOL:
    case TTAMD_U8: return 1;
    case TTAMD_I16: return 2;
    case TTAMD_I32:
    case TTAMD_F32: return 4;
    case TTAMD_I64:
    case TTAMD_F64: return 8;
    }
    return 0;
}

#define TTAMD_HIP_CHECK(expr)                                                                  \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess) {                                                                \
            ::ttamd::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return TTAMD_ERR_LAUNCH;                                                           \
        }                                                                                      \
    } while (0)

// Exact unsigned division by a runtime-invariant divisor (Granlund & Montgomery): q = x / d for all 32-bit x.
struct FastDiv {
    uint32_t mul, sh1, sh2, d;
    __device__ __forceinline__ uint32_t div(uint32_t x) const {
        const uint32_t t = __umulhi(mul, x);
        return (t + ((x - t) >> sh1)) >> sh2;
    }
    __device__ __forceinline__ void divmod(uint32_t x, uint32_t &q, uint32_t &r) const {
        q = div(x);
        r = x - q * d;
    }
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f{};
    f.d = d;
    uint32_t L = 0;
    while ((1ull << L) < d) ++L;
    f.mul = static_cast<uint32_t>(((1ull << 32) * ((1ull << L) - d)) / d + 1);
    f.sh1 = L < 1 ? L : 1;
    f.sh2 = L > 0 ? L - 1 : 0;
    return f;
}

// Device scratch owned by the library, one growing buffer per (device, stream): kernels enqueued on one stream
// run in order, so consecutive calls on that stream may share it; calls on different streams get different
// buffers.  Growing allocates (hipMalloc, at least double the size); the outgrown buffer is kept until the process
// ends, because kernels in flight and captured graphs may still refer to it.
ttamd_status stream_scratch(int device, hipStream_t stream, size_t bytes, void **out);
// Whole-device synchronisations (ttamd_device_synchronize) of `device`: how many have started, how many have finished.
// A use of shared memory that notes `started` at its launch is known to be over once `completed` exceeds that note.
uint64_t device_sync_started(int device);
uint64_t device_sync_completed(int device);

// One GEMM problem as the kernels see it.  Conventional letters inside the kernels:
// C[M,N] = A[M,K] . B[K,N]  (the C ABI's N,K,M map to M,K,N here).
// Pointers already include the view's element offset.
struct GemmArgs {
    const void *A;
    const void *B;
    void *C;
    int64_t a_sb, a_sm, a_sk;  // element strides of A: batch, row (m), column (k)
    int64_t b_sb, b_sk, b_sn;  // element strides of B: batch, row (k), column (n)
    int M, N, K, batch;
    const void *bias;
    int bias_mode, relu, accumulate;
    // extensions of the store (mfma::EpilogueExt): second output max(value, 0); mask "0 where zmask < 0"; column sums
    void *relu_out;
    const void *zmask;
    void *colsum_out;      // [batch, N], written by the kernel that adds the partial rows
    void *colsum_partial;  // [batch, colsum_rows, N] partial sums, filled in by the launcher (scratch)
    int colsum_rows;
    // [batch, N] = B summed over k (B dense row-major), or null.  A launcher whose kernel writes it sets *rhs_colsum_done
    // (host side only); otherwise the dispatcher adds B's rows in a launch of its own after the product.
    void *rhs_colsum;
    bool *rhs_colsum_done;
};

// Launchers (defined in gemm_mfma.hip / gemm_simt.hip).  `variant_only`: fill *variant with the
// kernel name that would run and return without launching.  `fixed_scratch`: split-k partial tiles go to the
// library's fixed device array instead of the growing per-stream buffer (nothing is allocated; products whose
// partial tiles exceed the array are refused).
ttamd_status launch_gemm_mfma(ttamd_dtype dt, const GemmArgs &g, int device, hipStream_t stream, const char **variant,
                              bool variant_only, bool *handled, bool fixed_scratch = false);
ttamd_status launch_gemm_simt(ttamd_dtype dt, const GemmArgs &g, hipStream_t stream, const char **variant,
                              bool variant_only);
// Two independent products as one grid (gemm_mfma.hip) when both are dense fp32 products of 128 to 256 small tiles in the
// layouts of a product's two gradients; *handled = false: nothing was launched, run them one after the other.
ttamd_status launch_gemm_pair(ttamd_dtype dt, const GemmArgs &g0, const GemmArgs &g1, int device, hipStream_t stream, bool *handled);
// Products of at most 16 columns and a reduction long enough to share out, and products with a reduction of at most
// 16 (gemm_thin.hip): one launch; only the column sums of the second kind may take scratch.
// *handled says whether the product is one of them (nothing is launched otherwise).
ttamd_status launch_gemm_thin(ttamd_dtype dt, const GemmArgs &g, int device, hipStream_t stream, const char **variant,
                              bool variant_only, bool *handled, bool fixed_scratch = false);
// A Linear layer of at most 16 outputs with mse_loss, forward and backward, in two launches (gemm_thin.hip); f32.
ttamd_status launch_linear_mse_head(int device, int64_t rows, int64_t in_features, int64_t out_features, const void *input,
                                    const void *weight, const void *bias, const void *target, const void *relu_input, void *output,
                                    void *loss_out, void *grad_output_out, void *grad_input_out, void *grad_weight_out,
                                    void *grad_bias_out, hipStream_t stream, bool *handled);
// The GEMM launchers' scratch (the stream's growing buffer, or the library's fixed array when `fixed`) and the kernel
// that adds `rows` partial rows of column sums: out[b][n] = sum over r of partial[b][r][n], r ascending.
ttamd_status gemm_scratch(int device, hipStream_t stream, size_t bytes, bool fixed, void **out);
ttamd_status launch_colsum_reduce(ttamd_dtype dt, const void *partial, int rows, int N, int batch, void *out, hipStream_t stream);

// Stride-1 fp32 convolution served by conv_patch.hip (weights resident in LDS, input rows staged once per tile).
// The caller fills the first block; launch_conv_patch_f32 derives the rest and reports through *handled whether the
// geometry fits (otherwise nothing was launched and the caller takes its general kernels).
struct ConvPatchArgs {
    const float *x;        // input [B,C,H,W]: column stride 1, the other strides below (elements)
    const float *w;        // weight: tap t of (row, reduction channel) at element row * w_row + red * w_red + t
    const float *bias;     // [O] or null
    float *out;            // dense [B,O,Ho,Wo]
    int B, C, H, W, O, k, P, Ho, Wo;  // C: reduction channels (the input's), O: rows of the result
    int64_t xs_b;
    int32_t xs_c, xs_h;
    int64_t w_row, w_red;
    int w_flip;            // taps used in reverse order (gradient with respect to the input)
    int w_rows_fast;       // lanes of the weight loader run along the rows (the axis whose stride is k*k) instead of the channels
    int64_t image_bytes, weight_bytes;  // bytes reachable from an image's / the weight's first element
    // Optional second job of the launch: red_out[i] = sum over s < red_splits of red_partial[s * red_n + i], carried out by
    // workgroups appended to the grid (a sum that some earlier launch on the stream left in parts, e.g. grad_weight's partial
    // tiles, spared a launch of its own).  red_n a multiple of 4, both pointers 16-byte aligned, red_splits * red_n * 4 < 2^31;
    // red_splits == 0: none.
    const float *red_partial;
    float *red_out;
    int red_n, red_splits;
    // a second such sum (grad_bias's parts), same conditions
    const float *red2_partial;
    float *red2_out;
    int red2_n, red2_splits;
    // derived: appended workgroups in all, those of them for the second sum
    int red_blocks, red2_blocks;
    int K, lda, cpad, R, pitch, vecs_per_row, xh, last_vecs, n_items, stage_slots, cl_shift, tiles_m, tiles_n;
    int n_seg, seg_len, segs_per_pass, n_fast, n_wvec, w_dense, w_pass_vecs, n_buf;
    int bne, tail;  // positions per tile; those of them behind the tile's whole 32-position blocks (twelve waves: 4 or 8)
    FastDiv d_wfast, d_segv, d_k, d_ngrp, d_xh, d_R, d_cpad4, d_2P, d_P, d_Wo, d_tiles_n, d_tail;
};
ttamd_status launch_conv_patch_f32(ConvPatchArgs a, hipStream_t stream, int *variant, bool launch = true);

// grad_weight with both operands staged in LDS (conv_wgrad_patch.hip).  The plan depends on the shape alone.
struct ConvWgradPatchPlan {
    bool use;
    int RS, SPI;          // output rows per unit, units per image
    int RSS, n_sub;       // a unit is cut into n_sub stages of RSS rows
    int n_units;          // B * SPI
    int workgroups;       // = partial tiles written
    int blocks_per_wave;
    int sets;             // 0: four waves with every block of output channels; 2 or 4: sets of four waves that share out the
                          // positions, one block of 32 output channels per workgroup (workgroups = partial tiles x O / 32)
    int a_instr, x_instr; // sets: load instructions per grad_out row / per input channel of a stage
    size_t lds_bytes;
};
ConvWgradPatchPlan plan_conv_wgrad_patch(int B, int C, int H, int W, int O, int k, int S, int P);
struct ConvWgradPatchArgs {
    const float *gout;     // dense [B,O,Ho,Wo]
    const float *x;        // input [B,C,H,W]: column stride 1, the other strides below (elements)
    float *partial;        // [workgroups][O][C k k]
    int B, C, H, W, O, k, P, Ho, Wo;
    int64_t xs_b;
    int32_t xs_c, xs_h;
    int64_t image_bytes;   // bytes reachable from an image's first element
    // derived
    int RS, SPI, RSS, n_sub, n_units, R, pitch, plane, pitch_a, waves_per_ob, col_blocks, blocks_per_wave, a_instr, x_instr;
    FastDiv d_cblocks, d_k, d_2P, d_P, d_R, d_C, d_spi, d_vw, d_Wo, d_kvecs;
};
ttamd_status launch_conv_wgrad_patch_f32(ConvWgradPatchArgs a, const ConvWgradPatchPlan &plan, hipStream_t stream, bool *handled);

}  // namespace ttamd

#endif  // TTAMD_CSRC_COMMON_H_
