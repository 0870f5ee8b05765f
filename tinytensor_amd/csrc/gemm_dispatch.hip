// gemm_dispatch.hip — ttamd_batched_matmul: argument contract and kernel selection.
// Stands where BackendBase::batched_matmul does (tinytensor/tensor/backend_base.h:130); the
// frontend has already promoted dtypes, rejected bool and lifted 1-D/2-D operands to 3-D
// (tinytensor/tensor/tensor.cpp:2390-2484), so this layer only re-checks what would otherwise
// become an out-of-bounds access on the device.
#include "common.h"

using namespace ttamd;

namespace {

ttamd_status build_args(ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs, const ttamd_view3 *rhs,
                        void *out, const ttamd_epilogue *ep, GemmArgs *g, bool need_pointers) {
    if (dtype == TTAMD_BOOL) {
        set_error("matmul does not support boolean tensors");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    const size_t esz = dtype_size(dtype);
    if (esz == 0 || dtype < TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("matmul: unknown dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (B < 0 || N < 0 || K < 0 || M < 0) {
        set_error("batched_matmul: negative extent (B=%d N=%d K=%d M=%d)", B, N, K, M);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (!lhs || !rhs) {
        set_error("batched_matmul: NULL operand view");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    for (int i = 0; i < 3; ++i) {
        if (lhs->stride[i] < 0 || rhs->stride[i] < 0) {
            set_error("batched_matmul: negative strides are not supported");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
    }
    if (lhs->offset < 0 || rhs->offset < 0) {
        set_error("batched_matmul: negative view offset");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const bool empty_out = B == 0 || N == 0 || M == 0;
    if (need_pointers && !empty_out) {
        if (!out) {
            set_error("batched_matmul: out is NULL");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        if (K > 0 && (!lhs->data || !rhs->data)) {
            set_error("batched_matmul: operand data pointer is NULL");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        if (reinterpret_cast<uintptr_t>(out) % esz != 0 || reinterpret_cast<uintptr_t>(lhs->data) % esz != 0 ||
            reinterpret_cast<uintptr_t>(rhs->data) % esz != 0) {
            set_error("batched_matmul: pointers must be aligned to the element size");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
    }
    if (ep) {
        if (ep->bias_mode < 0 || ep->bias_mode > 2 || (ep->bias_mode != 0 && !ep->bias)) {
            set_error("batched_matmul: invalid epilogue (bias_mode=%d, bias=%p)", ep->bias_mode, ep->bias);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        if ((ep->relu_out && ep->relu) || (ep->colsum_out && ep->accumulate)) {
            set_error("batched_matmul: invalid epilogue (relu_out excludes relu, colsum_out excludes accumulate)");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        if (ep->colsum_out && dtype != TTAMD_F32 && dtype != TTAMD_F64) {
            set_error("batched_matmul: colsum_out is implemented for f32 and f64");
            return TTAMD_ERR_UNSUPPORTED_DTYPE;
        }
        if (ep->rhs_colsum_out) {
            if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
                set_error("batched_matmul: rhs_colsum_out is implemented for f32 and f64");
                return TTAMD_ERR_UNSUPPORTED_DTYPE;
            }
            if (rhs->stride[2] != 1 || rhs->stride[1] != M || (B > 1 && rhs->stride[0] != static_cast<int64_t>(K) * M)) {
                set_error("batched_matmul: rhs_colsum_out needs a dense row-major right operand");
                return TTAMD_ERR_INVALID_ARGUMENT;
            }
        }
        if (reinterpret_cast<uintptr_t>(ep->relu_out) % esz != 0 || reinterpret_cast<uintptr_t>(ep->relu_grad_input) % esz != 0 ||
            reinterpret_cast<uintptr_t>(ep->colsum_out) % esz != 0 || reinterpret_cast<uintptr_t>(ep->rhs_colsum_out) % esz != 0) {
            set_error("batched_matmul: epilogue pointers must be aligned to the element size");
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
    }
    g->A = static_cast<const char *>(lhs->data) + lhs->offset * static_cast<int64_t>(esz);
    g->B = static_cast<const char *>(rhs->data) + rhs->offset * static_cast<int64_t>(esz);
    g->C = out;
    g->a_sb = lhs->stride[0];
    g->a_sm = lhs->stride[1];
    g->a_sk = lhs->stride[2];
    g->b_sb = rhs->stride[0];
    g->b_sk = rhs->stride[1];
    g->b_sn = rhs->stride[2];
    g->M = N;  // kernels use C[M,N] = A[M,K] . B[K,N]
    g->K = K;
    g->N = M;
    g->batch = B;
    g->bias = ep ? ep->bias : nullptr;
    g->bias_mode = ep ? ep->bias_mode : 0;
    g->relu = ep ? ep->relu : 0;
    g->accumulate = ep ? ep->accumulate : 0;
    g->relu_out = ep ? ep->relu_out : nullptr;
    g->zmask = ep ? ep->relu_grad_input : nullptr;
    g->colsum_out = ep ? ep->colsum_out : nullptr;
    g->colsum_partial = nullptr;
    g->colsum_rows = 0;
    g->rhs_colsum = ep ? ep->rhs_colsum_out : nullptr;
    g->rhs_colsum_done = nullptr;
    return TTAMD_OK;
}

ttamd_status run_product(ttamd_dtype dtype, const GemmArgs &g, int device, hipStream_t st, bool fixed_scratch) {
    const char *variant = nullptr;
    bool handled = false;
    if (g.K > 0) {
        if (ttamd_status s = launch_gemm_thin(dtype, g, device, st, &variant, false, &handled, fixed_scratch)) return s;
        if (handled) return TTAMD_OK;
        if (ttamd_status s = launch_gemm_mfma(dtype, g, device, st, &variant, false, &handled, fixed_scratch)) return s;
        if (handled) return TTAMD_OK;
    }
    // K == 0 also lands here: the vector-ALU kernel then stores the empty sum (0, + bias).  It uses no scratch.  The
    // column sums of the result, which that kernel does not form, are taken from the dense result afterwards (its rows
    // added in order).
    if (ttamd_status s = launch_gemm_simt(dtype, g, st, &variant, false)) return s;
    if (g.colsum_out) return launch_colsum_reduce(dtype, g.C, g.M, g.N, g.batch, g.colsum_out, st);
    return TTAMD_OK;
}

ttamd_status batched_matmul(int device, ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs,
                            const ttamd_view3 *rhs, void *out, const ttamd_epilogue *epilogue, void *stream, bool fixed_scratch) {
    GemmArgs g;
    if (ttamd_status s = build_args(dtype, B, N, K, M, lhs, rhs, out, epilogue, &g, true)) return s;
    // build_args has not looked at the data pointers of an empty product; the one such a call still reads (the right
    // operand, for its sums over k) is checked here, before any device work
    if (N == 0 && B > 0 && M > 0 && K > 0 && g.rhs_colsum &&
        (!rhs->data || reinterpret_cast<uintptr_t>(rhs->data) % dtype_size(dtype) != 0)) {
        set_error("batched_matmul: rhs_colsum_out needs the right operand's data (NULL or misaligned pointer)");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (B == 0 || N == 0 || M == 0) {
        // No product.  With batches and columns but no rows (N == 0) the sums over the rows exist all the same: the
        // result's column sums are zeros, the right operand's are what they always are.
        if (B > 0 && M > 0) {
            if (g.colsum_out)
                if (ttamd_status s = launch_colsum_reduce(dtype, nullptr, 0, g.N, g.batch, g.colsum_out, st)) return s;
            if (g.rhs_colsum) return launch_colsum_reduce(dtype, g.B, g.K, g.N, g.batch, g.rhs_colsum, st);
        }
        return TTAMD_OK;
    }
    bool rhs_sums_done = false;
    g.rhs_colsum_done = &rhs_sums_done;
    if (ttamd_status s = run_product(dtype, g, device, st, fixed_scratch)) return s;
    // The right operand's sums over k, unless the product's kernel has written them: its rows added in order.
    if (g.rhs_colsum && !rhs_sums_done) return launch_colsum_reduce(dtype, g.B, g.K, g.N, g.batch, g.rhs_colsum, st);
    return TTAMD_OK;
}

}  // namespace

extern "C" {

ttamd_status ttamd_batched_matmul(int device, ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs,
                                  const ttamd_view3 *rhs, void *out, const ttamd_epilogue *epilogue, void *stream) {
    return batched_matmul(device, dtype, B, N, K, M, lhs, rhs, out, epilogue, stream, false);
}

ttamd_status ttamd_batched_matmul_pair(int device, ttamd_dtype dtype, const ttamd_product *first, const ttamd_product *second,
                                       void *stream) {
    if (!first || !second) {
        set_error("batched_matmul_pair: NULL product");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const ttamd_product *const p[2] = {first, second};
    GemmArgs g[2];
    bool plain = true;  // both products have work on the device and nothing special about them
    for (int i = 0; i < 2; ++i) {
        if (ttamd_status s = build_args(dtype, p[i]->B, p[i]->N, p[i]->K, p[i]->M, p[i]->lhs, p[i]->rhs, p[i]->out, p[i]->epilogue,
                                        &g[i], true))
            return s;
        plain = plain && p[i]->B > 0 && p[i]->N > 0 && p[i]->M > 0 && p[i]->K > 0;
    }
    if (plain) {
        if (ttamd_status s = use_device(device)) return s;
        hipStream_t st = static_cast<hipStream_t>(stream);
        bool handled = false, sums_done = false;
        g[1].rhs_colsum_done = &sums_done;
        if (ttamd_status s = launch_gemm_pair(dtype, g[0], g[1], device, st, &handled)) return s;
        if (handled) {
            // the first product's right-operand sums (the pair's kernel does not form them) and the second's, unless written
            if (g[0].rhs_colsum)
                if (ttamd_status s = launch_colsum_reduce(dtype, g[0].B, g[0].K, g[0].N, g[0].batch, g[0].rhs_colsum, st)) return s;
            if (g[1].rhs_colsum && !sums_done) return launch_colsum_reduce(dtype, g[1].B, g[1].K, g[1].N, g[1].batch, g[1].rhs_colsum, st);
            return TTAMD_OK;
        }
    }
    for (int i = 0; i < 2; ++i)
        if (ttamd_status s = batched_matmul(device, dtype, p[i]->B, p[i]->N, p[i]->K, p[i]->M, p[i]->lhs, p[i]->rhs, p[i]->out,
                                            p[i]->epilogue, stream, false))
            return s;
    return TTAMD_OK;
}

ttamd_status ttamd_batched_matmul_noalloc(int device, ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs,
                                          const ttamd_view3 *rhs, void *out, const ttamd_epilogue *epilogue, void *stream) {
    return batched_matmul(device, dtype, B, N, K, M, lhs, rhs, out, epilogue, stream, true);
}

ttamd_status ttamd_linear_mse_head(int device, ttamd_dtype dtype, int64_t rows, int64_t in_features, int64_t out_features,
                                   const void *input, const void *weight, const void *bias, const void *target,
                                   const void *relu_input, void *output, void *loss_out, void *grad_output_out,
                                   void *grad_input_out, void *grad_weight_out, void *grad_bias_out, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("linear_mse_head: floating point dtypes only");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (rows < 1 || in_features < 1 || out_features < 1 || rows > 0x7fffffffLL || in_features > 0x7fffffffLL ||
        out_features > 64 || rows * in_features > 0x7fffffffLL) {
        set_error("linear_mse_head: rows %lld, in_features %lld, out_features %lld: each at least 1, at most 64 outputs, "
                  "fewer than 2^31 input elements", static_cast<long long>(rows), static_cast<long long>(in_features),
                  static_cast<long long>(out_features));
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (!input || !weight || !target || !output || !loss_out || !grad_output_out || !grad_input_out || !grad_weight_out) {
        set_error("linear_mse_head: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TTAMD_F32) {
        bool handled = false;
        if (ttamd_status s = launch_linear_mse_head(device, rows, in_features, out_features, input, weight, bias, target, relu_input,
                                                    output, loss_out, grad_output_out, grad_input_out, grad_weight_out,
                                                    grad_bias_out, st, &handled))
            return s;
        if (handled) return TTAMD_OK;
    }
    // The same results from the separate calls: y = x . W + b, the loss with dy and db, dx = (dy . W^T) * mask, dW = x^T . dy.
    const int R = static_cast<int>(rows), K = static_cast<int>(in_features), N = static_cast<int>(out_features);
    const ttamd_view3 x{input, 0, {rows * in_features, in_features, 1}}, xt{input, 0, {rows * in_features, 1, in_features}};
    const ttamd_view3 w{weight, 0, {in_features * out_features, out_features, 1}}, wt{weight, 0, {in_features * out_features, 1, out_features}};
    const ttamd_view3 dy{grad_output_out, 0, {rows * out_features, out_features, 1}};
    ttamd_epilogue fwd{};
    fwd.bias = bias;
    fwd.bias_mode = bias ? 1 : 0;
    if (ttamd_status s = batched_matmul(device, dtype, 1, R, K, N, &x, &w, output, &fwd, stream, false)) return s;
    if (ttamd_status s = ttamd_mse_loss(device, dtype, rows, out_features, output, target, loss_out, grad_output_out, grad_bias_out, stream))
        return s;
    ttamd_epilogue back{};
    back.relu_grad_input = relu_input;
    if (ttamd_status s = batched_matmul(device, dtype, 1, R, N, K, &dy, &wt, grad_input_out, &back, stream, false)) return s;
    return batched_matmul(device, dtype, 1, K, R, N, &xt, &dy, grad_weight_out, nullptr, stream, false);
}

const char *ttamd_batched_matmul_variant(ttamd_dtype dtype, int B, int N, int K, int M, const ttamd_view3 *lhs,
                                         const ttamd_view3 *rhs) {
    GemmArgs g;
    if (build_args(dtype, B, N, K, M, lhs, rhs, nullptr, nullptr, &g, false) != TTAMD_OK) return "invalid";
    if (B == 0 || N == 0 || M == 0) return "empty";
    const char *variant = "none";
    bool handled = false;
    if (K > 0) {
        if (launch_gemm_thin(dtype, g, 0, nullptr, &variant, true, &handled) != TTAMD_OK) return "invalid";
        if (handled) return variant;
        if (launch_gemm_mfma(dtype, g, 0, nullptr, &variant, true, &handled) != TTAMD_OK) return "invalid";
        if (handled) return variant;
    }
    if (launch_gemm_simt(dtype, g, nullptr, &variant, true) != TTAMD_OK) return "invalid";
    return variant;
}

}  // extern "C"
