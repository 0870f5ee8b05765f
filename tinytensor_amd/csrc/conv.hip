// conv.hip — conv2d forward / backward as implicit GEMM on the matrix cores (gfx950).
//
// Stands where BackendBase::conv2d / conv2d_backward do (tinytensor/tensor/backend_base.h:269-284).  The
// reference lowers each image to an explicit im2col matrix and runs one small GEMM per image
// (tinytensor/tensor/backend/cpu/conv.cpp:108-128, 208-272; index maps cpu/kernel/conv.hpp:12-118).
// Here the same three products run as batched GEMMs whose "column matrix" operand is never
// materialised: a gather stager computes the im2col address of every element it fetches and lets the
// buffer load return zero for padding.  With kk = (c, p, q) and n = (h, w):
//
//   forward      out[b][o][n]  = sum_kk  W[o][kk]      * x[b][c][S h + p - P][S w + q - P]     (+ bias[o])
//   grad_weight  gW[o][kk]     = sum_b sum_n g[b][o][n] * x[b][c][S h + p - P][S w + q - P]
//   grad_input   gX[b][c][y][x] = sum_(o,p,q) W[o][c][p][q] * g[b][o][(y+P-p)/S][(x+P-q)/S]   (when divisible, in range)
//
// grad_input is the gather form of the reference's col2im scatter-add (conv.hpp:83-118): every output
// element is owned by one lane, so there is no write race and the result is deterministic.  With a stride it runs as
// S*S dense unit-stride problems, one per class of input positions (DgradClass); with at most four input channels on
// the vector ALU (conv_dgrad_slots_kernel).
// grad_weight reduces over the batch (conv.cpp:239-244): one workgroup column per (group of images, slice of
// output positions) accumulates in registers, partial tiles go to the caller's workspace and are summed in a
// fixed order.  Integer dtypes (forward only; autograd never differentiates them) use a direct
// vector-ALU kernel with wrap-around arithmetic.
#include <cstdlib>
#include <type_traits>

#include "mfma_core.h"

namespace ttamd {
namespace {

using namespace mfma;

struct ConvGeom {
    int B, C, H, W, O, k, S, P, Ho, Wo;
    // grad_input's gather alone reads these: the kernel extent and the padding per axis.  They equal (k, k, P, P)
    // except in the dense sub-problems that a strided grad_input is split into (rectangular kernels, a padding per
    // axis); d_kk and d_k then divide by kh * kw and kw.
    int kh, kw, Ph, Pw;
    int64_t xs_b;              // input batch stride (elements)
    int32_t xs_c, xs_h, xs_w;  // input channel / row / column strides (elements)
    int64_t w_so;              // weight stride of the output channel; (c,p,q) are dense behind it
    FastDiv d_kk, d_k, d_Wo, d_W, d_S;
    // Not 0: the vector-gather kernels of forward and grad_input number their positions over rows of this many
    // columns, the row width (Wo, or W for grad_input) rounded up to whole 16-byte vectors, so that a vector never
    // crosses a row although the width is no multiple of it; the columns past the row are computed and dropped.
    int row_pad;
    FastDiv d_row_pad;
    // Not 0: this is one class of a strided grad_input (a unit-stride sub-problem over every sc_S-th row and column):
    // position (i, j) of its H x W positions is element (sc_y0 + sc_S * i, sc_x0 + sc_S * j) of a plane of
    // sc_H x sc_W elements, and the kernel writes it there instead of into a dense result of its own.
    int sc_S, sc_y0, sc_x0, sc_H, sc_W;
};

// ---------------------------------------------------------------------------------------------
// B operand of the forward product: Xu[kk][n] gathered from image b.  MC layout (n contiguous), one
// element per load.  A lane keeps one output position n for the whole kernel; the kk of a pass is
// wave-uniform, so its (c, p, q) decode runs on the scalar unit.
template <typename T, int ROWS, int BK, int PF = 1>
struct Im2colStager : TileLayout<T, ROWS, BK, false> {
    using L = TileLayout<T, ROWS, BK, false>;
    static constexpr int LPP = kThreads / ROWS;  // k lines per pass
    static constexpr int P = BK / LPP;
    static_assert(ROWS % 64 == 0 && BK % LPP == 0, "a wave must share its k line");
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = false;
    T reg[PF][P];
    __amdgpu_buffer_rsrc_t rsrc;
    const ConvGeom *g;
    int n_local, line0, k_next, K;
    int ih0, iw0;       // input coordinates of tap (0,0) for this lane's output position
    int32_t base_b;     // byte offset of (ih0, iw0) inside the image (may be negative under padding)
    bool n_ok;

    __device__ __forceinline__ explicit Im2colStager(const ConvGeom &geo_) : g(&geo_) {}

    __device__ __forceinline__ void init(const T *image, int64_t image_bytes, int tid, int n0) {
        const ConvGeom &geo = *g;
        rsrc = make_rsrc(image, image_bytes);
        n_local = tid % ROWS;
        line0 = __builtin_amdgcn_readfirstlane(tid / ROWS);
        k_next = 0;
        K = geo.C * geo.k * geo.k;
        const int n = n0 + n_local;
        n_ok = n < geo.Ho * geo.Wo;
        uint32_t h, w;
        geo.d_Wo.divmod(static_cast<uint32_t>(n_ok ? n : 0), h, w);
        ih0 = geo.S * static_cast<int>(h) - geo.P;
        iw0 = geo.S * static_cast<int>(w) - geo.P;
        base_b = (ih0 * geo.xs_h + iw0 * geo.xs_w) * static_cast<int32_t>(sizeof(T));
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int /*k_left*/) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int kk = k_next + p * LPP + line0;  // wave-uniform
            uint32_t c, r, pp, q;
            g->d_kk.divmod(static_cast<uint32_t>(kk), c, r);
            g->d_k.divmod(r, pp, q);
            const int32_t koff = (static_cast<int32_t>(c) * g->xs_c + static_cast<int32_t>(pp) * g->xs_h +
                                  static_cast<int32_t>(q) * g->xs_w) * static_cast<int32_t>(sizeof(T));
            const int ih = ih0 + static_cast<int>(pp), iw = iw0 + static_cast<int>(q);
            const bool ok = n_ok && kk < K && static_cast<unsigned>(ih) < static_cast<unsigned>(g->H) &&
                            static_cast<unsigned>(iw) < static_cast<unsigned>(g->W);
            reg[SLOT][p] = Vec<T, 1>::load(rsrc, ok ? static_cast<uint32_t>(base_b + koff) : kOob);
        }
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p) lds[(p * LPP + line0) * L::LD + n_local] = reg[SLOT][p];
    }
};

// ---------------------------------------------------------------------------------------------
// B operand of grad_weight: XuT[n][j] with n = output position (the reduction index) and j = (c,p,q)
// (the column index).  KC layout (n contiguous), one element per load.  The j of each pass is fixed for
// the whole kernel and decoded once; the n of a lane advances by BK per tile.
template <typename T, int ROWS, int BK, int PF = 1>
struct Im2colTStager : TileLayout<T, ROWS, BK, true> {
    using L = TileLayout<T, ROWS, BK, true>;
    static constexpr int RPP = kThreads / BK;  // j rows per pass
    static constexpr int P = ROWS / RPP;
    static_assert(ROWS % RPP == 0, "tile must split evenly");
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = false;
    T reg[PF][P];
    __amdgpu_buffer_rsrc_t rsrc;
    const ConvGeom *g;
    int32_t joff[P];  // byte offset of tap (c, p - P, q - P)
    int16_t dp[P], dq[P];
    bool j_ok[P];
    int k_local, row0, k_next, HoWo;

    __device__ __forceinline__ explicit Im2colTStager(const ConvGeom &geo_) : g(&geo_) {}

    __device__ __forceinline__ void init(int tid, int j0) {
        const ConvGeom &geo = *g;
        k_local = tid % BK;
        row0 = tid / BK;
        HoWo = geo.Ho * geo.Wo;
        const int J = geo.C * geo.k * geo.k;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int j = j0 + p * RPP + row0;
            j_ok[p] = j < J;
            uint32_t c, r, pp, q;
            geo.d_kk.divmod(static_cast<uint32_t>(j_ok[p] ? j : 0), c, r);
            geo.d_k.divmod(r, pp, q);
            dp[p] = static_cast<int16_t>(static_cast<int>(pp) - geo.P);
            dq[p] = static_cast<int16_t>(static_cast<int>(q) - geo.P);
            joff[p] = (static_cast<int32_t>(c) * geo.xs_c + dp[p] * geo.xs_h + dq[p] * geo.xs_w) *
                      static_cast<int32_t>(sizeof(T));
        }
    }

    // Points the stager at image `image` and restarts the reduction index at k0.
    __device__ __forceinline__ void set_image(const T *image, int64_t image_bytes, int k0) {
        rsrc = make_rsrc(image, image_bytes);
        k_next = k0;
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int /*k_left*/) {
        const int n = k_next + k_local;
        const bool n_ok = n < HoWo;
        uint32_t h, w;
        g->d_Wo.divmod(static_cast<uint32_t>(n_ok ? n : 0), h, w);
        const int ih0 = g->S * static_cast<int>(h), iw0 = g->S * static_cast<int>(w);
        const int32_t base_b = (ih0 * g->xs_h + iw0 * g->xs_w) * static_cast<int32_t>(sizeof(T));
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int ih = ih0 + dp[p], iw = iw0 + dq[p];
            const bool ok = n_ok && j_ok[p] && static_cast<unsigned>(ih) < static_cast<unsigned>(g->H) &&
                            static_cast<unsigned>(iw) < static_cast<unsigned>(g->W);
            reg[SLOT][p] = Vec<T, 1>::load(rsrc, ok ? static_cast<uint32_t>(base_b + joff[p]) : kOob);
        }
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p) lds[(p * RPP + row0) * L::LD + k_local] = reg[SLOT][p];
    }
};

// ---------------------------------------------------------------------------------------------
// B operand of grad_input: G[kk][n] = g[b][o][(y+P-p)/S][(x+P-q)/S], kk = (o,p,q), n = (y,x).  MC layout;
// the lane's input position is fixed, kk is wave-uniform per pass.
template <typename T, int ROWS, int BK, int PF = 1>
struct DgradStager : TileLayout<T, ROWS, BK, false> {
    using L = TileLayout<T, ROWS, BK, false>;
    static constexpr int LPP = kThreads / ROWS;
    static constexpr int P = BK / LPP;
    static_assert(ROWS % 64 == 0 && BK % LPP == 0, "a wave must share its k line");
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = false;
    T reg[PF][P];
    __amdgpu_buffer_rsrc_t rsrc;
    const ConvGeom *g;
    int n_local, line0, k_next, K, HoWo;
    int yP, xP;  // y + P, x + P for this lane's input position
    bool n_ok;

    __device__ __forceinline__ explicit DgradStager(const ConvGeom &geo_) : g(&geo_) {}

    __device__ __forceinline__ void init(const T *gout_image, int64_t bytes, int tid, int n0) {
        const ConvGeom &geo = *g;
        rsrc = make_rsrc(gout_image, bytes);
        n_local = tid % ROWS;
        line0 = __builtin_amdgcn_readfirstlane(tid / ROWS);
        k_next = 0;
        HoWo = geo.Ho * geo.Wo;
        K = geo.O * geo.kh * geo.kw;
        const int n = n0 + n_local;
        n_ok = n < geo.H * geo.W;
        uint32_t y, x;
        geo.d_W.divmod(static_cast<uint32_t>(n_ok ? n : 0), y, x);
        yP = static_cast<int>(y) + geo.Ph;
        xP = static_cast<int>(x) + geo.Pw;
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int /*k_left*/) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int kk = k_next + p * LPP + line0;  // wave-uniform
            uint32_t o, r, pp, q;
            g->d_kk.divmod(static_cast<uint32_t>(kk), o, r);
            g->d_k.divmod(r, pp, q);
            const int ty = yP - static_cast<int>(pp), tx = xP - static_cast<int>(q);
            bool ok = n_ok && kk < K && ty >= 0 && tx >= 0;
            uint32_t oh, rh, ow, rw;
            g->d_S.divmod(static_cast<uint32_t>(ok ? ty : 0), oh, rh);
            g->d_S.divmod(static_cast<uint32_t>(ok ? tx : 0), ow, rw);
            ok = ok && rh == 0 && rw == 0 && static_cast<int>(oh) < g->Ho && static_cast<int>(ow) < g->Wo;
            const uint32_t off = (o * static_cast<uint32_t>(HoWo) + oh * static_cast<uint32_t>(g->Wo) + ow) *
                                 static_cast<uint32_t>(sizeof(T));
            reg[SLOT][p] = Vec<T, 1>::load(rsrc, ok ? off : kOob);
        }
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p) lds[(p * LPP + line0) * L::LD + n_local] = reg[SLOT][p];
    }
};

// ---------------------------------------------------------------------------------------------
// Vector gathers for unit stride.  With S = 1 and a unit column stride, VEC consecutive positions of one
// plane row read VEC consecutive source elements src[ch][py + dy][px0 + dx .. + VEC - 1], so one 16-byte
// buffer load (any 4-byte alignment) fetches them; components that fall left or right of the row are
// cleared afterwards (the load itself stays inside the image: the descriptor checks its range per dword,
// and a vector that would begin before the image's first element is fetched element by element instead).
//
//   FLIP = false: taps (c, a, b) of the input image, positions = output pixels, dy = a - P  (forward, grad_weight)
//   FLIP = true:  taps (o, a, b) of grad_out,        positions = input pixels,  dy = P - a  (grad_input)
template <bool FLIP>
struct TapView {
    int taps, positions, src_h, src_w, k, pad, pad_h, pad_w;
    int pos_w;  // positions per row that exist (the row may be numbered over more columns, ConvGeom::row_pad)
    int32_t s_ch, s_h;
    FastDiv d_kk, d_k, d_pw;
    __device__ __forceinline__ explicit TapView(const ConvGeom &g) {
        k = g.k;
        pad = g.P;
        d_kk = g.d_kk;
        d_k = g.d_k;
        pad_h = FLIP ? g.Ph : g.P;
        pad_w = FLIP ? g.Pw : g.P;
        pos_w = FLIP ? g.W : g.Wo;
        if constexpr (FLIP) {
            taps = g.O * g.kh * g.kw;
            positions = g.H * (g.row_pad ? g.row_pad : g.W);
            src_h = g.Ho;
            src_w = g.Wo;
            s_ch = g.Ho * g.Wo;
            s_h = g.Wo;
            d_pw = g.row_pad ? g.d_row_pad : g.d_W;
        } else {
            taps = g.C * g.k * g.k;
            positions = g.Ho * (g.row_pad ? g.row_pad : g.Wo);
            src_h = g.H;
            src_w = g.W;
            s_ch = g.xs_c;
            s_h = g.xs_h;
            d_pw = g.row_pad ? g.d_row_pad : g.d_Wo;
        }
    }
    // (channel offset, dy, dx) of tap index t
    __device__ __forceinline__ void tap(uint32_t t, int32_t &ch_off, int &dy, int &dx) const {
        uint32_t ch, r, a, b;
        d_kk.divmod(t, ch, r);
        d_k.divmod(r, a, b);
        ch_off = static_cast<int32_t>(ch) * s_ch;
        dy = FLIP ? pad_h - static_cast<int>(a) : static_cast<int>(a) - pad_h;
        dx = FLIP ? pad_w - static_cast<int>(b) : static_cast<int>(b) - pad_w;
    }
};

// One gathered vector: elements e0 .. e0 + VEC - 1 of the image.  The components outside the row are NOT cleared
// here: touching the loaded registers would make the wave wait for the data before its MFMA work; the stagers
// keep the first column x0 and clear them in store(), just before the LDS write (clear_outside_row).
template <typename T, int VEC>
__device__ __forceinline__ typename Vec<T, VEC>::type gather_row_vector(__amdgpu_buffer_rsrc_t rsrc, bool row_ok, int32_t e0) {
    using V = typename Vec<T, VEC>::type;
    constexpr int32_t SZ = static_cast<int32_t>(sizeof(T));
    V v = Vec<T, VEC>::load(rsrc, (row_ok && e0 >= 0) ? static_cast<uint32_t>(e0 * SZ) : kOob);
    if (row_ok && e0 < 0) {  // top-left corner of the first plane under padding
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = Vec<T, 1>::load(rsrc, e0 + j >= 0 ? static_cast<uint32_t>((e0 + j) * SZ) : kOob);
    }
    return v;
}

// Columns x0 .. x0 + VEC - 1 of a row of width src_w: components outside the row become 0.
template <typename T, int VEC>
__device__ __forceinline__ typename Vec<T, VEC>::type clear_outside_row(typename Vec<T, VEC>::type v, int x0, int src_w) {
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        if (static_cast<unsigned>(x0 + j) >= static_cast<unsigned>(src_w)) v[j] = T(0);
    return v;
}

// The VEC positions of a lane at stride STRIDE: source columns x0, x0 + STRIDE, ...  They lie inside STRIDE consecutive
// vectors that start at x0 (gathered as they are, at any 4-byte alignment); this picks them out and clears the ones
// outside the row.  STRIDE = 1 is clear_outside_row.
template <typename T, int VEC, int STRIDE>
__device__ __forceinline__ typename Vec<T, VEC>::type pick_strided(const typename Vec<T, VEC>::type *v, int x0, int src_w) {
    if constexpr (STRIDE == 1) {
        return clear_outside_row<T, VEC>(v[0], x0, src_w);
    } else {
        typename Vec<T, VEC>::type out;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const T e = v[(j * STRIDE) / VEC][(j * STRIDE) % VEC];
            out[j] = static_cast<unsigned>(x0 + j * STRIDE) >= static_cast<unsigned>(src_w) ? T(0) : e;
        }
        return out;
    }
}

constexpr int kTapTableEntries = 128;  // window taps (k * k) served by a stager's (dy, dx) table; behind the tile buffers in LDS
constexpr size_t kTapTableBytes = kTapTableEntries * sizeof(int2);

// MC layout (positions contiguous in LDS), vectors along the positions: B operand of forward and of
// grad_input.  Requires positions-per-row % VEC == 0 so that a vector never crosses a plane row.
// STRIDE (forward only): the convolution's stride.  Position (py, px) then reads source element
// (STRIDE * py + dy, STRIDE * px + dx), and a lane's VEC positions come out of STRIDE gathered vectors (pick_strided).
template <typename T, int ROWS, int BK, int VEC, bool FLIP, int PF = 1, int STRIDE = 1>
struct TapStagerMC : TileLayout<T, ROWS, BK, false> {
    using L = TileLayout<T, ROWS, BK, false>;
    using V = typename Vec<T, VEC>::type;
    static constexpr int VPL = ROWS / VEC;       // vectors per k line
    static constexpr int LPP = kThreads / VPL;   // k lines per pass
    static constexpr int P = BK / LPP;
    static_assert(VEC > 1 && ROWS % VEC == 0 && kThreads % VPL == 0 && BK % LPP == 0, "tile must split evenly");
    static_assert(STRIDE == 1 || !FLIP, "the strided gather serves the forward product");
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = true;
    V reg[PF][P][STRIDE];
    int col0[PF][P];  // first source column of each gathered vector
    __amdgpu_buffer_rsrc_t rsrc;
    TapView<FLIP> tv;
    int n_local, line0, k_next;
    int py, px0;
    bool n_ok;
    // The reduction index of pass p, kept as (index, channel offset, tap within the window) and advanced by BK per
    // load -- a k tile on is BK / (window taps) channels and BK % (window taps) taps on, with at most one carry --
    // instead of two divisions per load; the tap's (dy, dx) comes from a table in LDS with one entry per window tap.
    int kk_p[P], r_p[P];
    int32_t ch_p[P];
    const int2 *tab;

    __device__ __forceinline__ explicit TapStagerMC(const ConvGeom &geo) : tv(geo), tab(nullptr) {}

    // The window's taps as (dy, dx), written by the first lanes of the workgroup (a barrier must follow before the first
    // load).  The host sends windows of more than kTapTableEntries taps to the element-wise stagers.
    __device__ __forceinline__ void fill_tap_table(int2 *table, int tid) {
        const int window = static_cast<int>(tv.d_kk.d);
        tab = table;
        if (tid < window && tid < kTapTableEntries) {
            int32_t ch_off;
            int dy, dx;
            tv.tap(static_cast<uint32_t>(tid), ch_off, dy, dx);
            table[tid] = int2{dy, dx};
        }
    }

    __device__ __forceinline__ void init(const T *image, int64_t image_bytes, int tid, int n0) {
        rsrc = make_rsrc(image, image_bytes);
        n_local = (tid % VPL) * VEC;
        line0 = tid / VPL;
        k_next = 0;
        const int n = n0 + n_local;
        n_ok = n < tv.positions;
        uint32_t y, x;
        tv.d_pw.divmod(static_cast<uint32_t>(n_ok ? n : 0), y, x);
        py = static_cast<int>(y);
        px0 = static_cast<int>(x);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            kk_p[p] = p * LPP + line0;
            uint32_t ch, r;
            tv.d_kk.divmod(static_cast<uint32_t>(kk_p[p]), ch, r);
            ch_p[p] = static_cast<int32_t>(ch) * tv.s_ch;
            r_p[p] = static_cast<int>(r);
        }
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int /*k_left*/) {
        const int window = static_cast<int>(tv.d_kk.d);
        const int step_r = BK % window;                                    // (wave-uniform: scalar arithmetic)
        const int32_t step_ch = static_cast<int32_t>(BK / window) * tv.s_ch;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int kk = kk_p[p];
            const bool k_ok = kk < tv.taps;
            const int2 t = tab[r_p[p]];
            const int32_t ch_off = ch_p[p];
            const int dy = t.x, dx = t.y;
            kk_p[p] = kk + BK;
            const int r = r_p[p] + step_r;
            const bool carry = r >= window;
            r_p[p] = carry ? r - window : r;
            ch_p[p] += carry ? step_ch + tv.s_ch : step_ch;
            const int y = STRIDE * py + dy, x0 = STRIDE * px0 + dx;
            const bool row_ok = n_ok && k_ok && static_cast<unsigned>(y) < static_cast<unsigned>(tv.src_h);
            const int32_t e0 = ch_off + y * tv.s_h + x0;
#pragma unroll
            for (int v = 0; v < STRIDE; ++v) reg[SLOT][p][v] = gather_row_vector<T, VEC>(rsrc, row_ok, e0 + v * VEC);
            col0[SLOT][p] = x0;
        }
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p)
            *reinterpret_cast<V *>(&lds[(p * LPP + line0) * L::LD + n_local]) = pick_strided<T, VEC, STRIDE>(reg[SLOT][p], col0[SLOT][p], tv.src_w);
    }
};

// KC layout (reduction index contiguous in LDS), vectors along the positions, which are the reduction
// index here: B operand of grad_weight.  The tap of each pass is fixed for the whole kernel.
// PADDED: the positions are numbered over padded rows; the vectors' components in the padding columns are cleared
// too (grad_out's stager clears its own), so that no value of either operand, finite or not, enters the sum there.
template <typename T, int ROWS, int BK, int VEC, int PF = 1, bool PADDED = false>
struct TapStagerKC : TileLayout<T, ROWS, BK, true> {
    using L = TileLayout<T, ROWS, BK, true>;
    using V = typename Vec<T, VEC>::type;
    static constexpr int VPL = BK / VEC;
    static constexpr int RPP = kThreads / VPL;  // tap rows per pass
    static constexpr int P = ROWS / RPP;
    static_assert(VEC > 1 && BK % VEC == 0 && kThreads % VPL == 0 && ROWS % RPP == 0, "tile must split evenly");
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = false;
    V reg[PF][P];
    int col0[PF];  // source column of the lane's first position, before the tap's dx
    __amdgpu_buffer_rsrc_t rsrc;
    TapView<false> tv;
    int32_t joff[P];
    int16_t dy[P], dx[P];
    bool j_ok[P];
    int k_local, row0, k_next;
    // PADDED only: several images in one reduction.  Every image takes joint_k positions (its own, rounded up to whole
    // k tiles; 0: one image per run), image_step elements apart; image_base is the current image's element offset.
    int joint_k, image_step, image_base;

    __device__ __forceinline__ explicit TapStagerKC(const ConvGeom &geo) : tv(geo) {}

    __device__ __forceinline__ void init(int tid, int j0) {
        k_local = (tid % VPL) * VEC;
        row0 = tid / VPL;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int j = j0 + p * RPP + row0;
            j_ok[p] = j < tv.taps;
            int32_t ch_off;
            int ddy, ddx;
            tv.tap(static_cast<uint32_t>(j_ok[p] ? j : 0), ch_off, ddy, ddx);
            dy[p] = static_cast<int16_t>(ddy);
            dx[p] = static_cast<int16_t>(ddx);
            joff[p] = ch_off + ddy * tv.s_h + ddx;
        }
    }

    __device__ __forceinline__ void set_image(const T *image, int64_t image_bytes, int k0) {
        rsrc = make_rsrc(image, image_bytes);
        k_next = k0;
        joint_k = 0;
        image_step = 0;
        image_base = 0;
    }

    // The images from `first` on as one reduction: span_bytes covers them all, `step` elements from one to the next.
    __device__ __forceinline__ void set_images(const T *first, int64_t span_bytes, int positions_per_image, int32_t step) {
        rsrc = make_rsrc(first, span_bytes);
        k_next = 0;
        joint_k = positions_per_image;
        image_step = step;
        image_base = 0;
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int /*k_left*/) {
        if constexpr (PADDED) {
            if (joint_k && k_next >= joint_k) {  // uniform: the next image starts with this tile
                k_next -= joint_k;
                image_base += image_step;
            }
        }
        const int n = k_next + k_local;
        const bool n_ok = n < tv.positions;
        uint32_t y, x;
        tv.d_pw.divmod(static_cast<uint32_t>(n_ok ? n : 0), y, x);
        const int py = static_cast<int>(y), px0 = static_cast<int>(x);
        const int32_t base = (PADDED ? image_base : 0) + py * tv.s_h + px0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int yy = py + dy[p];
            const bool row_ok = n_ok && j_ok[p] && static_cast<unsigned>(yy) < static_cast<unsigned>(tv.src_h);
            reg[SLOT][p] = gather_row_vector<T, VEC>(rsrc, row_ok, base + joff[p]);
        }
        col0[SLOT] = px0;
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            V v = clear_outside_row<T, VEC>(reg[SLOT][p], col0[SLOT] + dx[p], tv.src_w);
            if constexpr (PADDED) v = clear_outside_row<T, VEC>(v, col0[SLOT], tv.pos_w);
            *reinterpret_cast<V *>(&lds[(p * RPP + row0) * L::LD + k_local]) = v;
        }
    }
};

// A operand of grad_weight when the positions, its reduction index, are numbered over padded rows
// (ConvGeom::row_pad): row m is channel m0 + m of one image of grad_out [O][Ho * Wo], k = y * row_pad + x.  One vector
// load fetches columns x .. x + VEC - 1 of row y at any 4-byte alignment; the components in the padding columns
// (x >= Wo), which hold the next row's first elements, are cleared in store(), so that the gathered input values of
// those columns never reach the sum.  KC layout, same LDS image as Stager<T, ROWS, BK, true, VEC>.
template <typename T, int ROWS, int BK, int PF>
struct PaddedRowsStager : TileLayout<T, ROWS, BK, true> {
    using L = TileLayout<T, ROWS, BK, true>;
    static constexpr int VEC = Mfma<T>::VK;
    using V = typename Vec<T, VEC>::type;
    static constexpr int kPF = PF;
    static constexpr bool kTapTable = false;
    static constexpr int VPL = BK / VEC;
    static constexpr int RPP = kThreads / VPL;  // rows per pass
    static constexpr int P = ROWS / RPP;
    static_assert(BK % VEC == 0 && kThreads % VPL == 0 && ROWS % RPP == 0, "tile must split evenly");
    V reg[PF][P];
    int col0[PF];  // column x of the lane's vector in each slot
    uint32_t row_off[P];
    __amdgpu_buffer_rsrc_t rsrc;
    FastDiv d_row;
    int w, positions, k_local, row0, k_next;
    int joint_k;                     // several images in one reduction: positions per image (whole k tiles), or 0
    uint32_t image_step_b, image_b;  // bytes from one image to the next, byte offset of the current image

    // base: channel m0 of the (first) image; k0: first (padded) position of this workgroup's slice.  images > 1 with
    // positions_per_image (a multiple of BK) runs through that many images in one reduction.
    __device__ __forceinline__ void init(const T *base, int tid, int rows_left, const ConvGeom &geo, int k0, int images = 1,
                                         int positions_per_image = 0) {
        const int plane = geo.Ho * geo.Wo;
        const int rows = rows_left < ROWS ? rows_left : ROWS;
        const int64_t image_elems = static_cast<int64_t>(geo.O) * plane;
        rsrc = make_rsrc(base, ((images - 1) * image_elems + static_cast<int64_t>(rows) * plane) * static_cast<int64_t>(sizeof(T)));
        joint_k = positions_per_image;
        image_step_b = static_cast<uint32_t>(image_elems * static_cast<int64_t>(sizeof(T)));
        image_b = 0;
        d_row = geo.d_row_pad;
        w = geo.Wo;
        positions = geo.Ho * geo.row_pad;
        k_local = (tid % VPL) * VEC;
        row0 = tid / VPL;
        k_next = k0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int r = p * RPP + row0;
            row_off[p] = r < rows ? static_cast<uint32_t>(r * plane) * static_cast<uint32_t>(sizeof(T)) : kOob;
        }
    }

    template <bool MASK, int SLOT = 0>
    __device__ __forceinline__ void load(int k_left) {
        if (joint_k && k_next >= joint_k) {  // uniform: the next image starts with this tile
            k_next -= joint_k;
            image_b += image_step_b;
        }
        const int n = k_next + k_local;
        // slices are whole k tiles and the padded rows whole vectors: a vector lies inside the slice or outside it
        const bool ok = n < positions && k_local < k_left;
        uint32_t y, x;
        d_row.divmod(static_cast<uint32_t>(ok ? n : 0), y, x);
        const uint32_t pos_b = image_b + (y * static_cast<uint32_t>(w) + x) * static_cast<uint32_t>(sizeof(T));
#pragma unroll
        for (int p = 0; p < P; ++p) reg[SLOT][p] = Vec<T, VEC>::load(rsrc, (ok && row_off[p] != kOob) ? row_off[p] + pos_b : kOob);
        col0[SLOT] = static_cast<int>(x);
        k_next += BK;
    }

    template <int SLOT = 0>
    __device__ __forceinline__ void store(T *lds) const {
#pragma unroll
        for (int p = 0; p < P; ++p)
            *reinterpret_cast<V *>(&lds[(p * RPP + row0) * L::LD + k_local]) = clear_outside_row<T, VEC>(reg[SLOT][p], col0[SLOT], w);
    }
};

// ---------------------------------------------------------------------------------------------
// Tile shapes: 64x64 (2x2 waves) or, for products with at most 32 rows, 32x128 (1x4 waves): every wave owns a
// 32x32 block either way.
// Register prefetch distance of the conv kernels: tile t + kConvPF is requested while tile t is multiplied.  A k
// tile holds little MFMA work (32x32 per wave), so one tile of lookahead leaves part of the load latency exposed;
// two measured 1 - 4 % faster on 28x28 .. 56x56 layers, four slower (registers).
constexpr int kConvPF = 2;

template <typename T, int BM, int BN, int BK, class StA, class StB>
using ConvEngine = TileEngine<T, BM, BN, BK, BM == 32 ? 1 : 2, BM == 32 ? 4 : 2, StA, StB>;

// Store of a tile whose positions are numbered over padded rows (ConvGeom::row_pad): tile column n = y * row_pad + x
// goes to C[m][y * w + x] when x < w, C being [M, h * w]; bias (may be null) adds bias[m].  Pairs: n is even, the
// padded row a multiple of 4 and w even, so x + 1 < w whenever x < w.
template <typename T, class Engine>
__device__ __forceinline__ void store_tile_padded_rows(Engine &eng, T *__restrict__ C, int M_, int h, int w, const FastDiv &d_row, int m0,
                                                       int n0, const T *__restrict__ bias) {
    using pair_t = typename Mfma<T>::pair_t;
    constexpr uint32_t kSz = sizeof(T);
    const int plane = h * w;
    const int rows = M_ - m0 < Engine::kBM ? M_ - m0 : Engine::kBM;
    const __amdgpu_buffer_rsrc_t out = make_rsrc(C + static_cast<int64_t>(m0) * plane, static_cast<int64_t>(rows) * plane * kSz);
    const __amdgpu_buffer_rsrc_t bias_m = make_rsrc(bias, bias ? static_cast<int64_t>(M_) * kSz : 0);  // absent: loads 0
    auto offset_of = [&](int ml, int nl) {
        uint32_t y, x;
        d_row.divmod(static_cast<uint32_t>(n0 + nl), y, x);
        const bool inside = ml < rows && static_cast<int>(y) < h && static_cast<int>(x) < w;
        return inside ? static_cast<uint32_t>(ml * plane + static_cast<int>(y) * w + static_cast<int>(x)) * kSz : kOob;
    };
    auto bias_of = [&](int ml) { return Vec<T, 1>::load(bias_m, static_cast<uint32_t>(m0 + ml) * kSz); };
    const bool pairs_ok = (w % 2 == 0) && (reinterpret_cast<uintptr_t>(C) % (2 * sizeof(T)) == 0);
    // (phased walk: a block's bias loads go out together, then its stores)
    T bv[Mfma<T>::NACC];
    eng.template for_each<true, true>(
        pairs_ok,
        [&]<int PHASE>(int ml, int nl, T v, int, int e) {
            if constexpr (PHASE != 1) bv[e] = bias_of(ml);
            if constexpr (PHASE != 0) buffer_store(out, offset_of(ml, nl), v + bv[e]);
        },
        [&]<int PHASE>(int ml, int nl, T v0, T v1, int, int e) {
            if constexpr (PHASE != 1) bv[e] = bias_of(ml);
            if constexpr (PHASE != 0) {
                pair_t o;
                o[0] = v0 + bv[e];
                o[1] = v1 + bv[e];
                buffer_store(out, offset_of(ml, nl), o);
            }
        });
}

// Store of one class of a strided grad_input (ConvGeom::sc_S): tile column n = i * row + j, the class's positions
// numbered over rows of `row` columns (its own width or the padded one), goes to
// C[m][(sc_y0 + sc_S * i) * sc_W + sc_x0 + sc_S * j] when i, j lie inside the class, C being [M, sc_H * sc_W].
template <typename T, class Engine>
__device__ __forceinline__ void store_tile_class_scatter(Engine &eng, T *__restrict__ C, int M_, const ConvGeom &geo, const FastDiv &d_row,
                                                         int m0, int n0) {
    constexpr uint32_t kSz = sizeof(T);
    const int plane = geo.sc_H * geo.sc_W;
    const int rows = M_ - m0 < Engine::kBM ? M_ - m0 : Engine::kBM;
    const __amdgpu_buffer_rsrc_t out = make_rsrc(C + static_cast<int64_t>(m0) * plane, static_cast<int64_t>(rows) * plane * kSz);
    const int h = geo.H, w = geo.W;
    auto offset_of = [&](int ml, int nl) {
        uint32_t i, j;
        d_row.divmod(static_cast<uint32_t>(n0 + nl), i, j);
        const bool inside = ml < rows && static_cast<int>(i) < h && static_cast<int>(j) < w;
        const int e = (geo.sc_y0 + geo.sc_S * static_cast<int>(i)) * geo.sc_W + geo.sc_x0 + geo.sc_S * static_cast<int>(j);
        return inside ? static_cast<uint32_t>(ml * plane + e) * kSz : kOob;
    };
    eng.template for_each<true, false>(
        false, [&]<int PHASE>(int ml, int nl, T v, int, int) { buffer_store(out, offset_of(ml, nl), v); },
        [&]<int PHASE>(int, int, T, T, int, int) {});
}

// forward: M = O, N = Ho*Wo, K = C*k*k, one GEMM per image.  StB gathers the image.
template <typename T, int BM, int BN, int BK, int A_VEC, class StB>
__global__ void __launch_bounds__(kThreads, 2)
conv_fwd_kernel(ConvGeom geo, const T *x, const T *w, const T *bias, T *out, int64_t image_bytes, int tiles_m, int tiles_n) {
    using StA = Stager<T, BM, BK, true, A_VEC, kConvPF>;
    using Engine = ConvEngine<T, BM, BN, BK, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    int b, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, gridDim.x), tiles_m, tiles_n, b, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int M_ = geo.O, N_ = geo.Ho * geo.Wo, K = geo.C * geo.k * geo.k;
    StA sa;
    StB sb(geo);
    if constexpr (StB::kTapTable) {  // the window's (dy, dx) table, behind the tile buffers
        sb.fill_tap_table(reinterpret_cast<int2 *>(smem_raw + Engine::kLdsBytes), tid);
        __syncthreads();
    }
    sa.init(w + static_cast<int64_t>(m0) * geo.w_so, tid, M_ - m0, geo.w_so, 1, K);
    sb.init(x + static_cast<int64_t>(b) * geo.xs_b, image_bytes, tid, n0);
    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, K, false);
    if (geo.row_pad) store_tile_padded_rows<T>(eng, out + static_cast<int64_t>(b) * M_ * N_, M_, geo.Ho, geo.Wo, geo.d_row_pad, m0, n0, bias);
    else store_tile_dense<T, false>(eng, out + static_cast<int64_t>(b) * M_ * N_, M_, N_, m0, n0, bias, bias ? 2 : 0, 0, 0);
}

// wt[c][(o, a, b)] = w[o][c][a][b]: the A operand of grad_input with its reduction index contiguous.
template <typename T>
__global__ void __launch_bounds__(256) weight_transpose_kernel(ConvGeom geo, const T *__restrict__ w, T *__restrict__ wt, int total) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t k2 = static_cast<uint32_t>(geo.k * geo.k);
    const uint32_t row = k2 * static_cast<uint32_t>(geo.O);
    const uint32_t c = static_cast<uint32_t>(idx) / row, rem = static_cast<uint32_t>(idx) - c * row;
    uint32_t o, r;
    geo.d_kk.divmod(rem, o, r);
    wt[idx] = w[static_cast<int64_t>(o) * geo.w_so + c * k2 + r];
}

// A strided grad_input splits into S*S dense problems.  Input rows y with (y + P) mod S = ry meet only the taps
// p = ry, ry + S, ... (kp of them), and with y = y0 + S i, p = ry + S pi the output row (y + P - p) / S is
// i + ay - pi: a unit-stride grad_input with a kp x kq kernel and paddings (ay, ax) over the Hc x Wc positions of the
// class, which skips the taps that a stride makes zero (three quarters of the reduction at stride 2).
struct DgradClass {
    int ry, rx, kp, kq;  // first tap per axis, taps per axis (0: no window reaches these positions)
    int y0, x0, Hc, Wc;  // first position per axis, positions per axis
    int ay, ax;          // paddings of the sub-problem
    int64_t wt_off;      // element offset of the class's packed weight [C, O*kp*kq] in the workspace
    int64_t tmp_off;     // element offset of the class's dense result [B, C, Hc*Wc]
};
constexpr int kMaxDgradStride = 3;
struct DgradClasses {
    DgradClass cls[kMaxDgradStride * kMaxDgradStride];
};

// Class blockIdx.y of the table: wtc[c][(o, pi, qi)] = w[o][c][ry + S pi][rx + S qi], at the class's own offset in wt.
template <typename T>
__global__ void __launch_bounds__(256)
weight_class_pack_kernel(ConvGeom geo, const T *__restrict__ w, T *__restrict__ wt, DgradClasses tab) {
    const DgradClass &cl = tab.cls[blockIdx.y];
    const int kpq = cl.kp * cl.kq, row = geo.O * kpq, total = geo.C * row;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int c = idx / row, rem = idx - c * row;
    const int o = rem / kpq, r = rem - o * kpq;
    const int pi = r / cl.kq, qi = r - pi * cl.kq;
    wt[cl.wt_off + idx] = w[static_cast<int64_t>(o) * geo.w_so + (c * geo.k + cl.ry + geo.S * pi) * geo.k + cl.rx + geo.S * qi];
}

// gin[b][c][y][x] = the class result that owns (y, x), or 0 where no window reaches.
template <typename T>
__global__ void __launch_bounds__(256)
dgrad_interleave_kernel(ConvGeom geo, const T *__restrict__ tmp, T *__restrict__ gin, DgradClasses tab, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int HW = geo.H * geo.W;
    const int64_t bc = idx / HW;
    uint32_t y, x, qy, ry, qx, rx;
    geo.d_W.divmod(static_cast<uint32_t>(idx - bc * HW), y, x);
    geo.d_S.divmod(y + static_cast<uint32_t>(geo.P), qy, ry);
    geo.d_S.divmod(x + static_cast<uint32_t>(geo.P), qx, rx);
    const DgradClass &cl = tab.cls[ry * geo.S + rx];
    T v = T(0);
    if (cl.kp > 0 && cl.kq > 0) {
        const int i = (static_cast<int>(y) - cl.y0) / geo.S, j = (static_cast<int>(x) - cl.x0) / geo.S;
        v = tmp[cl.tmp_off + bc * (cl.Hc * cl.Wc) + i * cl.Wc + j];
    }
    gin[idx] = v;
}

// A small job that rides in a convolution launch as `blocks` workgroups appended to its grid (spared a launch of its
// own, which for these sizes is all launch floor): kind 1, dst[i] = sum over s < splits of src[s * n + i] (grad_weight's
// partial tiles, mfma::add_up_parts) and a second such sum (grad_bias's parts); kind 3, the packed class weights of a strided grad_input (weight_class_pack_kernel's work); kind 2, the transposed weight of grad_input (weight_transpose_kernel's work).
struct ConvRide {
    int kind = 0, blocks = 0;
    const void *src = nullptr;
    void *dst = nullptr;
    int n = 0, splits = 0;
    // kind 1: a second sum (grad_bias's parts) by the last blocks2 of the appended workgroups
    int blocks2 = 0;
    const void *src2 = nullptr;
    void *dst2 = nullptr;
    int n2 = 0, splits2 = 0;
};
template <typename T>
__device__ __forceinline__ void conv_ride(const ConvRide &r, const ConvGeom &geo, int block, T *smem, const DgradClasses *classes = nullptr) {
    if (r.kind == 3) {  // weight_class_pack_kernel's work: r.splits blocks per class of a strided grad_input
        const int ci = block / r.splits, idx = (block - ci * r.splits) * kThreads + static_cast<int>(threadIdx.x);
        const DgradClass &cl = classes->cls[ci];
        const int kpq = cl.kp * cl.kq, row = geo.O * kpq, total = geo.C * row;
        if (idx >= total) return;
        const int c = idx / row, rem = idx - c * row;
        const int o = rem / kpq, t = rem - o * kpq;
        const int pi = t / cl.kq, qi = t - pi * cl.kq;
        static_cast<T *>(r.dst)[cl.wt_off + idx] =
            static_cast<const T *>(r.src)[static_cast<int64_t>(o) * geo.w_so + (c * geo.k + cl.ry + geo.S * pi) * geo.k + cl.rx + geo.S * qi];
    } else if (r.kind == 1) {
        const int first = r.blocks - r.blocks2;
        if (block < first) add_up_parts<T, kThreads / 64>(static_cast<const T *>(r.src), static_cast<T *>(r.dst), r.n, r.splits, block, smem);
        else add_up_parts<T, kThreads / 64>(static_cast<const T *>(r.src2), static_cast<T *>(r.dst2), r.n2, r.splits2, block - first, smem);
    } else {
        const int idx = block * kThreads + static_cast<int>(threadIdx.x);
        if (idx >= r.n) return;
        const uint32_t k2 = static_cast<uint32_t>(geo.k * geo.k);
        const uint32_t row = k2 * static_cast<uint32_t>(geo.O);
        const uint32_t c = static_cast<uint32_t>(idx) / row, rem = static_cast<uint32_t>(idx) - c * row;
        uint32_t o, t;
        geo.d_kk.divmod(rem, o, t);
        static_cast<T *>(r.dst)[idx] = static_cast<const T *>(r.src)[static_cast<int64_t>(o) * geo.w_so + c * k2 + t];
    }
}

// grad_input: M = C, N = H*W, K = O*k*k, one GEMM per image.  wt is the transposed weight [C, O*k*k];
// StB gathers grad_out.
// SCATTER: the problem is one class of a strided grad_input and its result goes straight to that class's elements of
// grad_input (ConvGeom::sc_S, store_tile_class_scatter).
template <typename T, int BM, int BN, int BK, int A_VEC, class StB, bool SCATTER = false>
__global__ void __launch_bounds__(kThreads, 2)
conv_dgrad_kernel(ConvGeom geo, const T *gout, const T *wt, T *gin, int tiles_m, int tiles_n, ConvRide ride) {
    using StA = Stager<T, BM, BK, true, A_VEC, kConvPF>;
    using Engine = ConvEngine<T, BM, BN, BK, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    const unsigned conv_blocks = gridDim.x - static_cast<unsigned>(ride.blocks);
    if (blockIdx.x >= conv_blocks) {  // an appended workgroup
        conv_ride<T>(ride, geo, static_cast<int>(blockIdx.x - conv_blocks), smem);
        return;
    }
    int b, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, conv_blocks), tiles_m, tiles_n, b, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int M_ = geo.C, N_ = geo.H * geo.W, K = geo.O * geo.kh * geo.kw;
    const int64_t g_image = static_cast<int64_t>(geo.O) * geo.Ho * geo.Wo;
    StA sa;
    StB sb(geo);
    if constexpr (StB::kTapTable) {
        sb.fill_tap_table(reinterpret_cast<int2 *>(smem_raw + Engine::kLdsBytes), tid);
        __syncthreads();
    }
    sa.init(wt + static_cast<int64_t>(m0) * K, tid, M_ - m0, K, 1, K);
    sb.init(gout + static_cast<int64_t>(b) * g_image, g_image * static_cast<int64_t>(sizeof(T)), tid, n0);
    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, K, false);
    if constexpr (SCATTER)
        store_tile_class_scatter<T>(eng, gin + static_cast<int64_t>(b) * M_ * geo.sc_H * geo.sc_W, M_, geo, geo.row_pad ? geo.d_row_pad : geo.d_W, m0, n0);
    else if (geo.row_pad)
        store_tile_padded_rows<T>(eng, gin + static_cast<int64_t>(b) * M_ * N_, M_, geo.H, geo.W, geo.d_row_pad, m0, n0, static_cast<const T *>(nullptr));
    else
        store_tile_dense<T, true>(eng, gin + static_cast<int64_t>(b) * M_ * N_, M_, N_, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
}

// Every class of a strided grad_input in one launch: the classes are short products (a quarter of the taps each at stride
// 2, a reduction of O to 4 O), and launched one after the other each fills and drains the chip by itself.  Workgroups
// [first_block[i], first_block[i + 1]) run class i as conv_dgrad_kernel<..., SCATTER = true> would.
constexpr int kMaxDgradClasses = kMaxDgradStride * kMaxDgradStride;
struct DgradClassGeoms {
    ConvGeom geo[kMaxDgradClasses];
    int64_t wt_off[kMaxDgradClasses];  // element offset of the class's packed weight
    int first_block[kMaxDgradClasses + 1];
    int tiles_m[kMaxDgradClasses], tiles_n[kMaxDgradClasses];
    int n;
};
static_assert(sizeof(DgradClassGeoms) <= 3584, "kernel arguments are limited to 4 KiB");

template <typename T, int BM, int BN, int BK, int A_VEC, class StB>
__global__ void __launch_bounds__(kThreads, 2)
conv_dgrad_classes_kernel(DgradClassGeoms tab, const T *gout, const T *wt, T *gin, ConvRide ride) {
    using StA = Stager<T, BM, BK, true, A_VEC, kConvPF>;
    using Engine = ConvEngine<T, BM, BN, BK, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    if (static_cast<int>(blockIdx.x) >= tab.first_block[tab.n]) {  // an appended workgroup (sums only: no geometry needed)
        conv_ride<T>(ride, tab.geo[0], static_cast<int>(blockIdx.x) - tab.first_block[tab.n], smem);
        return;
    }
    int ci = 0;
    while (ci + 1 < tab.n && static_cast<int>(blockIdx.x) >= tab.first_block[ci + 1]) ++ci;  // (uniform, at most 8 steps)
    const ConvGeom &geo = tab.geo[ci];
    const int first = tab.first_block[ci], count = tab.first_block[ci + 1] - first;
    int b, tm, tn;
    decode_tile(remap_xcd(static_cast<int>(blockIdx.x) - first, count), tab.tiles_m[ci], tab.tiles_n[ci], b, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int M_ = geo.C, K = geo.O * geo.kh * geo.kw;
    const int64_t g_image = static_cast<int64_t>(geo.O) * geo.Ho * geo.Wo;
    StA sa;
    StB sb(geo);
    if constexpr (StB::kTapTable) {
        sb.fill_tap_table(reinterpret_cast<int2 *>(smem_raw + Engine::kLdsBytes), tid);
        __syncthreads();
    }
    sa.init(wt + tab.wt_off[ci] + static_cast<int64_t>(m0) * K, tid, M_ - m0, K, 1, K);
    sb.init(gout + static_cast<int64_t>(b) * g_image, g_image * static_cast<int64_t>(sizeof(T)), tid, n0);
    Engine eng;
    eng.init(tid);
    eng.run(sa, sb, smem, K, false);
    store_tile_class_scatter<T>(eng, gin + static_cast<int64_t>(b) * M_ * geo.sc_H * geo.sc_W, M_, geo, geo.row_pad ? geo.d_row_pad : geo.d_W, m0, n0);
}

// grad_weight: M = O, N = C*k*k, K = Ho*Wo per image.  Workgroup column `part` = (image group, k slice)
// accumulates slice [k0, k0 + k_chunk) of images [grp*group, min(B, (grp+1)*group)) in registers and writes one
// partial tile; k_chunk is a multiple of BK.
// PADDED: the positions are numbered over padded rows (geo.row_pad != 0), K = Ho * row_pad.  With joint_k != 0
// (PADDED only, kslices = 1) the group's images form one reduction of joint_k positions each, an image's own rounded up
// to whole k tiles: small images then share one run of the pipeline instead of filling and draining it per image.
template <typename T, int BK, int A_VEC, class StB, bool PADDED = false>
__global__ void __launch_bounds__(kThreads, 2)
conv_wgrad_kernel(ConvGeom geo, const T *gout, const T *x, T *partial, int64_t image_bytes, int group, int kslices, int k_chunk,
                  int tiles_m, int tiles_n, int joint_k, ConvRide ride, DgradClasses classes) {
    constexpr int BM = 64, BN = 64;
    using StA = std::conditional_t<PADDED, PaddedRowsStager<T, BM, BK, kConvPF>, Stager<T, BM, BK, true, A_VEC, kConvPF>>;
    using Engine = ConvEngine<T, BM, BN, BK, StA, StB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const smem = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    const unsigned conv_blocks = gridDim.x - static_cast<unsigned>(ride.blocks);
    if (blockIdx.x >= conv_blocks) {  // an appended workgroup
        conv_ride<T>(ride, geo, static_cast<int>(blockIdx.x - conv_blocks), smem, &classes);
        return;
    }
    int part, tm, tn;
    decode_tile(remap_xcd(blockIdx.x, conv_blocks), tiles_m, tiles_n, part, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int plane = geo.Ho * geo.Wo;
    const int M_ = geo.O, N_ = geo.C * geo.k * geo.k, K = PADDED ? geo.Ho * geo.row_pad : plane;
    const int grp = part / kslices, k0 = (part - grp * kslices) * k_chunk;
    const int k_len = K - k0 < k_chunk ? K - k0 : k_chunk;
    const int64_t g_image = static_cast<int64_t>(geo.O) * plane;
    StA sa;
    StB sb(geo);
    sb.init(tid, n0);
    Engine eng;
    eng.init(tid);
    const int b_end = (grp + 1) * group < geo.B ? (grp + 1) * group : geo.B;
    bool joint = false;
    if constexpr (PADDED) {
        if (joint_k) {
            joint = true;
            const int b0 = grp * group, images = b_end - b0;
            sa.init(gout + b0 * g_image + static_cast<int64_t>(m0) * plane, tid, M_ - m0, geo, 0, images, joint_k);
            sb.set_images(x + static_cast<int64_t>(b0) * geo.xs_b, (images - 1) * geo.xs_b * static_cast<int64_t>(sizeof(T)) + image_bytes,
                          joint_k, static_cast<int32_t>(geo.xs_b));
            eng.run(sa, sb, smem, images * joint_k, false);
        }
    }
    for (int b = grp * group; b < b_end && !joint; ++b) {
        if constexpr (PADDED) sa.init(gout + b * g_image + static_cast<int64_t>(m0) * plane, tid, M_ - m0, geo, k0);
        else sa.init(gout + b * g_image + static_cast<int64_t>(m0) * K + k0, tid, M_ - m0, K, 1, k_len);
        sb.set_image(x + static_cast<int64_t>(b) * geo.xs_b, image_bytes, k0);
        eng.run(sa, sb, smem, k_len, false);
        __syncthreads();  // the next image's prologue overwrites LDS buffer 0
    }
    store_tile_dense<T, true>(eng, partial + static_cast<int64_t>(part) * M_ * N_, M_, N_, m0, n0, static_cast<const T *>(nullptr), 0, 0, 0);
}

// out[i] = sum over parts of partial[s][i].  A workgroup owns 16 consecutive elements; its 16 lanes per element
// each add every 16th part in increasing order, and a fixed tree adds the 16 sums (deterministic).
template <typename T>
__global__ void __launch_bounds__(256) reduce_splits_kernel(const T *__restrict__ partial, T *__restrict__ out, int64_t n, int splits) {
    __shared__ T red[16][17];
    const int e = threadIdx.x % 16, lane_s = threadIdx.x / 16;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 16 + e;
    T acc = T(0);
    if (i < n)
        for (int s = lane_s; s < splits; s += 16) acc += partial[static_cast<int64_t>(s) * n + i];
    red[lane_s][e] = acc;
    __syncthreads();
    for (int h = 8; h > 0; h >>= 1) {
        if (lane_s < h) red[lane_s][e] += red[lane_s + h][e];
        __syncthreads();
    }
    if (lane_s == 0 && i < n) out[i] = red[0][e];
}

// The same sum for long outputs: one lane per 16-byte vector of out adds its parts in increasing order, every load a
// whole coalesced line of the wave (the kernel above reads 64 bytes per part and workgroup, and with few parts most of
// its lanes have nothing to add).  n is a multiple of the vector length; partial and out are 16-byte aligned.
template <typename T>
__global__ void __launch_bounds__(256) reduce_splits_stream_kernel(const T *__restrict__ partial, T *__restrict__ out, int64_t n, int splits) {
    using V = std::conditional_t<sizeof(T) == 4, float4, double2>;
    constexpr int VEC = sizeof(V) / sizeof(T);
    const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    V acc = *reinterpret_cast<const V *>(partial + i);
    T *a = reinterpret_cast<T *>(&acc);
#pragma unroll 4
    for (int s = 1; s < splits; ++s) {
        const V v = *reinterpret_cast<const V *>(partial + static_cast<int64_t>(s) * n + i);
        const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) a[j] += e[j];
    }
    *reinterpret_cast<V *>(out + i) = acc;
}

// The same sum for many parts of a tile of middling length (grad_weight's one partial tile per workgroup): a workgroup
// owns 64 consecutive elements, each of its eight waves adds a contiguous eighth of the parts in increasing order --
// every load a whole coalesced line of the wave, up to sixteen in flight (128 parts: one round trip per wave) -- and
// the eight sums are added in order.
template <typename T>
__global__ void __launch_bounds__(512) reduce_splits_ranges_kernel(const T *__restrict__ partial, T *__restrict__ out, int64_t n, int splits) {
    constexpr int kWaves = 8;
    __shared__ T red[kWaves][64];
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 64 + lane;
    const int per = (splits + kWaves - 1) / kWaves;
    const int s0 = w * per, s1 = s0 + per < splits ? s0 + per : splits;
    T acc = T(0);
    if (i < n) {
        int s = s0;
        for (; s + 16 <= s1; s += 16) {
            T v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = partial[static_cast<int64_t>(s + u) * n + i];
#pragma unroll
            for (int u = 0; u < 16; ++u) acc += v[u];
        }
        for (; s + 4 <= s1; s += 4) {
            T v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = partial[static_cast<int64_t>(s + u) * n + i];
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += v[u];
        }
        for (; s < s1; ++s) acc += partial[static_cast<int64_t>(s) * n + i];
    }
    red[w][lane] = acc;
    __syncthreads();
    if (w == 0 && i < n) {
        T v = red[0][lane];
#pragma unroll
        for (int k = 1; k < kWaves; ++k) v += red[k][lane];
        out[i] = v;
    }
}

// out[i] = sum over parts of partial[s][i], by whichever of the kernels suits the shape: the streaming one when
// there are enough vectors to fill the chip or too few parts to occupy the other's sixteen lanes per element.
template <typename T>
ttamd_status launch_reduce_splits(const T *partial, T *out, int64_t n, int splits, hipStream_t st) {
    constexpr int VEC = 16 / sizeof(T);
    const bool aligned = n % VEC == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (aligned && (n / VEC >= 65536 || splits <= 8)) {
        const int64_t blocks = (n / VEC + 255) / 256;
        reduce_splits_stream_kernel<T><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(partial, out, n, splits);
    } else if (splits >= 32 && n >= 4096) {
        reduce_splits_ranges_kernel<T><<<dim3(static_cast<unsigned>((n + 63) / 64)), dim3(512), 0, st>>>(partial, out, n, splits);
    } else {
        reduce_splits_kernel<T><<<dim3(static_cast<unsigned>((n + 15) / 16)), dim3(256), 0, st>>>(partial, out, n, splits);
    }
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

// grad_bias[o] = sum over batch and space of grad_out[b][o][.] (cpu/conv.cpp:289), in two steps so that the launch
// fills the chip whatever the channel count: workgroup (o, p) adds part p of channel o's B * HoWo elements (taken as
// vectors V of sizeof(V) / sizeof(T) elements, numbered image by image), and reduce_splits_kernel adds the parts.
template <typename T, typename V>
__global__ void __launch_bounds__(256)
bias_grad_kernel(const T *__restrict__ gout, T *__restrict__ partial, int O, int HoWo, uint32_t total, uint32_t chunk, FastDiv d_per_image) {
    constexpr int VEC = sizeof(V) / sizeof(T);
    __shared__ T red[256];
    const int o = blockIdx.x;
    const uint32_t begin = blockIdx.y * chunk, end = begin + chunk < total ? begin + chunk : total;
    T acc = T(0);
    for (uint32_t idx = begin + threadIdx.x; idx < end; idx += 256) {
        uint32_t b, i;
        d_per_image.divmod(idx, b, i);
        const V v = *reinterpret_cast<const V *>(gout + (static_cast<int64_t>(b) * O + o) * HoWo + static_cast<int64_t>(i) * VEC);
        const T *e = reinterpret_cast<const T *>(&v);
        T s = e[0];
#pragma unroll
        for (int j = 1; j < VEC; ++j) s += e[j];
        acc += s;
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (static_cast<int>(threadIdx.x) < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[static_cast<int64_t>(blockIdx.y) * O + o] = red[0];
}

// Direct forward for the integer dtypes: one lane per output element, wrap-around arithmetic in unsigned
// registers (same value modulo 2^n as the reference's SIMD lanes, cpu/kernel/simd.h:120-127).
template <typename T, typename Acc>
__global__ void __launch_bounds__(256)
conv_fwd_direct_kernel(ConvGeom geo, const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias, T *__restrict__ out, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int HoWo = geo.Ho * geo.Wo;
    const int n = static_cast<int>(idx % HoWo);
    const int o = static_cast<int>((idx / HoWo) % geo.O);
    const int b = static_cast<int>(idx / (static_cast<int64_t>(HoWo) * geo.O));
    const int h = n / geo.Wo, ww = n % geo.Wo;
    Acc acc = Acc(0);
    for (int c = 0; c < geo.C; ++c)
        for (int p = 0; p < geo.k; ++p)
            for (int q = 0; q < geo.k; ++q) {
                const int ih = geo.S * h + p - geo.P, iw = geo.S * ww + q - geo.P;
                if (ih < 0 || iw < 0 || ih >= geo.H || iw >= geo.W) continue;
                const Acc xv = static_cast<Acc>(x[b * geo.xs_b + static_cast<int64_t>(c) * geo.xs_c + static_cast<int64_t>(ih) * geo.xs_h + static_cast<int64_t>(iw) * geo.xs_w]);
                const Acc wv = static_cast<Acc>(w[o * geo.w_so + (c * geo.k + p) * geo.k + q]);
                acc += xv * wv;
            }
    T v = static_cast<T>(acc);
    if (bias) v = static_cast<T>(v + bias[o]);
    out[idx] = v;
}

// grad_input for layers with at most CMAX input channels (a network's first layer: 1 or 3), where the 32-row MFMA
// tile of conv_dgrad_kernel would be all but empty (C = 3: 29 of 32 rows multiply zeros) and, with a stride, most of
// its reduction too (the taps a stride skips).  One lane per input position (b, y, x) accumulates all its channels on
// the vector ALU, the weights in LDS as [o][p][q][c].  A position lies in at most NP x NP windows per output channel
// (NP >= ceil(k / S)): slot (i, j) is tap (p0 + i S, q0 + j S), p0 = (y + P) mod S, with output pixel
// (oh0 - i, ow0 - j).  A lane decodes its slots once; per output channel it then issues all NP * NP loads of grad_out
// at once (addresses clamped, invalid slots cleared by a select) and reads each slot's CMAX weights as one LDS
// vector, so the loads overlap instead of forming a dependent chain per tap.  The sum runs over (o, p, q) in that
// order, the order of conv_dgrad_kernel's reduction index.
// UNIT (stride 1, NP == k): slot (i, j) is tap (i, j) for every lane, so a weight is the same for the whole wave: it
// is read through the scalar cache straight from the weight tensor and multiplied as a scalar operand -- no LDS copy,
// no per-lane LDS read per product.
template <typename T, int CMAX, int NP, bool UNIT = false>
__global__ void __launch_bounds__(256)
conv_dgrad_slots_kernel(ConvGeom geo, const T *__restrict__ gout, const T *__restrict__ w, T *__restrict__ gin, int blocks_per_image,
                        ConvRide ride) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *const wl = reinterpret_cast<T *>(smem_raw);
    const unsigned conv_blocks = gridDim.x - static_cast<unsigned>(ride.blocks);
    if (blockIdx.x >= conv_blocks) {  // an appended workgroup (sums only; the launch reserves their 4 KB of LDS)
        conv_ride<T>(ride, geo, static_cast<int>(blockIdx.x - conv_blocks), wl);
        return;
    }
    const int kk = geo.k * geo.k, HW = geo.H * geo.W, HoWo = geo.Ho * geo.Wo;
    if constexpr (!UNIT) {
        for (int i = threadIdx.x; i < geo.O * kk * CMAX; i += 256) {
            const int c = i % CMAX, t = (i / CMAX) % kk, o = i / (CMAX * kk);
            wl[i] = c < geo.C ? w[static_cast<int64_t>(o) * geo.w_so + c * kk + t] : T(0);
        }
        __syncthreads();
    }
    const int b = blockIdx.x / blocks_per_image;
    const int n = (blockIdx.x - b * blocks_per_image) * 256 + threadIdx.x;
    if (n >= HW) return;
    uint32_t y, x;
    geo.d_W.divmod(static_cast<uint32_t>(n), y, x);
    uint32_t oh0, p0, ow0, q0;
    geo.d_S.divmod(y + static_cast<uint32_t>(geo.P), oh0, p0);
    geo.d_S.divmod(x + static_cast<uint32_t>(geo.P), ow0, q0);
    // grad_out of this image through a buffer descriptor: a slot's byte offset inside a channel plane stays in a
    // register for the whole kernel (invalid slots hold the out-of-range offset, which loads as zero) and the plane
    // advances through the scalar offset, so a load costs no address arithmetic and no select.
    const __amdgpu_buffer_rsrc_t grs = make_rsrc(gout + static_cast<int64_t>(b) * geo.O * HoWo,
                                                 static_cast<int64_t>(geo.O) * HoWo * static_cast<int64_t>(sizeof(T)));
    uint32_t goff[NP * NP];
    int woff[NP * NP];
#pragma unroll
    for (int i = 0; i < NP; ++i)
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            const int p = static_cast<int>(p0) + i * geo.S, q = static_cast<int>(q0) + j * geo.S;
            const int oh = static_cast<int>(oh0) - i, ow = static_cast<int>(ow0) - j;
            const bool v = (p < geo.k) & (q < geo.k) & (oh >= 0) & (oh < geo.Ho) & (ow >= 0) & (ow < geo.Wo);
            goff[i * NP + j] = v ? static_cast<uint32_t>(oh * geo.Wo + ow) * static_cast<uint32_t>(sizeof(T)) : kOob;
            woff[i * NP + j] = v ? (p * geo.k + q) * CMAX : 0;
        }
    T acc[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c) acc[c] = T(0);
    const T *wo = wl;
    const uint32_t plane_bytes = static_cast<uint32_t>(HoWo) * static_cast<uint32_t>(sizeof(T));
    uint32_t plane = 0;
    // kOU output channels to a round, their NP * NP * kOU loads in flight together; the sum still runs over (o, p, q)
    // in order.  (First layer of the MNIST example network, 1 -> 32 channels at batch 256: 28.7 us with one channel
    // per round and the weights in LDS, 27.5 with four, 24.5 with four and scalar weights -- what is left is the
    // 288 single-element loads per lane.)
    constexpr int kOU = 4;
    int o = 0;
    for (; o + kOU <= geo.O; o += kOU, plane += kOU * plane_bytes, wo += kOU * kk * CMAX) {
        T gv[kOU][NP * NP];
#pragma unroll
        for (int u = 0; u < kOU; ++u)
#pragma unroll
            for (int t = 0; t < NP * NP; ++t) gv[u][t] = Vec<T, 1>::load_at(grs, goff[t], plane + u * plane_bytes);
#pragma unroll
        for (int u = 0; u < kOU; ++u)
#pragma unroll
            for (int t = 0; t < NP * NP; ++t) {
#pragma unroll
                for (int c = 0; c < CMAX; ++c) {
                    if constexpr (UNIT) acc[c] += w[static_cast<int64_t>(o + u) * geo.w_so + c * kk + (t / NP) * geo.k + t % NP] * gv[u][t];
                    else acc[c] += wo[u * kk * CMAX + woff[t] + c] * gv[u][t];
                }
            }
    }
    for (; o < geo.O; ++o, plane += plane_bytes, wo += kk * CMAX) {
        T gv[NP * NP];
#pragma unroll
        for (int t = 0; t < NP * NP; ++t) gv[t] = Vec<T, 1>::load_at(grs, goff[t], plane);
#pragma unroll
        for (int t = 0; t < NP * NP; ++t) {
#pragma unroll
            for (int c = 0; c < CMAX; ++c) {
                if constexpr (UNIT) acc[c] += w[static_cast<int64_t>(o) * geo.w_so + c * kk + (t / NP) * geo.k + t % NP] * gv[t];
                else acc[c] += wo[woff[t] + c] * gv[t];
            }
        }
    }
    T *dst = gin + static_cast<int64_t>(b) * geo.C * HW + n;
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < geo.C) dst[static_cast<int64_t>(c) * HW] = acc[c];
}

// ---------------------------------------------------------------------------------------------
// host side

struct ConvPlan {
    ConvGeom geo;
    const void *x;
    const void *w;
    int64_t image_bytes;   // bytes reachable from an image's first element
    int64_t weight_bytes;  // bytes reachable from the weight's first element
};

ttamd_status make_plan(const char *who, ttamd_dtype dtype, const ttamd_view4 *input, const ttamd_view4 *weight, int B, int C,
                       int H, int W, int O, int k, int stride, int padding, ConvPlan *plan) {
    if (dtype == TTAMD_BOOL || dtype_size(dtype) == 0 || dtype < TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("%s does not support dtype code %d", who, static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (!input || !weight) {
        set_error("%s: NULL operand view", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || O <= 0 || k <= 0 || stride <= 0 || padding < 0) {
        set_error("%s: invalid geometry (B=%d C=%d H=%d W=%d O=%d k=%d stride=%d padding=%d)", who, B, C, H, W, O, k,
                  stride, padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (k >= (1 << 14) || padding >= (1 << 14)) {
        set_error("%s: kernel size and padding must be below 16384", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const int Ho = (H + 2 * padding - k) / stride + 1, Wo = (W + 2 * padding - k) / stride + 1;
    if (H + 2 * padding < k || W + 2 * padding < k || Ho <= 0 || Wo <= 0) {
        set_error("%s: kernel %d does not fit the padded input %dx%d", who, k, H + 2 * padding, W + 2 * padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    for (int i = 0; i < 4; ++i) {
        if (input->stride[i] < 0 || weight->stride[i] < 0) {
            set_error("%s: negative strides are not supported", who);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
    }
    if (input->offset < 0 || weight->offset < 0) {
        set_error("%s: negative view offset", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    // The weight is used as the matrix [O, C*k*k] (cpu/conv.cpp:69 reshapes it, cloning a non-dense view):
    // its (c,p,q) dimensions must already be dense; the adapter calls contiguous() otherwise.
    if ((C > 1 && weight->stride[1] != static_cast<int64_t>(k) * k) || (k > 1 && (weight->stride[2] != k || weight->stride[3] != 1))) {
        set_error("%s: weight dimensions (C,k,k) must be dense; make the weight contiguous first", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const size_t esz = dtype_size(dtype);
    const int64_t x_reach = (static_cast<int64_t>(C - 1) * input->stride[1] + static_cast<int64_t>(H - 1) * input->stride[2] +
                             static_cast<int64_t>(W - 1) * input->stride[3] + 1) * static_cast<int64_t>(esz);
    const int64_t w_reach = (static_cast<int64_t>(O - 1) * weight->stride[0] + static_cast<int64_t>(C) * k * k) * static_cast<int64_t>(esz);
    const int64_t limit = 0x7fffffffLL;
    if (x_reach >= limit || w_reach >= limit || static_cast<int64_t>(O) * Ho * Wo * static_cast<int64_t>(esz) >= limit ||
        static_cast<int64_t>(C) * H * W * static_cast<int64_t>(esz) >= limit ||
        static_cast<int64_t>(C) * k * k >= (1 << 24) || static_cast<int64_t>(O) * k * k >= (1 << 24) ||
        static_cast<int64_t>(H) * W >= limit / 8 || input->stride[1] >= limit / 8 || input->stride[2] >= limit / 8 ||
        input->stride[3] >= limit / 8) {
        set_error("%s: one image or the weight exceeds the 2 GiB addressing range of the kernels", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ConvGeom &g = plan->geo;
    g = ConvGeom{};
    g.B = B; g.C = C; g.H = H; g.W = W; g.O = O; g.k = k; g.S = stride; g.P = padding; g.Ho = Ho; g.Wo = Wo;
    g.kh = k; g.kw = k; g.Ph = padding; g.Pw = padding;
    g.xs_b = input->stride[0];
    g.xs_c = static_cast<int32_t>(input->stride[1]);
    g.xs_h = static_cast<int32_t>(input->stride[2]);
    g.xs_w = static_cast<int32_t>(input->stride[3]);
    g.w_so = weight->stride[0];
    g.d_kk = make_fastdiv(static_cast<uint32_t>(k) * k);
    g.d_k = make_fastdiv(static_cast<uint32_t>(k));
    g.d_Wo = make_fastdiv(static_cast<uint32_t>(Wo));
    g.d_W = make_fastdiv(static_cast<uint32_t>(W));
    g.d_S = make_fastdiv(static_cast<uint32_t>(stride));
    plan->x = static_cast<const char *>(input->data) + input->offset * static_cast<int64_t>(esz);
    plan->w = static_cast<const char *>(weight->data) + weight->offset * static_cast<int64_t>(esz);
    plan->image_bytes = x_reach;
    plan->weight_bytes = w_reach;
    return TTAMD_OK;
}

template <class Kernel>
ttamd_status set_lds(Kernel kernel, size_t lds_bytes) {
    if (lds_bytes > 48 * 1024)
        TTAMD_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            static_cast<int>(lds_bytes)));
    return TTAMD_OK;
}

// Which kernel family the calling thread's last forward ([0]), grad_input ([1]) and grad_weight ([2]) launches took: 0x100 the
// implicit-GEMM kernels of this file, 0x200 + 16 * waves + patch buffers the persistent kernel of conv_patch.hip,
// 0 anything else.  Read through ttamd_conv2d_last_kernel by the tests that mean to cover a particular kernel.
thread_local int t_last_kernel[4] = {0, 0, 0, 0};

// TTAMD_CONV_PATCH=0 keeps every convolution on the implicit-GEMM kernels of this file (for comparisons).
inline bool patch_kernel_enabled() {
    static const bool on = [] {
        const char *e = std::getenv("TTAMD_CONV_PATCH");
        return !(e && e[0] == '0');
    }();
    return on;
}

// TTAMD_CONV_STRIDED_VEC=0 keeps strided layers on the element-wise gathers (for comparisons).
inline bool strided_vector_gather_enabled() {
    static const bool on = [] {
        const char *e = std::getenv("TTAMD_CONV_STRIDED_VEC");
        return !(e && e[0] == '0');
    }();
    return on;
}

// TTAMD_CONV_MERGED_CLASSES=0 launches the classes of a strided grad_input one after the other (for comparisons).
inline bool merged_dgrad_classes_enabled() {
    static const bool on = [] {
        const char *e = std::getenv("TTAMD_CONV_MERGED_CLASSES");
        return !(e && e[0] == '0');
    }();
    return on;
}

template <typename T>
struct ConvTiles {
    static constexpr int BK = sizeof(T) == 4 ? 32 : 16;
};

// 16-byte loads of the weight / grad_out matrix need aligned rows.
template <typename T>
bool rows_vectorizable(const void *ptr, int64_t row_stride, int64_t image_stride) {
    constexpr int VK = Mfma<T>::VK;
    return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && row_stride % VK == 0 && image_stride % VK == 0;
}

template <class Kernel>
ttamd_status launch_conv(Kernel kernel, size_t lds, int64_t blocks, hipStream_t st, auto... args) {
    if (blocks > 0x7fffffff) {
        set_error("conv2d: too many workgroups");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = set_lds(kernel, lds)) return s;
    kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(kThreads), lds, st>>>(args...);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

// LDS bytes of the engine built from the weight/grad_out stager and gather stager StB.
template <typename T, int BM, int BN, int A_VEC, class StB>
constexpr size_t conv_lds_bytes() {
    constexpr int BK = ConvTiles<T>::BK;
    return ConvEngine<T, BM, BN, BK, Stager<T, BM, BK, true, A_VEC, kConvPF>, StB>::kLdsBytes + (StB::kTapTable ? kTapTableBytes : 0);
}

// Rows of `width` positions that are no whole number of 16-byte vectors: the padded row width with which the
// 16-byte gathers serve them, or 0 where the narrower gathers stay ahead (the padding columns are wasted work: at
// most a fifth more of it against the 8-byte gathers of an even width, at most double against element loads).
int padded_row_width(size_t esz, int width) {
    const int VK = static_cast<int>(16 / esz);
    if (width % VK == 0) return 0;
    const int padded = (width + VK - 1) / VK * VK;
    const bool pairs = esz == 4 && width % 2 == 0;
    return (pairs ? 5 * padded <= 6 * width : padded <= 2 * width) ? padded : 0;
}

template <typename T, int BM, int BN>
ttamd_status forward_mfma_tile(const ConvPlan &pl, const void *bias, void *out, hipStream_t st) {
    constexpr int BK = ConvTiles<T>::BK, VK = Mfma<T>::VK;
    ConvGeom g = pl.geo;
    const bool a_vec = rows_vectorizable<T>(pl.w, g.w_so, 0);
    const bool stride_two = g.S == 2 && strided_vector_gather_enabled();
    const bool table_ok = g.k * g.k <= kTapTableEntries;  // (the vector gathers read a window's taps from a table in LDS)
    if (a_vec && table_ok && (g.S == 1 || stride_two) && g.xs_w == 1) {
        g.row_pad = padded_row_width(sizeof(T), g.Wo);
        g.d_row_pad = make_fastdiv(static_cast<uint32_t>(g.row_pad ? g.row_pad : 1));
    }
    const int M_ = g.O, N_ = g.Ho * (g.row_pad ? g.row_pad : g.Wo);
    const int tiles_m = (M_ + BM - 1) / BM, tiles_n = (N_ + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.B;
    const bool b_vec = table_ok && g.S == 1 && g.xs_w == 1 && (g.row_pad || g.Wo % VK == 0);
    auto go = [&](auto kernel, size_t lds) {
        return launch_conv(kernel, lds, blocks, st, g, static_cast<const T *>(pl.x), static_cast<const T *>(pl.w),
                           static_cast<const T *>(bias), static_cast<T *>(out), pl.image_bytes, tiles_m, tiles_n);
    };
    using VecB = TapStagerMC<T, BN, BK, VK, false, kConvPF>;
    using OneB = Im2colStager<T, BN, BK, kConvPF>;
    if (a_vec && b_vec) return go(conv_fwd_kernel<T, BM, BN, BK, VK, VecB>, conv_lds_bytes<T, BM, BN, VK, VecB>());
    // stride 2 on dense rows with output rows of whole vectors: two 16-byte gathers per vector of positions
    if (a_vec && table_ok && stride_two && g.xs_w == 1 && (g.row_pad || g.Wo % VK == 0)) {
        using Vec2B = TapStagerMC<T, BN, BK, VK, false, kConvPF, 2>;
        t_last_kernel[0] = 0x102;
        return go(conv_fwd_kernel<T, BM, BN, BK, VK, Vec2B>, conv_lds_bytes<T, BM, BN, VK, Vec2B>());
    }
    if constexpr (sizeof(T) == 4) {  // rows of 2n elements: 8-byte gathers
        using PairB = TapStagerMC<T, BN, BK, 2, false, kConvPF>;
        if (a_vec && table_ok && g.S == 1 && g.xs_w == 1 && g.Wo % 2 == 0)
            return go(conv_fwd_kernel<T, BM, BN, BK, VK, PairB>, conv_lds_bytes<T, BM, BN, VK, PairB>());
    }
    if (a_vec) return go(conv_fwd_kernel<T, BM, BN, BK, VK, OneB>, conv_lds_bytes<T, BM, BN, VK, OneB>());
    if (b_vec) return go(conv_fwd_kernel<T, BM, BN, BK, 1, VecB>, conv_lds_bytes<T, BM, BN, 1, VecB>());
    return go(conv_fwd_kernel<T, BM, BN, BK, 1, OneB>, conv_lds_bytes<T, BM, BN, 1, OneB>());
}

template <typename T>
ttamd_status forward_mfma(const ConvPlan &pl, const void *bias, void *out, hipStream_t st) {
    if constexpr (std::is_same_v<T, float>) {
        // unit stride, dense rows and a weight block that fits in LDS: the persistent kernel of conv_patch.hip
        const ConvGeom &g = pl.geo;
        if (g.S == 1 && g.xs_w == 1 && patch_kernel_enabled()) {
            ConvPatchArgs a{};
            a.x = static_cast<const float *>(pl.x);
            a.w = static_cast<const float *>(pl.w);
            a.bias = static_cast<const float *>(bias);
            a.out = static_cast<float *>(out);
            a.B = g.B; a.C = g.C; a.H = g.H; a.W = g.W; a.O = g.O; a.k = g.k; a.P = g.P; a.Ho = g.Ho; a.Wo = g.Wo;
            a.xs_b = g.xs_b; a.xs_c = g.xs_c; a.xs_h = g.xs_h;
            a.w_row = g.w_so; a.w_red = static_cast<int64_t>(g.k) * g.k;  // lanes along the input channels
            a.image_bytes = pl.image_bytes;
            a.weight_bytes = pl.weight_bytes;
            int variant = 0;
            if (ttamd_status s = launch_conv_patch_f32(a, st, &variant)) return s;
            if (variant) {
                t_last_kernel[0] = 0x200 + variant;
                return TTAMD_OK;
            }
        }
    }
    t_last_kernel[0] = 0x100;
    if (pl.geo.O <= 32) return forward_mfma_tile<T, 32, 128>(pl, bias, out, st);
    return forward_mfma_tile<T, 64, 64>(pl, bias, out, st);
}

template <typename T, typename Acc>
ttamd_status forward_direct(const ConvPlan &pl, const void *bias, void *out, hipStream_t st) {
    const ConvGeom &g = pl.geo;
    const int64_t total = static_cast<int64_t>(g.B) * g.O * g.Ho * g.Wo;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) {
        set_error("conv2d: too many workgroups");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    conv_fwd_direct_kernel<T, Acc><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(
        g, static_cast<const T *>(pl.x), static_cast<const T *>(pl.w), static_cast<const T *>(bias), static_cast<T *>(out), total);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

// Images per grad_weight split: one per image unless that would need more than 64 MiB of partial tiles.
int wgrad_group(size_t esz, int B, int C, int O, int k) {
    const int64_t tile_bytes = static_cast<int64_t>(O) * C * k * k * static_cast<int64_t>(esz);
    const int64_t cap = 64LL << 20;
    int64_t max_splits = cap / (tile_bytes > 0 ? tile_bytes : 1);
    if (max_splits < 1) max_splits = 1;
    if (max_splits >= B) return 1;
    return static_cast<int>((B + max_splits - 1) / max_splits);
}

// The dense sub-problems of a strided grad_input and whether this build takes that road: strides 2 and 3, more
// channels than the vector-ALU kernel serves.  Decided by the geometry alone, so that the workspace query and the
// launch agree.  (Each class's packed weight starts on a 16-byte boundary; classes whose rows are whole 8- or 16-byte
// vectors gather with vector loads, the others element by element.)  wt_elems / tmp_elems: workspace elements for the packed weights and the dense class results.
struct DgradClassPlan {
    bool use = false;
    DgradClasses tab{};
    int64_t wt_elems = 0, tmp_elems = 0;
};

DgradClassPlan plan_dgrad_classes(size_t esz, int B, int C, int H, int W, int O, int k, int S, int P) {
    DgradClassPlan pl;
    if (S < 2 || S > kMaxDgradStride || C <= 4) return pl;
    const int vk = esz == 4 ? 4 : 2;
    for (int ry = 0; ry < S; ++ry)
        for (int rx = 0; rx < S; ++rx) {
            DgradClass &c = pl.tab.cls[ry * S + rx];
            c.ry = ry;
            c.rx = rx;
            c.kp = ry < k ? (k - ry + S - 1) / S : 0;
            c.kq = rx < k ? (k - rx + S - 1) / S : 0;
            c.y0 = ((ry - P) % S + S) % S;
            c.x0 = ((rx - P) % S + S) % S;
            c.Hc = c.y0 < H ? (H - c.y0 + S - 1) / S : 0;
            c.Wc = c.x0 < W ? (W - c.x0 + S - 1) / S : 0;
            c.ay = (c.y0 + P - ry) / S;
            c.ax = (c.x0 + P - rx) / S;
            c.wt_off = pl.wt_elems;
            c.tmp_off = pl.tmp_elems;
            const int64_t kc = static_cast<int64_t>(O) * c.kp * c.kq;
            pl.wt_elems += (static_cast<int64_t>(C) * kc + vk - 1) / vk * vk;
            pl.tmp_elems += static_cast<int64_t>(B) * C * c.Hc * c.Wc;
        }
    pl.use = true;
    return pl;
}

// Workspace layout of conv2d_backward: the transposed weight [C, O*k*k] (rounded up to 256 bytes), then, when
// grad_weight is computed in several parts, `parts` partial [O, C*k*k] tiles.  A part is (group of images,
// slice of the output positions): enough of them to give every compute unit a few workgroups.
struct BackwardWorkspace {
    size_t wt_bytes, partial_bytes;  // wt_bytes: the weight area plus, for a strided grad_input in classes, their dense results
    size_t class_tmp_offset;         // byte offset of those results (0: not used)
    int group, splits;     // images per group, number of groups
    int kslices, k_chunk;  // slices of the Ho*Wo reduction, positions per slice (a multiple of the k tile)
    size_t bias_bytes;     // per-part sums of grad_bias: kBiasGradParts rows of O elements
    int parts() const { return splits * kslices; }
    size_t total() const { return wt_bytes + partial_bytes + bias_bytes; }
};

// grad_bias is summed in at most this many parts per channel (about 2048 workgroups per launch, see bias_grad_parts).
constexpr int kBiasGradParts = 256;

// Number of parts for a channel's `vectors` loads: about 2048 workgroups in all, at least 512 loads per part.
inline int bias_grad_parts(int O, int64_t vectors) {
    int64_t parts = (2048 + O - 1) / O;
    if (parts > vectors / 512) parts = vectors / 512;
    if (parts > kBiasGradParts) parts = kBiasGradParts;
    return parts < 1 ? 1 : static_cast<int>(parts);
}

// wgrad_padded: grad_weight numbers its reduction over padded rows (wgrad_pads_rows and a unit column stride of the
// input); the workspace query, which does not see the strides, takes the larger of the two plans.
bool wgrad_pads_rows(size_t esz, int H, int W, int k, int stride, int padding) {
    return stride == 1 && padded_row_width(esz, (W + 2 * padding - k) / stride + 1) != 0;
}

// Images of at most this many k tiles (their positions numbered over rows of whole vectors) go through grad_weight's
// reduction several at a time.
constexpr int kJointTiles = 4;

// Positions per image in that joint reduction (whole k tiles), or 0 where it does not apply.
int wgrad_joint_positions(size_t esz, int H, int W, int k, int stride, int padding) {
    if (stride != 1) return 0;
    const int Ho = H + 2 * padding - k + 1, Wo = W + 2 * padding - k + 1;
    const int vk = static_cast<int>(16 / esz), bk = esz == 4 ? 32 : 16;
    const int row = Wo % vk == 0 ? Wo : padded_row_width(esz, Wo);
    if (row == 0) return 0;
    const int tiles = (Ho * row + bk - 1) / bk;
    return tiles <= kJointTiles ? tiles * bk : 0;
}

// wgrad_mode: 0 positions as they are, 1 over padded rows, 2 over rows of whole vectors with several images per reduction.
BackwardWorkspace backward_workspace(size_t esz, int B, int C, int H, int W, int O, int k, int stride, int padding, int wgrad_mode) {
    const bool wgrad_padded = wgrad_mode == 1;
    BackwardWorkspace w{};
    const size_t tile = static_cast<size_t>(O) * C * k * k * esz;
    w.wt_bytes = (tile + 255) & ~static_cast<size_t>(255);
    if (const DgradClassPlan dc = plan_dgrad_classes(esz, B, C, H, W, O, k, stride, padding); dc.use) {
        const size_t packed = static_cast<size_t>(dc.wt_elems) * esz;
        w.class_tmp_offset = ((packed > tile ? packed : tile) + 255) & ~static_cast<size_t>(255);
        w.wt_bytes = w.class_tmp_offset + ((static_cast<size_t>(dc.tmp_elems) * esz + 255) & ~static_cast<size_t>(255));
    }
    w.group = wgrad_group(esz, B, C, O, k);
    w.splits = (B + w.group - 1) / w.group;
    const int bk = esz == 4 ? 32 : 16;
    const int Ho = (H + 2 * padding - k) / stride + 1, Wo = (W + 2 * padding - k) / stride + 1;
    const int64_t K = static_cast<int64_t>(Ho) * (wgrad_padded ? padded_row_width(esz, Wo) : Wo);
    const int64_t k_tiles = (K + bk - 1) / bk;
    const int64_t tiles = static_cast<int64_t>((O + 63) / 64) * ((static_cast<int64_t>(C) * k * k + 63) / 64);
    // Slices of the reduction: the launch is as slow as its busiest CU, which runs ceil(workgroups / 256) of them,
    // each through its k tiles plus about three tiles' worth of prologue and epilogue; every part adds one tile to
    // the sum that follows.  Costs in microseconds: ~0.6 per k tile of a 64 x 64 workgroup that shares its CU,
    // ~4 MB per microsecond for the partial tiles.  At least 4 k tiles per slice, partial tiles <= 64 MiB.
    int64_t max_slices = k_tiles / 4;
    const int64_t room = (64LL << 20) / static_cast<int64_t>(tile ? tile : 1) / w.splits;
    if (max_slices > room) max_slices = room;
    if (max_slices < 1) max_slices = 1;
    int64_t chunk_tiles = k_tiles > 0 ? k_tiles : 1;
    double best = 0;
    for (int64_t want = 1; want <= max_slices; ++want) {
        const int64_t chunk = (k_tiles + want - 1) / want, slices = (k_tiles + chunk - 1) / chunk;
        const int64_t parts = slices * w.splits, wgs = tiles * parts;
        const double cost = static_cast<double>((wgs + 255) / 256) * static_cast<double>(chunk + 3) * 0.6 +
                            (parts > 1 ? static_cast<double>(parts) * static_cast<double>(tile) / 4e6 : 0.0);
        if (want == 1 || cost < best) {
            best = cost;
            chunk_tiles = chunk;
        }
    }
    w.k_chunk = static_cast<int>(chunk_tiles * bk);
    w.kslices = static_cast<int>((k_tiles + chunk_tiles - 1) / chunk_tiles);
    if (w.kslices < 1) w.kslices = 1;
    if (wgrad_mode == 2) {
        // Groups of images instead of slices of one: same cost model, a workgroup runs its group's k tiles in one go.
        // A group's grad_out and (dense) input stay inside the 2 GiB that one buffer descriptor addresses.
        const int joint_k = wgrad_joint_positions(esz, H, W, k, stride, padding);
        const int64_t tpi = joint_k / bk;
        const int64_t image_bytes = static_cast<int64_t>(esz) * (static_cast<int64_t>(O) * Ho * Wo > static_cast<int64_t>(C) * H * W
                                                                      ? static_cast<int64_t>(O) * Ho * Wo : static_cast<int64_t>(C) * H * W);
        int64_t max_group = (0x7fffffffLL / (image_bytes ? image_bytes : 1)) - 1;
        if (max_group < 1) max_group = 1;
        int64_t max_parts = (64LL << 20) / static_cast<int64_t>(tile ? tile : 1);
        if (max_parts < 1) max_parts = 1;
        int best_group = 0;
        for (int64_t want = 1; want <= B; ++want) {
            const int64_t group = (B + want - 1) / want, parts = (B + group - 1) / group;
            if (group > max_group || parts > max_parts) continue;
            const double cost = static_cast<double>((tiles * parts + 255) / 256) * static_cast<double>(group * tpi + 3) * 0.6 +
                                (parts > 1 ? static_cast<double>(parts) * static_cast<double>(tile) / 4e6 : 0.0);
            if (best_group == 0 || cost < best) {
                best = cost;
                best_group = static_cast<int>(group);
            }
        }
        if (best_group == 0) best_group = static_cast<int>(max_group < B ? max_group : B);
        w.group = best_group;
        w.splits = (B + w.group - 1) / w.group;
        w.kslices = 1;
        w.k_chunk = joint_k;
    }
    w.partial_bytes = w.parts() > 1 ? static_cast<size_t>(w.parts()) * tile : 0;
    if (esz == 4) {  // the LDS-staged grad_weight kernel writes one partial tile per workgroup
        const ConvWgradPatchPlan pp = plan_conv_wgrad_patch(B, C, H, W, O, k, stride, padding);
        if (pp.use && pp.workgroups > 1 && static_cast<size_t>(pp.workgroups) * tile > w.partial_bytes) w.partial_bytes = static_cast<size_t>(pp.workgroups) * tile;
    }
    w.partial_bytes = (w.partial_bytes + 255) & ~static_cast<size_t>(255);
    w.bias_bytes = static_cast<size_t>(kBiasGradParts) * O * esz;
    return w;
}

// Layers with at most this many input channels compute grad_input with conv_dgrad_slots_kernel when a position lies
// in at most 4 x 4 windows and the weights fit 64 KiB of LDS (7x7 stride-2 RGB stem on 224 x 224, batch 32: 0.3 ms
// against 7.3 ms on the padded MFMA tile; 3x3 stride-1 first layers of 28 x 28 and 32 x 32 images: 10 - 25 % faster).
constexpr int kDirectDgradChannels = 4;

// TTAMD_CONV_RIDE=0: every small job of a backward pass as a launch of its own (for comparisons).
bool conv_rides_enabled() {
    static const bool on = std::getenv("TTAMD_CONV_RIDE") == nullptr || std::atoi(std::getenv("TTAMD_CONV_RIDE")) != 0;
    return on;
}

template <typename T>
ttamd_status backward_mfma(const ConvPlan &pl, const void *gout, void *gin, void *gw, void *gb, void *ws, size_t ws_bytes,
                           hipStream_t st) {
    constexpr int BK = ConvTiles<T>::BK, VK = Mfma<T>::VK;
    const ConvGeom &g = pl.geo;
    const int HoWo = g.Ho * g.Wo;
    int wgrad_mode = g.xs_w == 1 && wgrad_pads_rows(sizeof(T), g.H, g.W, g.k, g.S, g.P) ? 1 : 0;
    const int joint_k = g.xs_w == 1 ? wgrad_joint_positions(sizeof(T), g.H, g.W, g.k, g.S, g.P) : 0;
    if (joint_k) {
        const BackwardWorkspace jp = backward_workspace(sizeof(T), g.B, g.C, g.H, g.W, g.O, g.k, g.S, g.P, 2);
        // the group's input images under one descriptor, the image behind the last one addressable too
        if ((static_cast<int64_t>(jp.group) + 1) * g.xs_b * static_cast<int64_t>(sizeof(T)) < 0x7fffffffLL) wgrad_mode = 2;
    }
    const bool wgrad_padded = wgrad_mode != 0;
    const BackwardWorkspace plan = backward_workspace(sizeof(T), g.B, g.C, g.H, g.W, g.O, g.k, g.S, g.P, wgrad_mode);
    if (!ws || ws_bytes < plan.total()) {
        set_error("conv2d_backward: workspace of %zu bytes is smaller than the %zu bytes required", ws_bytes, plan.total());
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    T *const wt = static_cast<T *>(ws);
    T *const partials = reinterpret_cast<T *>(static_cast<char *>(ws) + plan.wt_bytes);
    // grad_bias's parts first (they need grad_out alone): their sum can then ride in grad_input's launch
    int bias_parts_to_add = 0;
    T *bias_sums = nullptr;
    if (gb) {
        using V = std::conditional_t<sizeof(T) == 4, float4, double2>;
        const bool vec = rows_vectorizable<T>(gout, HoWo, static_cast<int64_t>(g.O) * HoWo);
        const int per_image = vec ? HoWo / VK : HoWo;
        const int64_t total = static_cast<int64_t>(g.B) * per_image;
        if (total > 0x7fffffff || g.O > 65535) {
            set_error("conv2d_backward: grad_bias over %lld loads per channel and %d channels exceeds the launch limits",
                      static_cast<long long>(total), g.O);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        const int bparts = bias_grad_parts(g.O, total);
        const uint32_t chunk = static_cast<uint32_t>((total + bparts - 1) / bparts);
        bias_sums = bparts > 1 ? reinterpret_cast<T *>(static_cast<char *>(ws) + plan.wt_bytes + plan.partial_bytes) : static_cast<T *>(gb);
        const dim3 grid(static_cast<unsigned>(g.O), static_cast<unsigned>(bparts));
        const FastDiv d = make_fastdiv(static_cast<uint32_t>(per_image));
        if (vec)
            bias_grad_kernel<T, V><<<grid, dim3(256), 0, st>>>(static_cast<const T *>(gout), bias_sums, g.O, HoWo, static_cast<uint32_t>(total), chunk, d);
        else
            bias_grad_kernel<T, T><<<grid, dim3(256), 0, st>>>(static_cast<const T *>(gout), bias_sums, g.O, HoWo, static_cast<uint32_t>(total), chunk, d);
        TTAMD_HIP_CHECK(hipGetLastError());
        if (bparts > 1) bias_parts_to_add = bparts;
    }
    // grad_weight by the LDS-staged kernel goes first where it applies: the sum over its partial tiles can then ride in
    // grad_input's launch (ConvPatchArgs::red_*) instead of one of its own.
    bool wgrad_staged = false;
    int parts_to_add = 0;  // partial tiles of grad_weight that still wait to be added up
    t_last_kernel[3] = 0;
    const int64_t gw_elems = static_cast<int64_t>(g.O) * g.C * g.k * g.k;
    if constexpr (std::is_same_v<T, float>) {
        // unit stride, channel counts that are multiples of 32, rows of whole vectors: both operands staged in LDS
        if (g.xs_w == 1 && patch_kernel_enabled()) {
            const ConvWgradPatchPlan pp = plan_conv_wgrad_patch(g.B, g.C, g.H, g.W, g.O, g.k, g.S, g.P);
            if (pp.use) {
                ConvWgradPatchArgs a{};
                a.gout = static_cast<const float *>(gout);
                a.x = static_cast<const float *>(pl.x);
                a.partial = pp.workgroups > 1 ? partials : static_cast<float *>(gw);
                a.B = g.B; a.C = g.C; a.H = g.H; a.W = g.W; a.O = g.O; a.k = g.k; a.P = g.P; a.Ho = g.Ho; a.Wo = g.Wo;
                a.xs_b = g.xs_b; a.xs_c = g.xs_c; a.xs_h = g.xs_h;
                a.image_bytes = pl.image_bytes;
                if (ttamd_status rc = launch_conv_wgrad_patch_f32(a, pp, st, &wgrad_staged)) return rc;
                if (wgrad_staged && pp.workgroups > 1) parts_to_add = pp.workgroups;
            }
        }
    }
    // grad_weight on the implicit-GEMM kernel, with `ride` appended to its grid; leaves its partial tiles (if any) in
    // parts_to_add for whoever adds them up.
    t_last_kernel[2] = wgrad_staged ? 0x200 : 0x100;
    bool wgrad_done = wgrad_staged;
    auto wgrad_implicit = [&](const ConvRide &ride, const DgradClasses &classes = DgradClasses{}) -> ttamd_status {
        const int M_ = g.O, N_ = g.C * g.k * g.k;
        const int parts = plan.parts();
        T *const partial = parts > 1 ? partials : static_cast<T *>(gw);
        const int tiles_m = (M_ + 63) / 64, tiles_n = (N_ + 63) / 64;
        const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * parts;
        const bool a_vec = rows_vectorizable<T>(gout, HoWo, static_cast<int64_t>(g.O) * HoWo);
        const bool b_vec = g.S == 1 && g.xs_w == 1 && g.Wo % VK == 0;
        ConvGeom gw_geo = g;
        if (wgrad_padded) {
            gw_geo.row_pad = g.Wo % VK == 0 ? g.Wo : padded_row_width(sizeof(T), g.Wo);  // whole vectors already: joint mode only
            gw_geo.d_row_pad = make_fastdiv(static_cast<uint32_t>(gw_geo.row_pad));
        }
        auto go = [&](auto kernel, size_t lds) {
            return launch_conv(kernel, lds, blocks + ride.blocks, st, gw_geo, static_cast<const T *>(gout), static_cast<const T *>(pl.x), partial,
                               pl.image_bytes, plan.group, plan.kslices, plan.k_chunk, tiles_m, tiles_n, wgrad_mode == 2 ? joint_k : 0, ride, classes);
        };
        using VecB = TapStagerKC<T, 64, BK, VK, kConvPF>;
        using OneB = Im2colTStager<T, 64, BK, kConvPF>;
        ttamd_status s;
        bool pair = false;
        if constexpr (sizeof(T) == 4) pair = a_vec && !b_vec && g.S == 1 && g.xs_w == 1 && g.Wo % 2 == 0;
        using PaddedB = TapStagerKC<T, 64, BK, VK, kConvPF, true>;
        if (wgrad_padded) s = go(conv_wgrad_kernel<T, BK, VK, PaddedB, true>, conv_lds_bytes<T, 64, 64, VK, PaddedB>());
        else if (a_vec && b_vec) s = go(conv_wgrad_kernel<T, BK, VK, VecB>, conv_lds_bytes<T, 64, 64, VK, VecB>());
        else if (pair) {
            if constexpr (sizeof(T) == 4) {
                using PairB = TapStagerKC<T, 64, BK, 2, kConvPF>;
                s = go(conv_wgrad_kernel<T, BK, VK, PairB>, conv_lds_bytes<T, 64, 64, VK, PairB>());
            } else {
                s = TTAMD_OK;
            }
        } else if (a_vec) s = go(conv_wgrad_kernel<T, BK, VK, OneB>, conv_lds_bytes<T, 64, 64, VK, OneB>());
        else if (b_vec) s = go(conv_wgrad_kernel<T, BK, 1, VecB>, conv_lds_bytes<T, 64, 64, 1, VecB>());
        else s = go(conv_wgrad_kernel<T, BK, 1, OneB>, conv_lds_bytes<T, 64, 64, 1, OneB>());
        if (s) return s;
        wgrad_done = true;
        if (parts > 1) parts_to_add = parts;
        return TTAMD_OK;
    };
    // the sum over grad_weight's partial tiles as a job appended to another launch, where vectors of 16 bytes can carry it
    auto sum_ride = [&]() {
        ConvRide r;
        if (!conv_rides_enabled()) return r;
        constexpr int VEC = 16 / static_cast<int>(sizeof(T));
        if (parts_to_add > 0 && gw_elems % VEC == 0 && reinterpret_cast<uintptr_t>(gw) % 16 == 0 && reinterpret_cast<uintptr_t>(partials) % 16 == 0 &&
            parts_to_add * gw_elems * static_cast<int64_t>(sizeof(T)) < 0x7fffffffLL) {
            r.kind = 1;
            r.blocks = static_cast<int>((gw_elems / VEC + 63) / 64);
            r.src = partials;
            r.dst = gw;
            r.n = static_cast<int>(gw_elems);
            r.splits = parts_to_add;
        }
        if (bias_parts_to_add > 0 && g.O % VEC == 0 && reinterpret_cast<uintptr_t>(gb) % 16 == 0 && reinterpret_cast<uintptr_t>(bias_sums) % 16 == 0) {
            r.kind = 1;
            r.blocks2 = (g.O / VEC + 63) / 64;
            r.blocks += r.blocks2;
            r.src2 = bias_sums;
            r.dst2 = gb;
            r.n2 = g.O;
            r.splits2 = bias_parts_to_add;
        }
        return r;
    };
    // (what a launch has taken along is no longer pending)
    auto rode = [&](const ConvRide &r) {
        if (r.kind != 1) return;
        if (r.blocks > r.blocks2) parts_to_add = 0, t_last_kernel[3] = 2;
        if (r.blocks2 > 0) bias_parts_to_add = 0;
    };
    // grad_input
    t_last_kernel[1] = 0;
    const int np = (g.k + g.S - 1) / g.S;
    const size_t slots_lds = static_cast<size_t>(g.O) * g.k * g.k * g.C * sizeof(T);
    if (g.C <= kDirectDgradChannels && np <= 4 && slots_lds <= 64 * 1024) {
        // grad_weight first: the sums over its partial tiles and grad_bias's parts ride in grad_input's launch
        if (!wgrad_done)
            if (ttamd_status rc = wgrad_implicit(ConvRide{})) return rc;
        const ConvRide sum = sum_ride();
        const size_t ride_lds = sum.kind ? kThreads / 64 * 64 * 16 : 0;  // add_up_parts: a 16-byte vector per lane
        const int bpi = (g.H * g.W + 255) / 256;
        const int64_t blocks = static_cast<int64_t>(g.B) * bpi;
        auto go = [&](auto kernel) -> ttamd_status {
            return launch_conv(kernel, slots_lds > ride_lds ? slots_lds : ride_lds, blocks + sum.blocks, st, g, static_cast<const T *>(gout),
                               static_cast<const T *>(pl.w), static_cast<T *>(gin), bpi, sum);
        };
        auto by_windows = [&]<int CMAX>() -> ttamd_status {  // CMAX = C: no padded channel is multiplied
            if (g.S == 1) {  // np == k: the weights are wave-uniform scalars, no LDS copy
                auto unit = [&](auto kernel) -> ttamd_status {
                    return launch_conv(kernel, ride_lds, blocks + sum.blocks, st, g, static_cast<const T *>(gout), static_cast<const T *>(pl.w),
                                       static_cast<T *>(gin), bpi, sum);
                };
                if (np == 1) return unit(conv_dgrad_slots_kernel<T, CMAX, 1, true>);
                if (np == 2) return unit(conv_dgrad_slots_kernel<T, CMAX, 2, true>);
                if (np == 3) return unit(conv_dgrad_slots_kernel<T, CMAX, 3, true>);
                return unit(conv_dgrad_slots_kernel<T, CMAX, 4, true>);
            }
            if (np == 1) return go(conv_dgrad_slots_kernel<T, CMAX, 1>);
            if (np == 2) return go(conv_dgrad_slots_kernel<T, CMAX, 2>);
            if (np == 3) return go(conv_dgrad_slots_kernel<T, CMAX, 3>);
            return go(conv_dgrad_slots_kernel<T, CMAX, 4>);
        };
        static_assert(kDirectDgradChannels == 4, "one instantiation per channel count");
        ttamd_status rc;
        if (g.C == 1) rc = by_windows.template operator()<1>();
        else if (g.C == 2) rc = by_windows.template operator()<2>();
        else if (g.C == 3) rc = by_windows.template operator()<3>();
        else rc = by_windows.template operator()<4>();
        if (rc) return rc;
        rode(sum);
    } else {
        // One unit-stride (or, without the class split, strided) grad_input GEMM: geometry gg, transposed weight wts
        // [C, O*kh*kw], dense result dst [B, C, gg.H*gg.W].
        auto dgrad_gemm = [&](const ConvGeom &gg, const T *wts, T *dst, const ConvRide &ride = ConvRide{}) -> ttamd_status {
          const int Kd = gg.O * gg.kh * gg.kw;
          auto run = [&]<int BM, int BN, bool SC>() -> ttamd_status {
            ConvGeom g = gg;
            const T *wt = wts;
            T *gin = dst;
            const bool a_vec = rows_vectorizable<T>(wt, Kd, 0);
            const bool table_ok = g.kh * g.kw <= kTapTableEntries;
            if (a_vec && table_ok && g.S == 1) {
                g.row_pad = padded_row_width(sizeof(T), g.W);
                g.d_row_pad = make_fastdiv(static_cast<uint32_t>(g.row_pad ? g.row_pad : 1));
            }
            const int M_ = g.C, N_ = g.H * (g.row_pad ? g.row_pad : g.W);
            const int tiles_m = (M_ + BM - 1) / BM, tiles_n = (N_ + BN - 1) / BN;
            const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.B;
            const bool b_vec = table_ok && g.S == 1 && (g.row_pad || g.W % VK == 0);
            auto go = [&](auto kernel, size_t lds) {
                return launch_conv(kernel, lds, blocks + ride.blocks, st, g, static_cast<const T *>(gout), static_cast<const T *>(wt),
                                   static_cast<T *>(gin), tiles_m, tiles_n, ride);
            };
            using VecB = TapStagerMC<T, BN, BK, VK, true, kConvPF>;
            using OneB = DgradStager<T, BN, BK, kConvPF>;
            if (a_vec && b_vec) return go(conv_dgrad_kernel<T, BM, BN, BK, VK, VecB, SC>, conv_lds_bytes<T, BM, BN, VK, VecB>());
            if constexpr (sizeof(T) == 4) {
                using PairB = TapStagerMC<T, BN, BK, 2, true, kConvPF>;
                if (a_vec && table_ok && g.S == 1 && g.W % 2 == 0)
                    return go(conv_dgrad_kernel<T, BM, BN, BK, VK, PairB, SC>, conv_lds_bytes<T, BM, BN, VK, PairB>());
            }
            if (a_vec) return go(conv_dgrad_kernel<T, BM, BN, BK, VK, OneB, SC>, conv_lds_bytes<T, BM, BN, VK, OneB>());
            if (b_vec) return go(conv_dgrad_kernel<T, BM, BN, BK, 1, VecB, SC>, conv_lds_bytes<T, BM, BN, 1, VecB>());
            return go(conv_dgrad_kernel<T, BM, BN, BK, 1, OneB, SC>, conv_lds_bytes<T, BM, BN, 1, OneB>());
          };
          if (gg.sc_S) return gg.C <= 32 ? run.template operator()<32, 128, true>() : run.template operator()<64, 64, true>();
          return gg.C <= 32 ? run.template operator()<32, 128, false>() : run.template operator()<64, 64, false>();
        };
        t_last_kernel[1] = 0x100;
        const DgradClassPlan dc = plan_dgrad_classes(sizeof(T), g.B, g.C, g.H, g.W, g.O, g.k, g.S, g.P);
        if (dc.use) {
            T *const tmp = reinterpret_cast<T *>(static_cast<char *>(ws) + plan.class_tmp_offset);
            // Every class's weights in one launch (an empty class has no elements).  When every class has taps, every
            // element of grad_input belongs to a class that writes it and the classes store straight into grad_input;
            // otherwise (k < S) they go to dense buffers and dgrad_interleave_kernel adds the zeros.
            int most = 0;
            bool every_class_has_taps = true;
            for (int ci = 0; ci < g.S * g.S; ++ci) {
                const DgradClass &cl = dc.tab.cls[ci];
                most = std::max(most, g.C * g.O * cl.kp * cl.kq);
                if (cl.kp == 0 || cl.kq == 0) every_class_has_taps = false;
            }
            // grad_weight first, the packing of the class weights appended to its grid; the sums over its partial tiles and
            // grad_bias's parts then ride in the classes' launch
            if (!wgrad_done && conv_rides_enabled()) {
                ConvRide pack;
                pack.kind = 3;
                pack.splits = (most + kThreads - 1) / kThreads;  // workgroups per class
                pack.blocks = pack.splits * g.S * g.S;
                pack.src = pl.w;
                pack.dst = wt;
                if (ttamd_status rc = wgrad_implicit(pack, dc.tab)) return rc;
            } else {
                weight_class_pack_kernel<T><<<dim3((most + 255) / 256, g.S * g.S), dim3(256), 0, st>>>(g, static_cast<const T *>(pl.w), wt, dc.tab);
                TTAMD_HIP_CHECK(hipGetLastError());
            }
            ConvRide sum = sum_ride();
            auto class_geometry = [&](const DgradClass &cl) {
                ConvGeom gc = g;  // the class as a unit-stride problem over its own positions
                gc.H = cl.Hc;
                gc.W = cl.Wc;
                gc.S = 1;
                gc.kh = cl.kp;
                gc.kw = cl.kq;
                gc.Ph = cl.ay;
                gc.Pw = cl.ax;
                gc.d_kk = make_fastdiv(static_cast<uint32_t>(cl.kp * cl.kq));
                gc.d_k = make_fastdiv(static_cast<uint32_t>(cl.kq));
                gc.d_W = make_fastdiv(static_cast<uint32_t>(cl.Wc));
                gc.d_S = make_fastdiv(1u);
                if (every_class_has_taps) {
                    gc.sc_S = g.S;
                    gc.sc_y0 = cl.y0;
                    gc.sc_x0 = cl.x0;
                    gc.sc_H = g.H;
                    gc.sc_W = g.W;
                }
                return gc;
            };
            // One launch for all classes when each of them takes the 16-byte gathers on both operands (the usual case:
            // class rows of whole vectors, or padded to them); otherwise a launch per class.
            bool merged = false;
            if (every_class_has_taps && merged_dgrad_classes_enabled()) {
                DgradClassGeoms tab{};
                const int BM = g.C <= 32 ? 32 : 64, BN = g.C <= 32 ? 128 : 64;
                int64_t blocks = 0;
                bool ok = true;
                for (int ci = 0; ci < g.S * g.S && ok; ++ci) {
                    const DgradClass &cl = dc.tab.cls[ci];
                    if (cl.Hc == 0 || cl.Wc == 0) continue;
                    ConvGeom gc = class_geometry(cl);
                    const int Kd = gc.O * gc.kh * gc.kw;
                    gc.row_pad = padded_row_width(sizeof(T), gc.W);
                    gc.d_row_pad = make_fastdiv(static_cast<uint32_t>(gc.row_pad ? gc.row_pad : 1));
                    ok = rows_vectorizable<T>(wt + cl.wt_off, Kd, 0) && (gc.row_pad || gc.W % VK == 0) && gc.kh * gc.kw <= kTapTableEntries;
                    const int N_ = gc.H * (gc.row_pad ? gc.row_pad : gc.W);
                    const int i = tab.n++;
                    tab.geo[i] = gc;
                    tab.wt_off[i] = cl.wt_off;
                    tab.tiles_m[i] = (gc.C + BM - 1) / BM;
                    tab.tiles_n[i] = (N_ + BN - 1) / BN;
                    tab.first_block[i] = static_cast<int>(blocks);
                    blocks += static_cast<int64_t>(tab.tiles_m[i]) * tab.tiles_n[i] * g.B;
                    ok = ok && blocks < 0x7fffffff;
                    tab.first_block[i + 1] = static_cast<int>(blocks);
                }
                if (ok && tab.n > 0) {
                    auto go = [&](auto kernel, size_t lds) {
                        return launch_conv(kernel, lds, blocks + sum.blocks, st, tab, static_cast<const T *>(gout), static_cast<const T *>(wt), static_cast<T *>(gin), sum);
                    };
                    ttamd_status rc;
                    if (g.C <= 32) {
                        using VecB = TapStagerMC<T, 128, BK, VK, true, kConvPF>;
                        rc = go(conv_dgrad_classes_kernel<T, 32, 128, BK, VK, VecB>, conv_lds_bytes<T, 32, 128, VK, VecB>());
                    } else {
                        using VecB = TapStagerMC<T, 64, BK, VK, true, kConvPF>;
                        rc = go(conv_dgrad_classes_kernel<T, 64, 64, BK, VK, VecB>, conv_lds_bytes<T, 64, 64, VK, VecB>());
                    }
                    if (rc) return rc;
                    merged = true;
                    t_last_kernel[1] = 0x101;
                    rode(sum);
                    sum = ConvRide{};
                }
            }
            for (int ci = 0; ci < g.S * g.S && !merged; ++ci) {
                const DgradClass &cl = dc.tab.cls[ci];
                if (cl.kp == 0 || cl.kq == 0 || cl.Hc == 0 || cl.Wc == 0) continue;
                const ConvGeom gc = class_geometry(cl);
                if (ttamd_status rc = dgrad_gemm(gc, wt + cl.wt_off, every_class_has_taps ? static_cast<T *>(gin) : tmp + cl.tmp_off, sum)) return rc;
                rode(sum);  // (the first class's launch takes the sums along)
                sum = ConvRide{};
            }
            if (!every_class_has_taps) {
                const int64_t total = static_cast<int64_t>(g.B) * g.C * g.H * g.W;
                const int64_t blocks = (total + 255) / 256;
                if (blocks > 0x7fffffff) {
                    set_error("conv2d_backward: too many workgroups");
                    return TTAMD_ERR_INVALID_ARGUMENT;
                }
                dgrad_interleave_kernel<T><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(g, tmp, static_cast<T *>(gin), dc.tab, total);
                TTAMD_HIP_CHECK(hipGetLastError());
            }
        } else {
            // Unit stride.  grad_input is the convolution of grad_out with the reversed taps, padding k - 1 - P and the
            // weight's two channel axes exchanged: the persistent kernel of conv_patch.hip reads the weight in that order
            // itself (no transposed copy) where its geometry fits; the implicit-GEMM kernel reads a transposed copy.
            // grad_weight goes first: the transposition then rides in its launch, and the sum over its partial tiles in
            // grad_input's.
            ConvPatchArgs a{};
            bool resident = false;
            if constexpr (std::is_same_v<T, float>) {
                if (g.S == 1 && g.kh == g.k && g.kw == g.k && g.P < g.k && patch_kernel_enabled()) {
                    a.x = static_cast<const float *>(gout);
                    a.w = static_cast<const float *>(pl.w);
                    a.bias = nullptr;
                    a.out = static_cast<float *>(gin);
                    a.B = g.B; a.C = g.O; a.H = g.Ho; a.W = g.Wo; a.O = g.C; a.k = g.k; a.P = g.k - 1 - g.P; a.Ho = g.H; a.Wo = g.W;
                    a.xs_b = static_cast<int64_t>(g.O) * HoWo; a.xs_c = HoWo; a.xs_h = g.Wo;
                    a.w_row = static_cast<int64_t>(g.k) * g.k; a.w_red = g.w_so; a.w_flip = 1; a.w_rows_fast = 1;
                    a.image_bytes = static_cast<int64_t>(g.O) * HoWo * 4;
                    a.weight_bytes = pl.weight_bytes;
                    int variant = 0;
                    if (ttamd_status rc = launch_conv_patch_f32(a, st, &variant, false)) return rc;  // (only asks)
                    resident = variant != 0;
                }
            }
            const int total = g.C * g.O * g.k * g.k;
            bool transposed = false;
            if (!wgrad_done) {
                ConvRide ride;
                if (!resident && conv_rides_enabled()) {
                    ride.kind = 2;
                    ride.blocks = (total + kThreads - 1) / kThreads;
                    ride.src = pl.w;
                    ride.dst = wt;
                    ride.n = total;
                    transposed = true;
                }
                if (ttamd_status rc = wgrad_implicit(ride)) return rc;
            }
            const ConvRide sum = sum_ride();
            if (resident) {
                if constexpr (std::is_same_v<T, float>) {
                    if (sum.blocks > sum.blocks2) {
                        a.red_partial = static_cast<const float *>(sum.src);
                        a.red_out = static_cast<float *>(sum.dst);
                        a.red_n = sum.n;
                        a.red_splits = sum.splits;
                    }
                    if (sum.blocks2 > 0) {
                        a.red2_partial = static_cast<const float *>(sum.src2);
                        a.red2_out = static_cast<float *>(sum.dst2);
                        a.red2_n = sum.n2;
                        a.red2_splits = sum.splits2;
                    }
                    int variant = 0;
                    if (ttamd_status rc = launch_conv_patch_f32(a, st, &variant)) return rc;
                    t_last_kernel[1] = 0x200 + variant;
                }
            } else {
                if (!transposed) {
                    weight_transpose_kernel<T><<<dim3((total + 255) / 256), dim3(256), 0, st>>>(g, static_cast<const T *>(pl.w), wt, total);
                    TTAMD_HIP_CHECK(hipGetLastError());
                }
                if (ttamd_status rc = dgrad_gemm(g, wt, static_cast<T *>(gin), sum)) return rc;
            }
            rode(sum);
        }
    }
    if (!wgrad_done)
        if (ttamd_status rc = wgrad_implicit(ConvRide{})) return rc;
    if (parts_to_add > 0) {
        if (ttamd_status rc = launch_reduce_splits<T>(partials, static_cast<T *>(gw), gw_elems, parts_to_add, st)) return rc;
        t_last_kernel[3] = 1;
    }
    if (bias_parts_to_add > 0)
        if (ttamd_status rc = launch_reduce_splits<T>(bias_sums, static_cast<T *>(gb), g.O, bias_parts_to_add, st)) return rc;
    return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" {

int ttamd_conv2d_last_kernel(int which) { return which >= 0 && which <= 3 ? ttamd::t_last_kernel[which] : 0; }

ttamd_status ttamd_conv2d_forward(int device, ttamd_dtype dtype, const ttamd_view4 *input, const ttamd_view4 *weight,
                                  const void *bias, void *out, int B, int C, int H, int W, int O, int k, int stride,
                                  int padding, void *stream) {
    ConvPlan pl;
    if (ttamd_status s = make_plan("conv2d", dtype, input, weight, B, C, H, W, O, k, stride, padding, &pl)) return s;
    if (ttamd_status s = use_device(device)) return s;
    t_last_kernel[0] = 0;
    if (B == 0) return TTAMD_OK;
    if (!input->data || !weight->data || !out) {
        set_error("conv2d: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case TTAMD_F32: return forward_mfma<float>(pl, bias, out, st);
    case TTAMD_F64: return forward_mfma<double>(pl, bias, out, st);
    case TTAMD_U8: return forward_direct<uint8_t, uint32_t>(pl, bias, out, st);
    case TTAMD_I16: return forward_direct<int16_t, uint32_t>(pl, bias, out, st);
    case TTAMD_I32: return forward_direct<int32_t, uint32_t>(pl, bias, out, st);
    case TTAMD_I64: return forward_direct<int64_t, uint64_t>(pl, bias, out, st);
    default: break;
    }
    set_error("conv2d does not support dtype code %d", static_cast<int>(dtype));
    return TTAMD_ERR_UNSUPPORTED_DTYPE;
}

ttamd_status ttamd_conv2d_backward_workspace(ttamd_dtype dtype, int B, int C, int H, int W, int O, int k, int stride,
                                             int padding, size_t *bytes) {
    if (!bytes) {
        set_error("conv2d_backward_workspace: bytes is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *bytes = 0;
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("conv2d_backward supports f32 and f64 only (autograd never differentiates integer tensors)");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (B <= 0 || C <= 0 || O <= 0 || k <= 0 || H <= 0 || W <= 0 || stride <= 0 || padding < 0 || H + 2 * padding < k ||
        W + 2 * padding < k)
        return TTAMD_OK;  // ttamd_conv2d_backward rejects the geometry itself
    const size_t esz = dtype_size(dtype);
    *bytes = backward_workspace(esz, B, C, H, W, O, k, stride, padding, 0).total();
    if (wgrad_pads_rows(esz, H, W, k, stride, padding)) {
        const size_t padded = backward_workspace(esz, B, C, H, W, O, k, stride, padding, 1).total();
        if (padded > *bytes) *bytes = padded;
    }
    if (wgrad_joint_positions(esz, H, W, k, stride, padding)) {
        const size_t joint = backward_workspace(esz, B, C, H, W, O, k, stride, padding, 2).total();
        if (joint > *bytes) *bytes = joint;
    }
    return TTAMD_OK;
}

ttamd_status ttamd_conv2d_backward(int device, ttamd_dtype dtype, const void *grad_out, const ttamd_view4 *input,
                                   const ttamd_view4 *weight, void *grad_input, void *grad_weight, void *grad_bias,
                                   int B, int C, int H, int W, int O, int k, int stride, int padding, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("conv2d_backward supports f32 and f64 only (autograd never differentiates integer tensors)");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    ConvPlan pl;
    if (ttamd_status s = make_plan("conv2d_backward", dtype, input, weight, B, C, H, W, O, k, stride, padding, &pl)) return s;
    if (ttamd_status s = use_device(device)) return s;
    if (!grad_weight || !input->data || !weight->data || (B > 0 && (!grad_out || !grad_input))) {
        set_error("conv2d_backward: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (B == 0) {
        // no images: the weight (and bias) gradients are empty sums
        if (ttamd_status s = ttamd_memset_zero(device, grad_weight, static_cast<size_t>(O) * C * k * k * dtype_size(dtype), stream)) return s;
        if (grad_bias) return ttamd_memset_zero(device, grad_bias, static_cast<size_t>(O) * dtype_size(dtype), stream);
        return TTAMD_OK;
    }
    if (dtype == TTAMD_F32) return backward_mfma<float>(pl, grad_out, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, st);
    return backward_mfma<double>(pl, grad_out, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, st);
}

}  // extern "C"
