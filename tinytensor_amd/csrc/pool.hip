// pool.hip — 2-D max / min / average pooling, forward and backward (gfx950).
//
// Stands where BackendBase::{max,min,avg}_pool2d and their *_backward do
// (tinytensor/tensor/backend_base.h:286-311; CPU form tinytensor/tensor/backend/cpu/conv.cpp:296-426 over the
// kernels of tinytensor/tensor/backend/cpu/kernel/conv.hpp:121-275, functors
// tinytensor/tensor/backend/common/kernel/reduce.hpp:28-140).  Both directions are bandwidth-bound streaming
// kernels: one lane per output element forward, one lane per input element (or four) backward.
//
// Forward visits the window in the reference's (p, q) order with the reference's arithmetic
//   max: out = (x > out) ? x : out from lowest();  min: out = (x < out) ? x : out from max();
//   avg: out = (x / n) + out from 0 with n = k*k (padding contributes 0 / n), integer inputs give f32,
// so results are bit-identical.  The input is read through its strides (the reference copies a non-dense input).
//
// Backward is the gather form of the reference's scatter-add: the lane that owns input (y, x) walks the outputs
// whose window contains it in increasing (h, w) — the order in which the reference's loop adds to that
// element — so the sums are bit-identical too, and nothing is written twice (no atomics, no zero-fill pass).
// For max / min a first pass over the outputs computes each output's share (gradient / number of window elements
// equal to the result) into the library's per-stream scratch, so the gather reads two values per covering output
// instead of recounting its window.
// On dense rows of 4n elements with at most 2 x 2 covering windows a lane owns four consecutive elements: it loads
// the block of covering outputs once and moves the input and the gradient as 16-byte vectors.
// For k == 3, stride == 2, padding == 1 on such rows (tests/test_conv.cpp:186-278) forward and the first backward
// pass own one output pair per lane and read their three input rows as vectors, the column between two lanes' vectors
// travelling by wave shuffle.
//
// Non-overlapping windows without padding (stride == k, padding == 0: the max_pool2d(x, 2, 2, 0) of
// examples/mnist_cnn_example.cpp:55) take a shorter road: an input element lies in at most one window, so backward
// is one pass with one lane per output that reads its window once, counts, and writes the window's gradients
// (plus zeros for rows / columns that no window reaches); with k == 2 and even dense rows both directions move
// their rows as 2-element vectors, so a wave reads and writes whole contiguous row segments.
#include "common.h"

#include <cfloat>
#include <climits>
#include <type_traits>

namespace ttamd {
namespace {

enum { POOL_MAX = 0, POOL_MIN = 1, POOL_AVG = 2 };

struct PoolGeom {
    int B, C, H, W, K, S, P, Ho, Wo;
    int64_t xs_b, xs_c, xs_h, xs_w;  // input strides (elements)
    // Work is laid out as (plane = b*C + c, block of 256 positions inside the plane) so that every index fits 32
    // bits and is split with exact multiply-shift division instead of 64-bit division.
    int out_blocks, in_blocks;        // blocks of 256 positions per output / input plane
    int quad_blocks;                  // blocks of 256 groups of four positions per input plane
    int opair_blocks;                 // blocks of 256 pairs of positions per output plane
    FastDiv d_out_blocks, d_in_blocks, d_quad_blocks, d_opair_blocks, d_C, d_Wo, d_W, d_S;
};

template <typename R, int OP>
__device__ __forceinline__ R pool_init() {
    if constexpr (OP == POOL_AVG) return R(0);
    else if constexpr (std::is_floating_point_v<R>) {
        constexpr R big = std::is_same_v<R, float> ? R(FLT_MAX) : R(DBL_MAX);
        return OP == POOL_MAX ? -big : big;
    } else if constexpr (std::is_unsigned_v<R>) {
        return OP == POOL_MAX ? R(0) : static_cast<R>(~R(0));
    } else {
        constexpr R lo = static_cast<R>(R(1) << (sizeof(R) * 8 - 1));
        return OP == POOL_MAX ? lo : static_cast<R>(~lo);
    }
}

// Input plane of (b, c) through the view's strides.
template <typename T>
__device__ __forceinline__ const T *plane_of(const PoolGeom &g, const T *x, uint32_t plane) {
    uint32_t b, c;
    g.d_C.divmod(plane, b, c);
    return x + static_cast<int64_t>(b) * g.xs_b + static_cast<int64_t>(c) * g.xs_c;
}

// KC: the window size when it is known at compile time (2 or 3), else 0.  With a fixed size the window is unrolled:
// all of its loads are issued before the first comparison instead of one load per loop iteration.
template <typename T, typename R, int OP, int KC>
__global__ void __launch_bounds__(256) pool_forward_kernel(PoolGeom g, const T *__restrict__ x, R *__restrict__ out) {
    uint32_t plane, blk;
    g.d_out_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = blk * 256 + threadIdx.x;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const T *src = plane_of(g, x, plane);
    const int K = KC ? KC : g.K;
    const R n = static_cast<R>(K * K);
    R acc = pool_init<R, OP>();
    auto visit = [&](R v) {
        if constexpr (OP == POOL_MAX) acc = (v > acc) ? v : acc;
        else if constexpr (OP == POOL_MIN) acc = (v < acc) ? v : acc;
        else acc = (v / n) + acc;
    };
    const int h0 = g.S * static_cast<int>(h) - g.P, w0 = g.S * static_cast<int>(w) - g.P;
    if constexpr (KC > 0) {
        R v[KC * KC];
#pragma unroll
        for (int p = 0; p < KC; ++p)
#pragma unroll
            for (int q = 0; q < KC; ++q) {
                const int hi = h0 + p, wi = w0 + q;
                const bool in = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
                // clamped address, so that the load needs no branch; the value is replaced when out of bounds
                const int hc = hi < 0 ? 0 : (hi >= g.H ? g.H - 1 : hi), wc = wi < 0 ? 0 : (wi >= g.W ? g.W - 1 : wi);
                const R got = static_cast<R>(src[hc * g.xs_h + wc * g.xs_w]);
                v[p * KC + q] = in ? got : pool_init<R, OP>();
            }
#pragma unroll
        for (int i = 0; i < KC * KC; ++i) visit(v[i]);
    } else {
        for (int p = 0; p < K; ++p) {
            const int hi = h0 + p;
            for (int q = 0; q < K; ++q) {
                const int wi = w0 + q;
                const bool in = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
                visit(in ? static_cast<R>(src[hi * g.xs_h + wi * g.xs_w]) : pool_init<R, OP>());
            }
        }
    }
    out[static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos] = acc;
}

// max / min backward, first pass (one lane per output): share = grad_out / (number of in-bounds window elements
// equal to the result), the amount each of those elements receives from this output (cpu/kernel/conv.hpp:188-203).
template <typename R, int KC>
__global__ void __launch_bounds__(256)
pool_share_kernel(PoolGeom g, const R *__restrict__ gout, const R *__restrict__ x, const R *__restrict__ res, R *__restrict__ share) {
    uint32_t plane, blk;
    g.d_out_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = blk * 256 + threadIdx.x;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const R *src = plane_of(g, x, plane);
    const int64_t o = static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos;
    const R target = res[o];
    const int h0 = g.S * static_cast<int>(h) - g.P, w0 = g.S * static_cast<int>(w) - g.P;
    R count = R(0);
    if constexpr (KC > 0) {  // fixed window: every load issued up front through clamped addresses
        R v[KC * KC];
        bool in[KC * KC];
#pragma unroll
        for (int p = 0; p < KC; ++p)
#pragma unroll
            for (int q = 0; q < KC; ++q) {
                const int hi = h0 + p, wi = w0 + q;
                in[p * KC + q] = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
                const int hc = hi < 0 ? 0 : (hi >= g.H ? g.H - 1 : hi), wc = wi < 0 ? 0 : (wi >= g.W ? g.W - 1 : wi);
                v[p * KC + q] = src[hc * g.xs_h + wc * g.xs_w];
            }
#pragma unroll
        for (int i = 0; i < KC * KC; ++i) count += (in[i] && v[i] == target) ? R(1) : R(0);
    } else {
        for (int p = 0; p < g.K; ++p)
            for (int q = 0; q < g.K; ++q) {
                const int hi = h0 + p, wi = w0 + q;
                const bool in = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
                count += (in && src[hi * g.xs_h + wi * g.xs_w] == target) ? R(1) : R(0);
            }
    }
    share[o] = gout[o] / count;
}

// Backward gather (one lane per input element): adds, in increasing (h, w), what each output whose window
// contains the element hands to it.  SELECT: `share` holds the per-output amounts of pool_share_kernel and only
// outputs whose result equals the element contribute; otherwise `share` is grad_out and every output
// contributes grad_out / (k*k).
// NW: compile-time bound on the outputs per axis whose window can contain one element (ceil(k / stride)) when it
// is 2, else 0 = loop over the run-time range.  With the bound the covering outputs are visited through clamped
// addresses and predicates, all loads issued up front; an output outside the range adds +0.
template <typename R, bool SELECT, int NW>
__global__ void __launch_bounds__(256)
pool_backward_kernel(PoolGeom g, const R *__restrict__ share, const R *__restrict__ x, const R *__restrict__ res, R *__restrict__ gin) {
    uint32_t plane, blk;
    g.d_in_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = blk * 256 + threadIdx.x;
    if (pos >= static_cast<uint32_t>(g.H * g.W)) return;
    uint32_t yh, xw;
    g.d_W.divmod(pos, yh, xw);
    const int64_t obase = static_cast<int64_t>(plane) * (g.Ho * g.Wo);
    const R *splane = share + obase;
    // outputs h with 0 <= yh + P - S*h < K, clipped to [0, Ho)
    const int ay = static_cast<int>(yh) + g.P, ax = static_cast<int>(xw) + g.P;
    int h_lo = ay - g.K >= 0 ? static_cast<int>(g.d_S.div(static_cast<uint32_t>(ay - g.K))) + 1 : 0;
    int w_lo = ax - g.K >= 0 ? static_cast<int>(g.d_S.div(static_cast<uint32_t>(ax - g.K))) + 1 : 0;
    int h_hi = static_cast<int>(g.d_S.div(static_cast<uint32_t>(ay))), w_hi = static_cast<int>(g.d_S.div(static_cast<uint32_t>(ax)));
    h_hi = h_hi >= g.Ho ? g.Ho - 1 : h_hi;
    w_hi = w_hi >= g.Wo ? g.Wo - 1 : w_hi;
    R acc = R(0);
    const R n = static_cast<R>(g.K * g.K);
    R mine = R(0);
    const R *rplane = res + obase;
    if constexpr (SELECT) mine = plane_of(g, x, plane)[static_cast<int64_t>(yh) * g.xs_h + static_cast<int64_t>(xw) * g.xs_w];
    if constexpr (NW > 0) {
        R amount[NW * NW], target[NW * NW];
        bool valid[NW * NW];
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int b = 0; b < NW; ++b) {
                const int h = h_lo + a, w = w_lo + b;
                valid[a * NW + b] = h <= h_hi && w <= w_hi;
                const int hc = h > g.Ho - 1 ? g.Ho - 1 : h, wc = w > g.Wo - 1 ? g.Wo - 1 : w;
                amount[a * NW + b] = splane[hc * g.Wo + wc];
                if constexpr (SELECT) target[a * NW + b] = rplane[hc * g.Wo + wc];
            }
#pragma unroll
        for (int i = 0; i < NW * NW; ++i) {
            if constexpr (SELECT) acc += (valid[i] && mine == target[i]) ? amount[i] : R(0);
            else acc += valid[i] ? amount[i] / n : R(0);
        }
    } else if constexpr (SELECT) {
        for (int h = h_lo; h <= h_hi; ++h)
            for (int w = w_lo; w <= w_hi; ++w) {
                // both loads are issued before the comparison (no dependent second access); an output that does not
                // select this element adds +0, which leaves the running sum's bits unchanged
                const R t = rplane[h * g.Wo + w], amount = splane[h * g.Wo + w];
                acc += (mine == t) ? amount : R(0);
            }
    } else {
        for (int h = h_lo; h <= h_hi; ++h)
            for (int w = w_lo; w <= w_hi; ++w) acc += splane[h * g.Wo + w] / n;
    }
    gin[static_cast<int64_t>(plane) * (g.H * g.W) + pos] = acc;
}

template <typename T>
using Pair = T __attribute__((ext_vector_type(2)));
template <typename T>
using Quad = T __attribute__((ext_vector_type(4)));

// The same gather for four consecutive elements of one input row per lane (W % 4 == 0, dense aligned rows, an
// element in at most 2 x 2 windows).  The outputs that cover the four elements form a block of 2 rows x NC columns
// (NC >= ceil((k + 3) / stride)); their amounts and results are loaded once instead of once per element, the input
// and the gradient move as one vector each, and every element still adds its own covering outputs in increasing
// (h, w), so the sums are the ones pool_backward_kernel produces.
// PAIRS (k == 3, stride == 2, padding == 1, NC == 3): the block's first column is even, so columns 0 and 1 of a
// block row are one aligned pair and column 2 is the first element of the pair that the lane to the right loads (a
// wave's last lane loads it): a wave reads whole contiguous segments of the output rows.
template <typename R, bool SELECT, int NC, bool PAIRS = false>
__global__ void __launch_bounds__(256)
pool_backward_quad_kernel(PoolGeom g, const R *__restrict__ share, const R *__restrict__ x, const R *__restrict__ res, R *__restrict__ gin) {
    uint32_t plane, blk;
    g.d_quad_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = (blk * 256 + threadIdx.x) * 4;
    if (pos >= static_cast<uint32_t>(g.H * g.W)) return;
    uint32_t yh, xw;
    g.d_W.divmod(pos, yh, xw);
    const int64_t obase = static_cast<int64_t>(plane) * (g.Ho * g.Wo);
    const R *splane = share + obase, *rplane = res + obase;
    const int ay = static_cast<int>(yh) + g.P, ax0 = static_cast<int>(xw) + g.P;
    int h_lo, h_hi, c_lo, w_lo[4], w_hi[4];
    if constexpr (PAIRS) {
        // k 3, stride 2, padding 1: row y lies in the windows of output rows y/2 and, for odd y, y/2 + 1; of the four
        // columns 4m .. 4m + 3 the first lies in output column 2m, the second in 2m and 2m + 1, the third in 2m + 1,
        // the fourth in 2m + 1 and 2m + 2 (kCovers below).
        h_lo = static_cast<int>(yh) >> 1;
        h_hi = (static_cast<int>(yh) + 1) >> 1;
        c_lo = static_cast<int>(xw) >> 1;
    } else {
        h_lo = ay - g.K >= 0 ? static_cast<int>(g.d_S.div(static_cast<uint32_t>(ay - g.K))) + 1 : 0;
        h_hi = static_cast<int>(g.d_S.div(static_cast<uint32_t>(ay)));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int ax = ax0 + j;
            w_lo[j] = ax - g.K >= 0 ? static_cast<int>(g.d_S.div(static_cast<uint32_t>(ax - g.K))) + 1 : 0;
            const int hi = static_cast<int>(g.d_S.div(static_cast<uint32_t>(ax)));
            w_hi[j] = hi >= g.Wo ? g.Wo - 1 : hi;
        }
        c_lo = w_lo[0];
    }
    h_hi = h_hi >= g.Ho ? g.Ho - 1 : h_hi;
    R amount[2 * NC], target[2 * NC];
    if constexpr (PAIRS) {
        static_assert(NC == 3, "pairs cover a block of three columns");
        const bool load_right = threadIdx.x % 64 == 63 && c_lo + 2 < g.Wo;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int h = h_lo + a;
            const int row = (h > g.Ho - 1 ? g.Ho - 1 : h) * g.Wo + c_lo;
            const Pair<R> am = *reinterpret_cast<const Pair<R> *>(splane + row);
            R am2 = __shfl_down(am[0], 1);
            if (load_right) am2 = splane[row + 2];
            amount[a * NC] = am[0];
            amount[a * NC + 1] = am[1];
            amount[a * NC + 2] = am2;
            if constexpr (SELECT) {
                const Pair<R> tg = *reinterpret_cast<const Pair<R> *>(rplane + row);
                R tg2 = __shfl_down(tg[0], 1);
                if (load_right) tg2 = rplane[row + 2];
                target[a * NC] = tg[0];
                target[a * NC + 1] = tg[1];
                target[a * NC + 2] = tg2;
            }
        }
    } else {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < NC; ++b) {
                const int h = h_lo + a, w = c_lo + b;
                const int hc = h > g.Ho - 1 ? g.Ho - 1 : h, wc = w > g.Wo - 1 ? g.Wo - 1 : w;
                amount[a * NC + b] = splane[hc * g.Wo + wc];
                if constexpr (SELECT) target[a * NC + b] = rplane[hc * g.Wo + wc];
            }
    }
    Quad<R> mine = {R(0), R(0), R(0), R(0)};
    if constexpr (SELECT)
        mine = *reinterpret_cast<const Quad<R> *>(plane_of(g, x, plane) + static_cast<int64_t>(yh) * g.xs_h + xw);
    if constexpr (!SELECT) {  // every covered element receives grad_out / k^2: divide once per output
        const R n = static_cast<R>(g.K * g.K);
#pragma unroll
        for (int i = 0; i < 2 * NC; ++i) amount[i] = amount[i] / n;
    }
    Quad<R> acc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        R sum = R(0);
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < NC; ++b) {
                const int w = c_lo + b;
                bool valid;
                if constexpr (PAIRS) {
                    constexpr bool kCovers[4][3] = {{true, false, false}, {true, true, false}, {false, true, false}, {false, true, true}};
                    if (!kCovers[j][b < 3 ? b : 0]) continue;  // (an output that does not cover the element would add +0)
                    valid = (h_lo + a <= h_hi) & (w < g.Wo);
                } else {
                    valid = (h_lo + a <= h_hi) & (w >= w_lo[j]) & (w <= w_hi[j]);
                }
                if constexpr (SELECT) sum += (valid && mine[j] == target[a * NC + b]) ? amount[a * NC + b] : R(0);
                else sum += valid ? amount[a * NC + b] : R(0);
            }
        acc[j] = sum;
    }
    *reinterpret_cast<Quad<R> *>(gin + static_cast<int64_t>(plane) * (g.H * g.W) + pos) = acc;
}


// Forward for k == 2, stride == 2, padding == 0 on rows that can be read as aligned pairs (the host checks).
// Same visiting order and arithmetic as pool_forward_kernel.
template <typename T, typename R, int OP>
__global__ void __launch_bounds__(256) pool_forward_k2_kernel(PoolGeom g, const T *__restrict__ x, R *__restrict__ out) {
    uint32_t plane, blk;
    g.d_out_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = blk * 256 + threadIdx.x;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const T *src = plane_of(g, x, plane) + static_cast<int64_t>(2 * h) * g.xs_h + 2 * w;
    const Pair<T> r0 = *reinterpret_cast<const Pair<T> *>(src), r1 = *reinterpret_cast<const Pair<T> *>(src + g.xs_h);
    const R v[4] = {static_cast<R>(r0[0]), static_cast<R>(r0[1]), static_cast<R>(r1[0]), static_cast<R>(r1[1])};
    R acc = pool_init<R, OP>();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (OP == POOL_MAX) acc = (v[i] > acc) ? v[i] : acc;
        else if constexpr (OP == POOL_MIN) acc = (v[i] < acc) ? v[i] : acc;
        else acc = (v[i] / R(4)) + acc;
    }
    out[static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos] = acc;
}

// Forward for k == 3, stride == 2, padding == 1 on dense rows of 4n elements (the host checks): a lane owns the
// output pair (h, 2m), (h, 2m + 1), whose windows span input columns 4m - 1 .. 4m + 3.  It loads columns
// 4m .. 4m + 3 of its three rows as one vector each and takes column 4m - 1 from the lane to its left (a wave's
// first lane loads it), so a wave reads whole contiguous row segments instead of every second element nine times.
// Same visiting order and arithmetic as pool_forward_kernel.
template <typename T, typename R, int OP>
__global__ void __launch_bounds__(256) pool_forward_k3s2_kernel(PoolGeom g, const T *__restrict__ x, R *__restrict__ out) {
    uint32_t plane, blk;
    g.d_opair_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = (blk * 256 + threadIdx.x) * 2;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const T *src = plane_of(g, x, plane);
    const int col = 2 * static_cast<int>(w);  // = 4m
    const bool load_left = threadIdx.x % 64 == 0 && col > 0;
    R v[3][5];
    bool rin[3];
#pragma unroll
    for (int p = 0; p < 3; ++p) {
        const int hi = 2 * static_cast<int>(h) - 1 + p;
        rin[p] = static_cast<unsigned>(hi) < static_cast<unsigned>(g.H);
        const T *row = src + static_cast<int64_t>(hi < 0 ? 0 : (hi >= g.H ? g.H - 1 : hi)) * g.xs_h + col;
        const Quad<T> own = *reinterpret_cast<const Quad<T> *>(row);
        T left = __shfl_up(own[3], 1);
        if (load_left) left = row[-1];
        v[p][0] = static_cast<R>(left);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][1 + j] = static_cast<R>(own[j]);
    }
    const R n = R(9);
    Pair<R> res;
#pragma unroll
    for (int o = 0; o < 2; ++o) {
        R acc = pool_init<R, OP>();
#pragma unroll
        for (int p = 0; p < 3; ++p)
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const bool in = rin[p] && (o == 1 || q > 0 || col > 0);  // only column -1 can be outside (W = 4n)
                const R e = in ? v[p][2 * o + q] : pool_init<R, OP>();
                if constexpr (OP == POOL_MAX) acc = (e > acc) ? e : acc;
                else if constexpr (OP == POOL_MIN) acc = (e < acc) ? e : acc;
                else acc = (e / n) + acc;
            }
        res[o] = acc;
    }
    *reinterpret_cast<Pair<R> *>(out + static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos) = res;
}

// First pass of max / min backward for the same geometry and row layout, one output pair per lane (same loads as
// pool_forward_k3s2_kernel): share = grad_out / (number of in-bounds window elements equal to the result).
template <typename R>
__global__ void __launch_bounds__(256)
pool_share_k3s2_kernel(PoolGeom g, const R *__restrict__ gout, const R *__restrict__ x, const R *__restrict__ res, R *__restrict__ share) {
    uint32_t plane, blk;
    g.d_opair_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = (blk * 256 + threadIdx.x) * 2;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const R *src = plane_of(g, x, plane);
    const int col = 2 * static_cast<int>(w);
    const bool load_left = threadIdx.x % 64 == 0 && col > 0;
    R v[3][5];
    bool rin[3];
#pragma unroll
    for (int p = 0; p < 3; ++p) {
        const int hi = 2 * static_cast<int>(h) - 1 + p;
        rin[p] = static_cast<unsigned>(hi) < static_cast<unsigned>(g.H);
        const R *row = src + static_cast<int64_t>(hi < 0 ? 0 : (hi >= g.H ? g.H - 1 : hi)) * g.xs_h + col;
        const Quad<R> own = *reinterpret_cast<const Quad<R> *>(row);
        R left = __shfl_up(own[3], 1);
        if (load_left) left = row[-1];
        v[p][0] = left;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][1 + j] = own[j];
    }
    const int64_t o0 = static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos;
    const Pair<R> target = *reinterpret_cast<const Pair<R> *>(res + o0), go = *reinterpret_cast<const Pair<R> *>(gout + o0);
    Pair<R> amount;
#pragma unroll
    for (int o = 0; o < 2; ++o) {
        R count = R(0);
#pragma unroll
        for (int p = 0; p < 3; ++p)
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const bool in = rin[p] && (o == 1 || q > 0 || col > 0);
                count += (in && v[p][2 * o + q] == target[o]) ? R(1) : R(0);
            }
        amount[o] = go[o] / count;
    }
    *reinterpret_cast<Pair<R> *>(share + o0) = amount;
}

// max / min backward for k == 3, stride == 2, padding == 1 on dense rows of 4n elements (at most kTileMaxWo output
// columns) in ONE launch: a workgroup owns kTileRows output rows h0 .. of one plane and the 2 * kTileRows input rows
// 2 h0 .. that receive from them.  First its lanes compute the shares of output rows h0 .. h0 + kTileRows (one more
// row than it owns: the last input row also receives from the row below), one output pair per lane with the loads of
// pool_share_k3s2_kernel, into LDS together with the results; after a barrier the lanes take the input rows four
// elements at a time and add the shares of the covering outputs from LDS, in increasing (h, w).  Shares and sums are
// formed exactly as the two kernels form them, but the shares never travel through memory (two launches move 870 MB
// for a [64,64,112,112] f32 input, the input, result and both gradients are 514 MB), and the input rows the second
// step reads were read by the first a moment ago.  (Counting the windows again in every lane that gathers -- no LDS,
// no barrier -- is no faster than the two launches: each share is then computed by some 4.5 lanes and the kernel is
// bound by its comparisons.)
constexpr int kTileRows = 8, kTileMaxWo = 256;

template <typename R>
__global__ void __launch_bounds__(256)
pool_backward_k3s2_tile_kernel(PoolGeom g, int tiles, FastDiv d_tiles, const R *__restrict__ gout, const R *__restrict__ x,
                               const R *__restrict__ res, R *__restrict__ gin) {
    __shared__ R s_share[(kTileRows + 1) * kTileMaxWo], s_target[(kTileRows + 1) * kTileMaxWo];
    uint32_t plane, tile;
    d_tiles.divmod(blockIdx.x, plane, tile);
    const int h0 = static_cast<int>(tile) * kTileRows;
    const R *src = plane_of(g, x, plane);
    const int64_t obase = static_cast<int64_t>(plane) * (g.Ho * g.Wo);
    // 1. shares of output rows h0 .. h0 + kTileRows (those that exist), one pair of outputs per lane and round
    const int out_rows = g.Ho - h0 < kTileRows + 1 ? g.Ho - h0 : kTileRows + 1;
    const uint32_t n_out = static_cast<uint32_t>(out_rows * g.Wo);
    for (uint32_t first = 0; first < n_out; first += 512) {  // (workgroup-uniform bound: every lane shuffles)
        const uint32_t want = first + threadIdx.x * 2;
        const bool live = want < n_out;
        const uint32_t pos = live ? want : n_out - 2;  // a lane beyond the end recomputes the last pair and drops it
        uint32_t hr, w;
        g.d_Wo.divmod(pos, hr, w);
        const int h = h0 + static_cast<int>(hr), col = 2 * static_cast<int>(w);  // col = 4m
        const bool load_left = threadIdx.x % 64 == 0 && col > 0;
        R v[3][5];
        bool rin[3];
#pragma unroll
        for (int p = 0; p < 3; ++p) {
            const int hi = 2 * h - 1 + p;
            rin[p] = static_cast<unsigned>(hi) < static_cast<unsigned>(g.H);
            const R *row = src + static_cast<int64_t>(hi < 0 ? 0 : (hi >= g.H ? g.H - 1 : hi)) * g.xs_h + col;
            const Quad<R> own = *reinterpret_cast<const Quad<R> *>(row);
            R left = __shfl_up(own[3], 1);
            if (load_left) left = row[-1];
            v[p][0] = left;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[p][1 + j] = own[j];
        }
        const int64_t o0 = obase + static_cast<int64_t>(h) * g.Wo + w;
        const Pair<R> target = *reinterpret_cast<const Pair<R> *>(res + o0), go = *reinterpret_cast<const Pair<R> *>(gout + o0);
#pragma unroll
        for (int o = 0; o < 2; ++o) {
            R count = R(0);
#pragma unroll
            for (int p = 0; p < 3; ++p)
#pragma unroll
                for (int q = 0; q < 3; ++q) {
                    const bool in = rin[p] && (o == 1 || q > 0 || col > 0);  // only column -1 can be outside (W = 4n)
                    count += (in && v[p][2 * o + q] == target[o]) ? R(1) : R(0);
                }
            if (live) {
                s_share[hr * kTileMaxWo + w + o] = go[o] / count;
                s_target[hr * kTileMaxWo + w + o] = target[o];
            }
        }
    }
    __syncthreads();
    // 2. input rows 2 h0 .. 2 h0 + 2 kTileRows - 1 (those that exist), four elements per lane and round
    const int y0 = 2 * h0;
    const int in_rows = g.H - y0 < 2 * kTileRows ? g.H - y0 : 2 * kTileRows;
    const uint32_t n_in = static_cast<uint32_t>(in_rows * g.W);
    for (uint32_t pos = threadIdx.x * 4; pos < n_in; pos += 1024) {
        uint32_t yr, xw;
        g.d_W.divmod(pos, yr, xw);
        const int y = y0 + static_cast<int>(yr);
        const Quad<R> mine = *reinterpret_cast<const Quad<R> *>(src + static_cast<int64_t>(y) * g.xs_h + xw);
        // row y lies in the windows of output rows y / 2 and, for odd y, y / 2 + 1; the four columns in those of
        // output columns 2m, 2m + 1, 2m + 2 (kCovers below)
        const int hr_lo = static_cast<int>(yr) >> 1, c_lo = static_cast<int>(xw) >> 1;
        int h_hi = (y + 1) >> 1;
        h_hi = h_hi >= g.Ho ? g.Ho - 1 : h_hi;
        const int n_rows = h_hi - (y >> 1) + 1;  // 1 or 2 covering output rows
        R amount[6], target[6];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 3; ++b) {
                const int c = c_lo + b < g.Wo ? c_lo + b : g.Wo - 1;  // (row hr_lo + 1 of the arrays always exists)
                amount[a * 3 + b] = s_share[(hr_lo + a) * kTileMaxWo + c];
                target[a * 3 + b] = s_target[(hr_lo + a) * kTileMaxWo + c];
            }
        Quad<R> acc;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            constexpr bool kCovers[4][3] = {{true, false, false}, {true, true, false}, {false, true, false}, {false, true, true}};
            R sum = R(0);
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b) {
                    if (!kCovers[j][b]) continue;  // (an output that does not cover the element would add +0)
                    const bool valid = (a < n_rows) & (c_lo + b < g.Wo);
                    sum += (valid && mine[j] == target[a * 3 + b]) ? amount[a * 3 + b] : R(0);
                }
            acc[j] = sum;
        }
        *reinterpret_cast<Quad<R> *>(gin + static_cast<int64_t>(plane) * (g.H * g.W) + static_cast<int64_t>(y) * g.W + xw) = acc;
    }
}

// Backward for non-overlapping windows (stride == k, padding == 0), one lane per output: the window's elements
// receive grad_out / (number of elements equal to the result) where they equal it (SELECT), or grad_out / k^2
// each; an element gets its single contribution as 0 + amount, the value the reference's zero-initialised sum
// ends with.  Input rows and columns beyond the last window are zero-filled by the lanes of the last output row /
// column.  K2: k == 2 on rows that can be moved as aligned pairs.
template <typename R, bool SELECT, bool K2>
__global__ void __launch_bounds__(256)
pool_backward_window_kernel(PoolGeom g, const R *__restrict__ gout, const R *__restrict__ x, const R *__restrict__ res,
                            R *__restrict__ gin) {
    uint32_t plane, blk;
    g.d_out_blocks.divmod(blockIdx.x, plane, blk);
    const uint32_t pos = blk * 256 + threadIdx.x;
    if (pos >= static_cast<uint32_t>(g.Ho * g.Wo)) return;
    uint32_t h, w;
    g.d_Wo.divmod(pos, h, w);
    const int64_t o = static_cast<int64_t>(plane) * (g.Ho * g.Wo) + pos;
    const int K = K2 ? 2 : g.K;
    const int y0 = static_cast<int>(h) * K, x0 = static_cast<int>(w) * K;
    const R *src = plane_of(g, x, plane);
    R *dst = gin + static_cast<int64_t>(plane) * (g.H * g.W);
    const R go = gout[o];
    if constexpr (K2) {
        Pair<R> d0, d1;
        if constexpr (SELECT) {
            const R *s0 = src + static_cast<int64_t>(y0) * g.xs_h + x0;
            const Pair<R> r0 = *reinterpret_cast<const Pair<R> *>(s0), r1 = *reinterpret_cast<const Pair<R> *>(s0 + g.xs_h);
            const R target = res[o];
            const R count = ((r0[0] == target) ? R(1) : R(0)) + ((r0[1] == target) ? R(1) : R(0)) +
                            ((r1[0] == target) ? R(1) : R(0)) + ((r1[1] == target) ? R(1) : R(0));
            const R share = go / count;
            d0[0] = R(0) + ((r0[0] == target) ? share : R(0));
            d0[1] = R(0) + ((r0[1] == target) ? share : R(0));
            d1[0] = R(0) + ((r1[0] == target) ? share : R(0));
            d1[1] = R(0) + ((r1[1] == target) ? share : R(0));
        } else {
            const R amount = R(0) + go / R(4);
            d0[0] = d0[1] = d1[0] = d1[1] = amount;
        }
        R *t0 = dst + static_cast<int64_t>(y0) * g.W + x0;
        *reinterpret_cast<Pair<R> *>(t0) = d0;
        *reinterpret_cast<Pair<R> *>(t0 + g.W) = d1;
    } else {
        R share;
        R target = R(0);
        if constexpr (SELECT) {
            target = res[o];
            R count = R(0);
            for (int p = 0; p < K; ++p)
                for (int q = 0; q < K; ++q)
                    count += (src[static_cast<int64_t>(y0 + p) * g.xs_h + static_cast<int64_t>(x0 + q) * g.xs_w] == target) ? R(1) : R(0);
            share = go / count;
        } else {
            share = go / static_cast<R>(K * K);
        }
        for (int p = 0; p < K; ++p)
            for (int q = 0; q < K; ++q) {
                bool take = true;
                if constexpr (SELECT) take = src[static_cast<int64_t>(y0 + p) * g.xs_h + static_cast<int64_t>(x0 + q) * g.xs_w] == target;
                dst[static_cast<int64_t>(y0 + p) * g.W + x0 + q] = R(0) + (take ? share : R(0));
            }
    }
    // rows and columns that no window covers
    const bool last_w = static_cast<int>(w) == g.Wo - 1, last_h = static_cast<int>(h) == g.Ho - 1;
    if (last_w)
        for (int p = 0; p < K; ++p)
            for (int c = g.Wo * K; c < g.W; ++c) dst[static_cast<int64_t>(y0 + p) * g.W + c] = R(0);
    if (last_h) {
        const int c_end = last_w ? g.W : x0 + K;
        for (int r = g.Ho * K; r < g.H; ++r)
            for (int c = x0; c < c_end; ++c) dst[static_cast<int64_t>(r) * g.W + c] = R(0);
    }
}

// Rows of the input (and of a dense tensor of the same shape) can be moved as aligned pairs of T.
template <typename T>
bool rows_pair_aligned(const PoolGeom &g, const void *x, const void *dense) {
    const auto even = [](int64_t v) { return v % 2 == 0; };
    return g.xs_w == 1 && g.W % 2 == 0 && even(g.xs_h) && even(g.xs_c) && even(g.xs_b) &&
           reinterpret_cast<uintptr_t>(x) % (2 * sizeof(T)) == 0 && reinterpret_cast<uintptr_t>(dense) % (2 * sizeof(T)) == 0;
}

// Rows of the input view (when it is read: x != nullptr) and of the dense gradient can be moved as aligned groups of
// four T.
template <typename T>
bool rows_quad_aligned(const PoolGeom &g, const void *x, const void *dense) {
    const auto by4 = [](int64_t v) { return v % 4 == 0; };
    if (g.W % 4 != 0 || reinterpret_cast<uintptr_t>(dense) % (4 * sizeof(T)) != 0) return false;
    if (!x) return true;
    return g.xs_w == 1 && by4(g.xs_h) && by4(g.xs_c) && by4(g.xs_b) && reinterpret_cast<uintptr_t>(x) % (4 * sizeof(T)) == 0;
}

ttamd_status make_pool_geom(const char *who, int op, const ttamd_view4 *input, int B, int C, int H, int W, int k, int stride,
                            int padding, PoolGeom *g) {
    if (op < POOL_MAX || op > POOL_AVG) {
        set_error("%s: unknown pooling op code %d", who, op);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (!input) {
        set_error("%s: NULL input view", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || k <= 0 || stride <= 0 || padding < 0) {
        set_error("%s: invalid geometry (B=%d C=%d H=%d W=%d k=%d stride=%d padding=%d)", who, B, C, H, W, k, stride, padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (H + 2 * padding < k || W + 2 * padding < k) {
        set_error("%s: kernel %d does not fit the padded input %dx%d", who, k, H + 2 * padding, W + 2 * padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (input->offset < 0 || input->stride[0] < 0 || input->stride[1] < 0 || input->stride[2] < 0 || input->stride[3] < 0) {
        set_error("%s: negative strides or offset are not supported", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *g = PoolGeom{};
    g->B = B; g->C = C; g->H = H; g->W = W; g->K = k; g->S = stride; g->P = padding;
    g->Ho = (H + 2 * padding - k) / stride + 1;
    g->Wo = (W + 2 * padding - k) / stride + 1;
    g->xs_b = input->stride[0]; g->xs_c = input->stride[1]; g->xs_h = input->stride[2]; g->xs_w = input->stride[3];
    const int64_t in_plane = static_cast<int64_t>(H) * W, out_plane = static_cast<int64_t>(g->Ho) * g->Wo;
    const int64_t planes = static_cast<int64_t>(B) * C;
    const int64_t in_blocks = (in_plane + 255) / 256, out_blocks = (out_plane + 255) / 256;
    if (in_plane >= 0x7fffffff || static_cast<int64_t>(H - 1) * g->xs_h + static_cast<int64_t>(W - 1) * g->xs_w >= 0x7fffffff ||
        planes * in_blocks >= 0x7fffffff || planes * (out_blocks > 0 ? out_blocks : 1) >= 0x7fffffff || k >= (1 << 14) ||
        padding >= (1 << 14)) {
        set_error("%s: the tensor exceeds the 32-bit plane / launch range of the pooling kernels", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    g->in_blocks = static_cast<int>(in_blocks);
    g->out_blocks = static_cast<int>(out_blocks > 0 ? out_blocks : 1);
    g->d_in_blocks = make_fastdiv(static_cast<uint32_t>(g->in_blocks));
    g->quad_blocks = static_cast<int>((in_plane / 4 + 255) / 256);
    g->d_quad_blocks = make_fastdiv(static_cast<uint32_t>(g->quad_blocks > 0 ? g->quad_blocks : 1));
    g->opair_blocks = static_cast<int>((out_plane / 2 + 255) / 256);
    g->d_opair_blocks = make_fastdiv(static_cast<uint32_t>(g->opair_blocks > 0 ? g->opair_blocks : 1));
    g->d_out_blocks = make_fastdiv(static_cast<uint32_t>(g->out_blocks));
    g->d_C = make_fastdiv(static_cast<uint32_t>(C));
    g->d_Wo = make_fastdiv(static_cast<uint32_t>(g->Wo > 0 ? g->Wo : 1));
    g->d_W = make_fastdiv(static_cast<uint32_t>(W));
    g->d_S = make_fastdiv(static_cast<uint32_t>(stride));
    return TTAMD_OK;
}

template <typename T, typename R, int OP>
ttamd_status launch_forward(const PoolGeom &g, const void *x, void *out, hipStream_t st) {
    const unsigned blocks = static_cast<unsigned>(static_cast<int64_t>(g.B) * g.C * g.out_blocks);
    if (g.K == 3 && g.S == 2 && g.P == 1 && rows_quad_aligned<T>(g, x, x) && reinterpret_cast<uintptr_t>(out) % (2 * sizeof(R)) == 0) {
        const unsigned pair_blocks = static_cast<unsigned>(static_cast<int64_t>(g.B) * g.C * g.opair_blocks);
        pool_forward_k3s2_kernel<T, R, OP><<<dim3(pair_blocks), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out));
    } else if (g.K == 2 && g.S == 2 && g.P == 0 && rows_pair_aligned<T>(g, x, x))
        pool_forward_k2_kernel<T, R, OP><<<dim3(blocks), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out));
    else if (g.K == 3)
        pool_forward_kernel<T, R, OP, 3><<<dim3(blocks), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out));
    else if (g.K == 2)
        pool_forward_kernel<T, R, OP, 2><<<dim3(blocks), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out));
    else
        pool_forward_kernel<T, R, OP, 0><<<dim3(blocks), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out));
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T>
ttamd_status forward_typed(int op, const PoolGeom &g, const void *x, void *out, hipStream_t st) {
    using Avg = std::conditional_t<std::is_floating_point_v<T>, T, float>;
    if (op == POOL_MAX) return launch_forward<T, T, POOL_MAX>(g, x, out, st);
    if (op == POOL_MIN) return launch_forward<T, T, POOL_MIN>(g, x, out, st);
    return launch_forward<T, Avg, POOL_AVG>(g, x, out, st);
}

template <typename R>
ttamd_status backward_typed(int device, int op, const PoolGeom &g, const void *gout, const void *x, const void *res, void *gin,
                            hipStream_t st) {
    const int64_t planes = static_cast<int64_t>(g.B) * g.C;
    const dim3 in_grid(static_cast<unsigned>(planes * g.in_blocks)), out_grid(static_cast<unsigned>(planes * g.out_blocks)), block(256);
    if (g.S == g.K && g.P == 0 && g.Ho > 0 && g.Wo > 0) {
        const R *go = static_cast<const R *>(gout), *xi = static_cast<const R *>(x), *rs = static_cast<const R *>(res);
        R *gi = static_cast<R *>(gin);
        const bool k2 = g.K == 2 && rows_pair_aligned<R>(g, x, gin);
        if (op == POOL_AVG) {
            if (k2) pool_backward_window_kernel<R, false, true><<<out_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else pool_backward_window_kernel<R, false, false><<<out_grid, block, 0, st>>>(g, go, xi, rs, gi);
        } else {
            if (k2) pool_backward_window_kernel<R, true, true><<<out_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else pool_backward_window_kernel<R, true, false><<<out_grid, block, 0, st>>>(g, go, xi, rs, gi);
        }
    } else {
        const R *go = static_cast<const R *>(gout), *xi = static_cast<const R *>(x), *rs = static_cast<const R *>(res);
        R *gi = static_cast<R *>(gin);
        const bool two = (g.K + g.S - 1) / g.S == 2;  // an element lies in at most 2 x 2 windows (k3 s2, k2 s1, k4 s2 ...)
        const int cols = (g.K + 3 + g.S - 1) / g.S;   // output columns that can cover four consecutive elements
        const bool quad = two && cols <= 5 && rows_quad_aligned<R>(g, op == POOL_AVG ? nullptr : x, gin);
        const dim3 quad_grid(static_cast<unsigned>(planes * g.quad_blocks));
        const auto pair_ok = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % (2 * sizeof(R)) == 0; };
        const bool k3s2p1 = g.K == 3 && g.S == 2 && g.P == 1;
        if (op == POOL_AVG) {
            if (quad && k3s2p1 && pair_ok(gout)) pool_backward_quad_kernel<R, false, 3, true><<<quad_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else if (quad && cols <= 3) pool_backward_quad_kernel<R, false, 3><<<quad_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else if (quad) pool_backward_quad_kernel<R, false, 5><<<quad_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else if (two) pool_backward_kernel<R, false, 2><<<in_grid, block, 0, st>>>(g, go, xi, rs, gi);
            else pool_backward_kernel<R, false, 0><<<in_grid, block, 0, st>>>(g, go, xi, rs, gi);
        } else {
            const int64_t tiles = (g.Ho + kTileRows - 1) / kTileRows;
            if (quad && k3s2p1 && pair_ok(gout) && pair_ok(res) && g.Wo <= kTileMaxWo && planes * tiles <= 0x7fffffff) {
                // one launch, the shares stay in LDS
                pool_backward_k3s2_tile_kernel<R><<<dim3(static_cast<unsigned>(planes * tiles)), block, 0, st>>>(
                    g, static_cast<int>(tiles), make_fastdiv(static_cast<uint32_t>(tiles)), go, xi, rs, gi);
                TTAMD_HIP_CHECK(hipGetLastError());
                return TTAMD_OK;
            }
            void *ws = nullptr;
            const size_t bytes = static_cast<size_t>(planes) * g.Ho * g.Wo * sizeof(R);
            if (ttamd_status s = stream_scratch(device, st, bytes ? bytes : sizeof(R), &ws)) return s;
            R *share = static_cast<R *>(ws);
            if (k3s2p1 && rows_quad_aligned<R>(g, x, x) && pair_ok(gout) && pair_ok(res))
                pool_share_k3s2_kernel<R><<<dim3(static_cast<unsigned>(planes * g.opair_blocks)), block, 0, st>>>(g, go, xi, rs, share);
            else if (g.K == 3) pool_share_kernel<R, 3><<<out_grid, block, 0, st>>>(g, go, xi, rs, share);
            else if (g.K == 2) pool_share_kernel<R, 2><<<out_grid, block, 0, st>>>(g, go, xi, rs, share);
            else pool_share_kernel<R, 0><<<out_grid, block, 0, st>>>(g, go, xi, rs, share);
            if (quad && k3s2p1 && pair_ok(res)) pool_backward_quad_kernel<R, true, 3, true><<<quad_grid, block, 0, st>>>(g, share, xi, rs, gi);
            else if (quad && cols <= 3) pool_backward_quad_kernel<R, true, 3><<<quad_grid, block, 0, st>>>(g, share, xi, rs, gi);
            else if (quad) pool_backward_quad_kernel<R, true, 5><<<quad_grid, block, 0, st>>>(g, share, xi, rs, gi);
            else if (two) pool_backward_kernel<R, true, 2><<<in_grid, block, 0, st>>>(g, share, xi, rs, gi);
            else pool_backward_kernel<R, true, 0><<<in_grid, block, 0, st>>>(g, share, xi, rs, gi);
        }
    }
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" {

ttamd_status ttamd_pool2d_forward(int device, ttamd_dtype dtype, int op, const ttamd_view4 *input, void *out, int B, int C, int H,
                                  int W, int k, int stride, int padding, void *stream) {
    if (dtype <= TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("pool2d does not support dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    PoolGeom g;
    if (ttamd_status s = make_pool_geom("pool2d", op, input, B, C, H, W, k, stride, padding, &g)) return s;
    if (ttamd_status s = use_device(device)) return s;
    if (B == 0) return TTAMD_OK;
    if (!input->data || !out) {
        set_error("pool2d: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *x = static_cast<const char *>(input->data) + input->offset * static_cast<int64_t>(dtype_size(dtype));
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case TTAMD_U8: return forward_typed<uint8_t>(op, g, x, out, st);
    case TTAMD_I16: return forward_typed<int16_t>(op, g, x, out, st);
    case TTAMD_I32: return forward_typed<int32_t>(op, g, x, out, st);
    case TTAMD_I64: return forward_typed<int64_t>(op, g, x, out, st);
    case TTAMD_F32: return forward_typed<float>(op, g, x, out, st);
    default: return forward_typed<double>(op, g, x, out, st);
    }
}

ttamd_status ttamd_pool2d_backward(int device, ttamd_dtype dtype, int op, const void *grad_out, const ttamd_view4 *input,
                                   const void *result, void *grad_input, int B, int C, int H, int W, int k, int stride,
                                   int padding, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("pool2d_backward supports f32 and f64 only (autograd never differentiates integer tensors)");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    PoolGeom g;
    if (ttamd_status s = make_pool_geom("pool2d_backward", op, input, B, C, H, W, k, stride, padding, &g)) return s;
    if (ttamd_status s = use_device(device)) return s;
    if (B == 0) return TTAMD_OK;
    if (!input->data || !grad_out || !result || !grad_input) {
        set_error("pool2d_backward: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *x = static_cast<const char *>(input->data) + input->offset * static_cast<int64_t>(dtype_size(dtype));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TTAMD_F32) return backward_typed<float>(device, op, g, grad_out, x, result, grad_input, st);
    return backward_typed<double>(device, op, g, grad_out, x, result, grad_input, st);
}

}  // extern "C"
