// Conv-logic kernels that accept any geometry (stride, padding, kernel size, image size, any tap
// selection).  They read taps straight from global memory with bounds checks.  The split layers
// (4 leaf gates per kernel, one tree level) always run here; the fused block uses these kernels
// when its LDS-tiled kernels (conv_block.hip) cannot take the shape.
//
// Launch shape: blockIdx.y is the logic kernel (output channel), so the channel is uniform per
// workgroup and its taps and folded coefficients live in scalar registers; threads run along
// output positions.  Gradients are deterministic: weight gradients are block-reduced in a fixed
// order into per-block partials that a second kernel sums in order; input gradients are gathered
// per input pixel (one writer per element, no atomics).
#include "conv_common.h"

namespace {

constexpr int kBlk = 256;

template <typename T>
struct alignas(sizeof(T) * 4) Quad {
    T v[4];
};
template <typename T>
struct alignas(sizeof(T) * 2) Pair {
    T v[2];
};

// ---------------------------------------------------------------------------------------------
// split layer: 4 leaf gates
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlk) void conv4_forward_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                           const int32_t *__restrict__ sel, T *__restrict__ y, Geom g)
{
    const int c = blockIdx.y;
    const int P = g.ho * g.wo;
    const int64_t item = (int64_t)blockIdx.x * kBlk + threadIdx.x;       // (sample, position)
    if (item >= (int64_t)g.n * P) return;
    const int n = (int)(item / P), pos = (int)(item - (int64_t)n * P);
    const int oy = pos / g.wo, ox = pos % g.wo;
    const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
    Quad<T> out;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const Coef<T> cf = fold16(w + (c * 4 + p) * 16);
        const T a = read_tap(xn, g, unpack_tap(sel[c * 8 + 2 * p], tap_limit(g)), oy, ox);
        const T b = read_tap(xn, g, unpack_tap(sel[c * 8 + 2 * p + 1], tap_limit(g)), oy, ox);
        out.v[p] = gate(cf, a, b);
    }
    reinterpret_cast<Quad<T> *>(y)[((int64_t)n * g.c + c) * P + pos] = out;
}

template <typename T>
__global__ __launch_bounds__(kBlk) void conv4_backward_w_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                              const int32_t *__restrict__ sel, T *__restrict__ partial,
                                                              Geom g)
{
    const int c = blockIdx.y, nb = gridDim.x;
    const int P = g.ho * g.wo;
    const int64_t items = (int64_t)g.n * P;
    Tap tap[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) tap[t] = unpack_tap(sel[c * 8 + t], tap_limit(g));
    T acc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) acc[k] = 0;
    for (int64_t it = (int64_t)blockIdx.x * kBlk + threadIdx.x; it < items; it += (int64_t)nb * kBlk) {
        const int n = (int)(it / P), pos = (int)(it % P);
        const int oy = pos / g.wo, ox = pos % g.wo;
        const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
        const Quad<T> q = reinterpret_cast<const Quad<T> *>(gy)[((int64_t)n * g.c + c) * P + pos];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const T a = read_tap(xn, g, tap[2 * p], oy, ox), b = read_tap(xn, g, tap[2 * p + 1], oy, ox);
            acc[4 * p + 0] = fma_t(q.v[p], a * b, acc[4 * p + 0]);
            acc[4 * p + 1] = fma_t(q.v[p], a, acc[4 * p + 1]);
            acc[4 * p + 2] = fma_t(q.v[p], b, acc[4 * p + 2]);
            acc[4 * p + 3] += q.v[p];
        }
    }
    block_sum_store<T, 16, kBlk>(acc, partial + ((int64_t)c * nb + blockIdx.x) * 16);
}

// out[row*G + q][i] = sum_k COEF[k][i] * (sum_blk partial[row][blk][q*4 + k]): the gradient w.r.t. the gate
// probabilities; with probs (the softmax output they came from) the gradient w.r.t. the logits instead.
// The 16 lanes of a gate split the sum: lane i adds component i & 3 over the blocks blk = i >> 2 (mod 4), the four
// stripes meet in a butterfly (same value in both partners), and every lane then holds the four totals.
template <typename T>
__global__ __launch_bounds__(256) void reduce_coef_partials_kernel(const T *__restrict__ partial, T *__restrict__ out, int64_t rows,
                                                                 int nb, int G, const T *__restrict__ probs)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int i = threadIdx.x & 15;
    const int64_t gate = e >> 4;                                     // row * G + q; a row of 16 lanes is live or dead as a whole
    if (gate >= rows * G) return;
    const int64_t row = gate / G;
    const int q = (int)(gate - row * G);
    const T *p = partial + (row * nb * G + q) * 4 + (i & 3);
    T acc = 0;
    int blk = i >> 2;
    for (; blk + 28 < nb; blk += 32) {                               // eight loads in flight, added in the same order as one by one
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[(int64_t)(blk + 4 * u) * G * 4];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; blk < nb; blk += 4) acc += p[(int64_t)blk * G * 4];
    acc += __shfl_xor(acc, 4, 16);
    acc += __shfl_xor(acc, 8, 16);
    const T s0 = __shfl(acc, 0, 16), s1 = __shfl(acc, 1, 16), s2 = __shfl(acc, 2, 16), s3 = __shfl(acc, 3, 16);
    T gi = coef_transpose_row<T>(i, s0, s1, s2, s3);
    if (probs != nullptr) gi = softmax16_backward(gi, probs[e]);
    out[e] = gi;
}

// One thread per input element; every (kernel, tap) that reads the element's channel is visited in
// a fixed order, so the sum is reproducible.  Gradient of the 4-leaf layer (grad arrives per leaf gate
// and conv position); the fused block uses convblock_backward_x_hits_kernel below.
template <typename T>
__global__ __launch_bounds__(kBlk) void conv_backward_x_gather_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                                    const T *__restrict__ w,
                                                                    const int32_t *__restrict__ sel,
                                                                    T *__restrict__ gx, Geom g)
{
    const int64_t total = (int64_t)g.n * g.cin * g.h * g.w;
    const int64_t e = (int64_t)blockIdx.x * kBlk + threadIdx.x;
    if (e >= total) return;
    const int ix = (int)(e % g.w), iy = (int)((e / g.w) % g.h);
    const int ch = (int)((e / ((int64_t)g.w * g.h)) % g.cin), n = (int)(e / ((int64_t)g.w * g.h * g.cin));
    const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
    const int P = g.ho * g.wo;
    T acc = 0;
    for (int c = 0; c < g.c; ++c) {
        for (int t = 0; t < 8; ++t) {
            const Tap tp = unpack_tap(sel[c * 8 + t], tap_limit(g));
            if (tp.ch != ch) continue;
            const int ny = iy + g.ph - tp.ry, nx = ix + g.pw - tp.rx;
            if (ny < 0 || nx < 0 || ny % g.sh != 0 || nx % g.sw != 0) continue;
            const int oy = ny / g.sh, ox = nx / g.sw;
            if (oy >= g.ho || ox >= g.wo) continue;
            const int p = t >> 1;
            const T gl = gy[(((int64_t)n * g.c + c) * P + oy * g.wo + ox) * 4 + p];
            const Coef<T> cf = fold16(w + (c * 4 + p) * 16);
            const T other = read_tap(xn, g, unpack_tap(sel[c * 8 + (t ^ 1)], tap_limit(g)), oy, ox);
            acc += gl * ((t & 1) ? gate_db(cf, other) : gate_da(cf, other));
        }
    }
    gx[e] = acc;
}

// Input gradient of the fused block for shapes the LDS kernels do not take: one thread per input element
// walks the list of kernels that read its channel (count / hits, built in increasing kernel order by the
// preparation kernel) and, where the stored argmax position of the touched pooled cell is the one that
// reads this element, recomputes that tree and adds the tap gradient.  One writer per element, fixed
// order: reproducible.
template <typename T>
__global__ __launch_bounds__(kBlk) void convblock_backward_x_hits_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                                       const T *__restrict__ folded,
                                                                       const int32_t *__restrict__ count,
                                                                       const int32_t *__restrict__ hits,
                                                                       const int32_t *__restrict__ sel,
                                                                       const uint8_t *__restrict__ argmax, T *__restrict__ gx,
                                                                       Geom g)
{
    const int64_t total = (int64_t)g.n * g.cin * g.h * g.w;
    const int64_t e = (int64_t)blockIdx.x * kBlk + threadIdx.x;
    if (e >= total) return;
    const int ix = (int)(e % g.w), iy = (int)((e / g.w) % g.h);
    const int ch = (int)((e / ((int64_t)g.w * g.h)) % g.cin), n = (int)(e / ((int64_t)g.w * g.h * g.cin));
    const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
    const int wp = g.wo / 2, I = (g.ho / 2) * wp;
    const int nhits = count[2 * ch];
    const int32_t *hit = hits + count[2 * ch + 1];
    T acc = 0;
    for (int k = 0; k < nhits; ++k) {
        const int ent = hit[k];
        const int c = ent & 0xFFFF, mask = (ent >> 16) & 0xFF;
        for (int t = 0; t < 8; ++t) {
            if (!((mask >> t) & 1)) continue;
            const Tap tp = unpack_tap(sel[c * 8 + t], tap_limit(g));
            const int ny = iy + g.ph - tp.ry, nx = ix + g.pw - tp.rx;
            if (ny < 0 || nx < 0 || ny % g.sh != 0 || nx % g.sw != 0) continue;
            const int oy = ny / g.sh, ox = nx / g.sw;
            if (oy >= g.ho || ox >= g.wo) continue;
            const int64_t cell = ((int64_t)n * g.c + c) * I + (oy >> 1) * wp + (ox >> 1);
            if (argmax[cell] != ((oy & 1) * 2 + (ox & 1))) continue;
            Tree<T> tr;
            const T *fc = folded + (int64_t)c * 28;
#pragma unroll
            for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
            T tap[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) tap[q] = read_tap(xn, g, unpack_tap(sel[c * 8 + q], tap_limit(g)), oy, ox);
            const TreeVals<T> v = eval_tree(tr, tap);
            const int p = t >> 1, m = p >> 1;
            const T g_mid = gy[cell] * (m ? gate_db(tr.g[6], v.mid[0]) : gate_da(tr.g[6], v.mid[1]));
            const T g_leaf = g_mid * ((p & 1) ? gate_db(tr.g[4 + m], v.leaf[p ^ 1]) : gate_da(tr.g[4 + m], v.leaf[p ^ 1]));
            acc += g_leaf * ((t & 1) ? gate_db(tr.g[p], tap[t ^ 1]) : gate_da(tr.g[p], tap[t ^ 1]));
        }
    }
    gx[e] = acc;
}

// ---------------------------------------------------------------------------------------------
// one tree level
// ---------------------------------------------------------------------------------------------
constexpr int kMaxTreeOut = 1024;

template <typename T, bool BACKWARD>
__global__ __launch_bounds__(kBlk) void tree_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                  const T *__restrict__ w, T *__restrict__ out, int C, int64_t positions,
                                                  int xo, int64_t blocks_per_nc)
{
    __shared__ Coef<T> cf[kMaxTreeOut];
    const int c = blockIdx.y;
    for (int p = threadIdx.x; p < xo; p += kBlk) cf[p] = fold16(w + ((int64_t)c * xo + p) * 16);
    __syncthreads();
    const int64_t n = blockIdx.x / blocks_per_nc;
    const int64_t e = (blockIdx.x % blocks_per_nc) * kBlk + threadIdx.x;  // over positions * xo
    if (e >= positions * xo) return;
    const int p = (int)(e % xo);
    const int64_t base = (n * C + c) * positions * xo + e;
    const Pair<T> in = reinterpret_cast<const Pair<T> *>(x)[base];
    if constexpr (!BACKWARD) {
        out[base] = gate(cf[p], in.v[0], in.v[1]);
    } else {
        const T gv = gy[base];
        Pair<T> r;
        r.v[0] = gv * gate_da(cf[p], in.v[1]);
        r.v[1] = gv * gate_db(cf[p], in.v[0]);
        reinterpret_cast<Pair<T> *>(out)[base] = r;
    }
}

// grid.y = c * xo + p; partial [c*xo+p][blk][4]
template <typename T>
__global__ __launch_bounds__(kBlk) void tree_backward_w_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                             T *__restrict__ partial, int64_t N, int C, int64_t positions,
                                                             int xo)
{
    const int c = blockIdx.y / xo, p = blockIdx.y % xo, nb = gridDim.x;
    const int64_t items = N * positions;
    T acc[4] = {0, 0, 0, 0};
    for (int64_t it = (int64_t)blockIdx.x * kBlk + threadIdx.x; it < items; it += (int64_t)nb * kBlk) {
        const int64_t n = it / positions, pos = it % positions;
        const int64_t base = ((n * C + c) * positions + pos) * xo + p;
        const Pair<T> in = reinterpret_cast<const Pair<T> *>(x)[base];
        const T gv = gy[base];
        acc[0] = fma_t(gv, in.v[0] * in.v[1], acc[0]);
        acc[1] = fma_t(gv, in.v[0], acc[1]);
        acc[2] = fma_t(gv, in.v[1], acc[2]);
        acc[3] += gv;
    }
    block_sum_store<T, 4, kBlk>(acc, partial + ((int64_t)blockIdx.y * nb + blockIdx.x) * 4);
}

// ---------------------------------------------------------------------------------------------
// fused block, any geometry
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlk) void convblock_forward_generic_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                       const int32_t *__restrict__ sel, T *__restrict__ y,
                                                                       uint8_t *__restrict__ argmax, Geom g)
{
    const int c = blockIdx.y;
    const int wp = g.wo / 2, I = (g.ho / 2) * wp;
    const int64_t item = (int64_t)blockIdx.x * kBlk + threadIdx.x;       // (sample, pooled cell)
    if (item >= (int64_t)g.n * I) return;
    const int n = (int)(item / I), cell = (int)(item - (int64_t)n * I);
    const int py = cell / wp, px = cell % wp;
    const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
    const Tree<T> tr = load_tree(w + c * 7 * 16);
    Tap tap[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) tap[t] = unpack_tap(sel[c * 8 + t], tap_limit(g));
    T best = -INFINITY;
    int code = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int oy = 2 * py + (q >> 1), ox = 2 * px + (q & 1);
        T v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, tap[t], oy, ox);
        const T r = eval_tree(tr, v).root;
        if (r > best) {
            best = r;
            code = q;
        }
    }
    const int64_t o = ((int64_t)n * g.c + c) * I + cell;
    y[o] = best;
    argmax[o] = (uint8_t)code;
}

template <typename T>
__global__ __launch_bounds__(kBlk) void convblock_intermediates_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                     const int32_t *__restrict__ sel, T *__restrict__ x2,
                                                                     T *__restrict__ x3, Geom g)
{
    const int c = blockIdx.y;
    const int P = g.ho * g.wo;
    const int64_t item = (int64_t)blockIdx.x * kBlk + threadIdx.x;       // (sample, position)
    if (item >= (int64_t)g.n * P) return;
    const int n = (int)(item / P), pos = (int)(item - (int64_t)n * P);
    const int oy = pos / g.wo, ox = pos % g.wo;
    const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
    const Tree<T> tr = load_tree(w + c * 7 * 16);
    T v[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, unpack_tap(sel[c * 8 + t], tap_limit(g)), oy, ox);
    const TreeVals<T> tv = eval_tree(tr, v);
    const int64_t o = ((int64_t)n * g.c + c) * P + pos;
    if (x2) {
        Quad<T> q;
#pragma unroll
        for (int p = 0; p < 4; ++p) q.v[p] = tv.leaf[p];
        reinterpret_cast<Quad<T> *>(x2)[o] = q;
    }
    if (x3) {
        Pair<T> pr;
        pr.v[0] = tv.mid[0];
        pr.v[1] = tv.mid[1];
        reinterpret_cast<Pair<T> *>(x3)[o] = pr;
    }
}

// 28 partial sums (7 gates x (ab, a, b, 1)) per kernel over all samples and pooled cells.
template <typename T>
__global__ __launch_bounds__(kBlk) void convblock_backward_w_generic_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                                          const T *__restrict__ w,
                                                                          const int32_t *__restrict__ sel,
                                                                          const uint8_t *__restrict__ argmax,
                                                                          T *__restrict__ partial, Geom g)
{
    const int c = blockIdx.y, nb = gridDim.x;
    const int wp = g.wo / 2, I = (g.ho / 2) * wp;
    const int64_t items = (int64_t)g.n * I;
    const Tree<T> tr = load_tree(w + c * 7 * 16);
    Tap tap[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) tap[t] = unpack_tap(sel[c * 8 + t], tap_limit(g));
    T acc[28];
#pragma unroll
    for (int k = 0; k < 28; ++k) acc[k] = 0;
    for (int64_t it = (int64_t)blockIdx.x * kBlk + threadIdx.x; it < items; it += (int64_t)nb * kBlk) {
        const int n = (int)(it / I), cell = (int)(it % I);
        const int64_t o = ((int64_t)n * g.c + c) * I + cell;
        const int code = argmax[o];
        const int oy = 2 * (cell / wp) + (code >> 1), ox = 2 * (cell % wp) + (code & 1);
        const T *xn = x + (int64_t)n * g.cin * g.h * g.w;
        T v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, tap[t], oy, ox);
        const TreeVals<T> tv = eval_tree(tr, v);
        T gate_in[7][2], gate_g[7];
        gate_g[6] = gy[o];
        gate_in[6][0] = tv.mid[0];
        gate_in[6][1] = tv.mid[1];
        gate_g[4] = gate_g[6] * gate_da(tr.g[6], tv.mid[1]);
        gate_g[5] = gate_g[6] * gate_db(tr.g[6], tv.mid[0]);
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            gate_in[4 + m][0] = tv.leaf[2 * m];
            gate_in[4 + m][1] = tv.leaf[2 * m + 1];
            gate_g[2 * m] = gate_g[4 + m] * gate_da(tr.g[4 + m], tv.leaf[2 * m + 1]);
            gate_g[2 * m + 1] = gate_g[4 + m] * gate_db(tr.g[4 + m], tv.leaf[2 * m]);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            gate_in[p][0] = v[2 * p];
            gate_in[p][1] = v[2 * p + 1];
        }
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            acc[4 * k + 0] = fma_t(gate_g[k], gate_in[k][0] * gate_in[k][1], acc[4 * k + 0]);
            acc[4 * k + 1] = fma_t(gate_g[k], gate_in[k][0], acc[4 * k + 1]);
            acc[4 * k + 2] = fma_t(gate_g[k], gate_in[k][1], acc[4 * k + 2]);
            acc[4 * k + 3] += gate_g[k];
        }
    }
    block_sum_store<T, 28, kBlk>(acc, partial + ((int64_t)c * nb + blockIdx.x) * 28);
}

int partial_blocks(int64_t items)
{
    const int64_t nb = clg_ceil_div(items, (int64_t)kBlk * 8);
    return (int)(nb < 1 ? 1 : (nb > 64 ? 64 : nb));
}

int check_dtype(int dtype, const char *name)
{
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "%s: dtype must be CLG_F32 or CLG_F64, got %d", name, dtype);
    return CLG_OK;
}

template <typename T>
int launch_reduce(const void *partial, void *out, int64_t rows, int nb, int G, hipStream_t st, const char *name,
                  const void *probs = nullptr)
{
    const int64_t total = rows * G * 16;
    hipLaunchKernelGGL(reduce_coef_partials_kernel<T>, dim3((unsigned)clg_ceil_div(total, 256)), dim3(256), 0, st,
                       (const T *)partial, (T *)out, rows, nb, G, (const T *)probs);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

}  // namespace

#define CLG_DISPATCH(dtype, ...)            \
    do {                                    \
        if ((dtype) == CLG_F32) {           \
            using T = float;                \
            __VA_ARGS__;                    \
        } else {                            \
            using T = double;               \
            __VA_ARGS__;                    \
        }                                   \
    } while (0)

static int check_grid(const Geom &g, int64_t blocks, const char *name)
{
    CLG_REQUIRE(g.c <= 65535, "%s: more than 65535 logic kernels are not supported", name);
    CLG_REQUIRE(blocks < (1ll << 31), "%s: batch too large for one launch", name);
    return CLG_OK;
}

extern "C" int clg_conv4_forward(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                 void *y, void *stream)
{
    Geom g;
    if (int e = clg_make_geom(gg, &g, "clg_conv4_forward")) return e;
    if (int e = check_dtype(dtype, "clg_conv4_forward")) return e;
    CLG_REQUIRE(x && w && selection && y, "clg_conv4_forward: null pointer argument");
    const int64_t blocks = clg_ceil_div((int64_t)g.n * g.ho * g.wo, kBlk);
    if (int e = check_grid(g, blocks, "clg_conv4_forward")) return e;
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(conv4_forward_kernel<T>, dim3((unsigned)blocks, g.c), dim3(kBlk), 0,
                                           clg_stream(stream), (const T *)x, (const T *)w, selection, (T *)y, g));
    CLG_CHECK_LAUNCH("clg_conv4_forward");
    return CLG_OK;
}

extern "C" int clg_conv4_backward_x(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                    const int32_t *selection, void *grad_x, void *stream)
{
    Geom g;
    if (int e = clg_make_geom(gg, &g, "clg_conv4_backward_x")) return e;
    if (int e = check_dtype(dtype, "clg_conv4_backward_x")) return e;
    CLG_REQUIRE(grad_y && x && w && selection && grad_x, "clg_conv4_backward_x: null pointer argument");
    const int64_t total = (int64_t)g.n * g.cin * g.h * g.w;
    CLG_REQUIRE(clg_ceil_div(total, kBlk) < (1ll << 31), "clg_conv4_backward_x: input too large for one launch");
    CLG_DISPATCH(dtype, hipLaunchKernelGGL((conv_backward_x_gather_kernel<T>), dim3((unsigned)clg_ceil_div(total, kBlk)),
                                           dim3(kBlk), 0, clg_stream(stream), (const T *)grad_y, (const T *)x, (const T *)w,
                                           selection, (T *)grad_x, g));
    CLG_CHECK_LAUNCH("clg_conv4_backward_x");
    return CLG_OK;
}

extern "C" int64_t clg_conv4_backward_w_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_make_geom(gg, &g, "clg_conv4_backward_w_scratch_bytes")) return -1;
    const int nb = partial_blocks((int64_t)g.n * g.ho * g.wo);
    return (int64_t)g.c * nb * 16 * (dtype == CLG_F64 ? 8 : 4);
}

extern "C" int clg_conv4_backward_w(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x,
                                    const int32_t *selection, void *grad_w, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_make_geom(gg, &g, "clg_conv4_backward_w")) return e;
    if (int e = check_dtype(dtype, "clg_conv4_backward_w")) return e;
    CLG_REQUIRE(grad_y && x && selection && grad_w && scratch, "clg_conv4_backward_w: null pointer argument");
    CLG_REQUIRE(g.c <= 65535, "clg_conv4_backward_w: more than 65535 logic kernels are not supported");
    const int nb = partial_blocks((int64_t)g.n * g.ho * g.wo);
    hipStream_t st = clg_stream(stream);
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(conv4_backward_w_kernel<T>, dim3(nb, g.c), dim3(kBlk), 0, st, (const T *)grad_y,
                                           (const T *)x, selection, (T *)scratch, g));
    CLG_CHECK_LAUNCH("clg_conv4_backward_w");
    CLG_DISPATCH(dtype, return launch_reduce<T>(scratch, grad_w, g.c, nb, 4, st, "clg_conv4_backward_w(reduce)"));
}

static int check_tree(int dtype, int64_t n, int64_t c, int64_t positions, int64_t xo, const char *name)
{
    if (int e = check_dtype(dtype, name)) return e;
    CLG_REQUIRE(n > 0 && c > 0 && positions > 0 && xo > 0, "%s: n, c, positions and xo must be positive", name);
    CLG_REQUIRE(xo <= kMaxTreeOut, "%s: at most %d gates per channel are supported, got %lld", name, kMaxTreeOut, (long long)xo);
    CLG_REQUIRE(c * xo <= 65535, "%s: channels * gates above 65535 is not supported", name);
    CLG_REQUIRE(n * clg_ceil_div(positions * xo, kBlk) < (1ll << 31), "%s: tensor too large for one launch", name);
    return CLG_OK;
}

extern "C" int clg_tree_forward(int dtype, const void *x, const void *w, void *y, int64_t n, int64_t c, int64_t positions,
                                int64_t xo, void *stream)
{
    if (int e = check_tree(dtype, n, c, positions, xo, "clg_tree_forward")) return e;
    CLG_REQUIRE(x && w && y, "clg_tree_forward: null pointer argument");
    const int64_t bpn = clg_ceil_div(positions * xo, kBlk);
    CLG_DISPATCH(dtype, hipLaunchKernelGGL((tree_kernel<T, false>), dim3((unsigned)(n * bpn), (unsigned)c), dim3(kBlk), 0,
                                           clg_stream(stream), (const T *)nullptr, (const T *)x, (const T *)w, (T *)y, (int)c,
                                           positions, (int)xo, bpn));
    CLG_CHECK_LAUNCH("clg_tree_forward");
    return CLG_OK;
}

extern "C" int clg_tree_backward_x(int dtype, const void *grad_y, const void *x, const void *w, void *grad_x, int64_t n,
                                   int64_t c, int64_t positions, int64_t xo, void *stream)
{
    if (int e = check_tree(dtype, n, c, positions, xo, "clg_tree_backward_x")) return e;
    CLG_REQUIRE(grad_y && x && w && grad_x, "clg_tree_backward_x: null pointer argument");
    const int64_t bpn = clg_ceil_div(positions * xo, kBlk);
    CLG_DISPATCH(dtype, hipLaunchKernelGGL((tree_kernel<T, true>), dim3((unsigned)(n * bpn), (unsigned)c), dim3(kBlk), 0,
                                           clg_stream(stream), (const T *)grad_y, (const T *)x, (const T *)w, (T *)grad_x,
                                           (int)c, positions, (int)xo, bpn));
    CLG_CHECK_LAUNCH("clg_tree_backward_x");
    return CLG_OK;
}

extern "C" int64_t clg_tree_backward_w_scratch_bytes(int dtype, int64_t n, int64_t c, int64_t positions, int64_t xo)
{
    if (n <= 0 || c <= 0 || positions <= 0 || xo <= 0) return -1;
    return c * xo * partial_blocks(n * positions) * 4 * (dtype == CLG_F64 ? 8 : 4);
}

extern "C" int clg_tree_backward_w(int dtype, const void *grad_y, const void *x, void *grad_w, void *scratch, int64_t n,
                                   int64_t c, int64_t positions, int64_t xo, void *stream)
{
    if (int e = check_tree(dtype, n, c, positions, xo, "clg_tree_backward_w")) return e;
    CLG_REQUIRE(grad_y && x && grad_w && scratch, "clg_tree_backward_w: null pointer argument");
    const int nb = partial_blocks(n * positions);
    hipStream_t st = clg_stream(stream);
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(tree_backward_w_kernel<T>, dim3(nb, (unsigned)(c * xo)), dim3(kBlk), 0, st,
                                           (const T *)grad_y, (const T *)x, (T *)scratch, n, (int)c, positions, (int)xo));
    CLG_CHECK_LAUNCH("clg_tree_backward_w");
    CLG_DISPATCH(dtype, return launch_reduce<T>(scratch, grad_w, c * xo, nb, 1, st, "clg_tree_backward_w(reduce)"));
}

int clg_launch_reduce_coef(int dtype, const void *partial, void *out, int64_t rows, int nb, int G, hipStream_t st, const char *name,
                           const void *probs)
{
    CLG_DISPATCH(dtype, return launch_reduce<T>(partial, out, rows, nb, G, st, name, probs));
}

// ---- fused block, generic entry points (called from conv_block.hip when no tiled kernel applies) ----
int clg_convblock_check(const clg_conv_geom *gg, Geom *g, int dtype, const char *name)
{
    if (int e = clg_make_geom(gg, g, name)) return e;
    if (int e = check_dtype(dtype, name)) return e;
    CLG_REQUIRE(g->ho % 2 == 0 && g->wo % 2 == 0,
                "%s: Output height and width after convolution must be divisible by 2 for 2x2 max pooling, but got H_out=%d, "
                "W_out=%d",
                name, g->ho, g->wo);
    return CLG_OK;
}

int clg_convblock_forward_generic(int dtype, const Geom &g, const void *x, const void *w, const int32_t *selection, void *y,
                                  uint8_t *argmax, hipStream_t st)
{
    const int64_t blocks = clg_ceil_div((int64_t)g.n * (g.ho / 2) * (g.wo / 2), kBlk);
    if (int e = check_grid(g, blocks, "clg_convblock_forward")) return e;
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(convblock_forward_generic_kernel<T>, dim3((unsigned)blocks, g.c), dim3(kBlk), 0, st,
                                           (const T *)x, (const T *)w, selection, (T *)y, argmax, g));
    CLG_CHECK_LAUNCH("clg_convblock_forward(generic)");
    return CLG_OK;
}

int clg_convblock_backward_x_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *folded,
                                     const int32_t *count, const int32_t *hits, const int32_t *selection, const uint8_t *argmax,
                                     void *grad_x, hipStream_t st)
{
    const int64_t total = (int64_t)g.n * g.cin * g.h * g.w;
    CLG_REQUIRE(clg_ceil_div(total, kBlk) < (1ll << 31), "clg_convblock_backward_x: input too large for one launch");
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(convblock_backward_x_hits_kernel<T>, dim3((unsigned)clg_ceil_div(total, kBlk)), dim3(kBlk),
                                           0, st, (const T *)grad_y, (const T *)x, (const T *)folded, count, hits, selection, argmax,
                                           (T *)grad_x, g));
    CLG_CHECK_LAUNCH("clg_convblock_backward_x(any shape)");
    return CLG_OK;
}

int clg_convblock_partial_blocks(const Geom &g) { return partial_blocks((int64_t)g.n * (g.ho / 2) * (g.wo / 2)); }

int clg_convblock_backward_w_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                                     hipStream_t st, const void *probs)
{
    CLG_REQUIRE(g.c <= 65535, "clg_convblock_backward_w: more than 65535 logic kernels are not supported");
    const int nb = clg_convblock_partial_blocks(g);
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(convblock_backward_w_generic_kernel<T>, dim3(nb, g.c), dim3(kBlk), 0, st,
                                           (const T *)grad_y, (const T *)x, (const T *)w, selection, argmax, (T *)scratch, g));
    CLG_CHECK_LAUNCH("clg_convblock_backward_w(generic)");
    CLG_DISPATCH(dtype, return launch_reduce<T>(scratch, grad_w, g.c, nb, 7, st, "clg_convblock_backward_w(reduce)", probs));
}

extern "C" int clg_convblock_intermediates(int dtype, const clg_conv_geom *gg, const void *x, const void *w,
                                           const int32_t *selection, void *x2, void *x3, void *stream)
{
    Geom g;
    if (int e = clg_make_geom(gg, &g, "clg_convblock_intermediates")) return e;
    if (int e = check_dtype(dtype, "clg_convblock_intermediates")) return e;
    CLG_REQUIRE(x && w && selection, "clg_convblock_intermediates: null pointer argument");
    const int64_t blocks = clg_ceil_div((int64_t)g.n * g.ho * g.wo, kBlk);
    if (int e = check_grid(g, blocks, "clg_convblock_intermediates")) return e;
    CLG_DISPATCH(dtype, hipLaunchKernelGGL(convblock_intermediates_kernel<T>, dim3((unsigned)blocks, g.c), dim3(kBlk), 0,
                                           clg_stream(stream), (const T *)x, (const T *)w, selection, (T *)x2, (T *)x3, g));
    CLG_CHECK_LAUNCH("clg_convblock_intermediates");
    return CLG_OK;
}
