// Device helpers shared by the conv-logic kernels.
#pragma once

#include "clg_common.h"

struct Geom {
    int n, cin, h, w, c, sh, sw, ph, pw, kh, kw, ho, wo;
    int y_fm;   // 1: the block's output and its gradient are laid out [c, ho/2, wo/2, n] (4x4 kernels only), else [n, c, ho/2, wo/2]
};

static inline int clg_make_geom(const clg_conv_geom *g, Geom *out, const char *name)
{
    CLG_REQUIRE(g != nullptr, "%s: null geometry", name);
    CLG_REQUIRE(g->n > 0 && g->c_in > 0 && g->h > 0 && g->w > 0 && g->c_out > 0, "%s: n, c_in, h, w, c_out must be positive",
                name);
    CLG_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->kernel_h > 0 && g->kernel_w > 0 && g->pad_h >= 0 && g->pad_w >= 0,
                "%s: stride and kernel must be positive, padding non-negative", name);
    CLG_REQUIRE(g->c_in <= 65536 && g->kernel_h <= 256 && g->kernel_w <= 256,
                "%s: selection packing allows at most 65536 input channels and a 256x256 kernel", name);
    const int ho = (g->h + 2 * g->pad_h - g->kernel_h) / g->stride_h + 1;
    const int wo = (g->w + 2 * g->pad_w - g->kernel_w) / g->stride_w + 1;
    CLG_REQUIRE(g->h + 2 * g->pad_h >= g->kernel_h && g->w + 2 * g->pad_w >= g->kernel_w && ho > 0 && wo > 0,
                "%s: Invalid output shape: H_out=%d, W_out=%d", name, ho, wo);
    CLG_REQUIRE((int64_t)g->c_in * g->h * g->w < (1ll << 31) && (int64_t)g->c_out * ho * wo * 4 < (1ll << 31),
                "%s: one sample must hold fewer than 2^31 elements", name);
    *out = Geom{g->n, g->c_in, g->h, g->w, g->c_out, g->stride_h, g->stride_w, g->pad_h, g->pad_w, g->kernel_h, g->kernel_w, ho, wo, 0};
    return CLG_OK;
}

#if defined(__HIPCC__)

__device__ __forceinline__ TapLimit tap_limit(const Geom &g) { return TapLimit{g.cin, g.kh, g.kw}; }

// Tap value of one sample (xn = x + n*cin*h*w) for conv output position (oy, ox); 0 outside.
template <typename T>
__device__ __forceinline__ T read_tap(const T *__restrict__ xn, const Geom &g, const Tap &t, int oy, int ox)
{
    const int iy = oy * g.sh + t.ry - g.ph, ix = ox * g.sw + t.rx - g.pw;
    const bool ok = (unsigned)iy < (unsigned)g.h && (unsigned)ix < (unsigned)g.w;
    return ok ? xn[(t.ch * g.h + iy) * g.w + ix] : T(0);
}

// The seven gates of one kernel: 0..3 leaves (tap pairs), 4..5 middle, 6 root.
template <typename T>
struct Tree {
    Coef<T> g[7];
};
template <typename T>
__device__ __forceinline__ Tree<T> load_tree(const T *__restrict__ w /* [7,16] of one kernel */)
{
    Tree<T> t;
#pragma unroll
    for (int k = 0; k < 7; ++k) t.g[k] = fold16(w + 16 * k);
    return t;
}

// A wave-uniform coefficient sits in a scalar register, and a vector instruction can read only one scalar register:
// an FMA "scalar * vector + scalar" costs an extra move per use.  Pinning the ADDENDS (a, one) of every gate in vector
// registers once per kernel visit leaves one scalar operand per FMA of gate() and gate_da(); the compiler cannot
// undo the copy (it would, to save registers, and re-make it in front of every use).  float only: a double tree would
// take 28 more registers than the kernels have.
template <typename T>
__device__ __forceinline__ void pin_addends(Tree<T> &t)
{
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            asm volatile("" : "+v"(t.g[k].a));
            asm volatile("" : "+v"(t.g[k].one));
        }
    }
}

template <typename T>
struct TreeVals {
    T leaf[4], mid[2], root;
};
template <typename T>
__device__ __forceinline__ TreeVals<T> eval_tree(const Tree<T> &t, const T (&tap)[8])
{
    TreeVals<T> v;
#pragma unroll
    for (int p = 0; p < 4; ++p) v.leaf[p] = gate(t.g[p], tap[2 * p], tap[2 * p + 1]);
    v.mid[0] = gate(t.g[4], v.leaf[0], v.leaf[1]);
    v.mid[1] = gate(t.g[5], v.leaf[2], v.leaf[3]);
    v.root = gate(t.g[6], v.mid[0], v.mid[1]);
    return v;
}

// Sums K per-thread values over the block (fixed order) and lets thread k < K write total k.
template <typename T, int K, int BLOCK>
__device__ __forceinline__ void block_sum_store(T (&acc)[K], T *__restrict__ dst)
{
    constexpr int kWaves = BLOCK / kWave;
    __shared__ T part[kWaves][K];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const T s = wave_sum(acc[k]);
        if (lane == 0) part[wave][k] = s;
    }
    __syncthreads();
    if (threadIdx.x < K) {
        T s = 0;
#pragma unroll
        for (int wv = 0; wv < kWaves; ++wv) s += part[wv][threadIdx.x];
        dst[threadIdx.x] = s;
    }
}

#endif
