// Fused conv-logic block on 4x4 images (3x3 kernel, stride 1, padding 1), one sample per lane -- or, for packed
// words, one group of 64 samples per lane (element policies of conv_ops.h).
//
// The last block of a network sees many channels and tiny images: a whole input plane is 16 elements, so the
// kernels that give a workgroup an image (or a padded copy of it) spend their time in set-up, staging and barriers
// (about 12x the FMA time at [128,16384,4,4] -> 32768).  Here the 64 lanes of a wavefront are 64 samples, so the
// kernel, its taps and the image position are uniform per wavefront.  Every lane keeps the two zero-padded 6x6
// planes its kernel reads in its own LDS slice (odd lane stride: lane = bank, no conflicts; the halo is written
// once and stays zero), a plane arrives as four 16-byte loads per lane that are requested one kernel ahead, and the
// 16 positions x 8 taps are LDS reads at (tap address + immediate position offset).  No barriers, no bounds checks.
// A kernel whose taps name more than two channels (possible with a caller-made selection) reads global memory.
#include <stdlib.h>

#include "conv_ops.h"

namespace {

constexpr int kLsWaves = 4;                        // wavefronts per workgroup
constexpr int kLsPlane = 36;                       // padded 6x6 plane
constexpr int kLsStride = 2 * kLsPlane + 1;        // elements per lane

// The taps of one kernel, sorted into at most two planes.
struct LaneTaps {
    int ch[8], ry[8], rx[8];
    int ch0, ch1;
    bool wide;
};
__device__ __forceinline__ LaneTaps lane_taps(const int32_t *__restrict__ sel, int c, const TapLimit &lim)
{
    LaneTaps t;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const Tap tp = unpack_tap(sel[c * 8 + k], lim);
        t.ch[k] = tp.ch, t.ry[k] = tp.ry, t.rx[k] = tp.rx;
    }
    t.ch0 = t.ch[0];
    t.ch1 = t.ch0;
#pragma unroll
    for (int k = 7; k >= 1; --k) t.ch1 = t.ch[k] != t.ch0 ? t.ch[k] : t.ch1;     // first channel that differs from ch0
    t.wide = false;
#pragma unroll
    for (int k = 1; k < 8; ++k) t.wide |= t.ch[k] != t.ch0 && t.ch[k] != t.ch1;
    return t;
}

template <typename T>
struct Planes {
    T v[32];                                       // 4x4 plane of ch0, then of ch1
};

template <typename T>
__device__ __forceinline__ void load_plane(T (&dst)[32], int at, const T *__restrict__ p)
{
    constexpr int PER = 16 / (int)sizeof(T);                       // elements per 16-byte load
#pragma unroll
    for (int q = 0; q < 16 / PER; ++q) {
        const u32x4 raw = reinterpret_cast<const u32x4 *>(p)[q];
        T part[PER];
        __builtin_memcpy(part, &raw, 16);
#pragma unroll
        for (int e = 0; e < PER; ++e) dst[at + q * PER + e] = part[e];
    }
}

// Requests the planes of kernel `tp` for this lane's sample (nothing for a dead lane or a wide kernel).
template <typename T>
__device__ __forceinline__ void fetch_planes(Planes<T> &pl, const LaneTaps &tp, const T *__restrict__ xn, bool live)
{
    if (!live || tp.wide) return;
    load_plane(pl.v, 0, xn + tp.ch0 * 16);
    if (tp.ch1 != tp.ch0) load_plane(pl.v, 16, xn + tp.ch1 * 16);
}

// grid: (64-sample blocks from sample n_first on, kernel tiles of ct kernels); LDS: kLsWaves * 64 * kLsStride elements.
// params: folded coefficients [c][28] (float gates) or gate ids uint8 [c][7] (packed words, argmax = null)
template <typename Ops>
__global__ __launch_bounds__(kLsWaves *kWave) void convblock_forward_4x4_kernel(const typename Ops::Elem *__restrict__ x,
                                                                              const void *__restrict__ params,
                                                                              const int32_t *__restrict__ sel,
                                                                              typename Ops::Elem *__restrict__ y,
                                                                              uint8_t *__restrict__ argmax, Geom g, int ct, int n_first)
{
    using T = typename Ops::Elem;
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    T *mine = reinterpret_cast<T *>(smem) + ((size_t)wave * kWave + lane) * kLsStride;
    const int64_t n = (int64_t)n_first + (int64_t)blockIdx.x * kWave + lane;
    const bool live = n < g.n;
    const T *xn = x + (live ? n : 0) * g.cin * 16;
#pragma unroll
    for (int e = 0; e < kLsStride; ++e) mine[e] = T(0);
    const int c0 = blockIdx.y * ct, c1 = min(g.c, c0 + ct);
    int c = c0 + wave;
    if (c >= c1) return;
    LaneTaps tp = lane_taps(sel, c, tap_limit(g));
    Planes<T> pl;
    fetch_planes(pl, tp, xn, live);
    while (true) {
        if (live && !tp.wide) {
#pragma unroll
            for (int e = 0; e < 16; ++e) mine[((e >> 2) + 1) * 6 + (e & 3) + 1] = pl.v[e];
            if (tp.ch1 != tp.ch0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) mine[kLsPlane + ((e >> 2) + 1) * 6 + (e & 3) + 1] = pl.v[16 + e];
            }
        }
        const typename Ops::Params pr = Ops::load_global(params, c);
        const LaneTaps cur = tp;
        const int cn = c + kLsWaves;
        const bool more = cn < c1;
        if (more) {                                                   // in flight while this kernel is evaluated
            tp = lane_taps(sel, cn, tap_limit(g));
            fetch_planes(pl, tp, xn, live);
        }
        const T *ta[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) ta[k] = mine + (cur.ch[k] != cur.ch0 ? kLsPlane : 0) + cur.ry[k] * 6 + cur.rx[k];
        T best[4];
        int codes = 0;
#pragma unroll
        for (int cell = 0; cell < 4; ++cell) {
            T r[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int oy = 2 * (cell >> 1) + (q >> 1), ox = 2 * (cell & 1) + (q & 1);
                T v[8];
                if (!cur.wide) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) v[k] = ta[k][oy * 6 + ox];
                } else {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const int iy = oy + cur.ry[k] - 1, ix = ox + cur.rx[k] - 1;
                        v[k] = T(0);
                        if ((unsigned)iy < 4u && (unsigned)ix < 4u && live) v[k] = xn[cur.ch[k] * 16 + iy * 4 + ix];
                    }
                }
                r[q] = Ops::root(pr, v);
            }
            int code;
            best[cell] = Ops::pool4(pr, r, code);
            codes |= code << (8 * cell);
        }
        if (live) {
            const int64_t o = (n * g.c + c) * 4;
            if (g.y_fm) {                                             // [c, 2, 2, n]: the lanes' samples are neighbours
#pragma unroll
                for (int cell = 0; cell < 4; ++cell) y[((int64_t)c * 4 + cell) * g.n + n] = best[cell];
            } else {
                constexpr int PER = 16 / (int)sizeof(T);
#pragma unroll
                for (int q = 0; q < 4 / PER; ++q) {
                    u32x4 raw;
                    __builtin_memcpy(&raw, &best[q * PER], 16);
                    reinterpret_cast<u32x4 *>(y + o)[q] = raw;
                }
            }
            if (argmax != nullptr) *reinterpret_cast<uint32_t *>(argmax + o) = (uint32_t)codes;
        }
        if (!more) break;
        c = cn;
    }
}

// Packed words, one group of 64 samples per lane, evaluated as two halves of 32 samples: the lane's LDS slice holds
// 4-byte elements, so a workgroup takes half the LDS of the 8-byte variant and two of them share a CU (the kernel is
// bound by what a wavefront has in flight, not by arithmetic).  The planes are fetched by the wavefront together:
// 8 lanes read the 128 contiguous bytes of one group's plane (8 lines per load instruction instead of 64) and every
// lane writes its two words into the slice of the lane that owns the group.  Order per kernel: low halves to LDS,
// evaluate, high halves to LDS, request the next kernel's planes, evaluate, store 64-bit words.
struct PackedPlanes {
    u32x4 raw[2][8];                               // [plane][load]: words 2 piece, 2 piece + 1 of group 8 load + lane / 8
};

__global__ __launch_bounds__(kLsWaves *kWave, 2) void convblock_eval_packed_4x4_kernel(const uint64_t *__restrict__ x,
                                                                                  const uint8_t *__restrict__ gates,
                                                                                  const int32_t *__restrict__ sel,
                                                                                  uint64_t *__restrict__ y, Geom g, int ct,
                                                                                  int ctiles, int sblocks)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    // Workgroups go round the 8 XCDs by their linear index; an XCD takes the blocks of 64 groups  xcd, xcd + 8, ...
    // one after the other with all kernel tiles of a block in a row, so that the block's planes (cin x 8 KiB) are
    // served by that XCD's L2 while the kernels pick channels at random.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int sblock = xcd + 8 * (slot / ctiles), tile = slot - (slot / ctiles) * ctiles;
    if (sblock >= sblocks) return;
    uint32_t *slices = reinterpret_cast<uint32_t *>(smem) + (size_t)wave * kWave * kLsStride;   // of this wavefront
    uint32_t *mine = slices + lane * kLsStride;
    const int64_t n = (int64_t)sblock * kWave + lane;
    constexpr bool live = true;                                      // the host sends full blocks of 64 groups only
    const uint64_t *xn = x + n * g.cin * 16;
#pragma unroll
    for (int e = 0; e < kLsStride; ++e) mine[e] = 0u;
    const int c0 = tile * ct, c1 = min(g.c, c0 + ct);
    int c = c0 + wave;
    if (c >= c1) return;
    // shared fetch: load j covers groups 8 j .. 8 j + 7 of the wavefront, this lane takes 16 bytes (words 2 piece and
    // 2 piece + 1) of group 8 j + sub
    const int piece = lane & 7, sub = lane >> 3;
    const uint64_t *xw = x + ((int64_t)sblock * kWave + sub) * g.cin * 16 + 2 * piece;   // load j: + 8 j groups
    const int64_t group_step = (int64_t)8 * g.cin * 16;
    uint32_t *put = slices + sub * kLsStride + ((piece >> 1) + 1) * 6 + 2 * (piece & 1) + 1;   // + 8 j slices, + plane
    PackedPlanes pl;
    // Only the channels of the next kernel are looked at ahead of time (its taps are read again when its turn comes:
    // scalar registers are scarce next to 28 gate masks).  Both planes are always fetched and written, also when a
    // kernel reads one channel only: one code path, so the registers of `pl` need no copies where paths meet.
    auto fetch = [&](int kernel) {
        const LaneTaps t = lane_taps(sel, kernel, tap_limit(g));
        if (t.wide) return;
#pragma unroll
        for (int j = 0; j < 8; ++j) pl.raw[0][j] = *reinterpret_cast<const u32x4 *>(xw + j * group_step + t.ch0 * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) pl.raw[1][j] = *reinterpret_cast<const u32x4 *>(xw + j * group_step + t.ch1 * 16);
    };
    fetch(c);
    while (true) {
        const BitOps::Params pr = BitOps::load_global(gates, c);
        const LaneTaps cur = lane_taps(sel, c, tap_limit(g));
        const int cn = c + kLsWaves;
        const bool more = cn < c1;
        const uint32_t *ta[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) ta[k] = mine + (cur.ch[k] != cur.ch0 ? kLsPlane : 0) + cur.ry[k] * 6 + cur.rx[k];
        if (cur.wide) {
            // taps in more than two channels (caller-made selection): 64-bit words straight from global memory, cell by
            // cell in a real loop so that the rare case costs no registers
            if (more) fetch(cn);
#pragma unroll 1
            for (int cell = 0; cell < 4; ++cell) {
                uint64_t pooled = 0;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int oy = 2 * (cell >> 1) + (q >> 1), ox = 2 * (cell & 1) + (q & 1);
                    uint64_t v[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const int iy = oy + cur.ry[k] - 1, ix = ox + cur.rx[k] - 1;
                        v[k] = 0;
                        if ((unsigned)iy < 4u && (unsigned)ix < 4u && live) v[k] = xn[cur.ch[k] * 16 + iy * 4 + ix];
                    }
                    pooled |= BitOps::root(pr, v);
                }
                if (live) y[g.y_fm ? ((int64_t)c * 4 + cell) * g.n + n : (n * g.c + c) * 4 + cell] = pooled;
            }
        } else {
            uint64_t best[4] = {0, 0, 0, 0};
#pragma unroll 1
            for (int half = 0; half < 2; ++half) {                    // a real loop: unrolled, the two passes pile up in registers
                // the lanes write into each other's slices: LDS serves a wavefront's instructions in order, the fences
                // keep the compiler from moving this lane's reads across the writes
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    uint32_t *dst = put + 8 * j * kLsStride;
                    dst[0] = half ? pl.raw[0][j].y : pl.raw[0][j].x;
                    dst[1] = half ? pl.raw[0][j].w : pl.raw[0][j].z;
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    uint32_t *dst = put + 8 * j * kLsStride + kLsPlane;
                    dst[0] = half ? pl.raw[1][j].y : pl.raw[1][j].x;
                    dst[1] = half ? pl.raw[1][j].w : pl.raw[1][j].z;
                }
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int cell = 0; cell < 4; ++cell) {
                    uint32_t pooled = 0;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int oy = 2 * (cell >> 1) + (q >> 1), ox = 2 * (cell & 1) + (q & 1);
                        uint32_t v[8];
#pragma unroll
                        for (int k = 0; k < 8; ++k) v[k] = ta[k][oy * 6 + ox];
                        pooled |= BitOps::root32(pr, v);
                    }
                    best[cell] |= (uint64_t)pooled << (32 * half);
                }
            }
            if (more) fetch(cn);
            if (live) {
                if (g.y_fm) {                                         // [c, 2, 2, groups]: the lanes' groups are neighbours
#pragma unroll
                    for (int cell = 0; cell < 4; ++cell) y[((int64_t)c * 4 + cell) * g.n + n] = best[cell];
                } else {
                    u32x4 *out = reinterpret_cast<u32x4 *>(y + (n * g.c + c) * 4);
                    out[0] = u32x4{(uint32_t)best[0], (uint32_t)(best[0] >> 32), (uint32_t)best[1], (uint32_t)(best[1] >> 32)};
                    out[1] = u32x4{(uint32_t)best[2], (uint32_t)(best[2] >> 32), (uint32_t)best[3], (uint32_t)(best[3] >> 32)};
                }
            }
        }
        if (!more) break;
        c = cn;
    }
}

// ---- gradients ---------------------------------------------------------------------------------
// Two passes, both with one sample per lane and no atomics:
//   convblock_backward_4x4_kernel      kernel-major, same plane staging as the forward: evaluates the tree at the
//                                      pooled arg-max position of the 4 cells once, accumulates the 28 weight-gradient
//                                      sums of its kernel over all samples (registers, then DPP and a fixed-order
//                                      combine of the 4 wavefronts) and writes the 4 x 8 tap gradients of every
//                                      (kernel, sample) to tg[c][n][cell][tap] (and its 4 arg-max codes to tcodes[c][n]);
//   convblock_backward_x_4x4_kernel    channel-major: a lane owns the gradient plane of (sample, channel) in its LDS
//                                      slice and adds the tap gradients of the kernels that read the channel, in
//                                      increasing kernel order, taps in order -- a fixed summation order.
// The tree and its derivatives are evaluated once per (kernel, sample, cell) for both gradients.

constexpr int kGradStride = kLsPlane + 1;          // gradient plane: padded 6x6 (taps of border cells fall into the halo)

template <typename T>
__global__ __launch_bounds__(kLsWaves *kWave) void convblock_backward_4x4_kernel(
    const T *__restrict__ x, const T *__restrict__ folded, const int32_t *__restrict__ sel, const T *__restrict__ gy,
    const uint8_t *__restrict__ argmax, T *__restrict__ tg, uint32_t *__restrict__ tcodes, T *__restrict__ gw,
    const T *__restrict__ probs, Geom g, int ct)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ T meet[kLsWaves][28];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    T *mine = reinterpret_cast<T *>(smem) + ((size_t)wave * kWave + lane) * kLsStride;
#pragma unroll
    for (int e = 0; e < kLsStride; ++e) mine[e] = T(0);
    const int sblocks = (g.n + kWave - 1) / kWave;
    const int c0 = blockIdx.x * ct, c1 = min(g.c, c0 + ct);
    for (int c = c0; c < c1; ++c) {
        const LaneTaps tp = lane_taps(sel, c, tap_limit(g));
        Tree<T> tr;
        const T *fc = folded + (int64_t)c * 28;
#pragma unroll
        for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
        const T *ta[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) ta[k] = mine + (tp.ch[k] != tp.ch0 ? kLsPlane : 0) + tp.ry[k] * 6 + tp.rx[k];
        T acc[28];
#pragma unroll
        for (int k = 0; k < 28; ++k) acc[k] = T(0);
        // the wavefronts of the workgroup deal the 64-sample blocks among themselves; planes one block ahead
        int sb = wave;
        Planes<T> pl;
        {
            const int64_t n = (int64_t)sb * kWave + lane;
            if (sb < sblocks) fetch_planes(pl, tp, x + (n < g.n ? n : 0) * g.cin * 16, n < g.n);
        }
        for (; sb < sblocks; sb += kLsWaves) {
            const int64_t n = (int64_t)sb * kWave + lane;
            const bool live = n < g.n;
            const T *xn = x + (live ? n : 0) * g.cin * 16;
            if (!tp.wide) {
#pragma unroll
                for (int e = 0; e < 16; ++e) mine[((e >> 2) + 1) * 6 + (e & 3) + 1] = live ? pl.v[e] : T(0);
                if (tp.ch1 != tp.ch0) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) mine[kLsPlane + ((e >> 2) + 1) * 6 + (e & 3) + 1] = live ? pl.v[16 + e] : T(0);
                }
            }
            const int64_t o = (n * g.c + c) * 4;
            T gout[4] = {T(0), T(0), T(0), T(0)};
            uint32_t codes = 0;
            if (live) {
#pragma unroll
                for (int cell = 0; cell < 4; ++cell) gout[cell] = g.y_fm ? gy[((int64_t)c * 4 + cell) * g.n + n] : gy[o + cell];
                codes = *reinterpret_cast<const uint32_t *>(argmax + o);
            }
            {
                const int sn = sb + kLsWaves;                          // next block's planes, in flight during the cells
                const int64_t nn = (int64_t)sn * kWave + lane;
                if (sn < sblocks) fetch_planes(pl, tp, x + (nn < g.n ? nn : 0) * g.cin * 16, nn < g.n);
            }
            T gt[32];
#pragma unroll
            for (int cell = 0; cell < 4; ++cell) {
                const int code = (codes >> (8 * cell)) & 3;
                const int oy = 2 * (cell >> 1) + (code >> 1), ox = 2 * (cell & 1) + (code & 1);
                T v[8];
                if (!tp.wide) {
                    const int po = oy * 6 + ox;                        // per lane: the pooled maximum's position
#pragma unroll
                    for (int k = 0; k < 8; ++k) v[k] = ta[k][po];
                } else {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const int iy = oy + tp.ry[k] - 1, ix = ox + tp.rx[k] - 1;
                        v[k] = T(0);
                        if ((unsigned)iy < 4u && (unsigned)ix < 4u && live) v[k] = xn[tp.ch[k] * 16 + iy * 4 + ix];
                    }
                }
                const TreeVals<T> tv = eval_tree(tr, v);
                const T go = gout[cell];                               // 0 for lanes without a sample
                const T g_m[2] = {go * gate_da(tr.g[6], tv.mid[1]), go * gate_db(tr.g[6], tv.mid[0])};
                T g_l[4];
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    g_l[2 * m] = g_m[m] * gate_da(tr.g[4 + m], tv.leaf[2 * m + 1]);
                    g_l[2 * m + 1] = g_m[m] * gate_db(tr.g[4 + m], tv.leaf[2 * m]);
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    gt[cell * 8 + 2 * q] = g_l[q] * gate_da(tr.g[q], v[2 * q + 1]);
                    gt[cell * 8 + 2 * q + 1] = g_l[q] * gate_db(tr.g[q], v[2 * q]);
                }
                // weight-gradient sums: (g a b, g a, g b, g) per gate
                auto add = [&](int q, T gg, T a, T b) {
                    acc[4 * q] = fma_t(gg, a * b, acc[4 * q]);
                    acc[4 * q + 1] = fma_t(gg, a, acc[4 * q + 1]);
                    acc[4 * q + 2] = fma_t(gg, b, acc[4 * q + 2]);
                    acc[4 * q + 3] += gg;
                };
#pragma unroll
                for (int q = 0; q < 4; ++q) add(q, g_l[q], v[2 * q], v[2 * q + 1]);
                add(4, g_m[0], tv.leaf[0], tv.leaf[1]);
                add(5, g_m[1], tv.leaf[2], tv.leaf[3]);
                add(6, go, tv.mid[0], tv.mid[1]);
            }
            if (tg != nullptr && live) {
                T *dst = tg + ((int64_t)c * g.n + n) * 32;
                tcodes[(int64_t)c * g.n + n] = codes;                  // kernel-major copy: the second pass reads it coalesced
                constexpr int PER = 16 / (int)sizeof(T);
#pragma unroll
                for (int q = 0; q < 32 / PER; ++q) {
                    u32x4 raw;
                    __builtin_memcpy(&raw, &gt[q * PER], 16);
                    reinterpret_cast<u32x4 *>(dst)[q] = raw;
                }
            }
        }
        // 28 sums of this kernel: lanes, then the wavefronts in order
#pragma unroll
        for (int k = 0; k < 28; ++k) {
            const T t = wave_sum(acc[k]);
            if (lane == 0) meet[wave][k] = t;
        }
        __syncthreads();
        if (threadIdx.x < 7 * 16) {
            const int q = threadIdx.x >> 4, i = threadIdx.x & 15;
            T sums[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) sums[k] = (meet[0][4 * q + k] + meet[1][4 * q + k]) + (meet[2][4 * q + k] + meet[3][4 * q + k]);
            T gi = coef_transpose_row<T>(i, sums[0], sums[1], sums[2], sums[3]);
            const int64_t e = ((int64_t)c * 7 + q) * 16 + i;
            if (probs != nullptr) gi = softmax16_backward(gi, probs[e]);       // gradient w.r.t. the logits
            gw[e] = gi;
        }
        __syncthreads();
    }
}

// grid: (64-sample blocks x channels) / kLsWaves.  count[2 ch] = kernels that read the channel, count[2 ch + 1] = where
// their list starts in hits; an entry is kernel | tap mask << 16.
template <typename T>
__global__ __launch_bounds__(kLsWaves *kWave) void convblock_backward_x_4x4_kernel(const T *__restrict__ tg,
                                                                                 const int32_t *__restrict__ count,
                                                                                 const int32_t *__restrict__ hits,
                                                                                 const int32_t *__restrict__ sel,
                                                                                 const uint32_t *__restrict__ tcodes,
                                                                                 T *__restrict__ gx, Geom g)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    const int sblocks = (g.n + kWave - 1) / kWave;
    const int item = uniform((int)blockIdx.x * kLsWaves + wave);      // channel fastest: a workgroup shares its samples
    if (item >= sblocks * g.cin) return;
    const int sb = item / g.cin, ch = item - sb * g.cin;
    const int64_t n = (int64_t)sb * kWave + lane;
    const bool live = n < g.n;
    const int64_t ns = live ? n : 0;
    T *plane = reinterpret_cast<T *>(smem) + ((size_t)wave * kWave + lane) * kGradStride;
#pragma unroll
    for (int e = 0; e < kGradStride; ++e) plane[e] = T(0);
    const int nhits = count[2 * ch];
    const int32_t *hit = hits + count[2 * ch + 1];
    constexpr int PER = 16 / (int)sizeof(T);
    auto fetch = [&](int k, T (&gt)[32], uint32_t &codes) {
        const int c = hit[k] & 0xFFFF;
        const T *src = tg + ((int64_t)c * g.n + ns) * 32;
#pragma unroll
        for (int q = 0; q < 32 / PER; ++q) {
            const u32x4 raw = reinterpret_cast<const u32x4 *>(src)[q];
            T part[PER];
            __builtin_memcpy(part, &raw, 16);
#pragma unroll
            for (int e = 0; e < PER; ++e) gt[q * PER + e] = part[e];
        }
        codes = tcodes[(int64_t)c * g.n + ns];
    };
    T cur[32], nxt[32];
    uint32_t cur_codes = 0, nxt_codes = 0;
    if (nhits > 0) fetch(0, cur, cur_codes);
    for (int k = 0; k < nhits; ++k) {
        if (k + 1 < nhits) fetch(k + 1, nxt, nxt_codes);              // in flight during the updates of hit k
        const int ent = hit[k];
        const int c = ent & 0xFFFF, mask = (ent >> 16) & 0xFF;
        int pc[4];                                                    // padded position of every cell's maximum
#pragma unroll
        for (int cell = 0; cell < 4; ++cell) {
            const int code = (cur_codes >> (8 * cell)) & 3;
            pc[cell] = (2 * (cell >> 1) + (code >> 1)) * 6 + 2 * (cell & 1) + (code & 1);
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if ((mask >> t) & 1) {                                    // wave-uniform: tap t of kernel c reads this channel
                const Tap tp = unpack_tap(sel[c * 8 + t], tap_limit(g));
                const int off = tp.ry * 6 + tp.rx;
                T old[4];
                // the four cells' targets of one tap are distinct elements; taps are applied one after the other
#pragma unroll
                for (int cell = 0; cell < 4; ++cell) old[cell] = plane[pc[cell] + off];
#pragma unroll
                for (int cell = 0; cell < 4; ++cell) plane[pc[cell] + off] = old[cell] + cur[cell * 8 + t];
            }
        }
#pragma unroll
        for (int e = 0; e < 32; ++e) cur[e] = nxt[e];
        cur_codes = nxt_codes;
    }
    if (live) {
        T out[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) out[e] = plane[((e >> 2) + 1) * 6 + (e & 3) + 1];
        T *dst = gx + (n * g.cin + ch) * 16;
#pragma unroll
        for (int q = 0; q < 16 / PER; ++q) {
            u32x4 raw;
            __builtin_memcpy(&raw, &out[q * PER], 16);
            reinterpret_cast<u32x4 *>(dst)[q] = raw;
        }
    }
}

}  // namespace

// The shapes this file covers: what the last block of a 32x32-input network sees (n counts 64-sample groups for packed words).
bool clg_convblock_is_4x4(const Geom &g)
{
    return g.h == 4 && g.w == 4 && g.kh == 3 && g.kw == 3 && g.sh == 1 && g.sw == 1 && g.ph == 1 && g.pw == 1 && g.n >= 32;
}

template <typename Ops>
static int launch_4x4(const Geom &g, const void *x, const void *params, const int32_t *sel, void *y, uint8_t *argmax, hipStream_t st,
                      const char *name, int n_first = 0)
{
    using T = typename Ops::Elem;
    const int sblocks = (g.n - n_first + kWave - 1) / kWave;
    int ct = 64;                                                      // 16 kernels per wavefront unless that starves the chip
    while (ct > kLsWaves && (int64_t)sblocks * ((g.c + ct - 1) / ct) < 1024) ct >>= 1;
    CLG_REQUIRE((g.c + ct - 1) / ct <= 65535, "%s: too many kernels for one launch (%d)", name, g.c);
    const dim3 grid((unsigned)sblocks, (unsigned)((g.c + ct - 1) / ct)), block(kLsWaves * kWave);
    const size_t lds = (size_t)kLsWaves * kWave * kLsStride * sizeof(T);
    if (int e = allow_lds(convblock_forward_4x4_kernel<Ops>, lds, name)) return e;
    hipLaunchKernelGGL(convblock_forward_4x4_kernel<Ops>, grid, block, lds, st, (const T *)x, params, sel, (T *)y, argmax, g, ct, n_first);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// folded: [c][28] coefficients (convblock_w_prepare_kernel).
int clg_convblock_forward_4x4(int dtype, const Geom &g, const void *x, const void *folded, const int32_t *sel, void *y, uint8_t *argmax,
                              hipStream_t st, const char *name)
{
    if (dtype == CLG_F32) return launch_4x4<FloatOps<float>>(g, x, folded, sel, y, argmax, st, name);
    return launch_4x4<FloatOps<double>>(g, x, folded, sel, y, argmax, st, name);
}

// gates: uint8 [c][7] gate ids; x, y: 64 samples per word.
int clg_convblock_eval_packed_4x4(const Geom &g, const uint64_t *x, const uint8_t *gates, const int32_t *sel, uint64_t *y, hipStream_t st,
                                  const char *name)
{
    const char *e_half = clg_knob(K_PACKED_4X4_HALVES);            // 0: one 64-bit pass per kernel (measurement)
    if (e_half && atoi(e_half) == 0) return launch_4x4<BitOps>(g, x, gates, sel, y, nullptr, st, name);
    // full blocks of 64 groups go to the half-word kernel, what is left of the batch to the 64-bit one
    const int sblocks = g.n / kWave;
    if (sblocks * kWave < g.n) {
        if (int e = launch_4x4<BitOps>(g, x, gates, sel, y, nullptr, st, name, sblocks * kWave)) return e;
        if (sblocks == 0) return CLG_OK;
    }
    int ct = 64;
    while (ct > kLsWaves && (int64_t)sblocks * ((g.c + ct - 1) / ct) < 2048) ct >>= 1;
    const int ctiles = (g.c + ct - 1) / ct;
    const int64_t wgs = (int64_t)8 * ((sblocks + 7) / 8) * ctiles;
    CLG_REQUIRE(wgs < (1ll << 31), "%s: problem too large for one launch", name);
    const size_t lds = (size_t)kLsWaves * kWave * kLsStride * sizeof(uint32_t);
    if (int e = allow_lds(convblock_eval_packed_4x4_kernel, lds, name)) return e;
    hipLaunchKernelGGL(convblock_eval_packed_4x4_kernel, dim3((unsigned)wgs), dim3(kLsWaves * kWave), lds, st, x, gates, sel, y, g, ct, ctiles,
                       sblocks);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// ---- gradients: launchers (the caller has run the prepare kernel: folded coefficients and per-channel kernel lists) ----
// tap gradients [c][n][32] followed by the arg-max codes [c][n] of the same (kernel, sample) pairs
static size_t tg_elems_bytes(int dtype, const Geom &g) { return (size_t)g.c * g.n * 32 * (dtype == CLG_F64 ? 8 : 4); }
size_t clg_convblock_backward_4x4_tg_bytes(int dtype, const Geom &g) { return tg_elems_bytes(dtype, g) + (size_t)g.c * g.n * 4; }

template <typename T>
static int launch_backward_4x4(const Geom &g, const void *x, const void *folded, const int32_t *sel, const void *gy, const uint8_t *argmax,
                               void *tg, void *gw, const void *probs, const int32_t *count, const int32_t *hits, void *gx, hipStream_t st,
                               const char *name)
{
    int ct = 16;                                                      // kernels per workgroup, at least ~1024 workgroups
    while (ct > 1 && (g.c + ct - 1) / ct < 1024) ct >>= 1;
    const size_t lds = (size_t)kLsWaves * kWave * kLsStride * sizeof(T);
    if (int e = allow_lds(convblock_backward_4x4_kernel<T>, lds + 1024, name)) return e;
    uint32_t *tcodes = reinterpret_cast<uint32_t *>(reinterpret_cast<unsigned char *>(tg) + tg_elems_bytes(sizeof(T) == 8 ? CLG_F64 : CLG_F32, g));
    hipLaunchKernelGGL(convblock_backward_4x4_kernel<T>, dim3((unsigned)((g.c + ct - 1) / ct)), dim3(kLsWaves * kWave), lds, st,
                       (const T *)x, (const T *)folded, sel, (const T *)gy, argmax, gx != nullptr ? (T *)tg : (T *)nullptr, tcodes, (T *)gw,
                       (const T *)probs, g, ct);
    CLG_CHECK_LAUNCH(name);
    if (gx == nullptr) return CLG_OK;
    const int64_t items = (int64_t)((g.n + kWave - 1) / kWave) * g.cin;
    CLG_REQUIRE((items + kLsWaves - 1) / kLsWaves < (1ll << 31), "%s: too many (sample block, channel) pairs for one launch", name);
    const size_t lds_x = (size_t)kLsWaves * kWave * kGradStride * sizeof(T);
    if (int e = allow_lds(convblock_backward_x_4x4_kernel<T>, lds_x, name)) return e;
    hipLaunchKernelGGL(convblock_backward_x_4x4_kernel<T>, dim3((unsigned)((items + kLsWaves - 1) / kLsWaves)), dim3(kLsWaves * kWave),
                       lds_x, st, (const T *)tg, count, hits, sel, (const uint32_t *)tcodes, (T *)gx, g);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// gw: gradient w.r.t. the probabilities, or w.r.t. the logits when probs (their softmax) is given; gx may be null.
int clg_convblock_backward_4x4(int dtype, const Geom &g, const void *x, const void *folded, const int32_t *sel, const void *gy,
                               const uint8_t *argmax, void *tg, void *gw, const void *probs, const int32_t *count, const int32_t *hits,
                               void *gx, hipStream_t st, const char *name)
{
    if (dtype == CLG_F32) return launch_backward_4x4<float>(g, x, folded, sel, gy, argmax, tg, gw, probs, count, hits, gx, st, name);
    return launch_backward_4x4<double>(g, x, folded, sel, gy, argmax, tg, gw, probs, count, hits, gx, st, name);
}
