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
__device__ __forceinline__ LaneTaps lane_taps(const int32_t *__restrict__ sel, int c)
{
    LaneTaps t;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const Tap tp = unpack_tap(sel[c * 8 + k]);
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

// grid: (64-sample blocks, kernel tiles of ct kernels); LDS: kLsWaves * 64 * kLsStride elements.
// params: folded coefficients [c][28] (float gates) or gate ids uint8 [c][7] (packed words, argmax = null)
template <typename Ops>
__global__ __launch_bounds__(kLsWaves *kWave) void convblock_forward_4x4_kernel(const typename Ops::Elem *__restrict__ x,
                                                                              const void *__restrict__ params,
                                                                              const int32_t *__restrict__ sel,
                                                                              typename Ops::Elem *__restrict__ y,
                                                                              uint8_t *__restrict__ argmax, Geom g, int ct)
{
    using T = typename Ops::Elem;
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    T *mine = reinterpret_cast<T *>(smem) + ((size_t)wave * kWave + lane) * kLsStride;
    const int64_t n = (int64_t)blockIdx.x * kWave + lane;
    const bool live = n < g.n;
    const T *xn = x + (live ? n : 0) * g.cin * 16;
#pragma unroll
    for (int e = 0; e < kLsStride; ++e) mine[e] = T(0);
    const int c0 = blockIdx.y * ct, c1 = min(g.c, c0 + ct);
    int c = c0 + wave;
    if (c >= c1) return;
    LaneTaps tp = lane_taps(sel, c);
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
            tp = lane_taps(sel, cn);
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
            best[cell] = Ops::pool4(r, code);
            codes |= code << (8 * cell);
        }
        if (live) {
            const int64_t o = (n * g.c + c) * 4;
            constexpr int PER = 16 / (int)sizeof(T);
#pragma unroll
            for (int q = 0; q < 4 / PER; ++q) {
                u32x4 raw;
                __builtin_memcpy(&raw, &best[q * PER], 16);
                reinterpret_cast<u32x4 *>(y + o)[q] = raw;
            }
            if (argmax != nullptr) *reinterpret_cast<uint32_t *>(argmax + o) = (uint32_t)codes;
        }
        if (!more) break;
        c = cn;
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
                      const char *name)
{
    using T = typename Ops::Elem;
    const int sblocks = (g.n + kWave - 1) / kWave;
    int ct = 64;                                                      // 16 kernels per wavefront unless that starves the chip
    while (ct > kLsWaves && (int64_t)sblocks * ((g.c + ct - 1) / ct) < 1024) ct >>= 1;
    CLG_REQUIRE((g.c + ct - 1) / ct <= 65535, "%s: too many kernels for one launch (%d)", name, g.c);
    const dim3 grid((unsigned)sblocks, (unsigned)((g.c + ct - 1) / ct)), block(kLsWaves * kWave);
    const size_t lds = (size_t)kLsWaves * kWave * kLsStride * sizeof(T);
    if (int e = allow_lds(convblock_forward_4x4_kernel<Ops>, lds, name)) return e;
    hipLaunchKernelGGL(convblock_forward_4x4_kernel<Ops>, grid, block, lds, st, (const T *)x, params, sel, (T *)y, argmax, g, ct);
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
    return launch_4x4<BitOps>(g, x, gates, sel, y, nullptr, st, name);
}
