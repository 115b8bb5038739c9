// Plans and small device helpers shared by the LDS-tiled conv-logic kernels.
#pragma once

#include "conv_common.h"

constexpr int kLdsLimit = 160 * 1024;

// Division of a 31-bit value by a runtime constant: q = umulhi(x, mul) >> shr (d == 1: q = x).
struct FastDiv {
    uint32_t mul, shr, d;
};
static inline FastDiv make_fastdiv(uint32_t d)
{
    if (d <= 1) return FastDiv{0, 0, 1};
    uint32_t lg = 0;
    while ((1ull << lg) < d) ++lg;
    const uint32_t p = 31 + lg;
    const uint32_t mul = (uint32_t)(((1ull << p) + d - 1) / d);
    return FastDiv{mul, p - 32, d};
}
__device__ __forceinline__ uint32_t fdiv(uint32_t x, const FastDiv &f) { return f.d == 1 ? x : (__umulhi(x, f.mul) >> f.shr); }

struct TilePlan {
    int S;              // samples per workgroup
    int G;              // samples sharing one wavefront pass (input gradient; 1 when a sample has >= 64 cells)
    int CT;             // kernels per workgroup (forward)
    int NW;             // wavefronts per workgroup
    int rs, chs;        // row and plane stride of the LDS image (elements)
    int xe;             // elements of one LDS image region (S samples + tail)
    int slots;          // per sample: (ho/2) * wo lane slots (forward) / pooled cells (input gradient)
    int band_rows, bands;  // input gradient: image rows per workgroup band, number of bands
    int hit_split;         // input gradient: workgroups sharing the kernels of one (sample, band), partial images
    int hsw;               // input gradient: wavefronts of one workgroup sharing the kernels of one gradient plane
    int dummy_in_halo;     // input gradient: masked updates go to halo elements instead of a region of their own
    int64_t part_stride;   // input gradient: elements between partial images (0 when hit_split == 1)
    int planes;            // forward: LDS planes per sample (all input channels, or 2 per kernel of the tile)
    int subset;            // forward: 1 = only the channels the kernel tile reads are staged
    int one_row;           // forward: 1 = a lane slot is one conv position (ho * wo per sample) instead of a column of two rows
    int w_logits;          // forward: 1 = the gate parameters handed to the kernel are logits (softmax taken while staging them)
    void *folded_out = nullptr;   // forward: where the first sample block writes the folded coefficients [c, 7, 4] of its kernels (or null)
    void *padded_out = nullptr;   // forward: where the first kernel tile writes its staged, zero-padded image: [n][sample_elems] (or null)
    int padded_sample_elems = 0;  // cin * chs + ph * rs + pw: one sample of that copy
    FastDiv d_hw, d_w, d_slots, d_wo, d_wp, d_planes;
    size_t lds_bytes;
};

template <typename T>
__device__ __forceinline__ T dpp_xor1(T v)
{
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)u, 0xB1, 0xF, 0xF, true);
        const uint32_t hi = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(u >> 32), 0xB1, 0xF, 0xF, true);
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    }
}

// value of the lane `delta` lanes up (ds_bpermute)
template <typename T>
__device__ __forceinline__ T lane_up(T v, int delta)
{
    const int src = (int)((threadIdx.x & 63) + delta) << 2;
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, v)));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = __builtin_amdgcn_ds_bpermute(src, (int)(uint32_t)u);
        const uint32_t hi = __builtin_amdgcn_ds_bpermute(src, (int)(uint32_t)(u >> 32));
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    }
}

// value of the lane DELTA lanes up inside a row of 16 lanes, as a DPP row shift (no LDS round trip); lanes whose
// source falls outside the row read 0
template <int DELTA, typename T>
__device__ __forceinline__ T row_up(T v)
{
    static_assert(DELTA > 0 && DELTA < 16, "row shift");
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + DELTA, 0xF, 0xF, true));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)u, 0x100 + DELTA, 0xF, 0xF, true);
        const uint32_t hi = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(u >> 32), 0x100 + DELTA, 0xF, 0xF, true);
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    }
}

template <typename T>
__device__ __forceinline__ T to_sgpr(T v)
{
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)u);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(u >> 32));
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    }
}

// Workgroup `bid` of a 1-D grid of `nb` runs on XCD bid % 8 (each XCD has its own L2).  Returns the logical block it
// should take so that every XCD works on a CONTIGUOUS range of logical blocks: neighbours that read the same rows then
// share one L2 instead of fetching them once per XCD.  A bijection of 0..nb-1 for any nb.
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned bid, unsigned nb)
{
    constexpr unsigned kXcds = 8;
    const unsigned q = nb / kXcds, r = nb % kXcds, xcd = bid % kXcds, idx = bid / kXcds;
    return xcd < r ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
}

// ---- plan helpers (host) ---------------------------------------------------------------------
static inline TapLimit host_tap_limit(const Geom &g) { return TapLimit{g.cin, g.kh, g.kw}; }
static inline void plan_common(const Geom &g, TilePlan *p)
{
    p->rs = g.w + g.pw;
    p->chs = (g.h + g.ph) * p->rs;
    p->one_row = 0;
    p->d_hw = make_fastdiv((uint32_t)(g.h * g.w));
    p->d_w = make_fastdiv((uint32_t)g.w);
    p->d_wo = make_fastdiv((uint32_t)g.wo);
    p->d_wp = make_fastdiv((uint32_t)(g.wo / 2));
}

static inline int64_t image_elems(const Geom &g, const TilePlan &p, int S) { return (int64_t)S * g.cin * p.chs + g.ph * p.rs + g.pw; }

// The last tap row/column must stay inside the padded image for the shared-halo layout to hold.
static inline bool taps_inside(const Geom &g) { return (g.ho - 1) * g.sh + g.kh <= g.h + 2 * g.ph && (g.wo - 1) * g.sw + g.kw <= g.w + 2 * g.pw; }

// Kernels that want more than 48 KiB of dynamic LDS must be told once; the largest size granted so
// far is remembered per kernel so that steady-state launches make no runtime call besides the launch.
int clg_allow_lds(const void *kernel, size_t bytes, const char *name);
template <typename K>
static inline int allow_lds(K kernel, size_t bytes, const char *name)
{
    return clg_allow_lds(reinterpret_cast<const void *>(kernel), bytes, name);
}

// ---- kernels shared by the paths that read taps from a padded global copy of x ------------------
#if defined(__HIPCC__)
// Element `index` of a buffer of fewer than 2^32 bytes: the unsigned 32-bit byte offset lets the load use a
// scalar base with a 32-bit vector offset instead of 64-bit address arithmetic per lane.
template <typename T>
__device__ __forceinline__ T load_at(const T *__restrict__ base, uint32_t index)
{
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(base) + (size_t)(index * (uint32_t)sizeof(T)));
}

// xp = zero-padded copy of x in the shared-halo layout: sample n at n * sample_elems, plane stride chs, row
// stride rs, pixel (iy, ix) at (iy + ph) * rs + ix + pw.  A job with total = 0 does nothing.
template <typename T>
struct PadJob {
    const T *x;
    T *xp;
    Geom g;
    FastDiv d_sample, d_chs, d_rs;
    int chs, rs, sample_elems;
    int64_t total;
};
template <typename T>
__device__ __forceinline__ void pad_image_elem(const PadJob<T> &j, int64_t e)
{
    if (e >= j.total) return;
    const uint32_t n = fdiv((uint32_t)e, j.d_sample), rem = (uint32_t)e - n * (uint32_t)j.sample_elems;
    const uint32_t plane = fdiv(rem, j.d_chs), r2 = rem - plane * (uint32_t)j.chs;
    const uint32_t row = fdiv(r2, j.d_rs), col = r2 - row * (uint32_t)j.rs;
    T v = T(0);
    if (plane < (uint32_t)j.g.cin && row - (uint32_t)j.g.ph < (uint32_t)j.g.h && col >= (uint32_t)j.g.pw)   // chs may hold more rows than h + ph
        v = j.x[(((int64_t)n * j.g.cin + plane) * j.g.h + (row - j.g.ph)) * j.g.w + (col - j.g.pw)];
    j.xp[e] = v;
}

template <typename T>
static inline PadJob<T> make_pad_job(const T *x, T *xp, const Geom &g, int rs, int chs, int sample_elems)
{
    PadJob<T> j;
    j.x = x, j.xp = xp, j.g = g, j.chs = chs, j.rs = rs, j.sample_elems = sample_elems;
    j.d_sample = make_fastdiv((uint32_t)sample_elems), j.d_chs = make_fastdiv((uint32_t)chs), j.d_rs = make_fastdiv((uint32_t)rs);
    j.total = (int64_t)sample_elems * g.n;
    return j;
}
template <typename T>
static inline PadJob<T> no_pad_job()
{
    PadJob<T> j = {};
    j.total = 0;
    return j;
}
template <typename T>
static inline unsigned pad_blocks(const PadJob<T> &j) { return (unsigned)clg_ceil_div(j.total, 256); }

// folded coefficients [c][28] and tap offsets [c][8] in the padded-image layout (either is skipped when null) in the
// first blocks of the launch, the padded copy in the blocks from pad_block0 on: one launch sets a kernel up.
// from_logits: w holds the logits, whose softmax goes to probs_out.
template <typename P, typename T>
__global__ __launch_bounds__(256) void convblock_w_prepare_kernel(const P *__restrict__ w, const int32_t *__restrict__ sel,
                                                                P *__restrict__ folded, int32_t *__restrict__ taps, int C, int rs,
                                                                int chs, TapLimit lim, PadJob<T> pad, int pad_block0, int from_logits = 0,
                                                                P *__restrict__ probs_out = nullptr)
{
    if ((int)blockIdx.x >= pad_block0) {
        pad_image_elem(pad, (int64_t)(blockIdx.x - pad_block0) * 256 + threadIdx.x);
        return;
    }
    const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (taps != nullptr && q < (int64_t)C * 8) {
        const Tap tp = unpack_tap(sel[q], lim);
        taps[q] = tp.ch * chs + tp.ry * rs + tp.rx;
    }
    if (folded != nullptr && q < (int64_t)C * 7) {
        P pr[16];
        if (from_logits) {                                           // w holds logits: softmax here, written out for the backward pass
            softmax16(w + q * 16, pr);
            if (probs_out != nullptr) {
#pragma unroll
                for (int i = 0; i < 16; ++i) probs_out[q * 16 + i] = pr[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) pr[i] = w[q * 16 + i];
        }
        const Coef<P> cf = fold16(pr);
        folded[q * 4 + 0] = cf.ab;
        folded[q * 4 + 1] = cf.a;
        folded[q * 4 + 2] = cf.b;
        folded[q * 4 + 3] = cf.one;
    }
}
#endif
