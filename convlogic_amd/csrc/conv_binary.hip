// Fused conv-logic block on BINARY inputs (every x in {0, 1}): the first block of a logic network, whose input is the
// thresholded image (src/convlogic/data.py:46-50).  float32, stride 1, images at most 32 columns wide.
//
// With binary taps the 7-gate tree of a kernel is a function of its 8 tap bits, so
//   forward          one 256-entry table per kernel, LUT_c[t] = tree_c(bits of t), made by the SAME three-FMA gate() the
//                    generic kernels evaluate (so values and pool arg-max are bit-identical to theirs); the image is kept as
//                    one 32-bit word per row, a lane owns a pair of conv rows of one sample, forms its 8 tap words with two
//                    shifts each, transposes them to 64 tap bytes (three butterfly stages per row) and pools four table
//                    reads per cell.  Besides y it stores one uint16 per pooled cell: arg-max code << 8 | tap byte.
//   weight gradient  grad_w[c] = sum_t H_c[t] * D_c[t] with H_c[t] = sum of grad_y over the cells of kernel c whose tap
//                    byte is t: a histogram streamed from (grad_y, tap byte) -- no image, no tree -- and a 256-term
//                    finish per kernel.  Bins are private to a lane (LDS [256][64]), so the order of additions is fixed.
//   input gradient   the walk of the generic kernels (one owner wavefront per (sample, input channel) plane, kernels of
//                    the channel in increasing order, read-add-write into an LDS plane nobody else touches), with the
//                    tap derivative as a product of two 16-entry table reads, d tree / d tap_i = F1[other nibble] *
//                    F2_i[own nibble], from a 640-byte LDS slot per wavefront (two taps of one nibble in one ds_read2_b32)
//                    instead of 8 tap reads and 49 FMAs.
// Replaces, for such inputs, src/convlogic/cuda/full_convlogic_kernel.cu:10-145 (forward), :233-363 (input gradient),
// :463-701 (weight gradient).
#include <stdlib.h>

#include <algorithm>

#include "conv_tile.h"

int clg_convblock_check(const clg_conv_geom *gg, Geom *g, int dtype, const char *name);

namespace {

constexpr int kFtab = 160;          // per kernel: F1[2][16], F2[8][16]

// ---- context: what the forward leaves for the backward pass (one device buffer) --------------------------------
struct BinCtx {
    size_t bits_off, lut_off, tapinfo_off, probs_off, folded_off, ftab_off, xtap_off, count_off, hits_off, total;
    int RP;         // rows of a bit plane: h + 2 ph
    int prs;        // row pitch of a gradient plane: w + pw (right halo of a row = left halo of the next)
    int plane;      // elements of a gradient plane incl. the last row's halo
};
size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
BinCtx bin_ctx(const Geom &g)
{
    BinCtx c;
    c.RP = g.h + 2 * g.ph;
    c.prs = g.w + g.pw;
    c.plane = (g.h + 2 * g.ph) * c.prs + g.pw + 1;
    c.bits_off = 0;
    c.lut_off = align256((size_t)g.n * g.cin * c.RP * 4);
    c.tapinfo_off = align256(c.lut_off + (size_t)g.c * 256 * 4);
    c.probs_off = align256(c.tapinfo_off + (size_t)g.c * 8 * 4);
    c.folded_off = align256(c.probs_off + (size_t)g.c * 112 * 4);
    c.ftab_off = align256(c.folded_off + (size_t)g.c * 28 * 4);
    c.xtap_off = align256(c.ftab_off + (size_t)g.c * kFtab * 4);
    c.count_off = align256(c.xtap_off + (size_t)g.c * 8 * 4);
    c.hits_off = align256(c.count_off + (size_t)g.cin * 8);
    c.total = align256(c.hits_off + (size_t)g.cin * g.c * 4);
    return c;
}

bool bin_supported(const Geom &g, int dtype)
{
    const int hp = g.ho / 2, wp = g.wo / 2;
    return dtype == CLG_F32 && g.sh == 1 && g.sw == 1 && g.w <= 32 && g.wo <= 32 && g.ho % 2 == 0 && g.wo % 2 == 0 && hp >= 1 && wp >= 1 &&
           hp * wp <= 256 && (hp * wp) % 4 == 0 && g.c <= 65535 && (int64_t)g.cin * (g.h + 2 * g.ph) < 65536 && (int64_t)g.cin * g.c <= (1ll << 22) && g.kw <= 32 && g.pw <= 31 && taps_inside(g) &&
           (int64_t)g.n * g.cin * (g.h + 2 * g.ph) < (1ll << 30) && (int64_t)g.n * g.c * hp * wp < (1ll << 31);
}

// ---- set-up launch ------------------------------------------------------------------------------------------------
// blocks [0, C): kernel c -- softmax / fold, the 256-entry table, the derivative tables, tap descriptors
// blocks [C, C + list_blocks): per input channel, the kernels that read it (increasing order) with their tap masks
// blocks from pack0 on: the image as bit rows, and the check that it is binary
struct PrepArgs {
    const float *x, *w;
    const int32_t *sel;
    uint32_t *bits;
    float *lut, *probs, *folded, *ftab;
    int32_t *tapinfo, *xtap, *count, *hits;
    int32_t *bad;            // set to 1 when some x is neither 0 nor 1 (may be host memory the device can write)
    int w_logits, list_blocks, pack0, RP, prs;
    FastDiv d_h, d_cinh;
};

__global__ __launch_bounds__(256) void convblock_bin_prepare_kernel(PrepArgs a, Geom g)
{
    const int tid = threadIdx.x, lane = tid & 63;
    if ((int)blockIdx.x < g.c) {
        __shared__ float cf[28];
        const int c = blockIdx.x;
        if (tid < 7) {
            const int64_t q = (int64_t)c * 7 + tid;
            float pr[16];
            if (a.w_logits) {
                softmax16(a.w + q * 16, pr);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = a.w[q * 16 + i];
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) a.probs[q * 16 + i] = pr[i];
            const Coef<float> k = fold16(pr);
            cf[4 * tid] = k.ab, cf[4 * tid + 1] = k.a, cf[4 * tid + 2] = k.b, cf[4 * tid + 3] = k.one;
            a.folded[q * 4] = k.ab, a.folded[q * 4 + 1] = k.a, a.folded[q * 4 + 2] = k.b, a.folded[q * 4 + 3] = k.one;
        }
        if (tid >= 64 && tid < 72) {
            const int t = tid - 64;
            const Tap tp = unpack_tap(a.sel[(int64_t)c * 8 + t], tap_limit(g));   // (forced into the layer's ranges)
            const int sh = tp.rx - g.pw;                              // tap word = row word >> sh (<< -sh)
            a.tapinfo[c * 8 + t] = ((tp.ch * a.RP + tp.ry) << 16) | ((sh < 0 ? -sh : 0) << 8) | (sh > 0 ? sh : 0);
            a.xtap[c * 8 + t] = tp.ry * a.prs + tp.rx;                 // offset of the tap in a gradient plane
        }
        __syncthreads();
        Tree<float> tr;
#pragma unroll
        for (int q = 0; q < 7; ++q) tr.g[q] = Coef<float>{cf[4 * q], cf[4 * q + 1], cf[4 * q + 2], cf[4 * q + 3]};
        float tap[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) tap[i] = (float)((tid >> i) & 1);
        const TreeVals<float> tv = eval_tree(tr, tap);
        a.lut[(int64_t)c * 256 + tid] = tv.root;
        if (tid < kFtab) {
            // F1[q][nib of the OTHER side] = d root / d mid_q; F2[i][own nibble] = d mid / d leaf * d leaf / d tap_i
            float v;
            const int nib = tid & 15;
            float nb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) nb[i] = (float)((nib >> i) & 1);
            auto coef = [&](int q) { return Coef<float>{cf[4 * q], cf[4 * q + 1], cf[4 * q + 2], cf[4 * q + 3]}; };   // (run-time gate index)
            if (tid < 32) {
                const int q = tid >> 4;                              // F1[q] is indexed by the nibble of side 1 - q
                const int o = 1 - q;
                const float l0 = gate(coef(2 * o), nb[0], nb[1]), l1 = gate(coef(2 * o + 1), nb[2], nb[3]);
                const float mo = gate(coef(4 + o), l0, l1);
                v = q == 0 ? gate_da(tr.g[6], mo) : gate_db(tr.g[6], mo);
            } else {
                const int i = (tid - 32) >> 4;                       // tap 0..7
                const int p = i >> 1, q = p >> 1, pl = p & 1, s = i & 1;   // leaf, side, leaf inside the side, operand
                const float pa = pl ? nb[0] : nb[2], pb = pl ? nb[1] : nb[3];            // taps of the partner leaf
                const float oa = pl ? nb[2] : nb[0], ob = pl ? nb[3] : nb[1];            // taps of the own leaf
                const float partner = gate(coef(2 * q + (1 - pl)), pa, pb);
                const float dm = pl == 0 ? gate_da(coef(4 + q), partner) : gate_db(coef(4 + q), partner);
                const float dl = s == 0 ? gate_da(coef(p), ob) : gate_db(coef(p), oa);
                v = dm * dl;
            }
            a.ftab[(int64_t)c * kFtab + tid] = v;
        }
        return;
    }
    if ((int)blockIdx.x < g.c + a.list_blocks) {
        // one wavefront per input channel: lanes test 64 kernels at a time, matches are appended in order
        const int ch = uniform((int)(blockIdx.x - g.c) * 4 + (tid >> 6));
        if (ch >= g.cin) return;
        int n = 0;
        for (int c0 = 0; c0 < g.c; c0 += kWave) {
            const int c = c0 + lane;
            int mask = 0;
            if (c < g.c) {
#pragma unroll
                for (int t = 0; t < 8; ++t) mask |= (tap_channel(a.sel[c * 8 + t], g.cin) == ch) << t;
            }
            const uint64_t vote = __ballot(mask != 0);
            if (mask) {
                const int before = __builtin_amdgcn_mbcnt_hi((uint32_t)(vote >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)vote, 0));
                a.hits[(int64_t)ch * g.c + n + before] = c | (mask << 16);
            }
            n += __popcll(vote);
        }
        if (lane == 0) {
            a.count[2 * ch] = n;
            a.count[2 * ch + 1] = ch * g.c;
        }
        return;
    }
    // bit rows: a wavefront packs two image rows per step (lane = row of the pair * 32 + column)
    const int64_t rows = (int64_t)g.n * g.cin * g.h;
    const int r = lane >> 5, col = lane & 31;
    const int64_t wave0 = (int64_t)(blockIdx.x - a.pack0) * 4 + (tid >> 6), nwaves = (int64_t)(gridDim.x - a.pack0) * 4;
    bool bad = false;
    for (int64_t pair = wave0; pair * 2 < rows; pair += nwaves) {
        const int64_t row = pair * 2 + r;
        const bool ok = row < rows && col < g.w;
        const float v = ok ? a.x[row * g.w + col] : 0.f;
        bad = bad || (v != 0.f && v != 1.f);
        const uint64_t m = __ballot(v != 0.f);
        if (col == 0 && row < rows) {
            const uint32_t plane = fdiv((uint32_t)row, a.d_h), iy = (uint32_t)row - plane * (uint32_t)g.h;
            uint32_t *dst = a.bits + (int64_t)plane * a.RP;
            dst[iy + g.ph] = (uint32_t)(r ? m >> 32 : m);
            if (iy == 0)
                for (int k = 0; k < g.ph; ++k) dst[k] = 0;
            if (iy == (uint32_t)g.h - 1)
                for (int k = 0; k < g.ph; ++k) dst[g.ph + g.h + k] = 0;
        }
    }
    if (bad) *a.bad = 1;
}

// ---- forward --------------------------------------------------------------------------------------------------------
struct BinFwd {
    int S, LB, CT, ktiles, RP, hp, wp;
    int tr_words;       // 32-bit words of a wavefront's buffer for the ordered write-out
    FastDiv d_hp, d_ktiles, d_lb, d_npc;
};

// 8 words of 32 columns -> per column one byte: afterwards byte g of word j holds bit (8 g + j) of the 8 input words
// (input word i in bit i).  Three stages of block swaps inside every byte column.
// (m & x) | (~m & y) in one instruction; the mask sits in a scalar register
__device__ __forceinline__ uint32_t bit_select(uint32_t m, uint32_t x, uint32_t y)
{
    uint32_t d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(m), "v"(x), "v"(y));
    return d;
}
__device__ __forceinline__ void transpose_bits8(uint32_t (&t)[8])
{
#define CLG_SWAP(a, b, m, s)                                     \
    do {                                                         \
        const uint32_t na = bit_select(m, t[a], t[b] << (s));    \
        const uint32_t nb = bit_select(m, t[a] >> (s), t[b]);    \
        t[a] = na, t[b] = nb;                                    \
    } while (0)
    CLG_SWAP(0, 1, 0x55555555u, 1); CLG_SWAP(2, 3, 0x55555555u, 1); CLG_SWAP(4, 5, 0x55555555u, 1); CLG_SWAP(6, 7, 0x55555555u, 1);
    CLG_SWAP(0, 2, 0x33333333u, 2); CLG_SWAP(1, 3, 0x33333333u, 2); CLG_SWAP(4, 6, 0x33333333u, 2); CLG_SWAP(5, 7, 0x33333333u, 2);
    CLG_SWAP(0, 4, 0x0F0F0F0Fu, 4); CLG_SWAP(1, 5, 0x0F0F0F0Fu, 4); CLG_SWAP(2, 6, 0x0F0F0F0Fu, 4); CLG_SWAP(3, 7, 0x0F0F0F0Fu, 4);
#undef CLG_SWAP
}

typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2u __attribute__((ext_vector_type(2), aligned(4)));
typedef float f32x2u __attribute__((ext_vector_type(2), aligned(4)));

// A piece of PC pooled cells of one row as it travels through the write-out buffer: PC floats of y, PC uint16 of taps.
template <int PC>
struct Piece;
template <>
struct Piece<4> {
    using Y = float4;
    using A = uint2;
    static __device__ __forceinline__ Y y(const float *v) { return make_float4(v[0], v[1], v[2], v[3]); }
    static __device__ __forceinline__ A a(const uint32_t *t) { return make_uint2(t[0] | (t[1] << 16), t[2] | (t[3] << 16)); }
    static __device__ __forceinline__ void store_y(float *dst, const Y &v) { *reinterpret_cast<f32x4u *>(dst) = f32x4u{v.x, v.y, v.z, v.w}; }
    static __device__ __forceinline__ void store_a(uint16_t *dst, const A &v) { *reinterpret_cast<u32x2u *>(dst) = u32x2u{v.x, v.y}; }
};
template <>
struct Piece<2> {
    using Y = float2;
    using A = uint32_t;
    static __device__ __forceinline__ Y y(const float *v) { return make_float2(v[0], v[1]); }
    static __device__ __forceinline__ A a(const uint32_t *t) { return t[0] | (t[1] << 16); }
    static __device__ __forceinline__ void store_y(float *dst, const Y &v) { *reinterpret_cast<f32x2u *>(dst) = f32x2u{v.x, v.y}; }
    static __device__ __forceinline__ void store_a(uint16_t *dst, const A &v) { *reinterpret_cast<uint32_t *>(dst) = v; }
};

// grid: (sample tiles x kernel tiles) flat.  LDS: tables of the CT kernels [CT][256], bit planes of the S samples and, with
// PC > 0 (rows of a multiple of PC = 4 or 2 cells), one write-out buffer per wavefront; PC = 0 writes rows directly.
template <int PC>
__global__ __launch_bounds__(512) void convblock_bin_forward_kernel(const uint32_t *__restrict__ bits, const float *__restrict__ lut,
                                                                  const int32_t *__restrict__ tapinfo, float *__restrict__ y,
                                                                  uint16_t *__restrict__ aux, Geom g, BinFwd p)
{
    extern __shared__ __align__(16) uint32_t smem_u[];
    float *lut_s = reinterpret_cast<float *>(smem_u);
    uint32_t *img = smem_u + p.CT * 256;
    uint32_t *trbuf = img + ((p.S * g.cin * p.RP + 3) & ~3);
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int lane = tid & (kWave - 1), wave = uniform(tid >> 6), nw = nthreads >> 6;
    const uint32_t b = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int stile = (int)fdiv(b, p.d_ktiles), ktile = (int)b - stile * p.ktiles;
    const int n0 = stile * p.S, s_cur = min(p.S, g.n - n0);
    const int c0 = ktile * p.CT, ct_cur = min(p.CT, g.c - c0);
    {
        const float4 *src = reinterpret_cast<const float4 *>(lut + (int64_t)c0 * 256);
        float4 *dst = reinterpret_cast<float4 *>(lut_s);
        for (int i = tid; i < ct_cur * 64; i += nthreads) dst[i] = src[i];
        const uint32_t *bsrc = bits + (int64_t)n0 * g.cin * p.RP;
        const int words = s_cur * g.cin * p.RP;
        for (int i = tid; i < words; i += nthreads) img[i] = bsrc[i];
    }
    __syncthreads();
    const int slots = s_cur * p.hp, P = p.hp * p.wp;
    const int units = p.LB * ct_cur;
    for (int u = wave; u < units; u += nw) {
        const int ct = (int)fdiv((uint32_t)u, p.d_lb), lb = u - ct * p.LB;     // wave-uniform
        const int v = lb * kWave + lane;
        const bool live = v < slots;
        const uint32_t vv = live ? (uint32_t)v : 0u;
        const uint32_t s = fdiv(vv, p.d_hp), rp = vv - s * (uint32_t)p.hp;
        const uint32_t *row0 = img + s * (uint32_t)(g.cin * p.RP) + 2 * rp;
        const int c = c0 + ct;
        const int32_t *ti = tapinfo + (int64_t)c * 8;
        uint32_t ta[8], tb[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t info = (uint32_t)ti[i];
            const uint32_t off = info >> 16, sl = (info >> 8) & 0xFF, sr = info & 0xFF;
            ta[i] = (row0[off] << sl) >> sr;
            tb[i] = (row0[off + 1] << sl) >> sr;
        }
        transpose_bits8(ta);
        transpose_bits8(tb);
        const float *L = lut_s + ct * 256;
        float yv[16];
        uint32_t ax[16];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const uint32_t i0 = (ta[2 * m] >> (8 * gq)) & 255u, i1 = (ta[2 * m + 1] >> (8 * gq)) & 255u;
                const uint32_t i2 = (tb[2 * m] >> (8 * gq)) & 255u, i3 = (tb[2 * m + 1] >> (8 * gq)) & 255u;
                const float v0 = L[i0], v1 = L[i1], v2 = L[i2], v3 = L[i3];
                float best = v0;                                      // first maximum in window order (0,0),(0,1),(1,0),(1,1)
                uint32_t t = i0;
                if (v1 > best) best = v1, t = i1 | 0x100u;
                if (v2 > best) best = v2, t = i2 | 0x200u;
                if (v3 > best) best = v3, t = i3 | 0x300u;
                yv[4 * gq + m] = best;
                ax[4 * gq + m] = t;
            }
            if (4 * gq + 4 >= p.wp) break;                            // wave-uniform
        }
        if constexpr (PC > 0) {
            // The lane holds one row of wp cells; rows of consecutive lanes are consecutive in memory.  Through a buffer of
            // the wavefront's own in LDS the rows go out as pieces of PC cells in lane order: every store instruction
            // writes one contiguous run per sample.
            using YP = typename Piece<PC>::Y;
            using AP = typename Piece<PC>::A;
            float *tb_y = reinterpret_cast<float *>(trbuf) + wave * p.tr_words;
            const int ys = p.wp + 4, npc = p.wp / PC;                 // padded row stride (floats); pieces per row
            constexpr int K = 16 / PC;
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (k < npc) *reinterpret_cast<YP *>(tb_y + lane * ys + PC * k) = Piece<PC>::y(yv + PC * k);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const uint32_t base = (uint32_t)((n0 * g.c + c) * P), sstep = (uint32_t)((g.c - 1) * P);
            // piece i of the wavefront = (row r, piece q of the row); its cell index in y / taps
            auto place = [&](int k, uint32_t &r, uint32_t &q, uint32_t &cell) {
                const uint32_t i = (uint32_t)(k * kWave + lane);
                r = fdiv(i, p.d_npc), q = i - r * (uint32_t)npc;
                const uint32_t vr = (uint32_t)(lb * kWave) + r;
                const bool ok = k < npc && (int)vr < slots;
                const uint32_t vs = ok ? vr : 0u;
                cell = base + vs * (uint32_t)p.wp + fdiv(vs, p.d_hp) * sstep + (uint32_t)PC * q;
                return ok;
            };
#pragma unroll
            for (int k = 0; k < K; ++k) {
                uint32_t r, q, cell;
                if (place(k, r, q, cell)) Piece<PC>::store_y(y + cell, *reinterpret_cast<const YP *>(tb_y + r * ys + PC * q));
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            uint32_t *tb_a = reinterpret_cast<uint32_t *>(tb_y);
            const int as = (p.wp >> 1) + 2;                            // padded row stride (dwords)
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (k < npc) *reinterpret_cast<AP *>(tb_a + lane * as + (PC / 2) * k) = Piece<PC>::a(ax + PC * k);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int k = 0; k < K; ++k) {
                uint32_t r, q, cell;
                if (place(k, r, q, cell)) Piece<PC>::store_a(aux + cell, *reinterpret_cast<const AP *>(tb_a + r * as + (PC / 2) * q));
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        } else if (live) {
            const int64_t cell0 = (((int64_t)(n0 + (int)s) * g.c + c) * p.hp + rp) * p.wp;
            float *yr = y + cell0;
            uint16_t *ar = aux + cell0;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                if (e < p.wp) {
                    yr[e] = yv[e];
                    ar[e] = (uint16_t)ax[e];
                }
            }
        }
    }
}

// ---- weight gradient: histogram of grad_y over the tap byte ---------------------------------------------------------
// One wavefront of HL active lanes per (kernel, part of the batch); lane-private bins bins[t][lane] (bank = lane: no
// conflicts, no atomics).  A wavefront's steps are a serial chain (tap bytes -> LDS reads -> adds -> LDS writes) and a CU
// holds 160 KiB / (256 * HL * 4 bytes) wavefronts; more wavefronts of fewer lanes do not pay (the chain per step stays as
// long), so HL = 64 is the default and the narrower instantiations are for measurement (CLG_BIN_HL).
// A lane takes 4 consecutive cells per step; equal tap bytes among them are chained in registers, the four stores then
// go out in order, so the bin holds the sum in program order.
struct BinHist {
    int C, P, Q, n, parts, per_part;      // Q = P / 4 quads per (sample, kernel) plane
    FastDiv d_q;
};
constexpr int kHistDepth = 8;           // steps whose loads are in flight together

// PLANE: a (sample, kernel) plane is exactly one step of the wavefront (P = 4 HL cells): the step index is the sample, so a
// step's addresses are a wave-uniform base plus a constant per lane and cost no vector arithmetic.
template <int HL, bool PLANE>
__global__ __launch_bounds__(HL) void convblock_bin_hist_kernel(const float *__restrict__ gy, const uint16_t *__restrict__ aux,
                                                                      float *__restrict__ hpart, BinHist p)
{
    extern __shared__ __align__(16) float bins[];                     // [256][HL]
    const int lane = threadIdx.x;
    const int c = blockIdx.x / p.parts, part = blockIdx.x - c * p.parts;
    const int s0 = part * p.per_part, s1 = min(p.n, s0 + p.per_part);
    {
        float4 *z = reinterpret_cast<float4 *>(bins);
        for (int i = lane; i < 256 * HL / 4; i += HL) z[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int items = (s1 - s0) * p.Q;                                // quads of this part
    const int64_t plane_stride = (int64_t)p.C * p.P;
    const float *gyc = gy + ((int64_t)s0 * p.C + c) * p.P;
    const uint16_t *axc = aux + ((int64_t)s0 * p.C + c) * p.P;
    float *mine = bins + lane;

    // loads never depend on a branch (an index past the end is clamped), so the compiler can count them and let a
    // whole group of steps stay in flight while the previous group is applied
    auto load = [&](int step, float4 &g4, uint2 &a2) {
        if constexpr (PLANE) {
            const int smp = min(step, s1 - s0 - 1);                   // wave-uniform (items = samples * HL)
            const float *gs = gyc + (int64_t)smp * plane_stride;
            const uint16_t *as = axc + (int64_t)smp * plane_stride;
            g4 = reinterpret_cast<const float4 *>(gs)[lane];
            a2 = reinterpret_cast<const uint2 *>(as)[lane];
        } else {
            int e = step * HL + lane;
            e = e < items ? e : items - 1;
            const uint32_t smp = fdiv((uint32_t)e, p.d_q), quad = (uint32_t)e - smp * (uint32_t)p.Q;
            const int64_t at = smp * plane_stride + quad * 4;
            g4 = *reinterpret_cast<const float4 *>(gyc + at);
            a2 = *reinterpret_cast<const uint2 *>(axc + at);
        }
    };
    auto apply = [&](const float4 &g4, const uint2 &a2) {
        const uint32_t t0 = a2.x & 255u, t1 = (a2.x >> 16) & 255u, t2 = a2.y & 255u, t3 = (a2.y >> 16) & 255u;
        float r0 = mine[t0 * HL], r1 = mine[t1 * HL], r2 = mine[t2 * HL], r3 = mine[t3 * HL];
        asm volatile("" : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3));   // all four reads in flight together
        const float v0 = r0 + g4.x;
        const float v1 = (t1 == t0 ? v0 : r1) + g4.y;
        const float v2 = (t2 == t1 ? v1 : (t2 == t0 ? v0 : r2)) + g4.z;
        const float v3 = (t3 == t2 ? v2 : (t3 == t1 ? v1 : (t3 == t0 ? v0 : r3))) + g4.w;
        mine[t0 * HL] = v0;
        mine[t1 * HL] = v1;
        mine[t2 * HL] = v2;
        mine[t3 * HL] = v3;
    };
    const int steps = (items + HL - 1) / HL;
    if (steps > 0) {
        float4 G[2][kHistDepth];
        uint2 A[2][kHistDepth];
        // a group of kHistDepth steps; in a group that reaches past the end the lanes without a quad add 0
        auto apply_group = [&](int s0, const float4 (&Gd)[kHistDepth], const uint2 (&Ad)[kHistDepth]) {
            if (s0 >= steps) return;                                  // wave-uniform
            if ((s0 + kHistDepth) * HL <= items) {
#pragma unroll
                for (int d = 0; d < kHistDepth; ++d) apply(Gd[d], Ad[d]);
            } else {
#pragma unroll
                for (int d = 0; d < kHistDepth; ++d) {
                    float4 g4 = Gd[d];
                    if ((s0 + d) * HL + lane >= items) g4 = make_float4(0.f, 0.f, 0.f, 0.f);
                    apply(g4, Ad[d]);
                }
            }
        };
#pragma unroll
        for (int d = 0; d < kHistDepth; ++d) load(d, G[0][d], A[0][d]);
        for (int st = 0; st < steps; st += 2 * kHistDepth) {
#pragma unroll
            for (int d = 0; d < kHistDepth; ++d) load(st + kHistDepth + d, G[1][d], A[1][d]);     // (clamped past the end; unused then)
            apply_group(st, G[0], A[0]);
#pragma unroll
            for (int d = 0; d < kHistDepth; ++d) load(st + 2 * kHistDepth + d, G[0][d], A[0][d]);
            apply_group(st + kHistDepth, G[1], A[1]);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // lane l sums bins l, l+64, l+128, l+192 over the 64 lane copies, starting at its own column (conflict-free, fixed order)
    float *out = hpart + ((int64_t)c * p.parts + part) * 256;
#pragma unroll
    for (int q = 0; q < 256 / HL; ++q) {
        const float *row = bins + (q * HL + lane) * HL;
        float acc = 0.f;
        for (int k0 = 0; k0 < HL; k0 += 8) {
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = row[(lane + k0 + k) & (HL - 1)];
#pragma unroll
            for (int k = 0; k < 8; ++k) acc += v[k];
        }
        out[q * HL + lane] = acc;
    }
}

// grid: C, 256 threads: thread t weights the derivative of the tree at tap byte t with the histogram; the 28 coefficient
// sums are added over t in a fixed order, then the transform to the 16 gates (and the softmax backward for logits).
__global__ __launch_bounds__(256) void convblock_bin_wgrad_finish_kernel(const float *__restrict__ hpart, const float *__restrict__ folded,
                                                                       const float *__restrict__ probs, float *__restrict__ gw, int parts)
{
    __shared__ float sums[28];
    const int c = blockIdx.x, t = threadIdx.x;
    float H = 0.f;
    const float *hp = hpart + (int64_t)c * parts * 256 + t;
    int k = 0;
    for (; k + 8 <= parts; k += 8) {                                  // eight loads in flight, added in the order of one by one
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = hp[(k + u) * 256];
#pragma unroll
        for (int u = 0; u < 8; ++u) H += v[u];
    }
    for (; k < parts; ++k) H += hp[k * 256];
    Tree<float> tr;
    const float *fc = folded + (int64_t)c * 28;
#pragma unroll
    for (int q = 0; q < 7; ++q) tr.g[q] = Coef<float>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
    float tap[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) tap[i] = (float)((t >> i) & 1);
    const TreeVals<float> tv = eval_tree(tr, tap);
    float acc[28];
    auto put = [&](int q, float g, float a, float b) {
        const float ga = g * a;
        acc[4 * q] = ga * b, acc[4 * q + 1] = ga, acc[4 * q + 2] = g * b, acc[4 * q + 3] = g;
    };
    put(6, H, tv.mid[0], tv.mid[1]);
    const float g_m0 = H * gate_da(tr.g[6], tv.mid[1]), g_m1 = H * gate_db(tr.g[6], tv.mid[0]);
    put(4, g_m0, tv.leaf[0], tv.leaf[1]);
    put(5, g_m1, tv.leaf[2], tv.leaf[3]);
    const float g_l0 = g_m0 * gate_da(tr.g[4], tv.leaf[1]), g_l1 = g_m0 * gate_db(tr.g[4], tv.leaf[0]);
    const float g_l2 = g_m1 * gate_da(tr.g[5], tv.leaf[3]), g_l3 = g_m1 * gate_db(tr.g[5], tv.leaf[2]);
    put(0, g_l0, tap[0], tap[1]);
    put(1, g_l1, tap[2], tap[3]);
    put(2, g_l2, tap[4], tap[5]);
    put(3, g_l3, tap[6], tap[7]);
    block_sum_store<float, 28, 256>(acc, sums);
    __syncthreads();
    if (t < 112) {
        const int q = t >> 4, i = t & 15;
        float gi = coef_transpose_row<float>(i, sums[4 * q], sums[4 * q + 1], sums[4 * q + 2], sums[4 * q + 3]);
        if (probs != nullptr) gi = softmax16_backward(gi, probs[(int64_t)c * 112 + t]);
        gw[(int64_t)c * 112 + t] = gi;
    }
}

// ---- input gradient ---------------------------------------------------------------------------------------------------
struct BinBwdX {
    int hsw;            // wavefronts sharing one (sample, channel) plane: each takes every hsw-th kernel of the channel's list
    int items_per_wg;   // (sample, channel) planes per workgroup
    int P, wp, prs, plane, plane_pad;
    int64_t items;      // n * cin
    FastDiv d_wp, d_cin;
};

// NB: blocks of 64 lanes that a plane's pooled cells (at most 256) fill.  FULL: they fill the last block too (no idle
// lanes, no sink element).
template <int NB, bool FULL>
__global__ __launch_bounds__(1024) void convblock_bin_backward_x_kernel(const float *__restrict__ gy, const uint16_t *__restrict__ aux,
                                                                      const float *__restrict__ ftab, const int32_t *__restrict__ xtap,
                                                                      const int32_t *__restrict__ count, const int32_t *__restrict__ hits,
                                                                      float *__restrict__ gx, Geom g, BinBwdX p)
{
    extern __shared__ __align__(16) float planes[];                   // [waves][plane_pad]
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = uniform(tid >> 6);
    const int slot = wave % p.hsw, local = wave / p.hsw;
    // planes in sample-major order, every XCD on a contiguous range of them: the channel planes of one sample read the
    // same gradient rows and then find them in one L2
    const int64_t item = (int64_t)xcd_contiguous_block(blockIdx.x, gridDim.x) * p.items_per_wg + local;
    const bool have = item < p.items;
    float *pl = planes + wave * p.plane_pad;
    for (int i = lane; i < p.plane_pad; i += kWave) pl[i] = 0.f;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    uint32_t n = 0, ch = 0;
    if (have) {
        n = fdiv((uint32_t)item, p.d_cin);
        ch = (uint32_t)item - n * (uint32_t)g.cin;
        int cellbase[NB];
        bool live[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int cell = j * kWave + lane;
            live[j] = FULL || cell < p.P;
            const uint32_t cl = live[j] ? (uint32_t)cell : 0u;
            const uint32_t cy = fdiv(cl, p.d_wp), cx = cl - cy * (uint32_t)p.wp;
            cellbase[j] = (int)(2 * cy) * p.prs + (int)(2 * cx);
        }
        const int sink = p.plane + lane;                              // private element for lanes without a cell
        const int nhits = count[2 * ch];
        const int32_t *hit = hits + count[2 * ch + 1];
        const int64_t nbase = (int64_t)n * g.c * p.P;
        struct Loads {
            float gyv[NB];
            uint32_t ax[NB];
            float tab[3];
        };
        auto issue = [&](int k, Loads &L) {
            const int c = hit[k] & 0xFFFF;
            const int64_t row = nbase + (int64_t)c * p.P;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                L.gyv[j] = 0.f;
                L.ax[j] = 0;
                if (live[j]) {
                    L.gyv[j] = gy[row + j * kWave + lane];
                    L.ax[j] = aux[row + j * kWave + lane];
                }
            }
            const float *ft = ftab + (int64_t)c * kFtab;
            L.tab[0] = ft[lane];
            L.tab[1] = ft[64 + lane];
            L.tab[2] = ft[128 + (lane & 31)];
        };
        Loads cur, nxt;
        if (slot < nhits) issue(slot, cur);
        // the kernel's derivative tables in the wavefront's own LDS slot: a lookup is a read at nibble + constant, and
        // two lookups with one nibble are one ds_read2_b32
        float *tabw = planes + (int)(blockDim.x >> 6) * p.plane_pad + wave * kFtab;
        for (int k = slot; k < nhits; k += p.hsw) {
            if (k + p.hsw < nhits) issue(k + p.hsw, nxt);
            const int ent = hit[k];
            const int c = ent & 0xFFFF, mask = (ent >> 16) & 0xFF;
            int to[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) to[t] = xtap[c * 8 + t];
            tabw[lane] = cur.tab[0];
            tabw[64 + lane] = cur.tab[1];
            if (lane < 32) tabw[128 + lane] = cur.tab[2];
            int pos[NB];
            const float *tl[NB], *th[NB];
            float u0[NB], u1[NB];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const uint32_t a = cur.ax[j];
                pos[j] = FULL || live[j] ? cellbase[j] + (int)((a >> 9) & 1) * p.prs + (int)((a >> 8) & 1) : sink;
                tl[j] = tabw + (a & 15u);
                th[j] = tabw + ((a >> 4) & 15u);
            }
            if (mask & 0x0F) {
#pragma unroll
                for (int j = 0; j < NB; ++j) u0[j] = cur.gyv[j] * th[j][0];                     // F1[0][hi]
            }
            if (mask & 0xF0) {
#pragma unroll
                for (int j = 0; j < NB; ++j) u1[j] = cur.gyv[j] * tl[j][16];                    // F1[1][lo]
            }
            // read-add-write of one tap for all cell blocks: reads first, so that they are in flight together
            auto add_tap = [&](int off, const float (&val)[NB]) {
                float old[NB];
#pragma unroll
                for (int j = 0; j < NB; ++j) old[j] = pl[pos[j] + off];
#pragma unroll
                for (int j = 0; j < NB; ++j) pl[pos[j] + off] = old[j] + val[j];
            };
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {                          // taps 2 pr and 2 pr + 1 share their nibble
                const int ta = 2 * pr, tb = ta + 1;
                const int both = (mask >> ta) & 3;                    // wave-uniform
                if (both == 0) continue;
                // F2[t][own nibble]: entry 32 + 16 t + nibble of the table
                float va[NB], vb[NB];
                if (both == 3) {
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const float *q = pr < 2 ? tl[j] : th[j];
                        const float fa = q[32 + 16 * ta], fb = q[32 + 16 * tb];
                        const float u = pr < 2 ? u0[j] : u1[j];
                        va[j] = u * fa, vb[j] = u * fb;
                    }
                    add_tap(to[ta], va);
                    add_tap(to[tb], vb);
                } else {
                    const int t = both == 1 ? ta : tb;
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const float *q = pr < 2 ? tl[j] : th[j];
                        va[j] = (pr < 2 ? u0[j] : u1[j]) * q[32 + 16 * t];
                    }
                    add_tap(both == 1 ? to[ta] : to[tb], va);
                }
            }
            cur = nxt;
        }
    }
    __syncthreads();
    // the wavefronts of a plane share its pixels; each adds the copies in order and writes its image elements out
    if (have) {
        float *dst = gx + ((int64_t)n * g.cin + ch) * g.h * g.w;
        const float *first = planes + (wave - slot) * p.plane_pad;
        const int total = g.h * g.w;
        for (int e = slot * kWave + lane; e < total; e += p.hsw * kWave) {
            const int iy = e / g.w, ix = e - iy * g.w;
            const int at = (iy + g.ph) * p.prs + ix + g.pw;
            float v = first[at];
            for (int k = 1; k < p.hsw; ++k) v += first[k * p.plane_pad + at];
            dst[e] = v;
        }
    }
}

}  // namespace

// ---- C ABI ------------------------------------------------------------------------------------------------------------
extern "C" int clg_convblock_bin_supported(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_bin_supported")) return 0;
    return bin_supported(g, dtype) ? 1 : 0;
}

extern "C" int clg_host_flag_device_pointer(void *host, void **device)
{
    CLG_REQUIRE(host && device, "clg_host_flag_device_pointer: null pointer argument");
    void *d = nullptr;
    const hipError_t e = hipHostGetDevicePointer(&d, host, 0);
    if (e != hipSuccess || d == nullptr) {
        (void)hipGetLastError();
        clg_set_error("clg_host_flag_device_pointer: not pinned host memory mapped for this device: %s", hipGetErrorString(e));
        return CLG_EINVAL;
    }
    *device = d;
    return CLG_OK;
}

extern "C" int64_t clg_convblock_bin_ctx_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_bin_ctx_bytes")) return -1;
    if (!bin_supported(g, dtype)) {
        clg_set_error("clg_convblock_bin_ctx_bytes: shape not supported by the binary-input kernels (clg_convblock_bin_supported)");
        return -1;
    }
    return (int64_t)bin_ctx(g).total;
}

extern "C" int clg_convblock_bin_forward(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                         void *y, uint16_t *taps, void *ctx, int flags, int32_t *not_binary, void *stream)
{
    const char *name = "clg_convblock_bin_forward";
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(bin_supported(g, dtype), "%s: shape not supported by the binary-input kernels (clg_convblock_bin_supported)", name);
    CLG_REQUIRE(x && w && selection && y && taps && ctx && not_binary, "%s: null pointer argument", name);
    CLG_REQUIRE((flags & ~CLG_FWD_W_LOGITS) == 0, "%s: unknown flags 0x%x", name, flags);
    const BinCtx cx = bin_ctx(g);
    unsigned char *base = reinterpret_cast<unsigned char *>(ctx);
    hipStream_t st = clg_stream(stream);

    PrepArgs a;
    a.x = (const float *)x, a.w = (const float *)w, a.sel = selection;
    a.bits = reinterpret_cast<uint32_t *>(base + cx.bits_off);
    a.lut = reinterpret_cast<float *>(base + cx.lut_off);
    a.probs = reinterpret_cast<float *>(base + cx.probs_off);
    a.folded = reinterpret_cast<float *>(base + cx.folded_off);
    a.ftab = reinterpret_cast<float *>(base + cx.ftab_off);
    a.tapinfo = reinterpret_cast<int32_t *>(base + cx.tapinfo_off);
    a.xtap = reinterpret_cast<int32_t *>(base + cx.xtap_off);
    a.count = reinterpret_cast<int32_t *>(base + cx.count_off);
    a.hits = reinterpret_cast<int32_t *>(base + cx.hits_off);
    a.bad = not_binary;
    a.w_logits = (flags & CLG_FWD_W_LOGITS) ? 1 : 0;
    a.list_blocks = (int)clg_ceil_div(g.cin, 4);
    a.pack0 = g.c + a.list_blocks;
    a.RP = cx.RP, a.prs = cx.prs;
    a.d_h = make_fastdiv((uint32_t)g.h);
    a.d_cinh = make_fastdiv((uint32_t)(g.cin * g.h));
    const int64_t row_pairs = clg_ceil_div((int64_t)g.n * g.cin * g.h, 2);
    const int pack_blocks = (int)std::min<int64_t>(clg_ceil_div(row_pairs, 4 * 8), 2048);   // about 8 row pairs per wavefront
    hipLaunchKernelGGL(convblock_bin_prepare_kernel, dim3((unsigned)(a.pack0 + std::max(pack_blocks, 1))), dim3(256), 0, st, a, g);
    CLG_CHECK_LAUNCH("clg_convblock_bin_forward(prepare)");

    BinFwd p;
    p.hp = g.ho / 2, p.wp = g.wo / 2, p.RP = cx.RP;
    // samples per workgroup: the smallest count that fills its last block of 64 lanes to at least 85 %
    int S = 1;
    for (int s = 1; s <= 32; s *= 2) {
        const int lanes = s * p.hp, blocks = (lanes + 63) / 64;
        S = s;
        if (lanes * 100 >= blocks * 64 * 85) break;
    }
    const size_t img_per_sample = (size_t)g.cin * cx.RP * 4;
    if (const char *e = clg_knob(K_BIN_S)) S = std::min(64, std::max(1, atoi(e)));
    while (S > 1 && S * img_per_sample > 64 * 1024) S /= 2;
    CLG_REQUIRE(S * img_per_sample <= 96 * 1024, "%s: the bit planes of one sample (%zu bytes) do not fit LDS", name, img_per_sample);
    if (S > g.n) S = g.n;
    p.S = S;
    p.LB = (S * p.hp + 63) / 64;
    const int stiles = (int)clg_ceil_div(g.n, S);
    int CT = 64;
    while (CT > 8 && (int64_t)stiles * clg_ceil_div(g.c, CT) < 512) CT /= 2;
    while (CT > 2 && (int64_t)stiles * clg_ceil_div(g.c, CT) < 256) CT /= 2;   // few kernels: a workgroup per CU first
    if (const char *e = clg_knob(K_BIN_CT)) CT = std::min(64, std::max(1, atoi(e)));
    if (CT > g.c) CT = g.c;
    p.CT = CT;
    p.ktiles = (int)clg_ceil_div(g.c, CT);
    p.d_hp = make_fastdiv((uint32_t)p.hp);
    p.d_ktiles = make_fastdiv((uint32_t)p.ktiles);
    p.d_lb = make_fastdiv((uint32_t)p.LB);
    int nw = p.LB * CT;
    nw = nw > 8 ? 8 : nw;
    if (const char *e = clg_knob(K_BIN_NW)) nw = std::min(8, std::max(1, atoi(e)));
    int pc = p.wp % 4 == 0 ? 4 : (p.wp % 2 == 0 ? 2 : 0);
    if (const char *e = clg_knob(K_BIN_PIECE)) pc = atoi(e) == 0 ? 0 : (atoi(e) == 2 && pc ? 2 : pc);   // narrower pieces / rows written directly
    p.tr_words = pc ? kWave * (p.wp + 4) : 0;
    p.d_npc = make_fastdiv((uint32_t)std::max(1, pc ? p.wp / pc : 1));
    const size_t lds = (size_t)CT * 1024 + (((size_t)S * g.cin * cx.RP + 3) & ~(size_t)3) * 4 + (size_t)nw * p.tr_words * 4;
#define CLG_BIN_FWD(PC)                                                                                                          \
    do {                                                                                                                         \
        if (int e = allow_lds(convblock_bin_forward_kernel<PC>, lds, name)) return e;                                            \
        hipLaunchKernelGGL(convblock_bin_forward_kernel<PC>, dim3((unsigned)(stiles * p.ktiles)), dim3(nw * kWave), lds, st,     \
                           (const uint32_t *)a.bits, (const float *)a.lut, (const int32_t *)a.tapinfo, (float *)y, taps, g, p);  \
    } while (0)
    if (pc == 4) CLG_BIN_FWD(4);
    else if (pc == 2) CLG_BIN_FWD(2);
    else CLG_BIN_FWD(0);
#undef CLG_BIN_FWD
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

namespace {
int hist_lanes()
{
    if (const char *e = clg_knob(K_BIN_HL)) {
        const int v = atoi(e);
        if (v == 64 || v == 32 || v == 16) return v;
    }
    return 64;                                                       // measured at [256,9,32,32] -> 256: 28.7 us with 64 lanes, 33.3 with 32, 42.4 with 16
}
int hist_parts(const Geom &g)
{
    int parts = 512 * (64 / hist_lanes()) / g.c;
    if (parts < 1) parts = 1;
    if (const char *e = clg_knob(K_BIN_PARTS)) parts = std::max(1, atoi(e));
    if (parts > g.n) parts = g.n;
    return parts;
}
}  // namespace

extern "C" int64_t clg_convblock_bin_backward_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_bin_backward_scratch_bytes")) return -1;
    if (!bin_supported(g, dtype)) {
        clg_set_error("clg_convblock_bin_backward_scratch_bytes: shape not supported by the binary-input kernels");
        return -1;
    }
    return (int64_t)g.c * hist_parts(g) * 256 * 4;
}

extern "C" int clg_convblock_bin_backward(int dtype, const clg_conv_geom *gg, const void *grad_y, const uint16_t *taps, const void *ctx,
                                          void *grad_x, void *grad_w, int flags, void *scratch, void *stream)
{
    const char *name = "clg_convblock_bin_backward";
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(bin_supported(g, dtype), "%s: shape not supported by the binary-input kernels (clg_convblock_bin_supported)", name);
    CLG_REQUIRE(grad_y && taps && ctx && (grad_x || grad_w), "%s: null pointer argument", name);
    CLG_REQUIRE(!grad_w || scratch, "%s: the weight gradient needs the scratch buffer", name);
    CLG_REQUIRE((flags & ~CLG_BWD_WRT_LOGITS) == 0, "%s: unknown flags 0x%x", name, flags);
    const BinCtx cx = bin_ctx(g);
    const unsigned char *base = reinterpret_cast<const unsigned char *>(ctx);
    hipStream_t st = clg_stream(stream);
    const int hp = g.ho / 2, wp = g.wo / 2, P = hp * wp;

    if (grad_x != nullptr) {
        BinBwdX p;
        p.P = P, p.wp = wp, p.prs = cx.prs, p.plane = cx.plane;
        // behind the plane: one element per lane for the lanes without a cell, which add their zeros there at the tap's
        // offset like every other lane
        p.plane_pad = (cx.plane + 64 + (g.kh - 1) * cx.prs + g.kw + 3) & ~3;
        p.items = (int64_t)g.n * g.cin;
        // wavefronts per plane: enough of them to give every SIMD a few, bounded by the shortest useful list
        int hsw = 1;
        const int64_t avg_hits = std::max<int64_t>(1, (int64_t)g.c * 2 / g.cin);
        while (hsw < 16 && p.items * hsw * 2 <= 10240 && hsw * 2 * 4 <= avg_hits) hsw *= 2;
        // one round of the launch when three quarters of that fit the 256 x 32 wavefront slots and the power of two does not
        if (hsw >= 4 && p.items * hsw > 8192 && p.items * (hsw / 4 * 3) <= 8192) hsw = hsw / 4 * 3;
        if (const char *e = clg_knob(K_BIN_HSW)) hsw = std::min(16, std::max(1, atoi(e)));
        p.hsw = hsw;
        int per_wg = std::max(1, 4 / hsw);
        while (per_wg > 1 && (size_t)per_wg * hsw * (p.plane_pad + kFtab) * 4 > 64 * 1024) per_wg /= 2;
        p.items_per_wg = per_wg;
        p.d_wp = make_fastdiv((uint32_t)wp);
        p.d_cin = make_fastdiv((uint32_t)g.cin);
        const size_t lds = (size_t)per_wg * hsw * (p.plane_pad + kFtab) * 4;   // gradient planes, then a table slot per wavefront
        CLG_REQUIRE(lds <= (size_t)kLdsLimit, "%s: gradient planes of %zu bytes do not fit LDS", name, lds);
        const dim3 grid((unsigned)clg_ceil_div(p.items, per_wg)), block(per_wg * hsw * kWave);
#define CLG_BIN_BWDX(NB, FULL)                                                                                                   \
    do {                                                                                                                         \
        if (int e = allow_lds(convblock_bin_backward_x_kernel<NB, FULL>, lds, name)) return e;                                   \
        hipLaunchKernelGGL((convblock_bin_backward_x_kernel<NB, FULL>), grid, block, lds, st, (const float *)grad_y, taps,       \
                           reinterpret_cast<const float *>(base + cx.ftab_off), reinterpret_cast<const int32_t *>(base + cx.xtap_off), \
                           reinterpret_cast<const int32_t *>(base + cx.count_off), reinterpret_cast<const int32_t *>(base + cx.hits_off), \
                           (float *)grad_x, g, p);                                                                               \
    } while (0)
#define CLG_BIN_BWDX_NB(NB)                                                                                                      \
    do {                                                                                                                         \
        if (P == NB * kWave) CLG_BIN_BWDX(NB, true);                                                                             \
        else CLG_BIN_BWDX(NB, false);                                                                                            \
    } while (0)
        switch ((P + kWave - 1) / kWave) {
        case 1: CLG_BIN_BWDX_NB(1); break;
        case 2: CLG_BIN_BWDX_NB(2); break;
        case 3: CLG_BIN_BWDX_NB(3); break;
        default: CLG_BIN_BWDX_NB(4); break;
        }
#undef CLG_BIN_BWDX_NB
#undef CLG_BIN_BWDX
        CLG_CHECK_LAUNCH("clg_convblock_bin_backward(input gradient)");
    }
    if (grad_w != nullptr) {
        BinHist h;
        h.C = g.c, h.P = P, h.n = g.n;
        h.parts = hist_parts(g);
        const int hl = hist_lanes();
        h.per_part = (int)clg_ceil_div(g.n, h.parts);
        CLG_REQUIRE(P % 4 == 0, "%s: the pooled plane must hold a multiple of 4 cells", name);
        h.Q = P / 4;
        h.d_q = make_fastdiv((uint32_t)h.Q);
        CLG_REQUIRE((int64_t)h.per_part * h.Q < (1ll << 31) - 4096, "%s: batch too large", name);
        const size_t lds = (size_t)256 * hl * 4;
#define CLG_BIN_HIST(HL)                                                                                                         \
    do {                                                                                                                         \
        auto kern = h.Q == HL ? convblock_bin_hist_kernel<HL, true> : convblock_bin_hist_kernel<HL, false>;                      \
        if (int e = allow_lds(kern, lds, name)) return e;                                                                        \
        hipLaunchKernelGGL(kern, dim3((unsigned)(g.c * h.parts)), dim3(HL), lds, st, (const float *)grad_y, taps, (float *)scratch, h); \
    } while (0)
        if (hl == 64) CLG_BIN_HIST(64);
        else if (hl == 32) CLG_BIN_HIST(32);
        else CLG_BIN_HIST(16);
#undef CLG_BIN_HIST
        CLG_CHECK_LAUNCH("clg_convblock_bin_backward(histogram)");
        hipLaunchKernelGGL(convblock_bin_wgrad_finish_kernel, dim3((unsigned)g.c), dim3(256), 0, st, (const float *)scratch,
                           reinterpret_cast<const float *>(base + cx.folded_off),
                           (flags & CLG_BWD_WRT_LOGITS) ? reinterpret_cast<const float *>(base + cx.probs_off) : (const float *)nullptr,
                           (float *)grad_w, h.parts);
        CLG_CHECK_LAUNCH("clg_convblock_bin_backward(finish)");
    }
    return CLG_OK;
}
