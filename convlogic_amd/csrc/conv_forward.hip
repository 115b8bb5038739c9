// Fused conv-logic block, forward: LDS-tiled kernel for gfx950 in two element flavours.
//
//   float / double  relaxed gates in the folded form, 2x2 max pool with a 1-byte arg-max code
//   uint64_t        64 samples per element (bit s of word group g = sample 64 g + s), gates as bitwise
//                   multiplexers, 2x2 pool = OR, no arg-max
//
// Both read images laid out [n, c_in, h, w] (for packed words n counts 64-sample groups) and write
// [n, c_out, ho/2, wo/2], so staging, tap addressing and the lane mapping are shared.
//
// A workgroup owns (S samples) x (CT kernels) and stages zero-padded input planes in LDS with shared
// halos (row stride rs = w + pw, plane stride chs = (h + ph) * rs): either all input channels of its
// samples, or -- for layers with many input channels -- only the (at most two) channels each kernel of
// its tile reads, two LDS planes per kernel.  A kernel whose taps name more than two channels (possible
// with a caller-made selection) reads its taps from global memory instead.  Lanes run along conv-output
// columns, each lane evaluates the tree at conv rows 2r and 2r+1, the horizontal neighbour comes over
// DPP, and the even lane pools and writes.  The kernel index is uniform per wavefront, so gate
// parameters and tap offsets sit in scalar registers.
#include <stdlib.h>

#include <algorithm>

#include "conv_ops.h"

int clg_convblock_check(const clg_conv_geom *gg, Geom *g, int dtype, const char *name);
int clg_convblock_forward_generic(int dtype, const Geom &g, const void *x, const void *w, const int32_t *selection, void *y,
                                  uint8_t *argmax, hipStream_t st);
bool clg_convblock_is_4x4(const Geom &g);
int clg_convblock_forward_4x4(int dtype, const Geom &g, const void *x, const void *folded, const int32_t *sel, void *y, uint8_t *argmax,
                              hipStream_t st, const char *name);
int clg_convblock_eval_packed_4x4(const Geom &g, const uint64_t *x, const uint8_t *gates, const int32_t *sel, uint64_t *y, hipStream_t st,
                                  const char *name);

namespace {

// ---- kernel ------------------------------------------------------------------------------------
// ROWSTEP: elements between conv rows 2r and 2r+1 in the LDS image when known at compile time (the
// second row's reads then use the immediate offset of the LDS instruction), 0 = read it from the plan.
// SUBSET: stage two planes per kernel of the tile instead of all input channels.
// ONE_ROW: a lane slot is one conv position instead of a column of two rows (plan.one_row; compile-time so that the
// two-row loop carries nothing of it); ROWSTEP is then wo if that is 8 or 4 (and all channels are staged), else 0.
// At most 80 scalar registers: with the 83 the compiler takes by itself a SIMD holds 7 wavefronts, not 8, and the last
// eighth of a launch of 8192 waits for the first to end (the launch stalled on scalar registers; [256,32,16,16] -> 128:
// 25.2 -> 23.2 us).
template <typename Ops, int ROWSTEP, bool SUBSET, bool ONE_ROW>
__global__ __attribute__((amdgpu_num_sgpr(80))) void convblock_forward_tiled_kernel(const typename Ops::Elem *__restrict__ x, const void *__restrict__ params,
                                               const int32_t *__restrict__ sel, typename Ops::Elem *__restrict__ y,
                                               uint8_t *__restrict__ argmax, Geom g, TilePlan p, void *__restrict__ probs_out)
{
    using T = typename Ops::Elem;
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    T *coef = xs + ((p.xe + 3) & ~3);                                 // [CT][kParams]
    int *toff = reinterpret_cast<int *>(coef + ((p.CT * Ops::kParams + 1) & ~1));   // [CT][8]
    int *chan = toff + p.CT * 8;                                      // [2 CT]  channel of every LDS plane (SUBSET)
    int *wide = chan + 2 * p.CT;                                      // [CT]    kernel reads more than two channels (SUBSET)
    int2 *slot = reinterpret_cast<int2 *>(wide + ((p.CT + 1) & ~1));  // [S * slots]

    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int lane = tid & (kWave - 1), wave = uniform(tid >> 6);
    const int n0 = blockIdx.x * p.S, s_cur = min(p.S, g.n - n0);
    const int c0 = blockIdx.y * p.CT, ct_cur = min(p.CT, g.c - c0);
    const int wp = g.wo >> 1, I = (g.ho >> 1) * wp;
    const int hw = g.h * g.w;

    for (int i = tid; i < p.xe; i += nthreads) xs[i] = T(0);
    // logits in (plan.w_logits): every workgroup takes the softmax of its kernels, the first sample block writes it out
    Ops::stage_params(coef, params, c0, ct_cur, tid, nthreads, p.w_logits != 0, blockIdx.x == 0 ? probs_out : nullptr);
    if (!SUBSET) {
        for (int q = tid; q < ct_cur * 8; q += nthreads) {
            const Tap t = unpack_tap(sel[(int64_t)c0 * 8 + q], tap_limit(g));
            toff[q] = t.ch * p.chs + t.ry * p.rs + t.rx;
        }
    } else {
        for (int q = tid; q < p.CT; q += nthreads) {
            int ch_a = 0, ch_b = 0, wd = 0;
            if (q < ct_cur) {
                const int32_t *sq = sel + ((int64_t)c0 + q) * 8;
                ch_a = ch_b = unpack_tap(sq[0], tap_limit(g)).ch;
                for (int t = 7; t >= 1; --t)
                    if (unpack_tap(sq[t], tap_limit(g)).ch != ch_a) ch_b = unpack_tap(sq[t], tap_limit(g)).ch;   // ends on the first other channel
                for (int t = 0; t < 8; ++t) {
                    const Tap tp = unpack_tap(sq[t], tap_limit(g));
                    int pl = 2 * q;
                    if (tp.ch == ch_b) pl = 2 * q + 1;
                    if (tp.ch == ch_a) pl = 2 * q;
                    if (tp.ch != ch_a && tp.ch != ch_b) wd = 1;
                    toff[q * 8 + t] = pl * p.chs + tp.ry * p.rs + tp.rx;
                }
            }
            chan[2 * q] = ch_a;
            chan[2 * q + 1] = ch_b;
            wide[q] = wd;
        }
    }
    const int U = s_cur * p.slots;
    constexpr int rows_per_slot = ONE_ROW ? 1 : 2;                   // conv rows a lane slot covers
    for (int u = tid; u < U; u += nthreads) {
        const uint32_t s = fdiv(u, p.d_slots), r = u - s * (uint32_t)p.slots;
        const uint32_t rp = fdiv(r, p.d_wo), ox = r - rp * (uint32_t)g.wo;        // rp: row pair, or row with one_row
        const uint32_t oy = rp * rows_per_slot;
        slot[u] = make_int2((int)(s * p.planes * p.chs + (oy * g.sh) * p.rs + ox * g.sw), (int)((s * g.c) * I + (oy >> 1) * wp + (ox >> 1)));
    }
    __syncthreads();
    {
        // planes of the samples into the zeroed LDS image, four global loads in flight per thread
        const T *src = x + (int64_t)n0 * g.cin * hw;
        const uint32_t total = (uint32_t)(s_cur * p.planes) * (uint32_t)hw;
        for (uint32_t e0 = tid; e0 < total; e0 += 4 * nthreads) {
            T v[4];
            int at[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t e = e0 + k * nthreads;
                at[k] = -1;
                if (e < total) {
                    const uint32_t plane = fdiv(e, p.d_hw), rem = e - plane * (uint32_t)hw;
                    const uint32_t iy = fdiv(rem, p.d_w), ix = rem - iy * (uint32_t)g.w;
                    at[k] = (int)(plane * p.chs + (iy + g.ph) * p.rs + ix + g.pw);
                    if (!SUBSET) {
                        v[k] = src[e];
                    } else {
                        const uint32_t s = fdiv(plane, p.d_planes), pl = plane - s * (uint32_t)p.planes;
                        v[k] = src[((int64_t)s * g.cin + chan[pl]) * hw + rem];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (at[k] >= 0) xs[at[k]] = v[k];
        }
    }
    __syncthreads();
    if constexpr (!SUBSET) {
        // The staged image IS the zero-padded copy of x that the direct input gradient and the padded weight gradient read
        // (same row and plane strides): the kernel tiles of a sample block, which all hold it, each leave their share of it
        // in global memory, and the backward call needs no launch to make it.  A sample's tail (the halo behind its last
        // plane) reads as zeros here: it is the top halo of the next sample's first plane, or the image's own tail.
        if (p.padded_out != nullptr) {
            T *po = reinterpret_cast<T *>(p.padded_out);
            const int se = p.padded_sample_elems;
            for (int s = 0; s < s_cur; ++s) {
                T *dst = po + (int64_t)(n0 + s) * se;
                const T *img = xs + s * p.planes * p.chs;
                for (int e = (int)blockIdx.y * nthreads + tid; e < se; e += nthreads * (int)gridDim.y) dst[e] = img[e];
            }
        }
    }
    if constexpr (Ops::kParams == 28) {                              // float gates: the folded coefficients for the backward pass
        if (p.folded_out != nullptr && blockIdx.x == 0) {
            T *fo = reinterpret_cast<T *>(p.folded_out) + (int64_t)c0 * 28;
            for (int i = tid; i < ct_cur * 28; i += nthreads) fo[i] = coef[i];
        }
    }

    const int row_step = ROWSTEP ? ROWSTEP : g.sh * p.rs;
    // lanes that pool and write: even columns, and with one position per lane even rows only
    const bool writer_lane = !(lane & 1) && !(ONE_ROW && ((lane / g.wo) & 1));
    // work items = (kernel, block of 64 slots), kernel-major; every wavefront takes a contiguous range, so
    // the scalar parameters are reloaded only when its range crosses into the next kernel
    const int nblk = (U + kWave - 1) / kWave;
    const int items = ct_cur * nblk;
    const int per = (items + p.NW - 1) / p.NW;
    const int first = wave * per, last = min(items, first + per);
    if constexpr (ONE_ROW && !SUBSET) {
        // One block of lane slots (at most 64 positions per workgroup), so an item is a kernel.  The wavefront holds few
        // instructions in flight per kernel (parameters -> tap reads -> gates -> pooling), and the workgroup's LDS
        // image keeps other workgroups off the CU: two kernels per step double what is in flight.
        const bool valid = lane < U;
        const int2 e = slot[valid ? lane : 0];
        const bool store_lane = valid && writer_lane;
        const int64_t obase = ((int64_t)n0 * g.c + c0) * I + e.y;
        // the row below sits wo lanes up: a DPP row shift when ROWSTEP names wo (8 or 4), else ds_bpermute
        auto below = [&](T v) {
            if constexpr (ROWSTEP == 8 || ROWSTEP == 4) return row_up<ROWSTEP>(v);
            else return lane_up(v, g.wo);
        };
        constexpr int K = 2;                                          // 1: 2 % slower, 4: the same
        for (int lc = first; lc < last; lc += K) {
            int lk[K];
            typename Ops::Params pr[K];
            T v[K][8], r[K], ro[K], r1[K], r1o[K];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                lk[k] = min(lc + k, last - 1);
                pr[k] = Ops::load_once(coef, lk[k]);
            }
#pragma unroll
            for (int k = 0; k < K; ++k) {
#pragma unroll
                for (int t = 0; t < 8; ++t) v[k][t] = xs[e.x + toff[lk[k] * 8 + t]];    // offsets stay vector values
            }
#pragma unroll
            for (int k = 0; k < K; ++k) {
                r[k] = Ops::root(pr[k], v[k]);
                ro[k] = dpp_xor1(r[k]);
                if constexpr (Ops::kOrPool) {                         // the row first, then one exchange with the row below
                    ro[k] = Ops::join(pr[k], r[k], ro[k]);
                    r1o[k] = below(ro[k]);
                } else {
                    r1[k] = below(r[k]);
                    r1o[k] = below(ro[k]);
                }
            }
            if (store_lane) {
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    if (k > 0 && lc + k >= last) continue;
                    if constexpr (Ops::kOrPool) y[obase + lk[k] * I] = Ops::join_last(pr[k], ro[k], r1o[k]);
                    else Ops::pool_store(r[k], ro[k], r1[k], r1o[k], y + obase, argmax ? argmax + obase : nullptr, lk[k] * I);
                }
            }
        }
        return;
    }
    int lc = first / nblk, blk = first - lc * nblk;
    for (int item = first; item < last;) {
        const typename Ops::Params pr = Ops::load(coef, lc);
        int to[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) to[t] = uniform(toff[lc * 8 + t]);
        const bool from_global = SUBSET && uniform(wide[lc]) != 0;
        const int64_t obase = ((int64_t)n0 * g.c + c0 + lc) * I;
        T *yb = y + obase;
        uint8_t *ab = argmax ? argmax + obase : nullptr;
        for (; blk < nblk && item < last; ++blk, ++item) {
            const int u = blk * kWave + lane;
            const bool valid = u < U;
            const int2 e = slot[valid ? u : 0];
            T v[8];
            T r0, r1 = T(0);
            if (!from_global) {
#pragma unroll
                for (int t = 0; t < 8; ++t) v[t] = xs[e.x + to[t]];
                r0 = Ops::root(pr, v);
                if (!ONE_ROW) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) v[t] = xs[e.x + row_step + to[t]];
                    r1 = Ops::root(pr, v);
                }
            } else {
                const uint32_t uu = valid ? u : 0;
                const uint32_t s = fdiv(uu, p.d_slots), r = uu - s * (uint32_t)p.slots;
                const uint32_t rp = fdiv(r, p.d_wo), ox = r - rp * (uint32_t)g.wo;
                const uint32_t oy = rp * rows_per_slot;
                const T *xn = x + (int64_t)(n0 + s) * g.cin * hw;
                const int32_t *sq = sel + ((int64_t)c0 + lc) * 8;
#pragma unroll
                for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, unpack_tap(sq[t], tap_limit(g)), (int)oy, (int)ox);
                r0 = Ops::root(pr, v);
                if (!ONE_ROW) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, unpack_tap(sq[t], tap_limit(g)), (int)(oy + 1), (int)ox);
                    r1 = Ops::root(pr, v);
                }
            }
            if constexpr (Ops::kOrPool) {                             // OR pool: any order, one exchange per direction
                T m;
                if (ONE_ROW) {
                    m = Ops::join(pr, r0, dpp_xor1(r0));
                    m = Ops::join_last(pr, m, lane_up(m, g.wo));
                } else {
                    m = Ops::join(pr, r0, r1);
                    m = Ops::join_last(pr, m, dpp_xor1(m));
                }
                if (valid && writer_lane) yb[e.y] = m;
            } else {
                const T r0o = dpp_xor1(r0);
                T r1o;
                if (ONE_ROW) {                                        // the row below sits wo lanes up (2 wo divides 64)
                    r1 = lane_up(r0, g.wo);
                    r1o = lane_up(r0o, g.wo);
                } else {
                    r1o = dpp_xor1(r1);
                }
                if (valid && writer_lane) Ops::pool_store(r0, r0o, r1, r1o, yb, ab, e.y);
            }
        }
        blk = 0;
        ++lc;
    }
}

// Forward with one KERNEL per lane: for deep blocks on small images -- hundreds of kernels, at most 16 pooled cells per
// sample, all input planes of a sample in LDS.  With lanes along positions (the kernel above) every wavefront fetches a
// kernel's 28 coefficients and 8 tap offsets from LDS for ONE block of 64 positions: 9 of its 17 LDS instructions per
// kernel.  Here a lane keeps its kernel's coefficients and tap offsets in registers for the whole sample and walks the
// conv positions cell by cell: 8 LDS gathers per position and nothing else, the 2x2 pool is a running maximum in
// registers (first maximum wins, in window order), and a lane's pooled values leave as whole 16-byte vectors.
// folded = [c][7][4] coefficients made by convblock_w_prepare_kernel.  Same values bit for bit: the same gate().
constexpr int kKplMaxCells = 16;
template <typename T>
__global__ __launch_bounds__(512) void convblock_forward_kpl_kernel(const T *__restrict__ x, const T *__restrict__ folded,
                                                                  const int32_t *__restrict__ sel, T *__restrict__ y,
                                                                  uint8_t *__restrict__ argmax, Geom g, TilePlan p, int kernels_per_wg)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int n = blockIdx.x, c0 = blockIdx.y * kernels_per_wg;
    const int hw = g.h * g.w;
    for (int i = tid; i < p.xe; i += nthreads) xs[i] = T(0);
    __syncthreads();
    {
        const T *src = x + (int64_t)n * g.cin * hw;
        const uint32_t total = (uint32_t)g.cin * (uint32_t)hw;
        for (uint32_t e0 = tid; e0 < total; e0 += 4 * nthreads) {
            T v[4];
            int at[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t e = e0 + k * nthreads;
                at[k] = -1;
                if (e < total) {
                    const uint32_t plane = fdiv(e, p.d_hw), rem = e - plane * (uint32_t)hw;
                    const uint32_t iy = fdiv(rem, p.d_w), ix = rem - iy * (uint32_t)g.w;
                    at[k] = (int)(plane * p.chs + (iy + g.ph) * p.rs + ix + g.pw);
                    v[k] = src[e];
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (at[k] >= 0) xs[at[k]] = v[k];
        }
    }
    __syncthreads();
    if (p.padded_out != nullptr) {                                    // the staged image = the padded copy for the backward pass
        T *dst = reinterpret_cast<T *>(p.padded_out) + (int64_t)n * p.padded_sample_elems;
        for (int e = (int)blockIdx.y * nthreads + tid; e < p.padded_sample_elems; e += nthreads * (int)gridDim.y) dst[e] = xs[e];
    }
    const int k = c0 + tid;
    if (tid >= kernels_per_wg || k >= g.c) return;
    Tree<T> tr;
    const T *fc = folded + (int64_t)k * 28;
#pragma unroll
    for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
    int to[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const Tap tp = unpack_tap(sel[(int64_t)k * 8 + t], tap_limit(g));
        to[t] = tp.ch * p.chs + tp.ry * p.rs + tp.rx;
    }
    const int wp = g.wo >> 1, I = (g.ho >> 1) * wp;
    T best[kKplMaxCells];
    uint32_t codes = 0;
#pragma unroll
    for (int cell = 0; cell < kKplMaxCells; ++cell) {
        best[cell] = T(0);
        if (cell < I) {                                               // wave-uniform
            const int cy = cell / wp, cx = cell - cy * wp;
            int code = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int off = ((2 * cy + (q >> 1)) * g.sh) * p.rs + (2 * cx + (q & 1)) * g.sw;
                T v[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) v[t] = xs[to[t] + off];
                const T r = eval_tree(tr, v).root;
                if (q == 0) {
                    best[cell] = r;
                } else if (r > best[cell]) {
                    best[cell] = r;
                    code = q;
                }
            }
            codes |= (uint32_t)code << (2 * cell);
        }
    }
    const int64_t o = ((int64_t)n * g.c + k) * I;
    if (I == kKplMaxCells && sizeof(T) == 4) {
        float4 *yo = reinterpret_cast<float4 *>(y + o);
        uint32_t packed[4];
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
            yo[v4] = make_float4((float)best[4 * v4], (float)best[4 * v4 + 1], (float)best[4 * v4 + 2], (float)best[4 * v4 + 3]);
            const uint32_t c8 = (codes >> (8 * v4)) & 0xFFu;      // four 2-bit codes -> four bytes
            packed[v4] = (c8 & 3u) | ((c8 & 12u) << 6) | ((c8 & 48u) << 12) | ((c8 & 192u) << 18);
        }
        *reinterpret_cast<uint4 *>(argmax + o) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    } else {
#pragma unroll
        for (int cell = 0; cell < kKplMaxCells; ++cell)
            if (cell < I) {
                y[o + cell] = best[cell];
                argmax[o + cell] = (uint8_t)((codes >> (2 * cell)) & 3u);
            }
    }
}

// Forward without LDS: for layers whose input channels do not fit LDS or whose images leave lanes idle.
// Taps come from a zero-padded global copy of x (shared-halo layout, served by L1/L2), so there is no
// staging, no barrier and no bounds check.  A wavefront keeps one set of 64 lane slots (sample, conv row
// pair, column) and runs the CT kernels of its tile over it; gate parameters and tap offsets are scalar loads.
template <typename Ops>
__global__ __launch_bounds__(256) void convblock_forward_direct_kernel(const typename Ops::Elem *__restrict__ xp,
                                                                     const void *__restrict__ params,
                                                                     const int32_t *__restrict__ taps,
                                                                     typename Ops::Elem *__restrict__ y,
                                                                     uint8_t *__restrict__ argmax, Geom g, TilePlan p,
                                                                     int sample_elems, int nblk)
{
    using T = typename Ops::Elem;
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    const int groups = (g.n + p.G - 1) / p.G;
    const int set = uniform((int)blockIdx.x * 4 + wave);
    if (set >= groups * nblk) return;
    const int grp = set / nblk, blk = set - grp * nblk;
    const int n0 = grp * p.G, g_here = min(p.G, g.n - n0);
    const int U = g_here * p.slots;
    const int u = blk * kWave + lane;
    const bool valid = u < U;
    const uint32_t uu = valid ? u : 0;
    const uint32_t s = fdiv(uu, p.d_slots), r = uu - s * (uint32_t)p.slots;
    const uint32_t rp = fdiv(r, p.d_wo), ox = r - rp * (uint32_t)g.wo;
    const int wp = g.wo >> 1, I = (g.ho >> 1) * wp;
    const int base = (int)((n0 + s) * (uint32_t)sample_elems + (2 * rp * g.sh) * p.rs + ox * g.sw);
    const int64_t obase = ((int64_t)(n0 + s) * g.c) * I + rp * wp + (ox >> 1);
    const int row_step = g.sh * p.rs;
    const int c0 = blockIdx.y * p.CT, c1 = min(g.c, c0 + p.CT);
    const bool writer = valid && !(lane & 1);
    for (int c = c0; c < c1; ++c) {
        const typename Ops::Params pr = Ops::load_global(params, c);
        int to[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) to[t] = taps[c * 8 + t];
        T v0[8], v1[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v0[t] = load_at(xp, (uint32_t)(base + to[t]));
#pragma unroll
        for (int t = 0; t < 8; ++t) v1[t] = load_at(xp, (uint32_t)(base + row_step + to[t]));
        const T r0 = Ops::root(pr, v0), r1 = Ops::root(pr, v1);
        if constexpr (Ops::kOrPool) {
            const T m = Ops::join(pr, r0, r1), pooled = Ops::join_last(pr, m, dpp_xor1(m));
            if (writer) y[obase + (int64_t)c * I] = pooled;
        } else {
            const T r0o = dpp_xor1(r0), r1o = dpp_xor1(r1);
            if (writer) Ops::pool_store(r0, r0o, r1, r1o, y + obase + (int64_t)c * I, argmax ? argmax + obase + (int64_t)c * I : nullptr, 0);
        }
    }
}

// Any shape, packed: one thread per (group, kernel, pooled cell), taps from global memory with bounds checks.
__global__ __launch_bounds__(256) void convblock_packed_generic_kernel(const uint64_t *__restrict__ x, const uint8_t *__restrict__ gid,
                                                                     const int32_t *__restrict__ sel, uint64_t *__restrict__ y,
                                                                     Geom g)
{
    const int c = blockIdx.y;
    const int wp = g.wo / 2, I = (g.ho / 2) * wp;
    const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (item >= (int64_t)g.n * I) return;
    const int n = (int)(item / I), cell = (int)(item - (int64_t)n * I);
    const int py = cell / wp, px = cell - py * wp;
    const BitOps::Params pr = BitOps::load_global(gid, c);
    const uint64_t *xn = x + (int64_t)n * g.cin * g.h * g.w;
    uint64_t acc = 0;
    for (int q = 0; q < 4; ++q) {
        uint64_t v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = read_tap(xn, g, unpack_tap(sel[c * 8 + t], tap_limit(g)), 2 * py + (q >> 1), 2 * px + (q & 1));
        acc |= BitOps::root_true(pr, v);
    }
    y[((int64_t)n * g.c + c) * I + cell] = acc;
}

// ---- plan --------------------------------------------------------------------------------------
size_t forward_lds_bytes(const TilePlan &p, int elem, int params_per_kernel)
{
    return (size_t)((p.xe + 3) & ~3) * elem + (size_t)((p.CT * params_per_kernel + 1) & ~1) * elem + (size_t)p.CT * 8 * 4 +
           (size_t)p.CT * 2 * 4 + (size_t)((p.CT + 1) & ~1) * 4 + (size_t)p.S * p.slots * 8;
}

bool plan_forward(const Geom &g, int elem, int params_per_kernel, TilePlan *p)
{
    if (!taps_inside(g)) return false;
    plan_common(g, p);
    p->slots = (g.ho / 2) * g.wo;
    p->G = 1;
    // 16 wavefronts share one staged image: measured 69 us against 109 us with 4 at [256,9,32,32] -> 256
    p->NW = 16;
    p->d_slots = make_fastdiv((uint32_t)p->slots);
    const int64_t tail = g.ph * p->rs + g.pw;
    auto util_of = [&](int S) {
        const int64_t U = (int64_t)S * p->slots;
        return (double)U / (double)(clg_ceil_div(U, kWave) * kWave);
    };
    // (a) all input channels staged: best lane utilisation within a 64 KiB image, smallest S on ties
    int sa = 0;
    double ua = 0;
    for (int S = 1; S <= 16 && S <= g.n; ++S) {
        const int64_t bytes = ((int64_t)S * g.cin * p->chs + tail) * elem + (int64_t)S * p->slots * 8;
        if (S > 1 && bytes > 64 * 1024) break;
        if (bytes > kLdsLimit - 8 * 1024) break;
        if (util_of(S) > ua + 0.02) { ua = util_of(S); sa = S; }
    }
    // (b) two planes per kernel of an 8-kernel tile: the largest S within 64 KiB among the best utilisations
    const int ctb = g.c < 8 ? g.c : 8;
    int sb = 0;
    double ub = 0;
    for (int S = 1; S <= 32 && S <= g.n; ++S) {
        const int64_t bytes = ((int64_t)S * 2 * ctb * p->chs + tail) * elem + (int64_t)S * p->slots * 8;
        if (S > 1 && bytes > 64 * 1024) break;
        if (bytes > kLdsLimit - 8 * 1024) break;
        if (util_of(S) > ub + 0.02 || (util_of(S) > ub - 0.02 && (int64_t)S * p->slots <= 4 * kWave)) {
            ub = util_of(S) > ub ? util_of(S) : ub;
            sb = S;
        }
    }
    // Staging all channels wins whenever it fits with reasonable lane use (measured on 8x8 and 16x16 layers
    // with 32..128 input channels); the two-planes-per-kernel staging is for what is left.
    bool subset = sb > 0 && (sa == 0 || ua < 0.4);
    if (const char *e = clg_knob(K_FWD_SUBSET)) subset = sb > 0 && (atoi(e) != 0 || sa == 0);
    const double util = subset ? ub : ua;
    if ((subset ? sb : sa) == 0 || util < 0.4) return false;
    p->subset = subset ? 1 : 0;
    p->S = subset ? sb : sa;
    if (subset) {
        p->CT = g.c < 8 ? g.c : 8;
        p->NW = 8;
    } else {
        // as many kernels per staged image as leave about two workgroups per CU (the prologue -- zero, stage,
        // two barriers -- is what small layers pay for)
        const int64_t groups = clg_ceil_div(g.n, p->S);
        const int64_t ct_cap = 32768 / ((int64_t)params_per_kernel * elem);   // at most 32 KiB of gate parameters
        int64_t ct = g.c < ct_cap ? g.c : ct_cap;
        while (ct > 4 && groups * clg_ceil_div(g.c, ct) < 512) ct = (ct + 1) / 2;
        ct = clg_ceil_div(g.c, clg_ceil_div(g.c, ct));               // equal tiles
        p->CT = (int)ct;
    }
    // measurement overrides
    if (const char *e = clg_knob(K_FWD_S)) p->S = atoi(e) < g.n ? atoi(e) : g.n;
    if (const char *e = clg_knob(K_FWD_CT)) p->CT = atoi(e) < g.c ? atoi(e) : g.c;
    if (const char *e = clg_knob(K_FWD_NW)) p->NW = atoi(e);
    if (p->S < 1 || p->CT < 1 || p->NW < 1 || p->NW > 16) return false;
    // A workgroup whose samples fill at most half a wavefront with (row pair, column) slots gives every conv position
    // a lane of its own instead (the pooling partner one row down is wo lanes up, so 2 wo has to divide 64), two
    // kernels per step.  Measured on [*,128,8,8] -> 512: packed words 174 -> 102 us, float32 39 -> 32 us.
    p->w_logits = 0;
    p->one_row = 0;
    if ((int64_t)p->S * p->slots * 2 <= kWave && g.wo <= 32 && (g.wo & (g.wo - 1)) == 0) p->one_row = 1;
    if (const char *e = clg_knob(K_FWD_ONE_ROW)) p->one_row = p->one_row && atoi(e) != 0;   // 0: never
    if (p->one_row) {
        p->slots = g.ho * g.wo;
        p->d_slots = make_fastdiv((uint32_t)p->slots);
    }
    for (;;) {
        p->planes = subset ? 2 * p->CT : g.cin;
        p->xe = (int)((int64_t)p->S * p->planes * p->chs + tail);
        p->lds_bytes = forward_lds_bytes(*p, elem, params_per_kernel);
        if (p->lds_bytes <= (size_t)kLdsLimit || p->CT <= 4) break;
        p->CT = (p->CT + 1) / 2;                                      // the gate parameters of the tile share LDS with the image
    }
    p->d_planes = make_fastdiv((uint32_t)p->planes);
    if (p->lds_bytes > (size_t)kLdsLimit) return false;
    if (clg_ceil_div(g.c, p->CT) > 65535) return false;
    return (int64_t)p->S * p->planes * p->chs < (1ll << 30) && (int64_t)p->S * g.c * ((g.ho / 2) * (g.wo / 2)) < (1ll << 31) &&
           (int64_t)p->S * p->planes * g.h * g.w < (1ll << 31);
}

// ---- direct (padded global copy) plan ----------------------------------------------------------
struct DirectPlan {
    TilePlan p;
    int sample_elems, nblk;
    size_t folded_off, taps_off, xp_off, total;   // scratch: [folded] | taps | padded x
};
bool plan_forward_direct(const Geom &g, int elem, bool needs_folded, DirectPlan *d)
{
    if (!taps_inside(g) || g.c > 65535) return false;
    TilePlan *p = &d->p;
    plan_common(g, p);
    p->slots = (g.ho / 2) * g.wo;
    p->d_slots = make_fastdiv((uint32_t)p->slots);
    int G = p->slots >= kWave ? 1 : kWave / p->slots;
    if (G > g.n) G = g.n;
    p->G = G;
    p->S = G;
    p->NW = 4;
    const int64_t se = (int64_t)g.cin * p->chs + g.ph * p->rs + g.pw;
    const int64_t I = (int64_t)(g.ho / 2) * (g.wo / 2);
    if (se * g.n * elem >= (1ll << 32)) return false;
    d->sample_elems = (int)se;
    d->nblk = (int)clg_ceil_div((int64_t)G * p->slots, kWave);
    const int64_t sets = clg_ceil_div(g.n, G) * d->nblk, wgs_x = clg_ceil_div(sets, 4);
    // kernels per wavefront: enough to amortise the lane set-up, few enough for about 16 workgroups per CU
    int64_t ct = g.c;
    while (ct > 16 && wgs_x * clg_ceil_div(g.c, ct) < 4096) ct = (ct + 1) / 2;
    ct = clg_ceil_div(g.c, clg_ceil_div(g.c, ct));
    if (const char *e = clg_knob(K_FWD_CT)) ct = atoi(e) < g.c ? atoi(e) : g.c;
    if (ct < 1) ct = 1;
    p->CT = (int)ct;
    if (wgs_x >= (1ll << 31) || clg_ceil_div(g.c, ct) > 65535) return false;
    d->folded_off = 0;
    d->taps_off = needs_folded ? (((size_t)g.c * 28 * elem + 255) & ~(size_t)255) : 0;
    d->xp_off = (d->taps_off + (size_t)g.c * 8 * 4 + 255) & ~(size_t)255;
    d->total = d->xp_off + (size_t)se * g.n * elem;
    return true;
}

// Which forward path a shape takes: 0 = tiled (all channels in LDS), 1 = tiled with channel subsets,
// 2 = direct from a padded copy (needs scratch), 3 = any-shape kernel, 4 = one sample per lane on 4x4 images
// (float gates; needs scratch for the folded coefficients), 5 = one kernel per lane (float gates, at most 16 pooled
// cells, all planes of a sample in LDS, at least 256 kernels; needs scratch for the folded coefficients).
int choose_forward(const Geom &g, int elem, int params_per_kernel, bool have_scratch, TilePlan *tp, DirectPlan *dp)
{
    bool lane_sample = have_scratch && params_per_kernel > 1 && clg_convblock_is_4x4(g);
    if (const char *e = clg_knob(K_FWD_4X4)) lane_sample = lane_sample && atoi(e) != 0;
    if (lane_sample) return 4;
    const bool tiled = plan_forward(g, elem, params_per_kernel, tp);
    {
        // one kernel per lane: 40.4 -> 21.2 us (+ 3.9 us for the launch that folds the coefficients) at [256,128,8,8] -> 512
        const int I = (g.ho / 2) * (g.wo / 2);
        bool kpl = have_scratch && params_per_kernel > 1 && tiled && !tp->subset && tp->one_row && tp->S == 1 && I <= kKplMaxCells && g.c >= 256 &&
                   g.ho % 2 == 0 && g.wo % 2 == 0;
        if (const char *e = clg_knob(K_FWD_KPL)) kpl = kpl && atoi(e) != 0;
        if (kpl) return 5;
    }
    const bool direct = have_scratch && plan_forward_direct(g, elem, params_per_kernel > 1, dp);
    // 4-byte elements: direct beats the channel-subset staging (354 -> 163 us at [256,256,16,16] -> 1024); 8-byte
    // elements load twice the bytes per tap and stay on the staged kernels (200 vs 329 us at [256,4096,4,4] -> 8192)
    // (4x4 images: the padded copy is 1.6x the image and both paths tie, 30 vs 35 us at [256,512,4,4] -> 1024).
    bool use_direct = direct && (!tiled || (tp->subset && elem == 4 && g.h * g.w >= 64));
    if (const char *e = clg_knob(K_FWD_DIRECT)) use_direct = direct && (atoi(e) != 0 || !tiled);
    if (use_direct) return 2;
    if (tiled) return tp->subset ? 1 : 0;
    return 3;
}

template <typename Ops, typename P>
int launch_forward_direct(const Geom &g, const DirectPlan &d, const void *x, const void *params, const int32_t *sel, void *y,
                          uint8_t *argmax, void *scratch, hipStream_t st, const char *name, bool from_logits = false,
                          void *probs_out = nullptr, void *padded_out = nullptr)
{
    using T = typename Ops::Elem;
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    int32_t *taps = reinterpret_cast<int32_t *>(base + d.taps_off);
    // the padded copy this path reads: in the scratch, or where the caller keeps it for the backward call
    T *xp = padded_out != nullptr ? reinterpret_cast<T *>(padded_out) : reinterpret_cast<T *>(base + d.xp_off);
    // one launch: folded coefficients (float gates only), tap offsets and the padded copy
    const bool fold = Ops::kParams > 1;
    const void *kernel_params = fold ? (const void *)base : params;
    const PadJob<T> job = make_pad_job((const T *)x, xp, g, d.p.rs, d.p.chs, d.sample_elems);
    const unsigned prep = (unsigned)clg_ceil_div((int64_t)g.c * 8, 256);
    hipLaunchKernelGGL((convblock_w_prepare_kernel<P, T>), dim3(prep + pad_blocks(job)), dim3(256), 0, st,
                       fold ? (const P *)params : (const P *)nullptr, sel, fold ? reinterpret_cast<P *>(base) : (P *)nullptr, taps, g.c,
                       d.p.rs, d.p.chs, host_tap_limit(g), job, (int)prep, fold && from_logits ? 1 : 0, reinterpret_cast<P *>(probs_out));
    CLG_CHECK_LAUNCH(name);
    const int64_t sets = clg_ceil_div(g.n, d.p.G) * d.nblk;
    hipLaunchKernelGGL(convblock_forward_direct_kernel<Ops>, dim3((unsigned)clg_ceil_div(sets, 4), (unsigned)clg_ceil_div(g.c, d.p.CT)),
                       dim3(256), 0, st, (const T *)xp, kernel_params, (const int32_t *)taps, (T *)y, argmax, g, d.p, d.sample_elems,
                       d.nblk);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// ---- launch ------------------------------------------------------------------------------------
// one kernel per lane (path 5): tp = the tiled plan of the shape (strides and size of the LDS image of one sample)
template <typename T>
int launch_forward_kpl(const Geom &g, TilePlan tp, const void *x, const void *folded, const int32_t *sel, void *y, uint8_t *argmax,
                       void *padded_out, hipStream_t st, const char *name)
{
    int per_wg = 512;
    if (const char *e = clg_knob(K_FWD_CT)) per_wg = std::min(512, std::max(64, atoi(e) / 64 * 64));
    per_wg = std::min(per_wg, (int)clg_ceil_div(g.c, 64) * 64);
    tp.padded_out = padded_out;
    tp.padded_sample_elems = g.cin * tp.chs + g.ph * tp.rs + g.pw;
    const size_t lds = (size_t)tp.xe * sizeof(T);
    if (int e = allow_lds(convblock_forward_kpl_kernel<T>, lds, name)) return e;
    hipLaunchKernelGGL(convblock_forward_kpl_kernel<T>, dim3((unsigned)g.n, (unsigned)clg_ceil_div(g.c, per_wg)), dim3(per_wg), lds, st,
                       (const T *)x, (const T *)folded, sel, (T *)y, argmax, g, tp, per_wg);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

template <typename Ops, int ROWSTEP, bool SUBSET, bool ONE_ROW = false>
int launch_forward_one(const Geom &g, const TilePlan &p, const void *x, const void *params, const int32_t *sel, void *y,
                       uint8_t *argmax, hipStream_t st, const char *name, void *probs_out = nullptr)
{
    using T = typename Ops::Elem;
    if (int e = allow_lds(convblock_forward_tiled_kernel<Ops, ROWSTEP, SUBSET, ONE_ROW>, p.lds_bytes, name)) return e;
    const dim3 grid((unsigned)clg_ceil_div(g.n, p.S), (unsigned)clg_ceil_div(g.c, p.CT));
    hipLaunchKernelGGL((convblock_forward_tiled_kernel<Ops, ROWSTEP, SUBSET, ONE_ROW>), grid, dim3(p.NW * kWave), p.lds_bytes, st, (const T *)x,
                       params, sel, (T *)y, argmax, g, p, probs_out);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// Row steps of 3x3 / padding 1 / stride 1 blocks on 32, 28, 16, 8 and 4 pixel wide images get their own
// instantiation; everything else reads the step from the plan.
template <typename Ops>
int launch_forward_tiled(const Geom &g, const TilePlan &p, const void *x, const void *params, const int32_t *sel, void *y,
                         uint8_t *argmax, hipStream_t st, const char *name, void *probs_out = nullptr)
{
#define CLG_FWD_CASE(RS)                                                                                              \
    case RS:                                                                                                          \
        return p.subset ? launch_forward_one<Ops, RS, true>(g, p, x, params, sel, y, argmax, st, name, probs_out)                \
                        : launch_forward_one<Ops, RS, false>(g, p, x, params, sel, y, argmax, st, name, probs_out)
    if (p.one_row) {                                                 // ROWSTEP names wo when a DPP row shift reaches the row below
        if (p.subset) return launch_forward_one<Ops, 0, true, true>(g, p, x, params, sel, y, argmax, st, name, probs_out);
        if (g.wo == 8) return launch_forward_one<Ops, 8, false, true>(g, p, x, params, sel, y, argmax, st, name, probs_out);
        if (g.wo == 4) return launch_forward_one<Ops, 4, false, true>(g, p, x, params, sel, y, argmax, st, name, probs_out);
        return launch_forward_one<Ops, 0, false, true>(g, p, x, params, sel, y, argmax, st, name, probs_out);
    }
    switch (g.sh * p.rs) {
        CLG_FWD_CASE(33);
        CLG_FWD_CASE(29);
        CLG_FWD_CASE(17);
        CLG_FWD_CASE(9);
        CLG_FWD_CASE(5);
    default:
        return p.subset ? launch_forward_one<Ops, 0, true>(g, p, x, params, sel, y, argmax, st, name, probs_out)
                        : launch_forward_one<Ops, 0, false>(g, p, x, params, sel, y, argmax, st, name, probs_out);
    }
#undef CLG_FWD_CASE
}

}  // namespace

extern "C" int clg_convblock_forward(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                     void *y, uint8_t *argmax, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_forward")) return e;
    CLG_REQUIRE(x && w && selection && y && argmax, "clg_convblock_forward: null pointer argument");
    TilePlan p;
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32) {
        if (plan_forward(g, 4, FloatOps<float>::kParams, &p))
            return launch_forward_tiled<FloatOps<float>>(g, p, x, w, selection, y, argmax, st, "clg_convblock_forward");
    } else {
        if (plan_forward(g, 8, FloatOps<double>::kParams, &p))
            return launch_forward_tiled<FloatOps<double>>(g, p, x, w, selection, y, argmax, st, "clg_convblock_forward");
    }
    return clg_convblock_forward_generic(dtype, g, x, w, selection, y, argmax, st);
}

extern "C" int clg_convblock_eval_packed(const clg_conv_geom *gg, const uint64_t *x, const uint8_t *gates, const int32_t *selection,
                                         uint64_t *y, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, CLG_F64, "clg_convblock_eval_packed")) return e;
    CLG_REQUIRE(x && gates && selection && y, "clg_convblock_eval_packed: null pointer argument");
    CLG_REQUIRE(x != y, "clg_convblock_eval_packed: x and y must not overlap");
    TilePlan p;
    hipStream_t st = clg_stream(stream);
    const char *e_4x4 = clg_knob(K_FWD_4X4);
    if (clg_convblock_is_4x4(g) && (!e_4x4 || atoi(e_4x4) != 0))
        return clg_convblock_eval_packed_4x4(g, x, gates, selection, y, st, "clg_convblock_eval_packed");
    if (plan_forward(g, 8, BitOps::kParams, &p)) {
        // one position per lane: a wavefront meets every kernel once, so the gates take the form without vector masks
        if (p.one_row && !p.subset) {
            const char *name = "clg_convblock_eval_packed";
            if (g.wo == 8) return launch_forward_one<BitOpsAnf, 8, false, true>(g, p, x, gates, selection, y, nullptr, st, name);
            if (g.wo == 4) return launch_forward_one<BitOpsAnf, 4, false, true>(g, p, x, gates, selection, y, nullptr, st, name);
            return launch_forward_one<BitOpsAnf, 0, false, true>(g, p, x, gates, selection, y, nullptr, st, name);
        }
        return launch_forward_tiled<BitOps>(g, p, x, gates, selection, y, nullptr, st, "clg_convblock_eval_packed");
    }
    const int64_t blocks = clg_ceil_div((int64_t)g.n * (g.ho / 2) * (g.wo / 2), 256);
    CLG_REQUIRE(g.c <= 65535 && blocks < (1ll << 31), "clg_convblock_eval_packed: problem too large for one launch");
    hipLaunchKernelGGL(convblock_packed_generic_kernel, dim3((unsigned)blocks, (unsigned)g.c), dim3(256), 0, st, x, gates, selection, y,
                       g);
    CLG_CHECK_LAUNCH("clg_convblock_eval_packed(any shape)");
    return CLG_OK;
}

extern "C" int64_t clg_convblock_forward_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_forward_scratch_bytes")) return -1;
    TilePlan tp;
    DirectPlan dp;
    const int elem = dtype == CLG_F64 ? 8 : 4;
    const int path = choose_forward(g, elem, 28, true, &tp, &dp);
    return path == 2 ? (int64_t)dp.total : (path == 4 || path == 5 ? (int64_t)g.c * 28 * elem : 0);
}

extern "C" int clg_convblock_forward_ws(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                        void *y, uint8_t *argmax, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_forward_ws")) return e;
    CLG_REQUIRE(x && w && selection && y && argmax, "clg_convblock_forward_ws: null pointer argument");
    TilePlan tp;
    DirectPlan dp;
    const int elem = dtype == CLG_F64 ? 8 : 4;
    const int path = choose_forward(g, elem, 28, scratch != nullptr, &tp, &dp);
    hipStream_t st = clg_stream(stream);
    if (path == 4 || path == 5) {
        const dim3 pgrid((unsigned)clg_ceil_div((int64_t)g.c * 7, 256));
        if (dtype == CLG_F32)
            hipLaunchKernelGGL((convblock_w_prepare_kernel<float, float>), pgrid, dim3(256), 0, st, (const float *)w, selection,
                               (float *)scratch, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<float>(), (int)pgrid.x);
        else
            hipLaunchKernelGGL((convblock_w_prepare_kernel<double, double>), pgrid, dim3(256), 0, st, (const double *)w, selection,
                               (double *)scratch, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<double>(), (int)pgrid.x);
        CLG_CHECK_LAUNCH("clg_convblock_forward_ws");
        if (path == 5) {
            if (dtype == CLG_F32)
                return launch_forward_kpl<float>(g, tp, x, scratch, selection, y, argmax, nullptr, st, "clg_convblock_forward_ws");
            return launch_forward_kpl<double>(g, tp, x, scratch, selection, y, argmax, nullptr, st, "clg_convblock_forward_ws");
        }
        return clg_convblock_forward_4x4(dtype, g, x, scratch, selection, y, argmax, st, "clg_convblock_forward_ws");
    }
    if (path != 2) return clg_convblock_forward(dtype, gg, x, w, selection, y, argmax, stream);
    if (dtype == CLG_F32)
        return launch_forward_direct<FloatOps<float>, float>(g, dp, x, w, selection, y, argmax, scratch, st, "clg_convblock_forward_ws");
    return launch_forward_direct<FloatOps<double>, double>(g, dp, x, w, selection, y, argmax, scratch, st, "clg_convblock_forward_ws");
}

namespace {
// probabilities of a [rows, 16] logit table: for the any-shape forward, whose kernel takes probabilities
template <typename T>
__global__ __launch_bounds__(256) void softmax16_rows_kernel(const T *__restrict__ logits, T *__restrict__ probs, int64_t rows)
{
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= rows) return;
    T pr[16];
    softmax16(logits + q * 16, pr);
#pragma unroll
    for (int i = 0; i < 16; ++i) probs[q * 16 + i] = pr[i];
}
}  // namespace

// Forward of the complete block with options (flags: CLG_FWD_W_LOGITS, CLG_FWD_Y_FEATURE_MAJOR).
int64_t clg_convblock_backward_padded_sample_elems(int dtype, const Geom &g);

static int forward_ex_impl(const char *name, int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                           void *y, uint8_t *argmax, void *probs_out, int flags, void *scratch, void *padded_out, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(x && w && selection && y && argmax, "%s: null pointer argument", name);
    CLG_REQUIRE((flags & ~(CLG_FWD_W_LOGITS | CLG_FWD_Y_FEATURE_MAJOR | CLG_FWD_FOLDED_OUT | CLG_FWD_FOLDED_IN)) == 0, "%s: unknown flags 0x%x",
                name, flags);
    const bool given = (flags & CLG_FWD_FOLDED_IN) != 0;                // probabilities and coefficients are in probs_out already
    CLG_REQUIRE(!given || ((flags & CLG_FWD_W_LOGITS) && (flags & CLG_FWD_FOLDED_OUT)), "%s: CLG_FWD_FOLDED_IN goes with CLG_FWD_W_LOGITS | "
                "CLG_FWD_FOLDED_OUT (it says that their outputs are there already)", name);
    bool logits = (flags & CLG_FWD_W_LOGITS) != 0;
    const bool fm = (flags & CLG_FWD_Y_FEATURE_MAJOR) != 0;
    bool want_folded = (flags & CLG_FWD_FOLDED_OUT) != 0;
    CLG_REQUIRE(!logits || probs_out, "%s: CLG_FWD_W_LOGITS needs probs_out [c_out, 7, 16]", name);
    CLG_REQUIRE(!want_folded || probs_out, "%s: CLG_FWD_FOLDED_OUT needs probs_out with room for [c_out, 7, 16] + [c_out, 7, 4]", name);
    CLG_REQUIRE(!fm || (scratch && clg_convblock_fm_supported(dtype, gg)), "%s: CLG_FWD_Y_FEATURE_MAJOR needs scratch and a shape for "
                "which clg_convblock_fm_supported() holds (4x4 images, 3x3 kernel, stride 1, padding 1, n >= 32)", name);
    TilePlan tp;
    DirectPlan dp;
    const int elem = dtype == CLG_F64 ? 8 : 4;
    const int path = fm ? 4 : choose_forward(g, elem, 28, scratch != nullptr, &tp, &dp);
    hipStream_t st = clg_stream(stream);
    // the folded coefficients [c_out, 7, 4] follow the probabilities in probs_out
    void *folded_out = want_folded ? reinterpret_cast<unsigned char *>(probs_out) + (size_t)g.c * 112 * elem : nullptr;
    // paths whose kernels do not write them themselves: one small launch folds the probabilities (after the forward launches)
    auto fold_after = [&](int e) {
        if (e != CLG_OK || !want_folded) return e;
        const dim3 pgrid((unsigned)clg_ceil_div((int64_t)g.c * 7, 256));
        const void *pr = logits ? probs_out : w;
        if (dtype == CLG_F32)
            hipLaunchKernelGGL((convblock_w_prepare_kernel<float, float>), pgrid, dim3(256), 0, st, (const float *)pr, selection,
                               (float *)folded_out, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<float>(), (int)pgrid.x);
        else
            hipLaunchKernelGGL((convblock_w_prepare_kernel<double, double>), pgrid, dim3(256), 0, st, (const double *)pr, selection,
                               (double *)folded_out, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<double>(), (int)pgrid.x);
        CLG_CHECK_LAUNCH(name);
        return CLG_OK;
    };
    if (path == 4 || path == 5) {
        g.y_fm = fm ? 1 : 0;
        void *fold_to = want_folded ? folded_out : scratch;             // the kernels read them from wherever they are
        const dim3 pgrid((unsigned)clg_ceil_div((int64_t)g.c * 7, 256));
        if (given) {
            // folded by the caller (clg_fold_many): no set-up launch
        } else if (dtype == CLG_F32)
            hipLaunchKernelGGL((convblock_w_prepare_kernel<float, float>), pgrid, dim3(256), 0, st, (const float *)w, selection,
                               (float *)fold_to, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<float>(), (int)pgrid.x, logits ? 1 : 0,
                               (float *)probs_out);
        else
            hipLaunchKernelGGL((convblock_w_prepare_kernel<double, double>), pgrid, dim3(256), 0, st, (const double *)w, selection,
                               (double *)fold_to, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<double>(), (int)pgrid.x, logits ? 1 : 0,
                               (double *)probs_out);
        CLG_CHECK_LAUNCH(name);
        if (path == 5) {
            if (dtype == CLG_F32) return launch_forward_kpl<float>(g, tp, x, fold_to, selection, y, argmax, padded_out, st, name);
            return launch_forward_kpl<double>(g, tp, x, fold_to, selection, y, argmax, padded_out, st, name);
        }
        return clg_convblock_forward_4x4(dtype, g, x, fold_to, selection, y, argmax, st, name);
    }
    if (given) {                                                     // the other kernels take the probabilities as their weights
        w = probs_out;
        logits = false;
        want_folded = false;                                         // (the coefficients are there: nothing to fold afterwards)
    }
    if (path == 2) {
        if (dtype == CLG_F32)
            return fold_after(launch_forward_direct<FloatOps<float>, float>(g, dp, x, w, selection, y, argmax, scratch, st, name, logits, probs_out,
                                                                            padded_out));
        return fold_after(launch_forward_direct<FloatOps<double>, double>(g, dp, x, w, selection, y, argmax, scratch, st, name, logits, probs_out,
                                                                          padded_out));
    }
    // The staged kernels take the softmax per workgroup while they set their gate parameters up, as long as that is at
    // most two rows of 16 logits per thread (C3 graph step 66.7 -> 63.7 us against a small launch of its own; with the
    // 512 kernels of [256,128,8,8] -> 512 in one tile it is four rows and costs 7 us where the launch costs 3); beyond
    // that, and for the any-shape kernel, the probabilities come from that small launch.
    const bool staged = path == 0 || path == 1;
    bool in_kernel = staged && logits && clg_ceil_div((int64_t)tp.CT * 7, (int64_t)tp.NW * kWave) <= 2;
    if (const char *e = clg_knob(K_FWD_SOFTMAX_IN_KERNEL)) in_kernel = staged && logits && atoi(e) != 0;
    if (logits && !in_kernel) {
        const int64_t rows = (int64_t)g.c * 7;
        if (dtype == CLG_F32)
            hipLaunchKernelGGL(softmax16_rows_kernel<float>, dim3((unsigned)clg_ceil_div(rows, 256)), dim3(256), 0, st, (const float *)w,
                               (float *)probs_out, rows);
        else
            hipLaunchKernelGGL(softmax16_rows_kernel<double>, dim3((unsigned)clg_ceil_div(rows, 256)), dim3(256), 0, st, (const double *)w,
                               (double *)probs_out, rows);
        CLG_CHECK_LAUNCH(name);
        w = probs_out;
    }
    if (staged) {
        tp.w_logits = in_kernel ? 1 : 0;
        tp.folded_out = folded_out;                                  // written by the first sample block of every kernel tile
        if (padded_out != nullptr) {
            tp.padded_out = padded_out;                              // written by the first kernel tile of every sample block
            tp.padded_sample_elems = g.cin * tp.chs + g.ph * tp.rs + g.pw;
        }
        if (dtype == CLG_F32) return launch_forward_tiled<FloatOps<float>>(g, tp, x, w, selection, y, argmax, st, name, probs_out);
        return launch_forward_tiled<FloatOps<double>>(g, tp, x, w, selection, y, argmax, st, name, probs_out);
    }
    return fold_after(clg_convblock_forward_generic(dtype, g, x, w, selection, y, argmax, st));
}

extern "C" int clg_convblock_forward_ex(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                        void *y, uint8_t *argmax, void *probs_out, int flags, void *scratch, void *stream)
{
    return forward_ex_impl("clg_convblock_forward_ex", dtype, gg, x, w, selection, y, argmax, probs_out, flags, scratch, nullptr, stream);
}

// Elements of the padded copy of x that clg_convblock_forward_padded leaves for clg_convblock_backward_planned_padded, or 0
// when the pair has no use for one at this shape: the forward must stage or read the copy anyway (all channels in LDS, or
// the direct kernel) and the backward must be the one that reads its taps from such a copy.
extern "C" int64_t clg_convblock_padded_elems(int dtype, const clg_conv_geom *gg, int have_scratch)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_padded_elems")) return -1;
    TilePlan tp;
    DirectPlan dp;
    const int elem = dtype == CLG_F64 ? 8 : 4;
    const int path = choose_forward(g, elem, 28, have_scratch != 0, &tp, &dp);
    if (path != 0 && path != 2 && path != 5) return 0;
    const int64_t se = clg_convblock_backward_padded_sample_elems(dtype, g);
    if (se <= 0) return 0;
    const int64_t mine = path == 2 ? dp.sample_elems : (int64_t)g.cin * tp.chs + g.ph * tp.rs + g.pw;
    return se == mine ? se * g.n : 0;
}

extern "C" int clg_convblock_forward_padded(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                            void *y, uint8_t *argmax, void *probs_out, int flags, void *scratch, void *padded_out,
                                            void *stream)
{
    const char *name = "clg_convblock_forward_padded";
    CLG_REQUIRE(padded_out, "%s: null pointer argument", name);
    CLG_REQUIRE((flags & CLG_FWD_Y_FEATURE_MAJOR) == 0 && clg_convblock_padded_elems(dtype, gg, scratch != nullptr) > 0,
                "%s: no padded copy at this shape (clg_convblock_padded_elems)", name);
    return forward_ex_impl(name, dtype, gg, x, w, selection, y, argmax, probs_out, flags, scratch, padded_out, stream);
}

// Which shapes the feature-major variants take: the one-sample-per-lane kernels for 4x4 images (conv_small.hip).
extern "C" int clg_convblock_fm_supported(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (gg == nullptr || (dtype != CLG_F32 && dtype != CLG_F64)) return 0;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_fm_supported")) return 0;
    const char *e_fwd = clg_knob(K_FWD_4X4), *e_bwd = clg_knob(K_BWD_4X4);
    if ((e_fwd && atoi(e_fwd) == 0) || (e_bwd && atoi(e_bwd) == 0)) return 0;
    return clg_convblock_is_4x4(g) && g.c <= 65535 ? 1 : 0;
}

extern "C" int clg_convblock_forward_fm(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                        void *y, uint8_t *argmax, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_forward_fm")) return e;
    CLG_REQUIRE(x && w && selection && y && argmax && scratch, "clg_convblock_forward_fm: null pointer argument");
    CLG_REQUIRE(clg_convblock_fm_supported(dtype, gg), "clg_convblock_forward_fm: needs 4x4 images, a 3x3 kernel, stride 1, padding 1 and "
                "at least 32 samples (clg_convblock_fm_supported)");
    g.y_fm = 1;
    hipStream_t st = clg_stream(stream);
    const dim3 pgrid((unsigned)clg_ceil_div((int64_t)g.c * 7, 256));
    if (dtype == CLG_F32)
        hipLaunchKernelGGL((convblock_w_prepare_kernel<float, float>), pgrid, dim3(256), 0, st, (const float *)w, selection,
                           (float *)scratch, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<float>(), (int)pgrid.x);
    else
        hipLaunchKernelGGL((convblock_w_prepare_kernel<double, double>), pgrid, dim3(256), 0, st, (const double *)w, selection,
                           (double *)scratch, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), no_pad_job<double>(), (int)pgrid.x);
    CLG_CHECK_LAUNCH("clg_convblock_forward_fm");
    return clg_convblock_forward_4x4(dtype, g, x, scratch, selection, y, argmax, st, "clg_convblock_forward_fm");
}

extern "C" int clg_convblock_eval_packed_fm_supported(const clg_conv_geom *gg)
{
    Geom g;
    if (gg == nullptr || clg_convblock_check(gg, &g, CLG_F64, "clg_convblock_eval_packed_fm_supported")) return 0;
    const char *e_4x4 = clg_knob(K_FWD_4X4);
    return clg_convblock_is_4x4(g) && (!e_4x4 || atoi(e_4x4) != 0) ? 1 : 0;
}

extern "C" int clg_convblock_eval_packed_fm(const clg_conv_geom *gg, const uint64_t *x, const uint8_t *gates, const int32_t *selection,
                                            uint64_t *y, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, CLG_F64, "clg_convblock_eval_packed_fm")) return e;
    CLG_REQUIRE(x && gates && selection && y, "clg_convblock_eval_packed_fm: null pointer argument");
    CLG_REQUIRE(x != y, "clg_convblock_eval_packed_fm: x and y must not overlap");
    CLG_REQUIRE(clg_convblock_eval_packed_fm_supported(gg), "clg_convblock_eval_packed_fm: needs 4x4 images, a 3x3 kernel, stride 1, "
                "padding 1 and at least 32 word groups (clg_convblock_eval_packed_fm_supported)");
    g.y_fm = 1;
    return clg_convblock_eval_packed_4x4(g, x, gates, selection, y, clg_stream(stream), "clg_convblock_eval_packed_fm");
}

extern "C" int64_t clg_convblock_eval_packed_scratch_bytes(const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, CLG_F64, "clg_convblock_eval_packed_scratch_bytes")) return -1;
    TilePlan tp;
    DirectPlan dp;
    return choose_forward(g, 8, 1, true, &tp, &dp) == 2 ? (int64_t)dp.total : 0;
}

extern "C" int clg_convblock_eval_packed_ws(const clg_conv_geom *gg, const uint64_t *x, const uint8_t *gates, const int32_t *selection,
                                            uint64_t *y, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, CLG_F64, "clg_convblock_eval_packed_ws")) return e;
    CLG_REQUIRE(x && gates && selection && y, "clg_convblock_eval_packed_ws: null pointer argument");
    CLG_REQUIRE(x != y, "clg_convblock_eval_packed_ws: x and y must not overlap");
    TilePlan tp;
    DirectPlan dp;
    if (choose_forward(g, 8, 1, scratch != nullptr, &tp, &dp) != 2) return clg_convblock_eval_packed(gg, x, gates, selection, y, stream);
    return launch_forward_direct<BitOps, float>(g, dp, x, gates, selection, y, nullptr, scratch, clg_stream(stream),
                                                "clg_convblock_eval_packed_ws");
}
