// Fused conv-logic block (tap gather -> 4 leaf gates -> 2 gates -> root gate -> 2x2/2 max pool):
// LDS-tiled kernels for gfx950, shape dispatch and the C entry points.
//
// LDS image layout.  A workgroup stages the zero-padded input planes of S samples (all input
// channels) in LDS.  Padding is shared: a row holds pw halo elements and then the w pixels, so the
// right halo of a row is the left halo of the next row (row stride rs = w + pw), and the bottom halo
// rows of a plane are the top halo rows of the next plane (plane stride chs = (h + ph) * rs).  A tap
// (ch, ry, rx) of a kernel is then one scalar offset ch*chs + ry*rs + rx that is added to a per-lane
// base, with no bounds checks in the inner loops.
//
// Forward: a workgroup owns (S samples) x (CT kernels).  Lanes run along conv-output columns, each
// lane evaluates the tree at conv rows 2r and 2r+1, the horizontal neighbour comes over DPP, and the
// even lane keeps the first maximum in window order and writes the pooled value and a 1-byte code.
// The kernel index is uniform per wavefront, so the 28 folded coefficients and 8 tap offsets sit in
// scalar registers.
//
// Input gradient: deterministic without float atomics in global memory.  Every (sample, input
// channel) plane of the gradient has exactly one owner wavefront, which walks all kernels that read
// its channel in increasing order, recomputes their tree at the stored argmax position of every
// pooled cell and accumulates the tap gradients of ITS channel into an LDS plane that only it
// touches (the plane has the same shared-halo layout as the input image, so out-of-image taps fall
// into halo elements that are never read back).  The order of additions is program order.
#include <stdlib.h>

#include <mutex>

#include "conv_tile.h"

int clg_convblock_check(const clg_conv_geom *gg, Geom *g, int dtype, const char *name);
int clg_convblock_forward_generic(int dtype, const Geom &g, const void *x, const void *w, const int32_t *selection, void *y,
                                  uint8_t *argmax, hipStream_t st);
int clg_convblock_backward_x_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *folded,
                                     const int32_t *count, const int32_t *hits, const int32_t *selection, const uint8_t *argmax,
                                     void *grad_x, hipStream_t st);
int clg_convblock_backward_w_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                                     hipStream_t st, const void *probs);
int clg_convblock_partial_blocks(const Geom &g);
bool clg_convblock_is_4x4(const Geom &g);
size_t clg_convblock_backward_4x4_tg_bytes(int dtype, const Geom &g);
int clg_convblock_backward_4x4(int dtype, const Geom &g, const void *x, const void *folded, const int32_t *sel, const void *gy,
                               const uint8_t *argmax, void *tg, void *gw, const void *probs, const int32_t *count, const int32_t *hits,
                               void *gx, hipStream_t st, const char *name);
int clg_launch_reduce_coef(int dtype, const void *partial, void *out, int64_t rows, int nb, int G, hipStream_t st, const char *name,
                           const void *probs);

namespace {

// ---------------------------------------------------------------------------------------------
// input gradient
// ---------------------------------------------------------------------------------------------
// Scratch of the input-gradient kernels, written by the preparation launches:
//   folded [c][7][4]   coefficients (ab, a, b, one) of every gate
//   count  [cin][2]    (number of kernels that read input channel ch, offset of its list in hits)
//   hits               those kernels in increasing order, entry = kernel | tap mask << 16
// (the reverse map "input channel -> kernels and taps reading it", built in a fixed order).  Small maps
// are dense, hits[cin][c], filled by one wavefront per channel.  Large ones (cin * c above 2^20) are
// compressed: lists back to back (at most 8 c entries), filled through integer atomics and then sorted per
// channel, so the order of the lists -- and with it the order of the float additions -- stays fixed.
struct BwdScratch {
    size_t folded_bytes, count_off, cursor_off, hits_off, unsorted_off, taps_off, part_off, total;
    int csr;
};
constexpr int kMaxHitSplit = 16;
bool hits_compressed(const Geom &g)
{
    if (const char *e = clg_knob(K_BWDX_CSR)) return atoi(e) != 0;
    return (int64_t)g.cin * g.c > (1ll << 20);
}
BwdScratch bwd_scratch_layout(const Geom &g, int elem, int hit_split)
{
    BwdScratch b;
    b.csr = hits_compressed(g) ? 1 : 0;
    const size_t list_bytes = b.csr ? (size_t)g.c * 8 * 4 : (size_t)g.cin * g.c * 4;
    b.folded_bytes = (size_t)g.c * 28 * elem;
    b.count_off = (b.folded_bytes + 63) & ~(size_t)63;
    b.cursor_off = (b.count_off + (size_t)g.cin * 8 + 63) & ~(size_t)63;
    b.hits_off = (b.cursor_off + (b.csr ? (size_t)g.cin * 4 : 0) + 63) & ~(size_t)63;
    b.unsorted_off = (b.hits_off + list_bytes + 63) & ~(size_t)63;
    b.taps_off = (b.unsorted_off + (b.csr ? list_bytes : 0) + 63) & ~(size_t)63;
    b.part_off = (b.taps_off + (size_t)g.c * 16 * 4 + 255) & ~(size_t)255;   // taps: 8 offsets in the image, 8 in the plane
    b.total = b.part_off + (hit_split > 1 ? (size_t)hit_split * g.n * g.cin * g.h * g.w * elem : 0);   // partial images
    return b;
}

template <typename T>
__global__ __launch_bounds__(256) void convblock_prepare_kernel(const T *__restrict__ w, const int32_t *__restrict__ sel,
                                                              T *__restrict__ folded, int32_t *__restrict__ count,
                                                              int32_t *__restrict__ hits, int32_t *__restrict__ taps, int C,
                                                              int cin, int fold_blocks, int rs, int chs, PadJob<T> pad, int pad_block0,
                                                              TapLimit lim)
{
    if ((int)blockIdx.x >= pad_block0) {                            // tail of the launch: the padded copy of x
        pad_image_elem(pad, (int64_t)(blockIdx.x - pad_block0) * 256 + threadIdx.x);
        return;
    }
    if ((int)blockIdx.x < fold_blocks) {
        const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (q < (int64_t)C * 8) {                                   // tap offsets of the LDS window layout
            const Tap tp = unpack_tap(sel[q], lim);
            const int rel = tp.ry * rs + tp.rx;
            const int64_t c = q >> 3, t = q & 7;
            taps[c * 16 + t] = tp.ch * chs + rel;
            taps[c * 16 + 8 + t] = rel;
        }
        if (w != nullptr && q < (int64_t)C * 7) {                    // (a plan is made without weights)
            const Coef<T> cf = fold16(w + q * 16);
            folded[q * 4 + 0] = cf.ab;
            folded[q * 4 + 1] = cf.a;
            folded[q * 4 + 2] = cf.b;
            folded[q * 4 + 3] = cf.one;
        }
        return;
    }
    // one wavefront per input channel: lanes test 64 kernels at a time, matches are appended in order
    const int lane = threadIdx.x & (kWave - 1);
    const int ch = uniform((int)(blockIdx.x - fold_blocks) * 4 + (int)(threadIdx.x >> 6));
    if (ch >= cin || hits == nullptr) return;
    int n = 0;
    for (int c0 = 0; c0 < C; c0 += kWave) {
        const int c = c0 + lane;
        int mask = 0;
        if (c < C) {
#pragma unroll
            for (int t = 0; t < 8; ++t) mask |= (tap_channel(sel[c * 8 + t], cin) == ch) << t;
        }
        const uint64_t vote = __ballot(mask != 0);
        if (mask) {
            const int before = __builtin_amdgcn_mbcnt_hi((uint32_t)(vote >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)vote, 0));
            hits[(int64_t)ch * C + n + before] = c | (mask << 16);
        }
        n += __popcll(vote);
    }
    if (lane == 0) {
        count[2 * ch] = n;
        count[2 * ch + 1] = ch * C;
    }
}

// ---- compressed lists ------------------------------------------------------------------------
// tap mask of kernel c for the channel of its tap t, or 0 when an earlier tap names the same channel
__device__ __forceinline__ int first_use_mask(const int32_t *__restrict__ sq, int t, int cin)
{
    const int ch = tap_channel(sq[t], cin);
    int mask = 0;
    for (int u = 0; u < 8; ++u) {
        if (tap_channel(sq[u], cin) == ch) {
            if (u < t) return 0;
            mask |= 1 << u;
        }
    }
    return mask;
}
__global__ __launch_bounds__(256) void hits_zero_kernel(int32_t *__restrict__ count, int32_t *__restrict__ cursor, int cin)
{
    const int ch = blockIdx.x * 256 + threadIdx.x;
    if (ch >= cin) return;
    count[2 * ch] = 0;
    count[2 * ch + 1] = 0;
    cursor[ch] = 0;
}
__global__ __launch_bounds__(256) void hits_count_kernel(const int32_t *__restrict__ sel, int32_t *__restrict__ count, int C, int cin)
{
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int32_t *sq = sel + (int64_t)c * 8;
    for (int t = 0; t < 8; ++t)
        if (first_use_mask(sq, t, cin)) atomicAdd(count + 2 * tap_channel(sq[t], cin), 1);
}
// exclusive prefix sum of the counts into the offsets, one workgroup
__global__ __launch_bounds__(1024) void hits_scan_kernel(int32_t *__restrict__ count, int cin)
{
    __shared__ int part[1024];
    const int tid = threadIdx.x;
    const int per = (cin + 1023) / 1024;
    const int lo = tid * per, hi = min(cin, lo + per);
    int sum = 0;
    for (int ch = lo; ch < hi; ++ch) sum += count[2 * ch];
    part[tid] = sum;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int v = tid >= d ? part[tid - d] : 0;
        __syncthreads();
        part[tid] += v;
        __syncthreads();
    }
    int run = part[tid] - sum;
    for (int ch = lo; ch < hi; ++ch) {
        count[2 * ch + 1] = run;
        run += count[2 * ch];
    }
}
__global__ __launch_bounds__(256) void hits_fill_kernel(const int32_t *__restrict__ sel, const int32_t *__restrict__ count,
                                                      int32_t *__restrict__ cursor, int32_t *__restrict__ unsorted, int C, int cin)
{
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int32_t *sq = sel + (int64_t)c * 8;
    for (int t = 0; t < 8; ++t) {
        const int mask = first_use_mask(sq, t, cin);
        if (mask) {
            const int ch = tap_channel(sq[t], cin);
            unsorted[count[2 * ch + 1] + atomicAdd(cursor + ch, 1)] = c | (mask << 16);
        }
    }
}
// one wavefront per channel: every entry goes to the position given by the number of smaller kernel
// indices in its list (a kernel occurs once per list)
__global__ __launch_bounds__(256) void hits_sort_kernel(const int32_t *__restrict__ count, const int32_t *__restrict__ unsorted,
                                                      int32_t *__restrict__ hits, int cin)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int ch = uniform((int)blockIdx.x * 4 + (int)(threadIdx.x >> 6));
    if (ch >= cin) return;
    const int n = count[2 * ch];
    const int32_t *src = unsorted + count[2 * ch + 1];
    int32_t *dst = hits + count[2 * ch + 1];
    for (int i = lane; i < n; i += kWave) {
        const int e = src[i], key = e & 0xFFFF;
        int rank = 0;
        for (int j = 0; j < n; ++j) rank += (src[j] & 0xFFFF) < key;
        dst[rank] = e;
    }
}

constexpr int kChunk = 4;  // cell blocks (of 64 lanes) whose grad_y / argmax loads are in flight together

template <typename T>
struct CellLoads {
    T gy[kChunk];
    uint32_t codes;            // the kChunk one-byte arg-max codes, block j in byte j
};

// Row band of the input image owned by one workgroup, the pooled cells whose taps can reach it and
// the padded rows those cells read.  Identical arithmetic on host (LDS sizing) and device.
struct Band {
    int r0, r1;      // image rows [r0, r1) whose gradient this workgroup produces
    int cell_lo, cb; // first pooled cell and number of pooled cells to visit
    int R0, rows;    // first staged padded row and number of staged rows
};
__host__ __device__ inline Band make_band(const Geom &g, int band, int band_rows)
{
    Band b;
    const int wp = g.wo / 2;
    if (band_rows >= g.h) {                                         // one band: the whole image
        b.r0 = 0; b.r1 = g.h; b.cell_lo = 0; b.cb = (g.ho / 2) * wp; b.R0 = 0; b.rows = g.h + 2 * g.ph;
        return b;
    }
    b.r0 = band * band_rows;
    b.r1 = b.r0 + band_rows < g.h ? b.r0 + band_rows : g.h;
    const int num = b.r0 + g.ph - g.kh + 1;                       // smallest oy*sh that can reach row r0
    int oy_lo = num <= 0 ? 0 : (num + g.sh - 1) / g.sh;
    int oy_hi = (b.r1 + g.ph - 1) / g.sh;
    if (oy_hi > g.ho - 1) oy_hi = g.ho - 1;
    int R0 = b.r0 + g.ph, R1 = b.r1 + g.ph;                       // the window always holds the owned rows
    b.cell_lo = 0;
    b.cb = 0;
    if (oy_lo <= oy_hi) {
        const int py_lo = oy_lo / 2, py_hi = oy_hi / 2;
        b.cell_lo = py_lo * wp;
        b.cb = (py_hi - py_lo + 1) * wp;
        const int t0 = 2 * py_lo * g.sh, t1 = (2 * py_hi + 1) * g.sh + g.kh;   // padded rows the cells read
        if (t0 < R0) R0 = t0;
        if (t1 > R1) R1 = t1;
        if (R1 > g.h + 2 * g.ph) R1 = g.h + 2 * g.ph;
    }
    b.R0 = R0;
    b.rows = R1 - R0;
    return b;
}

// grid: (sample groups, bands, hit split).  LDS: input window xs, gradient window gs (same layout: planes
// of `wrows` rows x rs elements, left halo shared with the previous row's right halo) and, unless halo
// elements can take them, one sink element per thread for masked updates.  With a hit split > 1 the
// workgroups blockIdx.z = 0..HS-1 of one (sample group, band) take every HS-th kernel of each channel's
// list and write partial gradient images that sum_partial_images adds in a fixed order.  Inside a workgroup,
// p.hsw wavefronts can share one (sample group, channel) the same way: each takes every hsw-th of those
// kernels and accumulates into its own copy of the gradient window; the copies are added in order on the
// way out.
// FULL: every wavefront pass has all of its kChunk * 64 cells (whole images, every sample group complete): no lane is
// ever redirected, and the per-lane liveness tests drop out of the loops.
// (float: two workgroups of 9 wavefronts share a compute unit only with 6 wavefronts per SIMD, i.e. at most 80 registers)
template <typename T, bool BANDED, bool SHARED, bool FULL>
__global__ __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? 6 : 4))) void convblock_backward_x_tiled_kernel(const T *__restrict__ gy, const T *__restrict__ x,
                                                  const T *__restrict__ folded, const int32_t *__restrict__ count,
                                                  const int32_t *__restrict__ hits, const int32_t *__restrict__ taps,
                                                  const uint8_t *__restrict__ argmax, T *__restrict__ gx, Geom g, TilePlan p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int xe4 = (p.xe + 3) & ~3;
    T *xs = reinterpret_cast<T *>(smem);
    T *gs = xs + xe4;
    const int gs_off = xe4;
    // sink of masked updates: the first (halo) row of the gradient window, or a region after it
    const int hsw = SHARED ? p.hsw : 1;                              // SHARED = false keeps the one-owner code as lean as it was
    const int sink_base = (1 + hsw) * xe4;

    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int lane = tid & (kWave - 1), wave = uniform(tid >> 6);
    const int n0 = blockIdx.x * p.S, s_cur = min(p.S, g.n - n0);
    const int wp = g.wo >> 1, I = p.slots;
    const Band bd = make_band(g, blockIdx.y, p.band_rows);
    const int chs = p.chs;                                          // plane stride of the windows

    const int zero_n = sink_base + (p.dummy_in_halo ? 0 : nthreads);
    for (int i = tid; i < zero_n; i += nthreads) xs[i] = T(0);
    __syncthreads();
    // stage the image rows that fall into the window (padded row = image row + ph)
    const int ir0 = bd.R0 - g.ph > 0 ? bd.R0 - g.ph : 0;
    const int ir1 = bd.R0 + bd.rows - g.ph < g.h ? bd.R0 + bd.rows - g.ph : g.h;
    const int irows = ir1 > ir0 ? ir1 - ir0 : 0;
    const int planes = s_cur * g.cin;
    const T *src = x + (int64_t)n0 * g.cin * g.h * g.w;
    for (int pr = wave; pr < planes * irows; pr += p.NW) {
        const int plane = uniform(pr / irows), iy = ir0 + (pr - plane * irows);
        const T *row = src + ((int64_t)plane * g.h + iy) * g.w;
        T *dst = xs + plane * chs + (iy + g.ph - bd.R0) * p.rs + g.pw;
        for (int ix = lane; ix < g.w; ix += kWave) dst[ix] = row[ix];
    }
    __syncthreads();

    // plane-relative range of elements this workgroup owns (rows r0..r1-1 of every plane)
    const uint32_t own_lo = (uint32_t)((bd.r0 + g.ph - bd.R0) * p.rs);
    const uint32_t own_len = (uint32_t)((bd.r1 - bd.r0) * p.rs);

    // work items: (group of G samples, input channel); a wavefront owns the gradient planes of its item
    const int groups = (s_cur + p.G - 1) / p.G;
    const int items = groups * g.cin;
    const int row_step = g.sh * p.rs;
    for (int witem = wave; witem < items * hsw; witem += p.NW) {
        const int item = SHARED ? witem / hsw : witem, slot = SHARED ? witem - item * hsw : 0;
        const int gw_off = gs_off + slot * xe4;                      // this wavefront's copy of the gradient window
        const int dummy_off = p.dummy_in_halo ? gw_off + (lane & 31) : sink_base + (int)threadIdx.x;
        const int grp = item / g.cin, ch = item - grp * g.cin;
        const int s0 = grp * p.G;
        const int v_here = min(p.G, s_cur - s0) * bd.cb;
        const int chunks = (v_here + kChunk * kWave - 1) / (kChunk * kWave);
        const int img0 = s0 * g.cin * chs;                          // LDS offset of the group's first plane
        const int64_t gbase = ((int64_t)(n0 + s0) * g.c) * I;       // global offset of the group's first cell row
        const int nhits = v_here > 0 ? count[2 * ch] : 0;
        const int32_t *hit = hits + count[2 * ch + 1];

        // chunk-major: the cell table entries of a chunk stay in registers while all kernels that read
        // this channel are applied to it (hits in increasing kernel order inside every chunk)
        for (int chunk = 0; chunk < chunks; ++chunk) {
            int cx[kChunk], cy[kChunk];
            bool live[kChunk];
#pragma unroll
            for (int j = 0; j < kChunk; ++j) {
                if (FULL && j > 0) {                                 // whole rows of cells per block: a uniform step from block 0
                    live[j] = true;
                    cx[j] = cx[0] + j * (kWave / wp) * 2 * row_step;
                    cy[j] = cy[0] + j * kWave;
                    continue;
                }
                const int v = (chunk * kChunk + j) * kWave + lane;
                live[j] = FULL || v < v_here;
                uint32_t sm = 0, cl = live[j] ? v : 0;              // sample inside the group, cell inside the band
                if (!BANDED && !FULL) {
                    sm = fdiv(cl, p.d_slots);
                    cl -= sm * (uint32_t)I;
                }
                const uint32_t cell = bd.cell_lo + cl;
                const uint32_t py = fdiv(cell, p.d_wp), px = cell - py * (uint32_t)wp;
                cx[j] = img0 + (int)(sm * g.cin * chs + (2 * py * g.sh - bd.R0) * p.rs + 2 * px * g.sw);
                cy[j] = (int)((sm * g.c) * I + cell);
            }
            // grad_y and the argmax code of hit k: requested one hit ahead of their use
            auto issue = [&](int k, CellLoads<T> &L) {
                const int64_t crow = gbase + (int64_t)(hit[k] & 0xFFFF) * I;
                const uint8_t *am = argmax + crow;
                const T *gr = gy + crow;
                uint32_t code[kChunk];
#pragma unroll
                for (int j = 0; j < kChunk; ++j) {
                    L.gy[j] = T(0);
                    code[j] = 0;
                    if (live[j]) {
                        code[j] = am[cy[j]];
                        L.gy[j] = gr[cy[j]];
                    }
                }
                L.codes = code[0];
#pragma unroll
                for (int j = 1; j < kChunk; ++j) L.codes |= code[j] << (8 * j);
            };
            CellLoads<T> cur, nxt;
            const int hs0 = blockIdx.z + gridDim.z * slot, hsn = gridDim.z * hsw;
            if (hs0 < nhits) issue(hs0, cur);
            for (int k = hs0; k < nhits; k += hsn) {
                if (k + hsn < nhits) issue(k + hsn, nxt);
                const int ent = hit[k];
                const int c = ent & 0xFFFF, mask = (ent >> 16) & 0xFF;
                int to[8];                                          // tap offsets inside the group's planes
                int tr_[8];                                         // the same, relative to the tap's own plane
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    to[t] = taps[c * 16 + t];
                    tr_[t] = BANDED ? taps[c * 16 + 8 + t] : 0;
                }
                Tree<T> tr;
                const T *fc = folded + (int64_t)c * 28;
#pragma unroll
                for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
                pin_addends(tr);
                // Two cell blocks at a time (the pinned addends serve both; the tap gradients of only two blocks are live):
                // phase 1: tree and tap gradients of the pair (registers only).  No per-lane control flow: a lane
                // without a cell recomputes cell 0 with a zero gradient.
                // phase 2: read-add-write per tap.  For one tap the targets of all cells (all lanes, both blocks) are
                // distinct elements, so the blocks of a pair go together; taps may collide with each other and are
                // applied one after the other, and the pairs one after the other.  Only this wavefront touches the
                // plane rows it owns.  Lanes without a cell, and (with bands) targets outside the owned rows, are
                // redirected to a private dummy element per lane, so the whole phase is straight-line code with the
                // LDS reads of a tap in flight together.
#pragma unroll
                for (int jp = 0; jp < kChunk; jp += 2) {
                    int pos[2];
                    T gt[2][8];
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        const int j = jp + jj;
                        const T gout = cur.gy[j];                   // 0 for lanes without a cell
                        pos[jj] = cx[j] + (int)((cur.codes >> (8 * j + 1)) & 1) * row_step + (int)((cur.codes >> (8 * j)) & 1) * g.sw;
                        T tv[8];
#pragma unroll
                        for (int t = 0; t < 8; ++t) tv[t] = xs[pos[jj] + to[t]];
                        const TreeVals<T> tvv = eval_tree(tr, tv);
                        const T g_m0 = gout * gate_da(tr.g[6], tvv.mid[1]);
                        const T g_m1 = gout * gate_db(tr.g[6], tvv.mid[0]);
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if ((mask >> (2 * q)) & 3) {             // wave-uniform: a tap of this leaf is ours
                                const int m = q >> 1;
                                const T g_mid = m ? g_m1 : g_m0;
                                const T g_leaf = g_mid * ((q & 1) ? gate_db(tr.g[4 + m], tvv.leaf[q ^ 1])
                                                                   : gate_da(tr.g[4 + m], tvv.leaf[q ^ 1]));
                                gt[jj][2 * q] = g_leaf * gate_da(tr.g[q], tv[2 * q + 1]);
                                gt[jj][2 * q + 1] = g_leaf * gate_db(tr.g[q], tv[2 * q]);
                            }
                        }
                    }
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        if ((mask >> t) & 1) {                       // wave-uniform
                            T old[2];
                            int at[2];
#pragma unroll
                            for (int jj = 0; jj < 2; ++jj) {
                                if (FULL && !BANDED) {
                                    at[jj] = gw_off + pos[jj] + to[t];
                                } else {
                                    bool mine = live[jp + jj];
                                    if (BANDED) mine = mine && ((uint32_t)(pos[jj] - img0 + tr_[t]) - own_lo) < own_len;
                                    at[jj] = mine ? gw_off + pos[jj] + to[t] : dummy_off;
                                }
                            }
#pragma unroll
                            for (int jj = 0; jj < 2; ++jj) old[jj] = xs[at[jj]];
#pragma unroll
                            for (int jj = 0; jj < 2; ++jj) xs[at[jj]] = old[jj] + gt[jj][t];
                        }
                    }
                }
                cur = nxt;
            }
        }
    }
    __syncthreads();
    // write the owned rows of the gradient planes back
    const int orows = bd.r1 - bd.r0;
    T *dstg = gx + (int64_t)blockIdx.z * p.part_stride + (int64_t)n0 * g.cin * g.h * g.w;
    for (int pr = wave; pr < planes * orows; pr += p.NW) {
        const int plane = uniform(pr / orows), iy = bd.r0 + (pr - plane * orows);
        const T *row = gs + plane * chs + (iy + g.ph - bd.R0) * p.rs + g.pw;
        T *dst = dstg + ((int64_t)plane * g.h + iy) * g.w;
        for (int ix = lane; ix < g.w; ix += kWave) {
            T v = row[ix];
            for (int k = 1; k < hsw; ++k) v += row[k * xe4 + ix];
            dst[ix] = v;
        }
    }
}

// Input gradient without an LDS copy of the input: for blocks whose sample images are too large for LDS,
// or so small that one sample leaves most of a wavefront idle.  A wavefront owns the gradient planes of
// one input channel for G consecutive samples (lanes = (sample, pooled cell)), keeps only those planes in
// LDS (same shared-halo layout, private to the wavefront, so the kernel has no barriers) and reads the
// taps from a zero-padded copy of x in global memory, which the L2 serves.  Same walk as the tiled
// kernel: kernels that read the channel in increasing order, taps in order, read-add-write per tap.
// What a launch of 8192 owners costs (wall-clock stamps per wavefront at [256,128,8,8] -> 512 and [256,32,16,16] -> 128):
// 106 scalar registers leave 6 wavefronts per SIMD, so 6144 owners start at once and the last 2048 between 12 and 18 us;
// a hit takes 1.2-1.8 us of a wavefront's life (about 620 clocks issuing the ten gathers of the hits ahead, 520 waiting,
// 1240 in the tree and the read-add-write rounds, with five or six wavefronts sharing the SIMD), a list 4 to 16 hits.
// Measured without gain on that: hit records through LDS instead of the scalar cache, the owner's own channel from an
// LDS copy (half the gathers), five hits in flight instead of three, register budgets for 7 and 8 wavefronts per SIMD,
// wavefront priority by list length, longest lists first.
template <typename T>
__global__ __launch_bounds__(256) void convblock_backward_x_direct_kernel(const T *__restrict__ gy, const T *__restrict__ xp,
                                                                        const T *__restrict__ folded,
                                                                        const int32_t *__restrict__ count,
                                                                        const int32_t *__restrict__ hits,
                                                                        const int32_t *__restrict__ taps,
                                                                        const uint8_t *__restrict__ argmax, T *__restrict__ gx,
                                                                        Geom g, TilePlan p, int sample_elems)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    const int groups = (g.n + p.G - 1) / p.G;
    // channel fastest: a workgroup shares its samples, and so do its neighbours on the same XCD (they read the same
    // padded images through one L2)
    const int item = uniform((int)xcd_contiguous_block(blockIdx.x, gridDim.x) * p.NW + wave);
    if (item >= groups * g.cin) return;
    const int grp = item / g.cin, ch = item - grp * g.cin;
    const int n0 = grp * p.G, g_here = min(p.G, g.n - n0);
    const int wp = g.wo >> 1, I = p.slots;
    T *gs = reinterpret_cast<T *>(smem) + wave * (p.xe + kWave);       // G planes + tail, then one sink element per lane
    const int dummy = p.xe + lane;
    for (int i = lane; i < p.xe + kWave; i += kWave) gs[i] = T(0);

    const int v_here = g_here * I;
    const int nhits = count[2 * ch];
    const int32_t *hit = hits + count[2 * ch + 1];
    const int64_t gbase = (int64_t)n0 * g.c * I;
    const int row_step = g.sh * p.rs;
    for (int blk = 0; blk * kWave < v_here; ++blk) {
        const int v = blk * kWave + lane;
        const bool live = v < v_here;
        uint32_t cl = live ? v : 0;
        const uint32_t sm = fdiv(cl, p.d_slots);
        cl -= sm * (uint32_t)I;
        const uint32_t py = fdiv(cl, p.d_wp), px = cl - py * (uint32_t)wp;
        const int rel = (int)((2 * py * g.sh) * p.rs + 2 * px * g.sw);
        const int gp = (int)((n0 + sm) * (uint32_t)sample_elems) + rel;
        const int lp = (int)(sm * p.chs) + rel;
        const int cy = (int)((sm * g.c) * I + cl);
        // three hits in flight: grad_y / arg-max of hit k+2 and the taps of hit k+1 (which need the arg-max
        // loaded one step earlier) are requested before hit k is computed
        auto load_cell = [&](int k, int &code, T &gout) {
            const int64_t crow = gbase + (int64_t)(hit[k] & 0xFFFF) * I;
            code = 0;
            gout = T(0);
            if (live) {
                code = argmax[crow + cy];
                gout = gy[crow + cy];
            }
        };
        auto load_taps = [&](int k, int code, int &off, T (&tv)[8]) {
            const int c = hit[k] & 0xFFFF;
            off = (code >> 1) * row_step + (code & 1) * g.sw;
#pragma unroll
            for (int t = 0; t < 8; ++t) tv[t] = load_at(xp, (uint32_t)(gp + off + taps[c * 16 + t]));
        };
        int code1 = 0, code2 = 0, off0 = 0, off1 = 0;
        T gy0 = T(0), gy1 = T(0), gy2 = T(0);
        T tv0[8], tv1[8];
        if (nhits > 0) {
            load_cell(0, code1, gy0);
            load_taps(0, code1, off0, tv0);
        }
        if (nhits > 1) load_cell(1, code1, gy1);
        for (int k = 0; k < nhits; ++k) {
            if (k + 2 < nhits) load_cell(k + 2, code2, gy2);
            if (k + 1 < nhits) load_taps(k + 1, code1, off1, tv1);
            const int ent = hit[k];
            const int c = ent & 0xFFFF, mask = (ent >> 16) & 0xFF;
            int tr_[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) tr_[t] = taps[c * 16 + 8 + t];
            Tree<T> tr;
            const T *fc = folded + (int64_t)c * 28;
#pragma unroll
            for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
            const TreeVals<T> tvv = eval_tree(tr, tv0);
            const T g_m0 = gy0 * gate_da(tr.g[6], tvv.mid[1]);
            const T g_m1 = gy0 * gate_db(tr.g[6], tvv.mid[0]);
            T gt[8];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if ((mask >> (2 * q)) & 3) {                         // wave-uniform: a tap of this leaf is ours
                    const int m = q >> 1;
                    const T g_mid = m ? g_m1 : g_m0;
                    const T g_leaf = g_mid * ((q & 1) ? gate_db(tr.g[4 + m], tvv.leaf[q ^ 1]) : gate_da(tr.g[4 + m], tvv.leaf[q ^ 1]));
                    gt[2 * q] = g_leaf * gate_da(tr.g[q], tv0[2 * q + 1]);
                    gt[2 * q + 1] = g_leaf * gate_db(tr.g[q], tv0[2 * q]);
                }
            }
            // for one tap the targets of all lanes are distinct elements; taps are applied one after the other
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                if ((mask >> t) & 1) {                               // wave-uniform
                    const int at = live ? lp + off0 + tr_[t] : dummy;
                    gs[at] = gs[at] + gt[t];
                }
            }
            off0 = off1;
            gy0 = gy1;
            gy1 = gy2;
            code1 = code2;
#pragma unroll
            for (int t = 0; t < 8; ++t) tv0[t] = tv1[t];
        }
    }
    // interior of the G planes -> gx
    const int hw = g.h * g.w;
    for (int e = lane; e < g_here * hw; e += kWave) {
        const uint32_t sm = fdiv((uint32_t)e, p.d_hw), rem = (uint32_t)e - sm * (uint32_t)hw;
        const uint32_t iy = fdiv(rem, p.d_w), ix = rem - iy * (uint32_t)g.w;
        gx[((int64_t)(n0 + sm) * g.cin + ch) * hw + rem] = gs[sm * p.chs + (iy + g.ph) * p.rs + ix + g.pw];
    }
}

// gx = ((part[0] + part[1]) + part[2]) + ... : partial gradient images of a split hit list, fixed order
template <typename T>
__global__ __launch_bounds__(256) void sum_partial_images_kernel(const T *__restrict__ part, T *__restrict__ gx, int64_t total, int hs)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    T acc = part[e];
    for (int k = 1; k < hs; ++k) acc += part[(int64_t)k * total + e];
    gx[e] = acc;
}

// ---------------------------------------------------------------------------------------------
// weight gradient
// ---------------------------------------------------------------------------------------------
// Kernel-major with plenty of small workgroups: blockIdx.y = kernel (coefficients and tap offsets are
// scalar), threads run over (sample, pooled cell) and keep the 28 sums (7 gates x (ab, a, b, 1)) in
// registers across all their cells; one block reduction per workgroup, partial [c][blocks][28], summed in
// order by reduce_coef_partials.  Taps come from a zero-padded copy of x in global memory (written once
// per call into scratch, same shared-halo layout as the LDS images), so the loop has no bounds checks
// and 32-bit offsets only.
// FIXED: the pooled cells of a sample divide the 256 threads (I = 1, 2, 4 ... 256), so a thread keeps its cell and walks
// over samples only: cell decoding and the cell part of every offset leave the loop, and 32-bit offsets suffice (the plan
// checks the sizes).
template <typename T, bool FIXED>
__global__ __launch_bounds__(256) void convblock_backward_w_padded_kernel(const T *__restrict__ gy, const T *__restrict__ xp,
                                                                        const T *__restrict__ folded,
                                                                        const int32_t *__restrict__ taps,
                                                                        const uint8_t *__restrict__ argmax,
                                                                        T *__restrict__ partial, Geom g, TilePlan p,
                                                                        FastDiv d_cells, int sample_elems, int tap_stride)
{
    // Workgroups that read the same samples (one sample block, every kernel) take consecutive logical numbers, so they run
    // on one XCD and share its L2 (the hardware deals workgroups to the 8 XCDs round-robin over x + gridDim.x * y).
    const int nb = gridDim.x;
    const unsigned logical = xcd_contiguous_block(blockIdx.x + (unsigned)nb * blockIdx.y, (unsigned)nb * gridDim.y);
    const int c = uniform((int)(logical % gridDim.y));
    const uint32_t bx = uniform((int)(logical / gridDim.y));        // sample block
    const int wp = g.wo >> 1, I = (g.ho >> 1) * wp;
    const uint32_t items = (uint32_t)g.n * I;
    Tree<T> tr;
    const T *fc = folded + (int64_t)c * 28;
#pragma unroll
    for (int q = 0; q < 7; ++q) tr.g[q] = Coef<T>{fc[4 * q], fc[4 * q + 1], fc[4 * q + 2], fc[4 * q + 3]};
    int to[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) to[t] = taps[c * tap_stride + t];   // [c][8], or the first 8 of the input gradient's [c][16]
    const int row_step = g.sh * p.rs;
    const int64_t kernel_row = (int64_t)c * I;
    const int64_t sample_cells = (int64_t)g.c * I;
    T acc[28];
#pragma unroll
    for (int k = 0; k < 28; ++k) acc[k] = T(0);
    // FIXED: this thread's cell, its first sample and the samples it skips per step
    const uint32_t per_block = FIXED ? 256u / (uint32_t)I : 1u;
    const uint32_t f_cell = FIXED ? threadIdx.x % (uint32_t)I : 0u;
    const uint32_t f_py = fdiv(f_cell, p.d_wp), f_px = f_cell - f_py * (uint32_t)wp;
    const uint32_t f_pos = (2 * f_py) * row_step + (2 * f_px) * g.sw;
    const uint32_t f_out = (uint32_t)(kernel_row + f_cell);
    const uint32_t f_n0 = bx * per_block + threadIdx.x / (uint32_t)I, f_step = (uint32_t)nb * per_block;
    // tree, upstream gradients and the 28 sums of one pooled cell
    auto accumulate = [&](const T (&tv)[8], T gout) {
        const TreeVals<T> v = eval_tree(tr, tv);
        T gin[7][2], gg[7];
        gg[6] = gout;
        gin[6][0] = v.mid[0];
        gin[6][1] = v.mid[1];
        gg[4] = gout * gate_da(tr.g[6], v.mid[1]);
        gg[5] = gout * gate_db(tr.g[6], v.mid[0]);
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            gin[4 + m][0] = v.leaf[2 * m];
            gin[4 + m][1] = v.leaf[2 * m + 1];
            gg[2 * m] = gg[4 + m] * gate_da(tr.g[4 + m], v.leaf[2 * m + 1]);
            gg[2 * m + 1] = gg[4 + m] * gate_db(tr.g[4 + m], v.leaf[2 * m]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            gin[q][0] = tv[2 * q];
            gin[q][1] = tv[2 * q + 1];
        }
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            acc[4 * k + 0] = fma_t(gg[k], gin[k][0] * gin[k][1], acc[4 * k + 0]);
            acc[4 * k + 1] = fma_t(gg[k], gin[k][0], acc[4 * k + 1]);
            acc[4 * k + 2] = fma_t(gg[k], gin[k][1], acc[4 * k + 2]);
            acc[4 * k + 3] += gg[k];
        }
    };
    if (FIXED) {
        for (uint32_t it = f_n0; it < (uint32_t)g.n; it += f_step) {
            const uint32_t o = it * (uint32_t)sample_cells + f_out;
            const int code = load_at(argmax, o);
            const T gout = load_at(gy, o);
            const int pos = (int)(it * (uint32_t)sample_elems + f_pos) + (code >> 1) * row_step + (code & 1) * g.sw;
            T tv[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) tv[t] = load_at(xp, (uint32_t)(pos + to[t]));
            accumulate(tv, gout);
        }
    } else {
        for (uint32_t it = bx * 256 + threadIdx.x; it < items; it += (uint32_t)nb * 256) {
            const uint32_t n = fdiv(it, d_cells), cell = it - n * (uint32_t)I;
            const uint32_t py = fdiv(cell, p.d_wp), px = cell - py * (uint32_t)wp;
            const int64_t o = (int64_t)n * sample_cells + kernel_row + cell;
            const int code = argmax[o];
            const T gout = gy[o];
            const int pos = (int)(n * (uint32_t)sample_elems) + (int)((2 * py + (code >> 1)) * row_step + (2 * px + (code & 1)) * g.sw);
            T tv[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) tv[t] = load_at(xp, (uint32_t)(pos + to[t]));
            accumulate(tv, gout);
        }
    }
    block_sum_store<T, 28, 256>(acc, partial + ((int64_t)c * nb + bx) * 28);
}


// Weight gradient with the input images staged in LDS (the layout of the forward kernel): for blocks whose sample
// images fit LDS.  A workgroup owns 16 kernels (one per wavefront, for its whole life) and a run of `rounds` groups
// of S samples, which it stages one after the other; a wavefront walks the pooled cells of the staged samples
// (lanes = cells), recomputes the tree at the arg-max position from LDS and keeps its kernel's 28 sums (7 gates x
// (ab, a, b, 1)) in registers over all rounds, so the 64-lane reduction of the sums happens once per wavefront.
// The next group's image travels through registers while the current one is evaluated (at most kStagePerThread
// elements per thread, LDS positions computed once).  Folded coefficients and tap offsets are made by the wavefront
// itself from w and the selection: no set-up launch, no padded copy of x, every x element is read once per 16 kernels.
// partial [c][partial sums per kernel][28], added in order by reduce_coef_partials_kernel.  (Letting the wavefront that
// finishes a kernel last add them itself needs a device-wide release / acquire per wavefront, which on this multi-die
// part writes the L2 back every time: 65 -> 160 us at [256,9,32,32] -> 256.)
constexpr int kStagePerThread = 9;
constexpr int kTiledWWaves = 16;
constexpr int kTiledWMaxParts = 256;   // partial sums per kernel the scratch buffer holds
template <typename T, int V>
__global__ __launch_bounds__(kTiledWWaves * kWave) void convblock_backward_w_tiled_kernel(
    const T *__restrict__ gy, const T *__restrict__ x, const T *__restrict__ w, const int32_t *__restrict__ sel,
    const uint8_t *__restrict__ argmax, T *__restrict__ partial, Geom g, TilePlan p, int rounds)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    const int tid = threadIdx.x;
    constexpr int nthreads = kTiledWWaves * kWave;
    const int lane = tid & (kWave - 1), wave = uniform(tid >> 6);
    // p.CT kernels per workgroup; the 16 / p.CT wavefronts of a kernel take every (16 / p.CT)-th block of cells
    const int slices = kTiledWWaves / p.CT, slice = wave / p.CT;
    const int c = uniform((int)blockIdx.y * p.CT + wave % p.CT);
    const bool has_kernel = c < g.c;
    const int cc = has_kernel ? c : g.c - 1;
    const int wp = g.wo >> 1, I = (g.ho >> 1) * wp;
    const int hw = g.h * g.w;
    // this wavefront's kernel: folded coefficients and tap offsets in the LDS image
    const Tree<T> tr = load_tree(w + (int64_t)cc * 7 * 16);
    int to[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const Tap tp = unpack_tap(sel[(int64_t)cc * 8 + t], tap_limit(g));
        to[t] = uniform(tp.ch * p.chs + tp.ry * p.rs + tp.rx);
    }
    T acc[28];
#pragma unroll
    for (int k = 0; k < 28; ++k) acc[k] = T(0);
    auto accumulate = [&](const T (&tv)[8], T gout) {
        const TreeVals<T> v = eval_tree(tr, tv);
        T gin[7][2], gg[7];
        gg[6] = gout;
        gin[6][0] = v.mid[0];
        gin[6][1] = v.mid[1];
        gg[4] = gout * gate_da(tr.g[6], v.mid[1]);
        gg[5] = gout * gate_db(tr.g[6], v.mid[0]);
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            gin[4 + m][0] = v.leaf[2 * m];
            gin[4 + m][1] = v.leaf[2 * m + 1];
            gg[2 * m] = gg[4 + m] * gate_da(tr.g[4 + m], v.leaf[2 * m + 1]);
            gg[2 * m + 1] = gg[4 + m] * gate_db(tr.g[4 + m], v.leaf[2 * m]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            gin[q][0] = tv[2 * q];
            gin[q][1] = tv[2 * q + 1];
        }
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            acc[4 * k + 0] = fma_t(gg[k], gin[k][0] * gin[k][1], acc[4 * k + 0]);
            acc[4 * k + 1] = fma_t(gg[k], gin[k][0], acc[4 * k + 1]);
            acc[4 * k + 2] = fma_t(gg[k], gin[k][1], acc[4 * k + 2]);
            acc[4 * k + 3] += gg[k];
        }
    };
    // rowbase[r]: LDS position of image row r = (sample, channel, iy) of a staged group (built once)
    int *rowbase = reinterpret_cast<int *>(xs + ((p.xe + 3) & ~3));
    const uint32_t group_rows = (uint32_t)(p.S * g.cin * g.h), group_elems = group_rows * (uint32_t)g.w;
    for (uint32_t r = tid; r < group_rows; r += nthreads) {
        const uint32_t plane = fdiv(r, p.d_planes), iy = r - plane * (uint32_t)g.h;   // d_planes: division by h here
        rowbase[r] = (int)(plane * p.chs + (iy + g.ph) * p.rs + g.pw);
    }
    T stage[kStagePerThread];
    auto fetch = [&](int round) {                                     // image elements of a round's samples -> registers
        const int n0 = ((int)blockIdx.x * rounds + round) * p.S;
        const int s_here = n0 < g.n ? min(p.S, g.n - n0) : 0;
        const uint32_t total = (uint32_t)(s_here * g.cin) * (uint32_t)hw;
        const T *src = x + (int64_t)n0 * g.cin * hw;
#pragma unroll
        for (int k = 0; k < kStagePerThread; ++k) {
            const uint32_t e = tid + k * nthreads;
            stage[k] = T(0);
            if (e < total) stage[k] = src[e];
        }
    };
    // A lane takes V consecutive cells of a pooled row (V divides the row length), so one vector load brings the grad_y
    // of V visits and one V-byte load their arg-max codes; the loads of the next group are in flight while the current
    // one is evaluated, across round boundaries too (the kernel streams grad_y / arg-max from HBM).
    struct Group {
        T gout[V];
        uint32_t codes;
        int pos;
    };
    auto issue = [&](int round, int sb, Group &q) {
        const int n0 = ((int)blockIdx.x * rounds + round) * p.S;
        const int U = min(p.S, g.n - n0) * I;
        const int u = (sb * kWave + lane) * V;
        const uint32_t uu = u < U ? u : 0;
        const uint32_t sm = fdiv(uu, p.d_slots), cl = uu - sm * (uint32_t)I;
        const uint32_t py = fdiv(cl, p.d_wp), px = cl - py * (uint32_t)wp;
        q.pos = (int)(sm * g.cin * p.chs + (2 * py * g.sh) * p.rs + 2 * px * g.sw);
        q.codes = 0;
#pragma unroll
        for (int k = 0; k < V; ++k) q.gout[k] = T(0);
        if (u < U) {
            const int64_t o = ((int64_t)(n0 + sm) * g.c + c) * I + cl;
            const T *gp = gy + o;
            const uint8_t *ap = argmax + o;
            if constexpr (V == 4) {
                q.codes = *reinterpret_cast<const uint32_t *>(ap);
                if constexpr (sizeof(T) == 4) {
                    const float4 v = *reinterpret_cast<const float4 *>(gp);
                    q.gout[0] = v.x, q.gout[1] = v.y, q.gout[2] = v.z, q.gout[3] = v.w;
                } else {
                    const double2 v0 = *reinterpret_cast<const double2 *>(gp), v1 = *reinterpret_cast<const double2 *>(gp + 2);
                    q.gout[0] = v0.x, q.gout[1] = v0.y, q.gout[2] = v1.x, q.gout[3] = v1.y;
                }
            } else if constexpr (V == 2) {
                q.codes = *reinterpret_cast<const uint16_t *>(ap);
                if constexpr (sizeof(T) == 4) {
                    const float2 v = *reinterpret_cast<const float2 *>(gp);
                    q.gout[0] = v.x, q.gout[1] = v.y;
                } else {
                    const double2 v = *reinterpret_cast<const double2 *>(gp);
                    q.gout[0] = v.x, q.gout[1] = v.y;
                }
            } else {
                q.codes = *ap;
                q.gout[0] = *gp;
            }
        }
    };
    Group cur, nxt;
    bool have_cur = false;
    for (int i = tid; i < p.xe; i += nthreads) xs[i] = T(0);          // halos stay zero over all rounds
    fetch(0);
    const int row_step = g.sh * p.rs;
    for (int round = 0; round < rounds; ++round) {
        const int n0 = ((int)blockIdx.x * rounds + round) * p.S;
        if (n0 >= g.n) break;                                        // uniform over the workgroup
        const int s_cur = min(p.S, g.n - n0);
        __syncthreads();                                             // the previous round's reads (or the zero fill) are done
        // (the LDS positions below are the same in every round; computed afresh so that they do not sit in -- or spill
        // from -- nine registers while the round is evaluated)
        uint32_t e0 = tid;
        asm volatile("" : "+v"(e0));
#pragma unroll
        for (int k = 0; k < kStagePerThread; ++k) {
            const uint32_t e = e0 + k * nthreads;
            if (e < group_elems) {
                const uint32_t r = fdiv(e, p.d_w);
                xs[rowbase[r] + (int)(e - r * (uint32_t)g.w)] = stage[k];
            }
        }
        __syncthreads();
        if (round + 1 < rounds) fetch(round + 1);                    // in flight while this round is evaluated
        if (!has_kernel) continue;
        const int nsb = (s_cur * I + kWave * V - 1) / (kWave * V);
        if (!have_cur && slice < nsb) issue(round, slice, cur);
        for (int sb = slice; sb < nsb; sb += slices) {
            // the next group of V visits: of this round, or the first one of the next round (its loads cross the barriers)
            if (sb + slices < nsb) {
                issue(round, sb + slices, nxt);
            } else {
                const int n1 = ((int)blockIdx.x * rounds + round + 1) * p.S;
                have_cur = round + 1 < rounds && n1 < g.n && slice * kWave * V < min(p.S, g.n - n1) * I;
                if (have_cur) issue(round + 1, slice, nxt);
            }
#pragma unroll
            for (int k = 0; k < V; ++k) {
                const int code = (int)(cur.codes >> (8 * k)) & 3;
                const int here = cur.pos + 2 * k * g.sw + (code >> 1) * row_step + (code & 1) * g.sw;
                T tv[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) tv[t] = xs[here + to[t]];
                accumulate(tv, cur.gout[k]);                         // lanes without a cell carry a zero gradient
            }
            cur = nxt;
        }
    }
    if (!has_kernel) return;                                          // no workgroup barrier below
    const int nb = gridDim.x * slices;                                // partial sums per kernel
    T mine = T(0);                                                    // lane k < 28 ends up with total k
#pragma unroll
    for (int k = 0; k < 28; ++k) {
        const T s = wave_sum(acc[k]);
        mine = lane == k ? s : mine;
    }
    T *my_partial = partial + ((int64_t)c * nb + blockIdx.x * slices + slice) * 28;
    if (lane < 28) my_partial[lane] = mine;
}

// ---------------------------------------------------------------------------------------------
// plans
// ---------------------------------------------------------------------------------------------
bool plan_backward_x(const Geom &g, int elem, TilePlan *p)
{
    if (!taps_inside(g) || g.c > 65535) return false;
    plan_common(g, p);
    const int I = (g.ho / 2) * (g.wo / 2);
    p->slots = I;
    p->CT = 0;
    p->d_slots = make_fastdiv((uint32_t)I);
    p->NW = g.cin < 16 ? g.cin : 16;
    // two windows (input, gradient); a sink region of one element per thread unless halo elements serve
    auto size_for = [&](int G, int band_rows, int *rows_max, int *cb_max) {
        const int bands = (int)clg_ceil_div(g.h, band_rows);
        *rows_max = 0;
        *cb_max = 0;
        for (int b = 0; b < bands; ++b) {
            const Band bd = make_band(g, b, band_rows);
            if (bd.rows > *rows_max) *rows_max = bd.rows;
            if (bd.cb > *cb_max) *cb_max = bd.cb;
        }
        const int64_t xe = (int64_t)G * g.cin * *rows_max * p->rs + g.pw;
        const bool halo_sink = bands == 1 && g.ph >= 1 && p->rs >= 32;
        return (int64_t)2 * ((xe + 3) & ~3) * elem + (halo_sink ? 0 : (int64_t)p->NW * kWave * elem);
    };
    // samples sharing a wavefront pass when a sample has fewer than 64 cells (whole image, one band)
    int G = I >= kWave ? 1 : kWave / I;
    if (G > g.n) G = g.n;
    int rows_max, cb_max;
    while (G > 1 && size_for(G, g.h, &rows_max, &cb_max) > kLdsLimit) G /= 2;
    int band_rows = g.h;
    if (G == 1) {
        // One band (the whole image) unless it does not fit: the time of this kernel is set by the
        // dependent chain of steps per visited kernel, which every band would repeat (measured: bands
        // never paid off, not even at 256 wavefronts in flight).  CLG_BWDX_BANDS overrides for tuning.
        const char *e_b = clg_knob(K_BWDX_BANDS);
        int64_t want = e_b ? atoi(e_b) : 1;
        if (want > g.h / 4) want = g.h / 4;
        if (want < 1) want = 1;
        band_rows = (int)clg_ceil_div(g.h, want);
        // whole images that do not fit are split further until a band window fits
        while (band_rows > 1 && size_for(1, band_rows, &rows_max, &cb_max) > kLdsLimit) band_rows = (band_rows + 1) / 2;
    }
    const int64_t bytes = size_for(G, band_rows, &rows_max, &cb_max);
    if (bytes > kLdsLimit) return false;
    p->G = G;
    p->S = G;
    p->band_rows = band_rows;
    p->bands = (int)clg_ceil_div(g.h, band_rows);
    p->chs = rows_max * p->rs;
    p->xe = (int)((int64_t)G * g.cin * p->chs + g.pw);
    p->dummy_in_halo = (p->bands == 1 && g.ph >= 1 && p->rs >= 32) ? 1 : 0;
    if (p->bands > 65535) return false;
    if (G * I < kWave / 5 && p->bands == 1) return false;            // almost empty wavefronts: gather kernel instead
    // Few input channels leave most of the 16 wavefront slots of a workgroup empty: then several wavefronts
    // share each gradient plane, every one with its own copy of the gradient window (at least two kernels per
    // wavefront, windows within 96 KiB so that a second workgroup still fits on the CU).
    const int64_t avg_hits = g.cin == 1 ? g.c : (2 * (int64_t)g.c) / g.cin;
    const int64_t window = (int64_t)((p->xe + 3) & ~3) * elem;
    int64_t hsw = 16 / g.cin;
    if (const char *e = clg_knob(K_BWDX_HSW)) hsw = atoi(e);
    if (hsw > avg_hits / 2) hsw = avg_hits / 2;
    while (hsw > 1 && (1 + hsw) * window > 96 * 1024) --hsw;
    if (hsw < 1 || p->bands > 1) hsw = 1;
    p->hsw = (int)hsw;
    p->NW = (int)(g.cin * hsw < 16 ? g.cin * hsw : 16);
    const int64_t bytes_all = (1 + hsw) * window + (p->dummy_in_halo ? 0 : (int64_t)p->NW * kWave * elem);
    if (bytes_all > kLdsLimit) return false;
    p->lds_bytes = (size_t)bytes_all;
    // hit split: when (sample groups x bands) leave room for more resident workgroups, several workgroups
    // share the kernels of one image; each handles every HS-th kernel and writes a partial image
    int64_t per_cu = kLdsLimit / (int64_t)(bytes_all > 1024 ? bytes_all : 1024);
    if (per_cu > 20 / p->NW) per_cu = 20 / p->NW;                    // about 80 VGPRs per lane: 5 wavefronts per SIMD
    if (per_cu < 1) per_cu = 1;
    const int64_t wgs = clg_ceil_div(g.n, p->S) * p->bands;
    const char *e_hs = clg_knob(K_BWDX_SPLIT);
    int64_t hs = e_hs ? atoi(e_hs) : (256 * per_cu) / wgs;
    if (hs > kMaxHitSplit) hs = kMaxHitSplit;
    // every split workgroup stages the image and writes a partial image: worth it only with at least
    // about 4 kernels left per channel list (a kernel reads at most two channels)
    if (!e_hs && hs > avg_hits / (4 * hsw)) hs = avg_hits / (4 * hsw);
    if (hs < 1) hs = 1;
    p->hit_split = (int)hs;
    p->part_stride = hs > 1 ? (int64_t)g.n * g.cin * g.h * g.w : 0;
    return (int64_t)p->S * g.cin * p->chs < (1ll << 30) && (int64_t)p->S * g.c * I < (1ll << 31);
}

// Plan of the input-gradient kernel that reads taps from a padded global copy of x.
bool plan_backward_x_direct(const Geom &g, int elem, TilePlan *p, int *sample_elems)
{
    if (!taps_inside(g) || g.c > 65535) return false;
    plan_common(g, p);
    const int I = (g.ho / 2) * (g.wo / 2);
    if (I < 1) return false;
    p->slots = I;
    p->CT = 0;
    p->d_slots = make_fastdiv((uint32_t)I);
    int G = I >= kWave ? 1 : kWave / I;
    if (G > g.n) G = g.n;
    p->G = G;
    p->S = G;
    p->bands = 1;
    p->band_rows = g.h;
    p->hit_split = 1;
    p->hsw = 1;
    p->part_stride = 0;
    p->dummy_in_halo = 0;
    p->xe = (int)(((int64_t)G * p->chs + g.ph * p->rs + g.pw + 3) & ~3ll);
    int nw = 4;
    while (nw > 1 && (int64_t)nw * (p->xe + kWave) * elem > 64 * 1024) nw /= 2;
    p->NW = nw;
    p->lds_bytes = (size_t)nw * (p->xe + kWave) * elem;
    if (p->lds_bytes > (size_t)kLdsLimit) return false;
    const int64_t se = (int64_t)g.cin * p->chs + g.ph * p->rs + g.pw;
    if (se * g.n * elem >= (1ll << 32) || (int64_t)G * g.c * I >= (1ll << 31)) return false;
    if (clg_ceil_div(clg_ceil_div(g.n, G) * g.cin, nw) >= (1ll << 31)) return false;
    *sample_elems = (int)se;
    return true;
}

enum BwdXMode { kBwdXGather = 0, kBwdXTiled = 1, kBwdXDirect = 2 };

// Tiled (input image in LDS) when a wavefront pass is reasonably full there; the direct kernel when the
// image does not fit or fills at least twice as many lanes; the per-element gather for everything else.
BwdXMode choose_backward_x(const Geom &g, int elem, TilePlan *p, int *sample_elems)
{
    TilePlan pt, pd;
    int se = 0;
    const bool tiled = plan_backward_x(g, elem, &pt);
    const bool direct = plan_backward_x_direct(g, elem, &pd, &se);
    const int I = (g.ho / 2) * (g.wo / 2);
    auto lanes = [&](const TilePlan &q) { return q.G * I < kWave ? q.G * I : kWave; };
    // The direct kernel has one independent wavefront per (sample group, channel) and no barriers: it also wins
    // when there are thousands of such owners with short kernel lists (48 vs 88 us at [256,32,16,16] -> 128,
    // 74 vs 164 us at [256,64,16,16] -> 256; few channels with long lists stay tiled: 141 vs 248 us at C4).
    const int64_t owners = clg_ceil_div(g.n, pd.G) * g.cin, avg_hits = (2 * (int64_t)g.c) / g.cin;
    bool use_direct = direct && (!tiled || lanes(pd) >= 2 * lanes(pt) || (owners >= 4096 && avg_hits <= 16));
    if (const char *e = clg_knob(K_BWDX_DIRECT)) use_direct = direct && (atoi(e) != 0 || !tiled);
    if (use_direct) {
        *p = pd;
        *sample_elems = se;
        return kBwdXDirect;
    }
    if (tiled) {
        *p = pt;
        return kBwdXTiled;
    }
    return kBwdXGather;
}

size_t bwd_x_direct_xp_off(const BwdScratch &lay) { return (lay.total + 255) & ~(size_t)255; }

// weight gradient from the padded copy: scratch = partials | folded | taps | padded x
struct WScratch {
    int nb, sample_elems;
    size_t folded_off, taps_off, xp_off, total;
};
// The padded weight-gradient kernel keeps a thread on one pooled cell when the cells of a sample divide its 256 threads
// and grad_y / arg-max can be addressed with 32-bit byte offsets.
// Pooled cells a thread of the padded weight-gradient kernel sums before the block reduction (28 wavefront sums per
// block): 16 when a kernel has at least 64 Ki cells (89 vs 92 us at [256,9,32,32] -> 256), else 8 (25.5 vs 29 us at
// [256,32,16,16] -> 128, where more would leave too few workgroups).
int cells_per_thread(int64_t cells_per_kernel)
{
    if (const char *e = clg_knob(K_BWDW_CELLS)) return atoi(e) > 0 ? atoi(e) : 8;
    return cells_per_kernel >= 65536 ? 16 : 8;
}
bool fixed_cells(const Geom &g, int elem)
{
    const int64_t I = (int64_t)(g.ho / 2) * (g.wo / 2);
    return I <= 256 && 256 % I == 0 && (int64_t)g.n * g.c * I * elem < (1ll << 32);
}
bool plan_backward_w(const Geom &g, int elem, TilePlan *p, WScratch *ws)
{
    if (!taps_inside(g) || g.c > 65535) return false;
    plan_common(g, p);
    const int64_t I = (int64_t)(g.ho / 2) * (g.wo / 2);
    // the padded copy costs two extra launches: it pays from about 8M pooled values (measured 102 vs 124 us
    // at 16.8M, 30 vs 27 us at 1.6M)
    if ((int64_t)g.n * g.c * I < (8ll << 20) && !clg_knob(K_BWDW_PADDED)) return false;
    const int64_t sample_elems = (int64_t)g.cin * p->chs + g.ph * p->rs + g.pw;
    // the copy may be made by the tiled input gradient of the same call, whose planes keep both halo rows
    const int64_t sample_elems_max = (int64_t)g.cin * (g.h + 2 * g.ph) * p->rs + g.ph * p->rs + g.pw;
    if (sample_elems_max * g.n * elem >= (1ll << 32) || I * g.n >= (1ll << 31)) return false;
    p->d_slots = make_fastdiv((uint32_t)p->chs);                    // reused as "divide by plane stride"
    ws->sample_elems = (int)sample_elems;
    int64_t nb = clg_ceil_div(I * g.n, 256 * cells_per_thread(I * g.n));
    ws->nb = (int)(nb < 1 ? 1 : (nb > 64 ? 64 : nb));
    ws->folded_off = ((size_t)g.c * 64 * 28 * elem + 255) & ~(size_t)255;   // partials sized for 64 blocks
    ws->taps_off = (ws->folded_off + (size_t)g.c * 28 * elem + 255) & ~(size_t)255;
    ws->xp_off = (ws->taps_off + (size_t)g.c * 8 * 4 + 255) & ~(size_t)255;
    ws->total = ws->xp_off + (size_t)sample_elems_max * g.n * elem;
    return true;
}

// folded coefficients, per-channel kernel lists and tap offsets (for LDS rows of rs, planes of chs elements)
// (and, in the same launch, a padded copy of x when `pad` names one)
template <typename T>
int launch_prepare(const Geom &g, const BwdScratch &lay, int rs, int chs, const void *w, const int32_t *sel, void *scratch,
                   hipStream_t st, const PadJob<T> &pad)
{
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    int32_t *count = reinterpret_cast<int32_t *>(base + lay.count_off), *hits = reinterpret_cast<int32_t *>(base + lay.hits_off);
    const int fold_blocks = (int)clg_ceil_div((int64_t)g.c * 8, 256), list_blocks = lay.csr ? 0 : (int)clg_ceil_div(g.cin, 4);
    hipLaunchKernelGGL(convblock_prepare_kernel<T>, dim3((unsigned)(fold_blocks + list_blocks) + pad_blocks(pad)), dim3(256), 0, st,
                       (const T *)w, sel, reinterpret_cast<T *>(base), count, lay.csr ? nullptr : hits,
                       reinterpret_cast<int32_t *>(base + lay.taps_off), g.c, g.cin, fold_blocks, rs, chs, pad, fold_blocks + list_blocks,
                       host_tap_limit(g));
    if (lay.csr) {
        int32_t *cursor = reinterpret_cast<int32_t *>(base + lay.cursor_off), *unsorted = reinterpret_cast<int32_t *>(base + lay.unsorted_off);
        const unsigned cb = (unsigned)clg_ceil_div(g.c, 256);
        hipLaunchKernelGGL(hits_zero_kernel, dim3((unsigned)clg_ceil_div(g.cin, 256)), dim3(256), 0, st, count, cursor, g.cin);
        hipLaunchKernelGGL(hits_count_kernel, dim3(cb), dim3(256), 0, st, sel, count, g.c, g.cin);
        hipLaunchKernelGGL(hits_scan_kernel, dim3(1), dim3(1024), 0, st, count, g.cin);
        hipLaunchKernelGGL(hits_fill_kernel, dim3(cb), dim3(256), 0, st, sel, (const int32_t *)count, cursor, unsorted, g.c, g.cin);
        hipLaunchKernelGGL(hits_sort_kernel, dim3((unsigned)clg_ceil_div(g.cin, 4)), dim3(256), 0, st, (const int32_t *)count,
                           (const int32_t *)unsorted, hits, g.cin);
    }
    CLG_CHECK_LAUNCH("clg_convblock_backward_x(prepare)");
    return CLG_OK;
}

// The tables of a per-layer plan (clg_convblock_plan): everything the gradient kernels need that depends only on the
// selection and the geometry -- per-channel kernel lists and tap offsets -- and optionally the coefficients the forward
// launch folded.
struct PlanView {
    const int32_t *count = nullptr, *hits = nullptr, *taps = nullptr;
    const void *folded = nullptr;
    const void *padded = nullptr;   // the zero-padded copy of x the forward call left (clg_convblock_forward_padded), or null
};
// Where the gradient kernels of a call find their tables: in the call's scratch (written by the set-up launch) or in a plan.
struct BwdTables {
    const void *folded = nullptr;
    const int32_t *count = nullptr, *hits = nullptr, *taps = nullptr;
};
// Sets a call's tables up.  Without a plan: one launch folds the coefficients, builds lists and tap offsets (and pads x
// when `pad` names a job).  With a plan only what changes per step is left: folding (unless the forward launch did it)
// and the padded copy -- no launch at all when neither is needed.
template <typename T>
int prepare_tables(const Geom &g, const BwdScratch &lay, int rs, int chs, const void *w, const int32_t *sel, void *scratch,
                   hipStream_t st, const PadJob<T> &pad, const PlanView *pv, BwdTables *tb)
{
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    if (pv == nullptr) {
        tb->folded = base;
        tb->count = reinterpret_cast<const int32_t *>(base + lay.count_off);
        tb->hits = reinterpret_cast<const int32_t *>(base + lay.hits_off);
        tb->taps = reinterpret_cast<const int32_t *>(base + lay.taps_off);
        return launch_prepare<T>(g, lay, rs, chs, w, sel, scratch, st, pad);
    }
    const bool fold = pv->folded == nullptr;
    tb->folded = fold ? (const void *)base : pv->folded;
    tb->count = pv->count, tb->hits = pv->hits, tb->taps = pv->taps;
    if (!fold && pad.total == 0) return CLG_OK;
    const unsigned prep = fold ? (unsigned)clg_ceil_div((int64_t)g.c * 7, 256) : 0u;
    hipLaunchKernelGGL((convblock_w_prepare_kernel<T, T>), dim3(prep + pad_blocks(pad)), dim3(256), 0, st, (const T *)w, sel,
                       fold ? reinterpret_cast<T *>(base) : (T *)nullptr, (int32_t *)nullptr, g.c, 0, 0, host_tap_limit(g), pad, (int)prep);
    CLG_CHECK_LAUNCH("clg_convblock_backward_planned(fold / pad)");
    return CLG_OK;
}

template <typename T>
int launch_backward_x_tiled(const Geom &g, const TilePlan &p, const void *gy, const void *x, const void *w, const int32_t *sel,
                            const uint8_t *argmax, void *gx, void *scratch, hipStream_t st, const PadJob<T> &pad,
                            const PlanView *pv = nullptr, BwdTables *tables_out = nullptr)
{
    const BwdScratch lay = bwd_scratch_layout(g, (int)sizeof(T), p.hit_split);
    BwdTables tb;
    if (int e = prepare_tables<T>(g, lay, p.rs, p.chs, w, sel, scratch, st, pad, pv, &tb)) return e;
    if (tables_out != nullptr) *tables_out = tb;
    const T *folded = reinterpret_cast<const T *>(tb.folded);
    const int32_t *count = tb.count, *hits = tb.hits, *taps = tb.taps;
    const dim3 grid((unsigned)clg_ceil_div(g.n, p.S), (unsigned)p.bands, (unsigned)p.hit_split), block(p.NW * kWave);
    T *part = reinterpret_cast<T *>(reinterpret_cast<unsigned char *>(scratch) + lay.part_off);
    T *out = p.hit_split > 1 ? part : (T *)gx;
#define CLG_BWDX_TILED(BANDED, SHARED, FULL)                                                                                    \
    do {                                                                                                                        \
        if (int e = allow_lds(convblock_backward_x_tiled_kernel<T, BANDED, SHARED, FULL>, p.lds_bytes, "clg_convblock_backward_x")) \
            return e;                                                                                                           \
        hipLaunchKernelGGL((convblock_backward_x_tiled_kernel<T, BANDED, SHARED, FULL>), grid, block, p.lds_bytes, st,          \
                           (const T *)gy, (const T *)x, (const T *)folded, (const int32_t *)count, (const int32_t *)hits,        \
                           (const int32_t *)taps, argmax, out, g, p);                                                           \
    } while (0)
    // whole images, one sample per wavefront pass, a multiple of kChunk * 64 cells per image and whole rows of pooled cells
    // per block of 64: no idle lanes, and the cells of a lane are a uniform step apart
    const bool full = p.bands == 1 && p.G == 1 && p.slots % (kChunk * kWave) == 0 && kWave % (g.wo / 2) == 0;
    if (p.bands > 1) CLG_BWDX_TILED(true, false, false);
    else if (p.hsw > 1 && full) CLG_BWDX_TILED(false, true, true);
    else if (p.hsw > 1) CLG_BWDX_TILED(false, true, false);
    else if (full) CLG_BWDX_TILED(false, false, true);
    else CLG_BWDX_TILED(false, false, false);
#undef CLG_BWDX_TILED
    CLG_CHECK_LAUNCH("clg_convblock_backward_x(tiled)");
    if (p.hit_split > 1) {
        const int64_t total = (int64_t)g.n * g.cin * g.h * g.w;
        hipLaunchKernelGGL(sum_partial_images_kernel<T>, dim3((unsigned)clg_ceil_div(total, 256)), dim3(256), 0, st, (const T *)part,
                           (T *)gx, total, p.hit_split);
        CLG_CHECK_LAUNCH("clg_convblock_backward_x(sum)");
    }
    return CLG_OK;
}

// What the direct input gradient leaves in its scratch for the weight gradient of the same call: the padded
// copy of x, the folded coefficients and the tap offsets (first 8 of every 16) in that copy's layout.
struct SharedPad {
    const void *xp = nullptr, *folded = nullptr;
    const int32_t *taps = nullptr;
    int sample_elems = 0;
    TilePlan p;
};

template <typename T>
int launch_backward_x_direct(const Geom &g, const TilePlan &p, int sample_elems, const void *gy, const void *x, const void *w,
                             const int32_t *sel, const uint8_t *argmax, void *gx, void *scratch, hipStream_t st, SharedPad *shared,
                             const PlanView *pv = nullptr)
{
    const BwdScratch lay = bwd_scratch_layout(g, (int)sizeof(T), 1);
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    const bool have_copy = pv != nullptr && pv->padded != nullptr;   // made by the forward call: nothing to pad here
    T *xp = have_copy ? const_cast<T *>(reinterpret_cast<const T *>(pv->padded)) : reinterpret_cast<T *>(base + bwd_x_direct_xp_off(lay));
    BwdTables tb;
    if (int e = prepare_tables<T>(g, lay, p.rs, p.chs, w, sel, scratch, st,
                                  have_copy ? no_pad_job<T>() : make_pad_job((const T *)x, xp, g, p.rs, p.chs, sample_elems), pv, &tb))
        return e;
    if (shared != nullptr) {
        shared->xp = xp;
        shared->folded = tb.folded;
        shared->taps = tb.taps;
        shared->sample_elems = sample_elems;
        shared->p = p;
    }
    if (int e = allow_lds(convblock_backward_x_direct_kernel<T>, p.lds_bytes, "clg_convblock_backward_x")) return e;
    const int64_t items = clg_ceil_div(g.n, p.G) * g.cin;
    hipLaunchKernelGGL(convblock_backward_x_direct_kernel<T>, dim3((unsigned)clg_ceil_div(items, p.NW)), dim3(p.NW * kWave),
                       p.lds_bytes, st, (const T *)gy, (const T *)xp, reinterpret_cast<const T *>(tb.folded), tb.count, tb.hits, tb.taps,
                       argmax, (T *)gx, g, p, sample_elems);
    CLG_CHECK_LAUNCH("clg_convblock_backward_x(direct)");
    return CLG_OK;
}

template <typename T>
int launch_backward_w_padded(const Geom &g, const TilePlan &p, const WScratch &ws, const void *gy, const void *x, const void *w,
                             const int32_t *sel, const uint8_t *argmax, void *gw, void *scratch, hipStream_t st, const void *probs)
{
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    T *partial = reinterpret_cast<T *>(base);
    T *folded = reinterpret_cast<T *>(base + ws.folded_off);
    int32_t *taps = reinterpret_cast<int32_t *>(base + ws.taps_off);
    T *xp = reinterpret_cast<T *>(base + ws.xp_off);
    const PadJob<T> job = make_pad_job((const T *)x, xp, g, p.rs, p.chs, ws.sample_elems);
    const unsigned prep = (unsigned)clg_ceil_div((int64_t)g.c * 8, 256);
    hipLaunchKernelGGL((convblock_w_prepare_kernel<T, T>), dim3(prep + pad_blocks(job)), dim3(256), 0, st, (const T *)w, sel, folded, taps,
                       g.c, p.rs, p.chs, host_tap_limit(g), job, (int)prep);
    CLG_CHECK_LAUNCH("clg_convblock_backward_w(prepare)");
    const int I = (g.ho / 2) * (g.wo / 2);
    if (fixed_cells(g, (int)sizeof(T)))
        hipLaunchKernelGGL((convblock_backward_w_padded_kernel<T, true>), dim3((unsigned)ws.nb, (unsigned)g.c), dim3(256), 0, st,
                           (const T *)gy, (const T *)xp, (const T *)folded, (const int32_t *)taps, argmax, partial, g, p,
                           make_fastdiv((uint32_t)I), ws.sample_elems, 8);
    else
        hipLaunchKernelGGL((convblock_backward_w_padded_kernel<T, false>), dim3((unsigned)ws.nb, (unsigned)g.c), dim3(256), 0, st,
                           (const T *)gy, (const T *)xp, (const T *)folded, (const int32_t *)taps, argmax, partial, g, p,
                           make_fastdiv((uint32_t)I), ws.sample_elems, 8);
    CLG_CHECK_LAUNCH("clg_convblock_backward_w(padded)");
    return clg_launch_reduce_coef(sizeof(T) == 8 ? CLG_F64 : CLG_F32, partial, gw, g.c, ws.nb, 7, st, "clg_convblock_backward_w(reduce)",
                                  probs);
}

// weight gradient from the padded copy the input gradient of the same call has made
template <typename T>
int launch_backward_w_shared(const Geom &g, const SharedPad &sh, const void *gy, const uint8_t *argmax, void *gw, void *scratch,
                             hipStream_t st, const void *probs)
{
    const int64_t I = (int64_t)(g.ho / 2) * (g.wo / 2);
    int64_t nb = clg_ceil_div(I * g.n, 256 * cells_per_thread(I * g.n));
    nb = nb < 1 ? 1 : (nb > 64 ? 64 : nb);
    T *partial = reinterpret_cast<T *>(scratch);                      // [c][nb][28], within the any-shape kernel's [c][64][28]
    if (fixed_cells(g, (int)sizeof(T)))
        hipLaunchKernelGGL((convblock_backward_w_padded_kernel<T, true>), dim3((unsigned)nb, (unsigned)g.c), dim3(256), 0, st,
                           (const T *)gy, (const T *)sh.xp, (const T *)sh.folded, sh.taps, argmax, partial, g, sh.p,
                           make_fastdiv((uint32_t)I), sh.sample_elems, 16);
    else
        hipLaunchKernelGGL((convblock_backward_w_padded_kernel<T, false>), dim3((unsigned)nb, (unsigned)g.c), dim3(256), 0, st,
                           (const T *)gy, (const T *)sh.xp, (const T *)sh.folded, sh.taps, argmax, partial, g, sh.p,
                           make_fastdiv((uint32_t)I), sh.sample_elems, 16);
    CLG_CHECK_LAUNCH("clg_convblock_backward_w(padded, shared copy)");
    return clg_launch_reduce_coef(sizeof(T) == 8 ? CLG_F64 : CLG_F32, partial, gw, g.c, (int)nb, 7, st,
                                  "clg_convblock_backward_w(reduce)", probs);
}

// Plan of the LDS-staged weight gradient: S samples per staged group (their image elements travel through at most
// kStagePerThread registers per thread), `rounds` groups per workgroup, nb = workgroups along the batch (partial sums
// per kernel = nb x wavefronts per kernel, at most kTiledWMaxParts).
struct TiledWPlan {
    TilePlan p;
    int rounds, nb;
};
bool plan_backward_w_tiled(const Geom &g, int elem, TiledWPlan *tw)
{
    if (const char *e = clg_knob(K_BWDW_LDS))
        if (atoi(e) == 0) return false;
    if (!taps_inside(g) || g.c > 65535) return false;
    if (elem != 4) return false;                                      // float only: the 28 sums, a tree and the staged elements of a
                                                                     // double pass do not fit 128 registers (the padded-copy kernel serves double)
    TilePlan *p = &tw->p;
    plan_common(g, p);
    const int64_t I = (int64_t)(g.ho / 2) * (g.wo / 2);
    if (I < 1 || g.wo / 2 > 32768) return false;
    p->slots = (int)I;
    p->d_slots = make_fastdiv((uint32_t)I);
    p->G = 1;
    p->NW = kTiledWWaves;
    const int64_t tail = g.ph * p->rs + g.pw;
    const int64_t sample_elems = (int64_t)g.cin * g.h * g.w, sample_lds = (int64_t)g.cin * p->chs;
    const int64_t stage_cap = (int64_t)kStagePerThread * kTiledWWaves * kWave;
    int64_t S = stage_cap / sample_elems;                            // what the staging registers carry ...
    const int64_t lds_cap = (96 * 1024 / elem - tail) / sample_lds;   // ... within 96 KiB of LDS
    if (S > lds_cap) S = lds_cap;
    if (S > g.n) S = g.n;
    if (S > 64) S = 64;
    if (S < 1) return false;
    if (S * I < 2 * kWave) return false;                             // under two blocks of cells per staged group: the other kernels do better
    // kernels per workgroup: 16 (one per wavefront), fewer for layers with few kernels (the wavefronts of a kernel
    // then share its cells); rounds: at least 8 cell blocks per wavefront before its 28 reductions, at most 256 partial
    // sums per kernel, and as many more as still leave one workgroup per CU (its 16 wavefronts fill the CU's vector
    // registers; what a wavefront does once -- folding its kernel's coefficients, the 28 reductions -- costs as much
    // as 7 visits, so long runs pay: 101 -> 76 us at [256,9,32,32] -> 256 from 4 to 16 rounds)
    const int64_t groups = clg_ceil_div(g.n, S);
    int64_t kw = kTiledWWaves;
    while (kw > 4 && clg_ceil_div(g.c, kw) * groups < 1024) kw /= 2;
    const int64_t slices = kTiledWWaves / kw, ktiles = clg_ceil_div(g.c, kw);
    const int64_t blocks_per_round = clg_ceil_div(clg_ceil_div(S * I, kWave), slices);
    int64_t R = clg_ceil_div(8, blocks_per_round);
    while (clg_ceil_div(groups, R) * slices > kTiledWMaxParts) ++R;
    while (R < groups && clg_ceil_div(groups, R + 1) * ktiles >= 256) ++R;
    if (R > groups) R = groups;
    if (clg_ceil_div(groups, R) * slices > kTiledWMaxParts) return false;
    p->CT = (int)kw;
    p->S = (int)S;
    p->xe = (int)(S * sample_lds + tail);
    p->d_planes = make_fastdiv((uint32_t)g.h);                        // image row -> (plane, iy)
    p->lds_bytes = (size_t)((p->xe + 3) & ~3) * elem + (size_t)S * g.cin * g.h * 4;
    if (p->lds_bytes > (size_t)kLdsLimit) return false;
    tw->rounds = (int)R;
    tw->nb = (int)clg_ceil_div(groups, R);                           // workgroups along the batch; partial sums per kernel = nb * slices
    return S * sample_lds < (1ll << 30) && S * g.c * I < (1ll << 31) && (int64_t)g.n * g.c * I < (1ll << 62);
}

template <typename T>
int launch_backward_w_tiled(const Geom &g, const TiledWPlan &tw, const void *gy, const void *x, const void *w, const int32_t *sel,
                            const uint8_t *argmax, void *gw, void *scratch, hipStream_t st, const void *probs)
{
    const dim3 grid((unsigned)tw.nb, (unsigned)clg_ceil_div(g.c, tw.p.CT)), block(kTiledWWaves * kWave);
    const int nparts = tw.nb * (kTiledWWaves / tw.p.CT);
    // cells per lane and load: 4 or 2 when they divide the pooled row length and the pointers are aligned for the vector loads
    const int wp = g.wo / 2;
    const uintptr_t gy_a = (uintptr_t)gy, am_a = (uintptr_t)argmax;
    const int64_t group_cells = (int64_t)tw.p.S * (g.ho / 2) * wp, lanes_needed = (int64_t)kWave * (kTiledWWaves / tw.p.CT);
    int v = 1;                                                       // (wide loads only while they leave the wavefronts of a kernel full)
    if (wp % 4 == 0 && gy_a % (4 * sizeof(T)) == 0 && am_a % 4 == 0 && group_cells >= 4 * lanes_needed) v = 4;
    else if (wp % 2 == 0 && gy_a % (2 * sizeof(T)) == 0 && am_a % 2 == 0 && group_cells >= 2 * lanes_needed) v = 2;
#define CLG_BWDW_TILED(VV)                                                                                                        \
    do {                                                                                                                          \
        if (int e = allow_lds(convblock_backward_w_tiled_kernel<T, VV>, tw.p.lds_bytes, "clg_convblock_backward_w")) return e;    \
        hipLaunchKernelGGL((convblock_backward_w_tiled_kernel<T, VV>), grid, block, tw.p.lds_bytes, st, (const T *)gy, (const T *)x, \
                           (const T *)w, sel, argmax, (T *)scratch, g, tw.p, tw.rounds);                                          \
    } while (0)
    if (v == 4) CLG_BWDW_TILED(4);
    else if (v == 2) CLG_BWDW_TILED(2);
    else CLG_BWDW_TILED(1);
#undef CLG_BWDW_TILED
    CLG_CHECK_LAUNCH("clg_convblock_backward_w(tiled)");
    return clg_launch_reduce_coef(sizeof(T) == 8 ? CLG_F64 : CLG_F32, scratch, gw, g.c, nparts, 7, st, "clg_convblock_backward_w(reduce)",
                                  probs);
}

int elem_size(int dtype) { return dtype == CLG_F64 ? 8 : 4; }

}  // namespace

// Kernels that want more than 48 KiB of dynamic LDS must be told once; the largest size granted so
// far is remembered per kernel so that steady-state launches make no runtime call besides the launch.
int clg_allow_lds(const void *kernel, size_t bytes, const char *name)
{
    constexpr int kSlots = 256;                                      // (kernel instantiation, device) pairs remembered
    static std::mutex mu;
    static const void *known[kSlots];
    static int device_of[kSlots];
    static size_t granted[kSlots];
    static int used = 0;
    if (bytes <= 48 * 1024) return CLG_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;                    // the attribute is kept per device
    std::lock_guard<std::mutex> lock(mu);
    int slot = -1;
    for (int i = 0; i < used; ++i)
        if (known[i] == kernel && device_of[i] == dev) slot = i;
    if (slot >= 0 && granted[slot] >= bytes) return CLG_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
        clg_set_error("%s: cannot reserve %zu bytes of LDS: %s", name, bytes, hipGetErrorString(e));
        return CLG_ELAUNCH;
    }
    if (slot < 0 && used < kSlots) slot = used++;
    if (slot >= 0) {
        known[slot] = kernel;
        device_of[slot] = dev;
        granted[slot] = bytes;
    }
    return CLG_OK;
}

extern "C" int64_t clg_convblock_backward_x_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_x_scratch_bytes")) return -1;
    TilePlan p;
    int se = 0;
    const BwdXMode mode = choose_backward_x(g, elem_size(dtype), &p, &se);
    const BwdScratch lay = bwd_scratch_layout(g, elem_size(dtype), mode == kBwdXTiled ? p.hit_split : 1);
    if (mode == kBwdXDirect) return (int64_t)(bwd_x_direct_xp_off(lay) + (size_t)se * g.n * elem_size(dtype));
    return (int64_t)lay.total;
}

// What the tiled input gradient sets up for a padded weight gradient that follows in the same call: its prepare launch
// also writes the padded copy (planes of p.chs elements, the layout its tap offsets are made for) into the weight
// gradient's scratch, so that one neither folds nor computes tap offsets nor pads again.
template <typename T>
PadJob<T> share_from_tiled(const Geom &g, const TilePlan &p, const void *x, void *w_scratch, SharedPad *shared)
{
    TilePlan pw;
    WScratch ws;
    const char *e_pad = clg_knob(K_BWDW_PADDED);
    TiledWPlan tw;
    if (!(e_pad && atoi(e_pad) != 0) && plan_backward_w_tiled(g, (int)sizeof(T), &tw)) return no_pad_job<T>();   // that kernel stages x itself
    if (shared == nullptr || w_scratch == nullptr || p.bands != 1 || (e_pad && atoi(e_pad) == 0) || !plan_backward_w(g, (int)sizeof(T), &pw, &ws))
        return no_pad_job<T>();
    const int sample_elems = g.cin * p.chs + g.ph * p.rs + g.pw;
    T *xp = reinterpret_cast<T *>(reinterpret_cast<unsigned char *>(w_scratch) + ws.xp_off);
    shared->xp = xp;                                                  // folded / taps: filled in from the call's tables
    shared->sample_elems = sample_elems;
    shared->p = pw;
    return make_pad_job((const T *)x, xp, g, p.rs, p.chs, sample_elems);
}

static int convblock_backward_x_impl(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_x, void *scratch, void *stream,
                                     SharedPad *shared, void *w_scratch = nullptr, const PlanView *pv = nullptr)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_x")) return e;
    CLG_REQUIRE(grad_y && x && w && selection && argmax && grad_x && scratch, "clg_convblock_backward_x: null pointer argument");
    TilePlan p;
    int se = 0;
    const BwdXMode mode = choose_backward_x(g, elem_size(dtype), &p, &se);
    hipStream_t st = clg_stream(stream);
    if (mode == kBwdXTiled) {
        BwdTables tb;
        int e;
        if (dtype == CLG_F32)
            e = launch_backward_x_tiled<float>(g, p, grad_y, x, w, selection, argmax, grad_x, scratch, st,
                                               share_from_tiled<float>(g, p, x, w_scratch, shared), pv, &tb);
        else
            e = launch_backward_x_tiled<double>(g, p, grad_y, x, w, selection, argmax, grad_x, scratch, st,
                                                share_from_tiled<double>(g, p, x, w_scratch, shared), pv, &tb);
        if (shared != nullptr && shared->xp != nullptr) {
            shared->folded = tb.folded;
            shared->taps = tb.taps;
        }
        return e;
    }
    if (mode == kBwdXDirect) {
        if (dtype == CLG_F32)
            return launch_backward_x_direct<float>(g, p, se, grad_y, x, w, selection, argmax, grad_x, scratch, st, shared, pv);
        return launch_backward_x_direct<double>(g, p, se, grad_y, x, w, selection, argmax, grad_x, scratch, st, shared, pv);
    }
    // any other shape: per-element gather driven by the same per-channel kernel lists
    const BwdScratch lay = bwd_scratch_layout(g, elem_size(dtype), 1);
    BwdTables tb;
    if (dtype == CLG_F32) {
        if (int e = prepare_tables<float>(g, lay, 0, 0, w, selection, scratch, st, no_pad_job<float>(), pv, &tb)) return e;
    } else {
        if (int e = prepare_tables<double>(g, lay, 0, 0, w, selection, scratch, st, no_pad_job<double>(), pv, &tb)) return e;
    }
    return clg_convblock_backward_x_generic(dtype, g, grad_y, x, tb.folded, tb.count, tb.hits, selection, argmax, grad_x, st);
}

extern "C" int64_t clg_convblock_backward_w_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_w_scratch_bytes")) return -1;
    TilePlan p;
    WScratch ws;
    TiledWPlan tw;
    const char *e_pad = clg_knob(K_BWDW_PADDED);
    const bool tiled = !(e_pad && atoi(e_pad) != 0) && plan_backward_w_tiled(g, elem_size(dtype), &tw);
    if (!tiled && plan_backward_w(g, elem_size(dtype), &p, &ws)) return (int64_t)ws.total;
    // partial sums of the LDS-staged (at most 256 per kernel) and of the any-shape kernel (at most 64)
    return (int64_t)g.c * (tiled ? kTiledWMaxParts : 64) * 28 * elem_size(dtype);
}

extern "C" int clg_convblock_backward_x(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                        const int32_t *selection, const uint8_t *argmax, void *grad_x, void *scratch,
                                        void *stream)
{
    return convblock_backward_x_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_x, scratch, stream, nullptr);
}

// grad_w w.r.t. the gate probabilities, or -- with probs = the softmax output w -- w.r.t. the logits
static int convblock_backward_w_impl(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch, void *stream,
                                     const void *probs, const char *name, const SharedPad *shared = nullptr)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(grad_y && x && w && selection && argmax && grad_w && scratch, "%s: null pointer argument", name);
    if (shared != nullptr && shared->xp != nullptr && g.c <= 65535) {
        if (dtype == CLG_F32) return launch_backward_w_shared<float>(g, *shared, grad_y, argmax, grad_w, scratch, clg_stream(stream), probs);
        return launch_backward_w_shared<double>(g, *shared, grad_y, argmax, grad_w, scratch, clg_stream(stream), probs);
    }
    TiledWPlan tw;
    const char *e_pad = clg_knob(K_BWDW_PADDED);
    if (!(e_pad && atoi(e_pad) != 0) && plan_backward_w_tiled(g, elem_size(dtype), &tw)) {     // images in LDS (CLG_BWDW_PADDED=1 forces the padded copy)
        return launch_backward_w_tiled<float>(g, tw, grad_y, x, w, selection, argmax, grad_w, scratch, clg_stream(stream), probs);
    }
    TilePlan p;
    WScratch ws;
    if ((!e_pad || atoi(e_pad) != 0) && plan_backward_w(g, elem_size(dtype), &p, &ws)) {
        if (dtype == CLG_F32)
            return launch_backward_w_padded<float>(g, p, ws, grad_y, x, w, selection, argmax, grad_w, scratch, clg_stream(stream), probs);
        return launch_backward_w_padded<double>(g, p, ws, grad_y, x, w, selection, argmax, grad_w, scratch, clg_stream(stream), probs);
    }
    return clg_convblock_backward_w_generic(dtype, g, grad_y, x, w, selection, argmax, grad_w, scratch, clg_stream(stream), probs);
}

extern "C" int clg_convblock_backward_w(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                        const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                                        void *stream)
{
    return convblock_backward_w_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_w, scratch, stream, nullptr,
                                     "clg_convblock_backward_w");
}

// 4x4 images with one sample per lane (conv_small.hip): scratch = prepare tables | tap gradients
static bool backward_4x4_wanted(const Geom &g)
{
    const char *e = clg_knob(K_BWD_4X4);
    return clg_convblock_is_4x4(g) && g.c <= 65535 && (!e || atoi(e) != 0);
}
static size_t backward_4x4_tg_off(const Geom &g, int dtype) { return (bwd_scratch_layout(g, elem_size(dtype), 1).total + 255) & ~(size_t)255; }

static int convblock_backward_4x4(int dtype, const Geom &g, const void *grad_y, const void *x, const void *w, const int32_t *selection,
                                  const uint8_t *argmax, void *grad_x, void *grad_w, void *scratch, void *stream, const void *probs,
                                  const char *name, const PlanView *pv = nullptr)
{
    CLG_REQUIRE(grad_y && x && w && selection && argmax && grad_w && scratch, "%s: null pointer argument", name);
    const BwdScratch lay = bwd_scratch_layout(g, elem_size(dtype), 1);
    unsigned char *base = reinterpret_cast<unsigned char *>(scratch);
    hipStream_t st = clg_stream(stream);
    BwdTables tb;
    if (dtype == CLG_F32) {
        if (int e = prepare_tables<float>(g, lay, 0, 0, w, selection, scratch, st, no_pad_job<float>(), pv, &tb)) return e;
    } else {
        if (int e = prepare_tables<double>(g, lay, 0, 0, w, selection, scratch, st, no_pad_job<double>(), pv, &tb)) return e;
    }
    return clg_convblock_backward_4x4(dtype, g, x, tb.folded, selection, grad_y, argmax, base + backward_4x4_tg_off(g, dtype), grad_w, probs,
                                      tb.count, tb.hits, grad_x, st, name);
}

extern "C" int64_t clg_convblock_backward_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    const int64_t a = clg_convblock_backward_x_scratch_bytes(dtype, gg), b = clg_convblock_backward_w_scratch_bytes(dtype, gg);
    if (a < 0 || b < 0) return -1;
    int64_t total = ((a + 255) & ~255ll) + b;
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_scratch_bytes")) return -1;
    if (backward_4x4_wanted(g)) {
        const int64_t small = (int64_t)(backward_4x4_tg_off(g, dtype) + clg_convblock_backward_4x4_tg_bytes(dtype, g));
        if (small > total) total = small;
    }
    return total;
}

extern "C" int clg_convblock_backward(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                      const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_w, void *scratch,
                                      void *stream)
{
    CLG_REQUIRE(scratch, "clg_convblock_backward: null pointer argument");
    {
        Geom g;
        if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward")) return e;
        if (backward_4x4_wanted(g)) {
            CLG_REQUIRE(grad_x, "clg_convblock_backward: null pointer argument");
            return convblock_backward_4x4(dtype, g, grad_y, x, w, selection, argmax, grad_x, grad_w, scratch, stream, nullptr,
                                          "clg_convblock_backward");
        }
    }
    const int64_t a = clg_convblock_backward_x_scratch_bytes(dtype, gg);
    if (a < 0) return CLG_EINVAL;
    SharedPad shared;
    void *w_scratch = reinterpret_cast<unsigned char *>(scratch) + ((a + 255) & ~255ll);
    if (int e = convblock_backward_x_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_x, scratch, stream, &shared, w_scratch)) return e;
    return convblock_backward_w_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_w, w_scratch, stream, nullptr,
                                     "clg_convblock_backward", &shared);
}

extern "C" int clg_convblock_fm_supported(int dtype, const clg_conv_geom *gg);

extern "C" int clg_convblock_backward_fm(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                         const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_w,
                                         int wrt_logits, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_fm")) return e;
    CLG_REQUIRE(clg_convblock_fm_supported(dtype, gg), "clg_convblock_backward_fm: needs 4x4 images, a 3x3 kernel, stride 1, padding 1 "
                "and at least 32 samples (clg_convblock_fm_supported)");
    g.y_fm = 1;
    return convblock_backward_4x4(dtype, g, grad_y, x, w, selection, argmax, grad_x, grad_w, scratch, stream, wrt_logits ? w : nullptr,
                                  "clg_convblock_backward_fm");
}

extern "C" int clg_convblock_backward_logits(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                             const int32_t *selection, const uint8_t *argmax, void *grad_x, void *grad_logits,
                                             void *scratch, void *stream)
{
    CLG_REQUIRE(scratch, "clg_convblock_backward_logits: null pointer argument");
    {
        Geom g;
        if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_logits")) return e;
        if (backward_4x4_wanted(g))
            return convblock_backward_4x4(dtype, g, grad_y, x, w, selection, argmax, grad_x, grad_logits, scratch, stream, w,
                                          "clg_convblock_backward_logits");
    }
    const int64_t a = clg_convblock_backward_x_scratch_bytes(dtype, gg);
    if (a < 0) return CLG_EINVAL;
    SharedPad shared;
    void *w_scratch = reinterpret_cast<unsigned char *>(scratch) + ((a + 255) & ~255ll);
    if (grad_x != nullptr)
        if (int e = convblock_backward_x_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_x, scratch, stream, &shared, w_scratch))
            return e;
    return convblock_backward_w_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_logits, w_scratch, stream, w,
                                     "clg_convblock_backward_logits", &shared);
}

// ---- per-layer plan --------------------------------------------------------------------------------
// plan = BwdScratch layout without partial images: (folded: unused) | count | cursor | hits | unsorted | taps
namespace {
struct PlanInfo {
    BwdScratch lay;
    int rs, chs;
    size_t total;
    int64_t signature;
};
PlanInfo plan_info(const Geom &g, int dtype)
{
    PlanInfo pi;
    const int elem = elem_size(dtype);
    int mode = 3, rs = 0, chs = 0;                                    // 3: one sample per lane on 4x4 images
    if (!backward_4x4_wanted(g)) {
        TilePlan p;
        int se = 0;
        mode = (int)choose_backward_x(g, elem, &p, &se);
        if (mode != kBwdXGather) rs = p.rs, chs = p.chs;
    }
    pi.lay = bwd_scratch_layout(g, elem, 1);
    pi.rs = rs, pi.chs = chs;
    pi.total = pi.lay.part_off;
    // what the tables were made for: a plan is rejected when geometry, element type or the path choice differ
    const int64_t fields[] = {mode, rs, chs, pi.lay.csr, elem, g.n, g.cin, g.h, g.w, g.c, g.sh, g.sw, g.ph, g.pw, g.kh, g.kw};
    uint64_t h = 1469598103934665603ull;
    for (int64_t f : fields) {
        h ^= (uint64_t)f;
        h *= 1099511628211ull;
    }
    pi.signature = (int64_t)(h & 0x7fffffffffffffffull);
    return pi;
}
}  // namespace

extern "C" int64_t clg_convblock_plan_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_plan_bytes")) return -1;
    return (int64_t)plan_info(g, dtype).total;
}

extern "C" int clg_convblock_plan(int dtype, const clg_conv_geom *gg, const int32_t *selection, void *plan, int64_t *signature,
                                  void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_plan")) return e;
    CLG_REQUIRE(selection && plan && signature, "clg_convblock_plan: null pointer argument");
    const PlanInfo pi = plan_info(g, dtype);
    hipStream_t st = clg_stream(stream);
    // lists and tap offsets by the set-up launch of the unplanned path (no weights: nothing is folded)
    if (dtype == CLG_F32) {
        if (int e = launch_prepare<float>(g, pi.lay, pi.rs, pi.chs, nullptr, selection, plan, st, no_pad_job<float>())) return e;
    } else {
        if (int e = launch_prepare<double>(g, pi.lay, pi.rs, pi.chs, nullptr, selection, plan, st, no_pad_job<double>())) return e;
    }
    *signature = pi.signature;
    return CLG_OK;
}

// One sample of the padded copy the planned backward pass reads when its input gradient is the direct kernel, else 0.
int64_t clg_convblock_backward_padded_sample_elems(int dtype, const Geom &g)
{
    if (backward_4x4_wanted(g)) return 0;
    TilePlan p;
    int se = 0;
    return choose_backward_x(g, elem_size(dtype), &p, &se) == kBwdXDirect ? se : 0;
}

static int backward_planned_impl(const char *name, int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                 const void *folded, const void *padded, const int32_t *selection, const uint8_t *argmax, void *plan,
                                 int64_t signature, void *grad_x, void *grad_w, int flags, void *scratch, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(grad_y && x && w && selection && argmax && plan && grad_w && scratch, "%s: null pointer argument", name);
    CLG_REQUIRE((flags & ~(CLG_BWD_WRT_LOGITS | CLG_BWD_GY_FEATURE_MAJOR)) == 0, "%s: unknown flags 0x%x", name, flags);
    const bool wrt_logits = (flags & CLG_BWD_WRT_LOGITS) != 0, fm = (flags & CLG_BWD_GY_FEATURE_MAJOR) != 0;
    CLG_REQUIRE(!fm || clg_convblock_fm_supported(dtype, gg), "%s: CLG_BWD_GY_FEATURE_MAJOR needs a shape for which "
                "clg_convblock_fm_supported() holds (4x4 images, 3x3 kernel, stride 1, padding 1, n >= 32)", name);
    const PlanInfo pi = plan_info(g, dtype);
    CLG_REQUIRE(signature == pi.signature, "%s: the plan was made for another geometry, element type or kernel choice (make a new one "
                "with clg_convblock_plan; the CLG_* knobs are part of the choice)", name);
    unsigned char *pb = reinterpret_cast<unsigned char *>(plan);
    PlanView pv;
    pv.count = reinterpret_cast<const int32_t *>(pb + pi.lay.count_off);
    pv.hits = reinterpret_cast<const int32_t *>(pb + pi.lay.hits_off);
    pv.taps = reinterpret_cast<const int32_t *>(pb + pi.lay.taps_off);
    pv.folded = folded;
    pv.padded = padded;
    const void *probs = wrt_logits ? w : nullptr;
    if (backward_4x4_wanted(g)) {
        g.y_fm = fm ? 1 : 0;
        return convblock_backward_4x4(dtype, g, grad_y, x, w, selection, argmax, grad_x, grad_w, scratch, stream, probs, name, &pv);
    }
    const int64_t a = clg_convblock_backward_x_scratch_bytes(dtype, gg);
    if (a < 0) return CLG_EINVAL;
    SharedPad shared;
    void *w_scratch = reinterpret_cast<unsigned char *>(scratch) + ((a + 255) & ~255ll);
    if (grad_x != nullptr)
        if (int e = convblock_backward_x_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_x, scratch, stream, &shared, w_scratch, &pv))
            return e;
    return convblock_backward_w_impl(dtype, gg, grad_y, x, w, selection, argmax, grad_w, w_scratch, stream, probs, name, &shared);
}

extern "C" int clg_convblock_backward_planned(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                              const void *folded, const int32_t *selection, const uint8_t *argmax, void *plan,
                                              int64_t signature, void *grad_x, void *grad_w, int flags, void *scratch, void *stream)
{
    return backward_planned_impl("clg_convblock_backward_planned", dtype, gg, grad_y, x, w, folded, nullptr, selection, argmax, plan, signature,
                                 grad_x, grad_w, flags, scratch, stream);
}

extern "C" int clg_convblock_backward_planned_padded(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                                     const void *folded, const void *padded, const int32_t *selection,
                                                     const uint8_t *argmax, void *plan, int64_t signature, void *grad_x, void *grad_w,
                                                     int flags, void *scratch, void *stream)
{
    const char *name = "clg_convblock_backward_planned_padded";
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, name)) return e;
    CLG_REQUIRE(padded == nullptr || (grad_x != nullptr && clg_convblock_backward_padded_sample_elems(dtype, g) > 0),
                "%s: a padded copy is only taken with grad_x and where clg_convblock_padded_elems() is not 0", name);
    return backward_planned_impl(name, dtype, gg, grad_y, x, w, folded, padded, selection, argmax, plan, signature, grad_x, grad_w, flags,
                                 scratch, stream);
}
