// Packed-bit inference: pack bool -> words, bitwise gate evaluation, per-class popcount.
//
// A word holds `bits` samples of one feature (sample s = bit s % bits of word s / bits, LSB first).
// Every gate is bitwise, so the evaluation kernel treats a row as a run of bytes and moves it with
// 16-byte vectors whatever the word type is; one wavefront evaluates one neuron (gate id, wiring
// and truth-table masks are wave-uniform) over a column chunk of its two input rows.
#include <stdlib.h>

#include "clg_common.h"

namespace {

// ---------------------------------------------------------------------------------------------
// evaluation
// ---------------------------------------------------------------------------------------------
constexpr int kEvalBlock = 256;
constexpr int kEvalWaves = kEvalBlock / kWave;

// Rows are `row_vecs` vectors of type V.  blockIdx.x enumerates (column chunk, neuron group) with
// the chunk as the slow index, so that all neurons of one column chunk run back to back and the
// second read of an input row segment finds it in the last-level cache.
template <typename V, int UNROLL>
__global__ __launch_bounds__(kEvalBlock) void eval_packed_kernel(const V *__restrict__ x, const int64_t *__restrict__ a,
                                                               const int64_t *__restrict__ b,
                                                               const uint8_t *__restrict__ gate, V *__restrict__ y,
                                                               int out_dim, int64_t row_vecs, int chunk_vecs,
                                                               int groups_per_chunk, int neurons_per_wave, int64_t in_dim)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int chunk = blockIdx.x / groups_per_chunk;
    const int group = blockIdx.x % groups_per_chunk;
    const int64_t v0 = (int64_t)chunk * chunk_vecs;
    const int64_t v1 = (v0 + chunk_vecs < row_vecs) ? v0 + chunk_vecs : row_vecs;
    const int j0 = (group * kEvalWaves + wave) * neurons_per_wave;
    for (int jj = 0; jj < neurons_per_wave; ++jj) {
        const int j = j0 + jj;
        if (j >= out_dim) break;
        const V *xa = x + clamp_index(a[j], in_dim) * row_vecs;    // (a bad index reads a wrong row; it never leaves x)
        const V *xb = x + clamp_index(b[j], in_dim) * row_vecs;
        V *yj = y + (int64_t)j * row_vecs;
        const Masks m = gate_masks(gate[j]);
        for (int64_t v = v0 + lane; v < v1; v += (int64_t)kWave * UNROLL) {
            V ra[UNROLL], rb[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int64_t vv = v + (int64_t)u * kWave;
                if (vv < v1) {
                    ra[u] = xa[vv];
                    rb[u] = xb[vv];
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int64_t vv = v + (int64_t)u * kWave;
                if (vv < v1) __builtin_nontemporal_store(gate_vec(m, ra[u], rb[u]), yj + vv);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// evaluation along a precomputed walk of the wiring graph
// ---------------------------------------------------------------------------------------------
// Input rows are vertices and neurons are edges of a multigraph.  The plan lists the neurons along
// trails of that graph, so that a neuron shares one input row with its predecessor; the wavefront
// keeps that row in registers and loads only the other one.  Every row chunk is then read about once
// (plus one extra row per segment start) instead of twice.
// plan[k] = neuron | use << 28 | keep << 30
//   use : 0 nothing carried, 1 carried row is input a, 2 carried row is input b, 3 it is both
//   keep: row carried to the next step, 0 = input a, 1 = input b
// Index of the first maximum of 16 float32 logits, a NaN counting as the maximum (the rule of gate_argmax_kernel and of
// torch.argmax), computed by the whole wavefront: lane l holds logit l % 16 (`v`) as an order-preserving integer key (-0
// and +0 equal, NaN on top), the row maximum comes over DPP, the first lane that holds it names the gate.  Wave-uniform.
__device__ __forceinline__ int argmax16_uniform(float v)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, v + 0.0f);
    const uint32_t key = v != v ? 0xFFFFFFFFu : (u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u));
    const uint32_t top = row16_max(key);
    const uint32_t first = (uint32_t)__ballot(key == top) & 0xFFFFu;
    return uniform(__builtin_ctz(first));
}

// gate[j] for a wave-uniform j through the scalar cache: the aligned 32-bit word that holds it (a byte load would be a
// vector load, and the wait for it would also wait for the row loads in flight).  The last word is read bytewise when
// it reaches past the table; the table starts at a 4-byte boundary or is read bytewise altogether.
__device__ __forceinline__ int gate_id_uniform(const uint8_t *__restrict__ gate, int j, int n)
{
    if ((reinterpret_cast<uintptr_t>(gate) & 3) == 0 && (j | 3) < n) {
        const uint32_t w = reinterpret_cast<const uint32_t *>(gate)[j >> 2];
        return (int)((w >> ((j & 3) * 8)) & 0xFFu);
    }
    return gate[j];
}

// LOGITS: `gate` points to float32 logits [out_dim, 16] and the wavefront takes their arg-max itself (the layer's eval
// call then needs no launch of its own for the gate ids); else to uint8 gate ids [out_dim].
template <int R, bool LOGITS>
__global__ __launch_bounds__(kEvalBlock) void eval_packed_walk_kernel(const u32x4 *__restrict__ x, const int64_t *__restrict__ a,
                                                                    const int64_t *__restrict__ b,
                                                                    const void *__restrict__ gate,
                                                                    const int32_t *__restrict__ plan, u32x4 *__restrict__ y,
                                                                    int steps, int seg_len, int64_t row_vecs, int64_t in_dim)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int k0 = (blockIdx.x * kEvalWaves + wave) * seg_len;
    if (k0 >= steps) return;
    const int k1 = k0 + seg_len < steps ? k0 + seg_len : steps;
    const int64_t col0 = (int64_t)blockIdx.y * (kWave * R) + lane;   // this lane's first vector in the row
    u32x4 ra[R], rb[R], carry[R];
#pragma unroll
    for (int r = 0; r < R; ++r) carry[r] = (u32x4)0u;
    for (int k = k0; k < k1; ++k) {
        const int p = plan[k];
        const int j = min(p & 0x0FFFFFFF, steps - 1), keep = (p >> 30) & 1;   // one plan entry per neuron
        const int use = k == k0 ? 0 : (p >> 28) & 3;
        const u32x4 *xa = x + clamp_index(a[j], in_dim) * row_vecs + col0;
        const u32x4 *xb = x + clamp_index(b[j], in_dim) * row_vecs + col0;
        float logit = 0.f;                                            // requested ahead of the rows: vector loads return in order
        if constexpr (LOGITS) logit = reinterpret_cast<const float *>(gate)[(int64_t)j * 16 + (lane & 15)];
        if (use != 1 && use != 3) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (col0 + r * kWave < row_vecs) ra[r] = xa[r * kWave];
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) ra[r] = carry[r];
        }
        if (use < 2) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (col0 + r * kWave < row_vecs) rb[r] = xb[r * kWave];
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) rb[r] = carry[r];
        }
        int id;
        if constexpr (LOGITS) id = argmax16_uniform(logit);
        else id = gate_id_uniform(reinterpret_cast<const uint8_t *>(gate), j, steps);
        const Masks m = gate_masks(id);
        u32x4 *yj = y + (int64_t)j * row_vecs + col0;
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (col0 + r * kWave < row_vecs) __builtin_nontemporal_store(gate_vec(m, ra[r], rb[r]), yj + r * kWave);
#pragma unroll
        for (int r = 0; r < R; ++r) carry[r] = keep ? rb[r] : ra[r];
    }
}

// bytewise tail / odd row sizes: one thread per byte of the output
__global__ void eval_packed_bytes_kernel(const uint8_t *__restrict__ x, const int64_t *__restrict__ a,
                                         const int64_t *__restrict__ b, const uint8_t *__restrict__ gate,
                                         uint8_t *__restrict__ y, int64_t out_dim, int64_t row_bytes, int64_t in_dim)
{
    const int64_t total = out_dim * row_bytes;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t j = i / row_bytes, c = i % row_bytes;
        const Masks m = gate_masks(gate[j]);
        y[i] = (uint8_t)gate_bits(m, x[clamp_index(a[j], in_dim) * row_bytes + c], x[clamp_index(b[j], in_dim) * row_bytes + c]);
    }
}

// ---------------------------------------------------------------------------------------------
// packing
// ---------------------------------------------------------------------------------------------
// 8 bool bytes (any non-zero value counts as true) -> 8 bits, byte k -> bit k.
__device__ __forceinline__ uint32_t squeeze8(uint64_t v)
{
    v |= v >> 4;
    v |= v >> 2;
    v |= v >> 1;
    v &= 0x0101010101010101ull;
    return (uint32_t)((v * 0x0102040810204080ull) >> 56);
}

// feature-major input t [F, B]: one thread per output byte (8 samples); the word type only fixes the
// padded row length, because words are little endian and samples fill them LSB first.
__global__ void pack_bits_kernel(const uint8_t *__restrict__ t, uint8_t *__restrict__ out, int64_t features, int64_t batch,
                                 int64_t row_bytes, bool aligned8)
{
    const int64_t total = features * row_bytes;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t f = i / row_bytes, c = i % row_bytes;
        const int64_t s0 = c * 8;
        const uint8_t *p = t + f * batch + s0;
        uint32_t bits = 0;
        if (aligned8 && s0 + 8 <= batch) {
            bits = squeeze8(*reinterpret_cast<const uint64_t *>(p));
        } else {
            for (int k = 0; k < 8; ++k)
                if (s0 + k < batch && p[k]) bits |= 1u << k;
        }
        out[i] = (uint8_t)bits;
    }
}

// sample-major input t [B, F]: lanes run along features (contiguous reads), each thread keeps the
// 64 samples of one feature in a 64-bit register and then stores 8 bytes of that feature's row.
// Consecutive 64-sample groups of the same features are handled by the same thread one after the
// other so that its partial-line stores merge in L2.
constexpr int kPackGroups = 16;  // 64-sample groups per thread
__global__ __launch_bounds__(256) void pack_bits_sm_kernel(const uint8_t *__restrict__ t, uint8_t *__restrict__ out,
                                                         int64_t features, int64_t batch, int64_t row_bytes)
{
    const int64_t f = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= features) return;
    const int64_t g0 = (int64_t)blockIdx.y * kPackGroups;
    for (int g = 0; g < kPackGroups; ++g) {
        const int64_t s0 = (g0 + g) * 64;
        if (s0 >= batch) break;
        uint64_t word = 0;
        const int64_t n = batch - s0 < 64 ? batch - s0 : 64;
        if (n == 64) {
#pragma unroll 16
            for (int k = 0; k < 64; ++k) word |= (uint64_t)(t[(s0 + k) * features + f] != 0) << k;
        } else {
            for (int k = 0; k < n; ++k) word |= (uint64_t)(t[(s0 + k) * features + f] != 0) << k;
        }
        uint8_t *dst = out + f * row_bytes + s0 / 8;
        const int64_t nbytes = row_bytes - s0 / 8 < 8 ? row_bytes - s0 / 8 : 8;
        if (nbytes == 8 && (row_bytes & 7) == 0) {
            *reinterpret_cast<uint64_t *>(dst) = word;
        } else {
            for (int k = 0; k < nbytes; ++k) dst[k] = (uint8_t)(word >> (8 * k));
        }
    }
}

// The same for feature counts that are multiples of 16: a lane takes 16 consecutive features, so a
// wavefront reads 1 KiB of a sample row per load.  Bytes are turned into bits four features at a time
// inside a 32-bit register: bit 7 of every byte is set where the byte is non-zero, and
// acc = (acc >> 1) | bits run over 8 samples leaves their 8 bits LSB first in every byte.
template <int V>
struct PackVec;
template <>
struct PackVec<1> {
    typedef uint32_t type;
    static __device__ __forceinline__ uint32_t get(uint32_t v, int) { return v; }
};
template <>
struct PackVec<2> {
    typedef u32x2 type;
    static __device__ __forceinline__ uint32_t get(u32x2 v, int q) { return v[q]; }
};
template <>
struct PackVec<4> {
    typedef u32x4 type;
    static __device__ __forceinline__ uint32_t get(u32x4 v, int q) { return v[q]; }
};
// V 32-bit registers (4 V features) per lane, G consecutive 64-sample groups per thread (its 8-byte stores
// to one feature row are then adjacent and merge into full lines in L2).
template <int V, int G>
__global__ __launch_bounds__(256) void pack_bits_smv_kernel(const uint8_t *__restrict__ t, uint8_t *__restrict__ out,
                                                          int64_t features, int64_t batch, int64_t row_bytes)
{
    typedef typename PackVec<V>::type Vec;
    const int64_t f0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * (4 * V);
    if (f0 >= features) return;
    const int64_t row_vecs = features / (4 * V);
    for (int g = 0; g < G; ++g) {
        const int64_t s0 = ((int64_t)blockIdx.y * G + g) * 64;
        if (s0 >= batch) break;
        const int n = batch - s0 < 64 ? (int)(batch - s0) : 64;
        const Vec *src = reinterpret_cast<const Vec *>(t + s0 * features + f0);
        uint32_t acc[8][V];
#pragma unroll
        for (int o = 0; o < 8; ++o) {
            Vec v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = o * 8 + j < n ? src[(int64_t)(o * 8 + j) * row_vecs] : Vec(0u);
#pragma unroll
            for (int q = 0; q < V; ++q) {
                uint32_t a = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t b = PackVec<V>::get(v[j], q);
                    const uint32_t nz = (((b & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | b) & 0x80808080u;
                    a = (a >> 1) | nz;
                }
                acc[o][q] = a;
            }
        }
        const int64_t byte0 = s0 / 8;
        const int64_t nbytes = row_bytes - byte0 < 8 ? row_bytes - byte0 : 8;
#pragma unroll
        for (int q = 0; q < V; ++q) {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int o = 0; o < 4; ++o) {
                    lo |= ((acc[o][q] >> (8 * b)) & 0xFFu) << (8 * o);
                    hi |= ((acc[4 + o][q] >> (8 * b)) & 0xFFu) << (8 * o);
                }
                uint8_t *dst = out + (f0 + 4 * q + b) * row_bytes + byte0;
                const uint64_t word = ((uint64_t)hi << 32) | lo;
                if (nbytes == 8 && (row_bytes & 7) == 0) {
                    *reinterpret_cast<uint64_t *>(dst) = word;
                } else {
                    for (int k = 0; k < nbytes; ++k) dst[k] = (uint8_t)(word >> (8 * k));
                }
            }
        }
    }
}

// The same bit gathering with the stores gone through LDS: a workgroup of FL feature lanes x SG sample groups packs
// 16 FL features x 64 SG samples, collects the words in LDS and writes SG consecutive words (8 SG bytes) of every feature
// row with consecutive lanes and streaming stores.  The 8-byte stores of the kernel above, scattered over rows, cost a
// third of its time (155 us against 100 us without them on bool [8192, 64000]).
template <int FL, int SG>
__global__ __launch_bounds__(FL *SG) void pack_bits_tile_kernel(const uint8_t *__restrict__ t, uint8_t *__restrict__ out,
                                                           int64_t features, int64_t batch, int64_t row_bytes)
{
    __shared__ uint64_t tile[FL * 16][SG + 1];
    const int fl = threadIdx.x % FL, sg = threadIdx.x / FL;
    const int64_t f0 = ((int64_t)blockIdx.x * FL + fl) * 16;
    const int64_t s0 = ((int64_t)blockIdx.y * SG + sg) * 64;
    uint32_t acc[8][4];
#pragma unroll
    for (int o = 0; o < 8; ++o)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[o][q] = 0;
    if (f0 < features && s0 < batch) {
        const int n = batch - s0 < 64 ? (int)(batch - s0) : 64;
        const int64_t row_vecs = features / 16;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(t + s0 * features + f0);
#pragma unroll
        for (int o = 0; o < 8; ++o) {
            u32x4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = o * 8 + j < n ? src[(int64_t)(o * 8 + j) * row_vecs] : u32x4(0u);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t a = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t b = v[j][q];
                    const uint32_t nz = (((b & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | b) & 0x80808080u;
                    a = (a >> 1) | nz;
                }
                acc[o][q] = a;
            }
        }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                lo |= ((acc[o][q] >> (8 * b)) & 0xFFu) << (8 * o);
                hi |= ((acc[4 + o][q] >> (8 * b)) & 0xFFu) << (8 * o);
            }
            tile[(4 * q + b) * FL + fl][sg] = ((uint64_t)hi << 32) | lo;   // feature-lane fastest: the lanes of a wavefront spread over the banks
        }
    }
    __syncthreads();
    const int64_t frow0 = (int64_t)blockIdx.x * FL * 16, grp0 = (int64_t)blockIdx.y * SG;
    for (int idx = threadIdx.x; idx < FL * 16 * SG; idx += FL * SG) {
        const int row = idx / SG, w = idx % SG;
        const int64_t f = frow0 + row, byte0 = (grp0 + w) * 8;
        if (f >= features || byte0 >= row_bytes) continue;
        const uint64_t word = tile[(row % 16) * FL + row / 16][w];
        uint8_t *dst = out + f * row_bytes + byte0;
        const int64_t nbytes = row_bytes - byte0 < 8 ? row_bytes - byte0 : 8;
        if (nbytes == 8 && (row_bytes & 7) == 0) {
            __builtin_nontemporal_store(word, reinterpret_cast<uint64_t *>(dst));
        } else {
            for (int k = 0; k < nbytes; ++k) dst[k] = (uint8_t)(word >> (8 * k));
        }
    }
}

template <int V, int G>
void launch_pack_smv(const uint8_t *t, void *words, int64_t features, int64_t batch, int64_t row_bytes, int64_t groups, hipStream_t st)
{
    hipLaunchKernelGGL((pack_bits_smv_kernel<V, G>), dim3((unsigned)clg_ceil_div(features / (4 * V), 256), (unsigned)clg_ceil_div(groups, G)),
                       dim3(256), 0, st, t, (uint8_t *)words, features, batch, row_bytes);
}

// ---------------------------------------------------------------------------------------------
// per-class bit counts
// ---------------------------------------------------------------------------------------------
// One wave per (class, 8-byte column): the 64 lanes are the 64 sample bits of that column; rows of
// the class are split over `slices` waves whose partial counts meet in integer atomics (exact, so the
// result does not depend on their order).
__global__ __launch_bounds__(256) void group_bit_sum_kernel(const uint8_t *__restrict__ x, int32_t *__restrict__ out,
                                                          int64_t class_rows, int64_t row_bytes, int64_t samples, int k,
                                                          int cols8, int slices)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int64_t item = (int64_t)blockIdx.x * 4 + wave;
    const int64_t total = (int64_t)k * cols8 * slices;
    if (item >= total) return;
    const int slice = (int)(item % slices);
    const int col = (int)((item / slices) % cols8);
    const int g = (int)(item / ((int64_t)slices * cols8));
    const int64_t r0 = class_rows * slice / slices, r1 = class_rows * (slice + 1) / slices;
    const int64_t byte0 = (int64_t)col * 8;
    const int nbytes = row_bytes - byte0 < 8 ? (int)(row_bytes - byte0) : 8;
    const uint8_t *base = x + (int64_t)g * class_rows * row_bytes + byte0;
    int32_t acc = 0;
    if (nbytes == 8 && (row_bytes & 7) == 0) {
        for (int64_t r = r0; r < r1; ++r) {
            const uint64_t wv = *reinterpret_cast<const uint64_t *>(base + r * row_bytes);
            acc += (int32_t)((wv >> lane) & 1);
        }
    } else {
        for (int64_t r = r0; r < r1; ++r) {
            uint64_t wv = 0;
            for (int b = 0; b < nbytes; ++b) wv |= (uint64_t)base[r * row_bytes + b] << (8 * b);
            acc += (int32_t)((wv >> lane) & 1);
        }
    }
    const int64_t s = byte0 * 8 + lane;
    if (s < samples) {
        if (slices == 1) out[s * k + g] = acc;
        else atomicAdd(out + s * k + g, acc);
    }
}

// Many samples: lanes along 8-byte columns, so a wavefront reads 512 contiguous bytes of a row.  A
// workgroup owns 64 columns of one class (and one row slice); its 8 wavefronts split the rows.  Every
// thread counts the 64 bit positions of its column with vertical counters (plane p holds bit p of the 64
// running counts): four words are combined by three carry-save adders and the resulting "fours" word
// ripples into planes 2 and up.  The wavefronts' planes meet in LDS, are added as binary numbers, and
// every wavefront expands 8 of the 64 bit positions into counts.
constexpr int kCountPlanes = 14;                                     // a wavefront counts at most 2^14 - 8 rows
constexpr int kCountWaves = 8;
__device__ __forceinline__ void csa(uint64_t &hi, uint64_t &lo, uint64_t a, uint64_t b, uint64_t c)
{
    const uint64_t u = a ^ b;
    hi = (a & b) | (u & c);
    lo = u ^ c;
}
__device__ __forceinline__ void count8(uint64_t (&plane)[kCountPlanes], const uint64_t (&w)[8])
{
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint64_t two_a, two_b, four;
        csa(two_a, plane[0], plane[0], w[4 * h], w[4 * h + 1]);
        csa(two_b, plane[0], plane[0], w[4 * h + 2], w[4 * h + 3]);
        csa(four, plane[1], plane[1], two_a, two_b);
#pragma unroll
        for (int q = 2; q < kCountPlanes; ++q) {
            const uint64_t t = plane[q] & four;
            plane[q] ^= four;
            four = t;
        }
    }
}
__global__ __launch_bounds__(kCountWaves *kWave) void group_bit_sum_columns_kernel(const uint64_t *__restrict__ x,
                                                                                  int32_t *__restrict__ out, int64_t class_rows,
                                                                                  int64_t row_words, int64_t samples, int k,
                                                                                  int slices)
{
    __shared__ uint64_t meet[kCountWaves][kCountPlanes][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = uniform((int)(threadIdx.x >> 6));
    const int64_t col = (int64_t)blockIdx.x * kWave + lane;
    const bool live = col < row_words;
    const int g = blockIdx.y;
    const int part = blockIdx.z * kCountWaves + wave, parts = slices * kCountWaves;
    const int64_t r0 = class_rows * part / parts, r1 = class_rows * (part + 1) / parts;
    const uint64_t *p = x + ((int64_t)g * class_rows + r0) * row_words + (live ? col : 0);
    uint64_t plane[kCountPlanes];
#pragma unroll
    for (int q = 0; q < kCountPlanes; ++q) plane[q] = 0;
    int64_t r = r0;
    if (r + 8 <= r1) {
        uint64_t cur[8], nxt[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) cur[j] = p[(int64_t)j * row_words];
        p += 8 * row_words;
        r += 8;
        for (; r + 8 <= r1; r += 8) {                                // next 8 rows are in flight while these are counted
#pragma unroll
            for (int j = 0; j < 8; ++j) nxt[j] = p[(int64_t)j * row_words];
            p += 8 * row_words;
            count8(plane, cur);
#pragma unroll
            for (int j = 0; j < 8; ++j) cur[j] = nxt[j];
        }
        count8(plane, cur);
    }
    for (; r < r1; ++r) {
        uint64_t carry = *p;
        p += row_words;
#pragma unroll
        for (int q = 0; q < kCountPlanes; ++q) {
            const uint64_t t = plane[q] & carry;
            plane[q] ^= carry;
            carry = t;
        }
    }
#pragma unroll
    for (int q = 0; q < kCountPlanes; ++q) meet[wave][q][lane] = plane[q];
    __syncthreads();
    // total = sum of the wavefronts' counters, as binary numbers spread over the planes (a total above
    // 2^14 - 1 cannot occur: the host keeps the rows of a workgroup below that)
#pragma unroll
    for (int q = 0; q < kCountPlanes; ++q) plane[q] = meet[0][q][lane];
    for (int wv = 1; wv < kCountWaves; ++wv) {
        uint64_t carry = 0;
#pragma unroll
        for (int q = 0; q < kCountPlanes; ++q) {
            const uint64_t b = meet[wv][q][lane], u = plane[q] ^ b;
            const uint64_t c = (plane[q] & b) | (u & carry);
            plane[q] = u ^ carry;
            carry = c;
        }
    }
    if (!live) return;
    const int64_t s0 = col * 64;
#pragma unroll
    for (int bb = 0; bb < 64 / kCountWaves; ++bb) {
        const int b = wave * (64 / kCountWaves) + bb;
        if (s0 + b >= samples) break;
        int32_t cnt = 0;
#pragma unroll
        for (int q = 0; q < kCountPlanes; ++q) cnt |= (int32_t)((plane[q] >> b) & 1) << q;
        if (slices == 1) out[(s0 + b) * k + g] = cnt;
        else atomicAdd(out + (s0 + b) * k + g, cnt);
    }
}

__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

int small_grid(int64_t items, int block)
{
    const int64_t g = clg_ceil_div(items, block);
    return (int)(g < 1 ? 1 : (g > 65536 * 16 ? 65536 * 16 : g));
}

template <typename V>
void launch_eval(const void *x, const int64_t *a, const int64_t *b, const uint8_t *gate, void *y, int64_t out_dim,
                 int64_t row_bytes, hipStream_t st, int64_t in_dim)
{
    const int64_t row_vecs = row_bytes / (int64_t)sizeof(V);
    // column chunks of at most 4 KiB per row: both uses of a row segment fall inside one chunk pass,
    // so the working set of a pass (in_dim x 4 KiB) can stay in the last-level cache (measured best on
    // 64000 x 8 KiB rows among 0.5..8 KiB).  CLG_EVAL_CHUNK_BYTES / CLG_EVAL_NPW override for tuning.
    const char *e_chunk = clg_knob(K_EVAL_CHUNK_BYTES), *e_npw = clg_knob(K_EVAL_NPW);
    const int max_chunk_vecs = (e_chunk ? atoi(e_chunk) : 4096) / (int)sizeof(V);
    const int chunk_vecs = row_vecs < max_chunk_vecs ? (int)row_vecs : max_chunk_vecs;
    const int chunks = (int)clg_ceil_div(row_vecs, chunk_vecs);
    const int neurons_per_wave = e_npw ? atoi(e_npw) : 1;
    const int groups = (int)clg_ceil_div(out_dim, (int64_t)kEvalWaves * neurons_per_wave);
    hipLaunchKernelGGL((eval_packed_kernel<V, 2>), dim3((unsigned)(chunks * groups)), dim3(kEvalBlock), 0, st, (const V *)x, a,
                       b, gate, (V *)y, (int)out_dim, row_vecs, chunk_vecs, groups, neurons_per_wave, in_dim);
}

bool valid_elem(int e) { return e == 1 || e == 2 || e == 4 || e == 8; }

}  // namespace

extern "C" int clg_fc_eval_packed(int elem_size, const void *x, const int64_t *a, const int64_t *b, const uint8_t *gate,
                                  void *y, int64_t in_dim, int64_t out_dim, int64_t words, void *stream)
{
    CLG_REQUIRE(valid_elem(elem_size), "clg_fc_eval_packed: elem_size must be 1, 2, 4 or 8, got %d", elem_size);
    CLG_REQUIRE(x && a && b && gate && y, "clg_fc_eval_packed: null pointer argument");
    CLG_REQUIRE(x != y, "clg_fc_eval_packed: x and y must not overlap");
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && words > 0, "clg_fc_eval_packed: in_dim, out_dim and words must be positive");
    CLG_REQUIRE(out_dim < (1ll << 31), "clg_fc_eval_packed: out_dim above 2^31-1 is not supported");
    const int64_t row_bytes = words * elem_size;
    const uintptr_t align = (uintptr_t)x | (uintptr_t)y | (uintptr_t)row_bytes;
    hipStream_t st = clg_stream(stream);
    const int64_t blocks_needed = clg_ceil_div(row_bytes, 2048) * clg_ceil_div(out_dim, 16);
    if (blocks_needed >= (1ll << 31)) {
        CLG_REQUIRE(false, "clg_fc_eval_packed: problem too large for one launch (%lld blocks)", (long long)blocks_needed);
    }
    if ((align & 15) == 0) launch_eval<u32x4>(x, a, b, gate, y, out_dim, row_bytes, st, in_dim);
    else if ((align & 7) == 0) launch_eval<u32x2>(x, a, b, gate, y, out_dim, row_bytes, st, in_dim);
    else if ((align & 3) == 0) launch_eval<uint32_t>(x, a, b, gate, y, out_dim, row_bytes, st, in_dim);
    else
        hipLaunchKernelGGL(eval_packed_bytes_kernel, dim3(small_grid(out_dim * row_bytes, 256)), dim3(256), 0, st,
                           (const uint8_t *)x, a, b, gate, (uint8_t *)y, out_dim, row_bytes, in_dim);
    CLG_CHECK_LAUNCH("clg_fc_eval_packed");
    return CLG_OK;
}

static int check_pack(const void *t, void *words, int64_t features, int64_t batch, int bit_count, const char *name)
{
    CLG_REQUIRE(t && words, "%s: null pointer argument", name);
    CLG_REQUIRE(bit_count == 8 || bit_count == 16 || bit_count == 32 || bit_count == 64,
                "%s: `bit_count` has to be in { 8, 16, 32, 64 }, got %d", name, bit_count);
    CLG_REQUIRE(features > 0 && batch > 0, "%s: features and batch must be positive", name);
    return CLG_OK;
}

extern "C" int clg_pack_bits(const uint8_t *t, void *words, int64_t features, int64_t batch, int bit_count, void *stream)
{
    if (int e = check_pack(t, words, features, batch, bit_count, "clg_pack_bits")) return e;
    const int64_t row_bytes = clg_ceil_div(batch, bit_count) * (bit_count / 8);
    const bool aligned8 = (batch % 8 == 0) && (((uintptr_t)t & 7) == 0);
    hipLaunchKernelGGL(pack_bits_kernel, dim3(small_grid(features * row_bytes, 256)), dim3(256), 0, clg_stream(stream), t,
                       (uint8_t *)words, features, batch, row_bytes, aligned8);
    CLG_CHECK_LAUNCH("clg_pack_bits");
    return CLG_OK;
}

extern "C" int clg_pack_bits_sample_major(const uint8_t *t, void *words, int64_t features, int64_t batch, int bit_count,
                                          void *stream)
{
    if (int e = check_pack(t, words, features, batch, bit_count, "clg_pack_bits_sample_major")) return e;
    const int64_t row_bytes = clg_ceil_div(batch, bit_count) * (bit_count / 8);
    const int64_t groups = clg_ceil_div(batch, 64);
    if (features % 16 == 0 && ((uintptr_t)t & 15) == 0 && ((uintptr_t)words & 7) == 0 && groups <= 65535) {
        // 16 features per lane, 2 groups per thread: best of 4..16 features x 2..16 groups (3.8 TB/s on bool [8192, 64000])
        // from 8 groups of 64 samples on, the words go through LDS and leave as 64 (8..15 groups) or 128 contiguous bytes per
        // feature row: 155 -> 121 us on bool [8192, 64000], 101 -> 52 us on [65536, 4096] with 32 feature lanes x 16 groups
        // (512 threads; 16 x 16 and 64 x 8 are 8 % slower); CLG_PACK_TILE=0 keeps the direct stores
        const char *e_tile = clg_knob(K_PACK_TILE);
        const bool tiled = !e_tile || atoi(e_tile) != 0;
        if (tiled && groups >= 16)
            hipLaunchKernelGGL((pack_bits_tile_kernel<32, 16>), dim3((unsigned)clg_ceil_div(features, 32 * 16), (unsigned)clg_ceil_div(groups, 16)),
                               dim3(512), 0, clg_stream(stream), t, (uint8_t *)words, features, batch, row_bytes);
        else if (tiled && groups >= 8)
            hipLaunchKernelGGL((pack_bits_tile_kernel<32, 8>), dim3((unsigned)clg_ceil_div(features, 32 * 16), (unsigned)clg_ceil_div(groups, 8)),
                               dim3(256), 0, clg_stream(stream), t, (uint8_t *)words, features, batch, row_bytes);
        else
            launch_pack_smv<4, 2>(t, words, features, batch, row_bytes, groups, clg_stream(stream));
    } else {
        const int64_t gy = clg_ceil_div(groups, kPackGroups);
        CLG_REQUIRE(gy <= 65535, "clg_pack_bits_sample_major: batch above %lld samples is not supported", 65535ll * kPackGroups * 64);
        hipLaunchKernelGGL(pack_bits_sm_kernel, dim3((unsigned)clg_ceil_div(features, 256), (unsigned)gy), dim3(256), 0,
                           clg_stream(stream), t, (uint8_t *)words, features, batch, row_bytes);
    }
    CLG_CHECK_LAUNCH("clg_pack_bits_sample_major");
    return CLG_OK;
}

extern "C" int clg_group_bit_sum(int elem_size, const void *x, int32_t *out, int64_t features, int64_t words, int64_t pad_len,
                                 int64_t k, void *stream)
{
    CLG_REQUIRE(valid_elem(elem_size), "clg_group_bit_sum: elem_size must be 1, 2, 4 or 8, got %d", elem_size);
    CLG_REQUIRE(x && out, "clg_group_bit_sum: null pointer argument");
    CLG_REQUIRE(features > 0 && words > 0 && k > 0, "clg_group_bit_sum: features, words and k must be positive");
    CLG_REQUIRE(features % k == 0, "in_dim (%lld) has to be divisible by k (%lld) but it is not", (long long)features, (long long)k);
    const int64_t row_bytes = words * elem_size, samples = row_bytes * 8 - pad_len;
    CLG_REQUIRE(pad_len >= 0 && samples > 0, "clg_group_bit_sum: pad_len %lld leaves no samples", (long long)pad_len);
    CLG_REQUIRE(k < (1 << 20), "clg_group_bit_sum: k too large");
    const int cols8 = (int)clg_ceil_div(row_bytes, 8);
    const int64_t class_rows = features / k;
    hipStream_t st = clg_stream(stream);
    if ((row_bytes & 7) == 0 && ((uintptr_t)x & 7) == 0 && cols8 >= 64 && k <= 65535) {
        // wide rows: lanes along columns, vertical counters.  One workgroup takes all rows of its 64 columns and
        // class (no atomics, no zero fill: measured 101 us against 164 us with two row slices at 64000 x 1024
        // words); rows are sliced only beyond the counter range of 2^14 - 8 rows per workgroup.
        const int64_t row_words = row_bytes / 8;
        const int64_t col_blocks = clg_ceil_div(row_words, kWave);
        const char *e_sl = clg_knob(K_GSUM_SLICES);
        int64_t slices = e_sl ? atoi(e_sl) : 1;
        if (slices > class_rows / (64 * kCountWaves)) slices = class_rows / (64 * kCountWaves);
        const int64_t need = clg_ceil_div(class_rows, (1 << kCountPlanes) - 8);
        if (slices < need) slices = need;
        if (slices < 1) slices = 1;
        CLG_REQUIRE(slices <= 65535 && col_blocks < (1ll << 31), "clg_group_bit_sum: problem too large for one launch");
        if (slices > 1)
            hipLaunchKernelGGL(fill_zero_i32_kernel, dim3(small_grid(samples * k, 256)), dim3(256), 0, st, out, samples * k);
        hipLaunchKernelGGL(group_bit_sum_columns_kernel, dim3((unsigned)col_blocks, (unsigned)k, (unsigned)slices),
                           dim3(kCountWaves * kWave), 0, st, (const uint64_t *)x, out, class_rows, row_words, samples, (int)k,
                           (int)slices);
        CLG_CHECK_LAUNCH("clg_group_bit_sum");
        return CLG_OK;
    }
    // enough waves to fill the GPU, at least 64 rows per slice
    int64_t slices = clg_ceil_div(16384, (int64_t)k * cols8);
    if (slices > class_rows / 64) slices = class_rows / 64;
    if (slices < 1) slices = 1;
    if (slices > 1)
        hipLaunchKernelGGL(fill_zero_i32_kernel, dim3(small_grid(samples * k, 256)), dim3(256), 0, st, out, samples * k);
    const int64_t items = k * cols8 * slices;
    CLG_REQUIRE(clg_ceil_div(items, 4) < (1ll << 31), "clg_group_bit_sum: problem too large for one launch");
    hipLaunchKernelGGL(group_bit_sum_kernel, dim3((unsigned)clg_ceil_div(items, 4)), dim3(256), 0, st, (const uint8_t *)x, out,
                       class_rows, row_bytes, samples, (int)k, cols8, (int)slices);
    CLG_CHECK_LAUNCH("clg_group_bit_sum");
    return CLG_OK;
}

// ---- walk plan (host side) --------------------------------------------------------------------
extern "C" int clg_fc_eval_plan(const int64_t *a, const int64_t *b, int64_t in_dim, int64_t out_dim, int32_t *plan)
{
    CLG_REQUIRE(a && b && plan, "clg_fc_eval_plan: null pointer argument");
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && out_dim < (1ll << 28), "clg_fc_eval_plan: out_dim must be in 1..2^28-1");
    // adjacency: edges (neurons) incident to each vertex (input row); a self-paired neuron is listed twice
    int64_t *start = (int64_t *)calloc((size_t)in_dim + 1, sizeof(int64_t));
    int32_t *adj = (int32_t *)malloc((size_t)out_dim * 2 * sizeof(int32_t));
    int64_t *fill = (int64_t *)malloc((size_t)in_dim * sizeof(int64_t));
    uint8_t *used = (uint8_t *)calloc((size_t)out_dim, 1);
    if (!start || !adj || !fill || !used) {
        free(start); free(adj); free(fill); free(used);
        clg_set_error("clg_fc_eval_plan: out of host memory");
        return CLG_EINVAL;
    }
    for (int64_t j = 0; j < out_dim; ++j) {
        if (a[j] < 0 || a[j] >= in_dim || b[j] < 0 || b[j] >= in_dim) {
            free(start); free(adj); free(fill); free(used);
            clg_set_error("clg_fc_eval_plan: neuron %lld is wired to a feature outside 0..%lld", (long long)j, (long long)in_dim - 1);
            return CLG_EINVAL;
        }
        ++start[a[j] + 1];
        ++start[b[j] + 1];
    }
    for (int64_t v = 0; v < in_dim; ++v) start[v + 1] += start[v];
    for (int64_t v = 0; v < in_dim; ++v) fill[v] = start[v];
    for (int64_t j = 0; j < out_dim; ++j) {
        adj[fill[a[j]]++] = (int32_t)j;
        adj[fill[b[j]]++] = (int32_t)j;
    }
    for (int64_t v = 0; v < in_dim; ++v) fill[v] = start[v];       // now: scan position per vertex
    int64_t n = 0;
    // trails start at odd-degree vertices first (pass 0), then anywhere edges remain (pass 1)
    for (int pass = 0; pass < 2; ++pass) {
        for (int64_t v0 = 0; v0 < in_dim; ++v0) {
            if (pass == 0 && ((start[v0 + 1] - start[v0]) & 1) == 0) continue;
            int64_t v = v0;
            bool carried = false;
            for (;;) {
                while (fill[v] < start[v + 1] && used[adj[fill[v]]]) ++fill[v];
                if (fill[v] == start[v + 1]) break;
                const int32_t e = adj[fill[v]++];
                used[e] = 1;
                const int64_t other = a[e] == v ? b[e] : a[e];
                int use = 0;
                if (carried) use = (a[e] == v ? 1 : 0) | (b[e] == v ? 2 : 0);
                const int keep = other == b[e] ? 1 : 0;
                plan[n++] = e | (use << 28) | (keep << 30);
                v = other;
                carried = true;
            }
        }
    }
    free(start); free(adj); free(fill); free(used);
    CLG_REQUIRE(n == out_dim, "clg_fc_eval_plan: internal error, %lld of %lld neurons placed", (long long)n, (long long)out_dim);
    return CLG_OK;
}

namespace {
// rows the walk kernel takes: whole 16-byte vectors at 16-byte aligned addresses, at least 1 KiB long (shorter rows gain
// nothing from carrying a row in registers)
bool walk_fits(int elem_size, const void *x, const void *y, int64_t words)
{
    const int64_t row_bytes = words * elem_size;
    const uintptr_t align = (uintptr_t)x | (uintptr_t)y | (uintptr_t)row_bytes;
    return (align & 15) == 0 && row_bytes >= 1024;
}

template <bool LOGITS>
int launch_walk(const char *name, int elem_size, const void *x, const int64_t *a, const int64_t *b, const void *gate, const int32_t *plan,
                void *y, int64_t in_dim, int64_t out_dim, int64_t words, void *stream)
{
    const int64_t row_vecs = words * elem_size / 16;
    const char *e_r = clg_knob(K_EVAL_WALK_R), *e_l = clg_knob(K_EVAL_WALK_SEG);
    int R = e_r ? atoi(e_r) : 4;
    while (R > 1 && (int64_t)kWave * (R / 2) >= row_vecs) R /= 2;
    const int seg = e_l ? atoi(e_l) : 8;
    const int64_t col_chunks = clg_ceil_div(row_vecs, (int64_t)kWave * R);
    CLG_REQUIRE(col_chunks <= 65535, "%s: rows above %lld bytes are not supported", name, 65535ll * kWave * R * 16);
    const dim3 grid((unsigned)clg_ceil_div(out_dim, (int64_t)kEvalWaves * seg), (unsigned)col_chunks), block(kEvalBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_WALK(RR)                                                                                                          \
    hipLaunchKernelGGL((eval_packed_walk_kernel<RR, LOGITS>), grid, block, 0, st, (const u32x4 *)x, a, b, gate, plan, (u32x4 *)y, \
                       (int)out_dim, seg, row_vecs, in_dim)
    switch (R) {
    case 1: CLG_WALK(1); break;
    case 2: CLG_WALK(2); break;
    case 4: CLG_WALK(4); break;
    default: CLG_WALK(8); break;
    }
#undef CLG_WALK
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}
}  // namespace

extern "C" int clg_fc_eval_packed_planned(int elem_size, const void *x, const int64_t *a, const int64_t *b, const uint8_t *gate,
                                          const int32_t *plan, void *y, int64_t in_dim, int64_t out_dim, int64_t words,
                                          void *stream)
{
    const char *name = "clg_fc_eval_packed_planned";
    CLG_REQUIRE(valid_elem(elem_size), "%s: elem_size must be 1, 2, 4 or 8, got %d", name, elem_size);
    CLG_REQUIRE(x && a && b && gate && plan && y, "%s: null pointer argument", name);
    CLG_REQUIRE(x != y, "%s: x and y must not overlap", name);
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && words > 0, "%s: in_dim, out_dim and words must be positive", name);
    CLG_REQUIRE(out_dim < (1ll << 28), "%s: out_dim above 2^28-1 is not supported", name);
    if (!walk_fits(elem_size, x, y, words)) return clg_fc_eval_packed(elem_size, x, a, b, gate, y, in_dim, out_dim, words, stream);
    return launch_walk<false>(name, elem_size, x, a, b, gate, plan, y, in_dim, out_dim, words, stream);
}

extern "C" int clg_fc_eval_walk_fits(int elem_size, const void *x, const void *y, int64_t words)
{
    return valid_elem(elem_size) && x && y && words > 0 && walk_fits(elem_size, x, y, words) ? 1 : 0;
}

extern "C" int clg_fc_eval_packed_planned_logits(int elem_size, const void *x, const int64_t *a, const int64_t *b, const float *logits,
                                                 const int32_t *plan, void *y, int64_t in_dim, int64_t out_dim, int64_t words,
                                                 void *stream)
{
    const char *name = "clg_fc_eval_packed_planned_logits";
    CLG_REQUIRE(valid_elem(elem_size), "%s: elem_size must be 1, 2, 4 or 8, got %d", name, elem_size);
    CLG_REQUIRE(x && a && b && logits && plan && y, "%s: null pointer argument", name);
    CLG_REQUIRE(x != y, "%s: x and y must not overlap", name);
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && words > 0, "%s: in_dim, out_dim and words must be positive", name);
    CLG_REQUIRE(out_dim < (1ll << 28), "%s: out_dim above 2^28-1 is not supported", name);
    CLG_REQUIRE(walk_fits(elem_size, x, y, words), "%s: rows must be whole 16-byte vectors of at least 1 KiB at 16-byte aligned addresses "
                "(clg_fc_eval_walk_fits); use clg_gate_argmax + clg_fc_eval_packed_planned otherwise", name);
    return launch_walk<true>(name, elem_size, x, a, b, logits, plan, y, in_dim, out_dim, words, stream);
}
