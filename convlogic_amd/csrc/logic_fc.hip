// Fully connected logic layer, feature-major: x [in_dim, batch], y [out_dim, batch].
//
// One wavefront owns one neuron (forward, weight gradient) or one input feature (input
// gradient) and streams its rows with 64 lanes x VEC samples, so every global access is a
// contiguous row segment.  The neuron index is wave-uniform: wiring indices and the 16 gate
// probabilities come through the scalar cache and are folded to 4 coefficients in SGPR-uniform
// registers; the per-sample work is one multiply and three FMAs.
#include <hip/hip_fp16.h>

#include <mutex>

#include "clg_common.h"

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * kWave;

template <typename T, int VEC>
struct VecT;
template <>
struct VecT<float, 4> { using type = float4; };
template <>
struct VecT<float, 1> { using type = float; };
template <>
struct VecT<double, 2> { using type = double2; };
template <>
struct VecT<double, 1> { using type = double; };

template <typename T, int VEC>
struct Pack {
    T v[VEC];
};

// Storage type S of a tensor and the type its values are computed in: half is a storage format only, the arithmetic
// of such tensors runs in float32.
template <typename S>
struct ComputeOf { using type = S; };
template <>
struct ComputeOf<__half> { using type = float; };

template <typename S, int VEC>
__device__ __forceinline__ Pack<typename ComputeOf<S>::type, VEC> load_vec(const S *p)
{
    using T = typename ComputeOf<S>::type;
    if constexpr (sizeof(S) == 2) {
        Pack<T, VEC> r;
        if constexpr (VEC == 8) {
            const u32x4 raw = *reinterpret_cast<const u32x4 *>(p);
            __half h[8];
            __builtin_memcpy(h, &raw, 16);
#pragma unroll
            for (int k = 0; k < 8; ++k) r.v[k] = __half2float(h[k]);
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = __half2float(p[k]);
        }
        return r;
    } else {
        using V = typename VecT<T, VEC>::type;
        const V r = *reinterpret_cast<const V *>(p);
        return __builtin_bit_cast(Pack<T, VEC>, r);
    }
}
template <typename S, int VEC>
__device__ __forceinline__ void store_vec(S *p, const Pack<typename ComputeOf<S>::type, VEC> &v)
{
    using T = typename ComputeOf<S>::type;
    if constexpr (sizeof(S) == 2) {
        if constexpr (VEC == 8) {
            __half h[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) h[k] = __float2half(v.v[k]);
            u32x4 raw;
            __builtin_memcpy(&raw, h, 16);
            *reinterpret_cast<u32x4 *>(p) = raw;
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) p[k] = __float2half(v.v[k]);
        }
    } else {
        using V = typename VecT<T, VEC>::type;
        *reinterpret_cast<V *>(p) = __builtin_bit_cast(V, v);
    }
}
template <typename S>
__device__ __forceinline__ typename ComputeOf<S>::type load_one(const S *p)
{
    if constexpr (sizeof(S) == 2) return __half2float(*p);
    else return *p;
}
template <typename S>
__device__ __forceinline__ void store_one(S *p, typename ComputeOf<S>::type v)
{
    if constexpr (sizeof(S) == 2) *p = __float2half(v);
    else *p = v;
}
// fold16 of 16 stored probabilities
template <typename S>
__device__ __forceinline__ Coef<typename ComputeOf<S>::type> fold16_stored(const S *__restrict__ w)
{
    if constexpr (sizeof(S) == 2) {
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = __half2float(w[i]);
        return fold16(t);
    } else {
        return fold16(w);
    }
}

// folded = 4 coefficients per neuron, written by fc_fold_kernel
template <typename T>
__device__ __forceinline__ Coef<T> load_coef(const T *__restrict__ f)
{
    Coef<T> c;
    if constexpr (sizeof(T) == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(f);
        c.ab = v.x, c.a = v.y, c.b = v.z, c.one = v.w;
    } else {
        const double2 u = *reinterpret_cast<const double2 *>(f), v = *reinterpret_cast<const double2 *>(f + 2);
        c.ab = u.x, c.a = u.y, c.b = v.x, c.one = v.y;
    }
    return c;
}

template <typename S, int VEC>
__global__ __launch_bounds__(kBlock) void fc_forward_kernel(const S *__restrict__ x, const int64_t *__restrict__ a,
                                                          const int64_t *__restrict__ b, const S *__restrict__ w,
                                                          S *__restrict__ y, int out_dim, int64_t batch, int in_dim)
{
    using T = typename ComputeOf<S>::type;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    for (int j = blockIdx.x * kWavesPerBlock + wave; j < out_dim; j += gridDim.x * kWavesPerBlock) {
        const S *xa = x + clamp_index(a[j], in_dim) * batch;
        const S *xb = x + clamp_index(b[j], in_dim) * batch;
        S *yj = y + (int64_t)j * batch;
        const Coef<T> c = fold16_stored(w + (int64_t)j * 16);
        for (int64_t s = (int64_t)lane * VEC; s < batch; s += kWave * VEC) {
            const Pack<T, VEC> va = load_vec<S, VEC>(xa + s), vb = load_vec<S, VEC>(xb + s);
            Pack<T, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = gate(c, va.v[k], vb.v[k]);
            store_vec<S, VEC>(yj + s, r);
        }
    }
}

// Sum over each group of LPR lanes: valid in the last 16 lanes of the group.
template <typename T, int LPR>
__device__ __forceinline__ T lane_group_sum(T v)
{
    if constexpr (LPR == 64) {
        return wave_sum(v);
    } else {
        v = row16_sum(v);
        if constexpr (LPR == 32) v += dpp_zero<0x142, 0xA>(v);   // row_bcast15: rows 1 and 3 add the row before them
        return v;
    }
}

// A neuron's row takes LPR lanes x VEC samples per pass, a wavefront 64/LPR neurons; the last 16 lanes of each
// group hold the four sums and write the 16 gate gradients.
template <typename S, int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void fc_backward_w_kernel(const S *__restrict__ x, const int64_t *__restrict__ a,
                                                             const int64_t *__restrict__ b,
                                                             const S *__restrict__ gy, S *__restrict__ gw, int out_dim,
                                                             int64_t batch, const S *__restrict__ probs, int in_dim)
{
    using T = typename ComputeOf<S>::type;
    constexpr int ROWS = kWave / LPR;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int sub = lane / LPR, l = lane % LPR;
    for (int64_t j0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * ROWS; j0 < out_dim;
         j0 += (int64_t)gridDim.x * kWavesPerBlock * ROWS) {
        const bool valid = j0 + sub < out_dim;
        const int64_t j = valid ? j0 + sub : out_dim - 1;           // every lane takes part in the reductions
        const S *xa = x + clamp_index(a[j], in_dim) * batch;
        const S *xb = x + clamp_index(b[j], in_dim) * batch;
        const S *gj = gy + j * batch;
        T sab = 0, sa = 0, sb = 0, s1 = 0;
        for (int64_t s = (int64_t)l * VEC; s < batch; s += LPR * VEC) {
            const Pack<T, VEC> va = load_vec<S, VEC>(xa + s), vb = load_vec<S, VEC>(xb + s),
                               vg = load_vec<S, VEC>(gj + s);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                sab = fma_t(vg.v[k], va.v[k] * vb.v[k], sab);
                sa = fma_t(vg.v[k], va.v[k], sa);
                sb = fma_t(vg.v[k], vb.v[k], sb);
                s1 += vg.v[k];
            }
        }
        sab = lane_group_sum<T, LPR>(sab);
        sa = lane_group_sum<T, LPR>(sa);
        sb = lane_group_sum<T, LPR>(sb);
        s1 = lane_group_sum<T, LPR>(s1);
        if (l >= LPR - 16) {
            const int i = lane & 15;
            T gi = coef_transpose_row<T>(i, sab, sa, sb, s1);
            if (probs != nullptr) gi = softmax16_backward(gi, load_one(probs + j * 16 + i));   // gradient w.r.t. the logits
            if (valid) store_one(gw + j * 16 + i, gi);
        }
    }
}

// Both gradients in one pass for layers in which every input feature is read by exactly one neuron operand
// (2 out_dim = in_dim with the reference's random wiring): the input gradient of such a feature is a single
// product, so the neuron that reads it writes its row and no gather over consumers is needed.  Same arithmetic
// as fc_backward_w_kernel and fc_backward_x_folded_kernel; 3 row reads and 2 row writes per neuron instead of 7 and 2.
// CLASSES: the layer feeds a GroupSum and gy is the gradient of ITS output, [batch, k]: the gradient of neuron j's row is
// gy[b][j / class_rows] * inv_tau, formed here instead of being written out by one kernel and read back by this one.
template <typename T, int VEC, int LPR, bool CLASSES = false>
__global__ __launch_bounds__(kBlock) void fc_backward_sole_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                                const int64_t *__restrict__ b, const T *__restrict__ folded,
                                                                const T *__restrict__ gy, T *__restrict__ gx,
                                                                T *__restrict__ gw, int out_dim, int64_t batch,
                                                                const T *__restrict__ probs, int k = 0, int64_t class_rows = 1,
                                                                T inv_tau = T(1))
{
    constexpr int ROWS = kWave / LPR;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int sub = lane / LPR, l = lane % LPR;
    for (int64_t j0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * ROWS; j0 < out_dim;
         j0 += (int64_t)gridDim.x * kWavesPerBlock * ROWS) {
        const bool valid = j0 + sub < out_dim;
        const int64_t j = valid ? j0 + sub : out_dim - 1;           // every lane takes part in the reductions
        const int64_t ia = clamp_index(a[j], 2 * (int64_t)out_dim), ib = clamp_index(b[j], 2 * (int64_t)out_dim);   // in_dim = 2 out_dim here
        const Coef<T> c = load_coef(folded + j * 4);
        const T *xa = x + ia * batch;
        const T *xb = x + ib * batch;
        const T *gj = CLASSES ? gy + j / class_rows : gy + j * batch;
        T sab = 0, sa = 0, sb = 0, s1 = 0;
        for (int64_t s = (int64_t)l * VEC; s < batch; s += LPR * VEC) {
            const Pack<T, VEC> va = load_vec<T, VEC>(xa + s), vb = load_vec<T, VEC>(xb + s);
            Pack<T, VEC> vg;
            if constexpr (CLASSES) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    vg.v[i] = gj[(s + i) * k] * inv_tau;             // (the product group_sum_backward writes out)
                    asm volatile("" : "+v"(vg.v[i]));                // the rounded product: no contraction into the sums below
                }
            } else {
                vg = load_vec<T, VEC>(gj + s);
            }
            Pack<T, VEC> ga, gb;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                sab = fma_t(vg.v[k], va.v[k] * vb.v[k], sab);
                sa = fma_t(vg.v[k], va.v[k], sa);
                sb = fma_t(vg.v[k], vb.v[k], sb);
                s1 += vg.v[k];
                ga.v[k] = fma_t(c.ab, vb.v[k], c.a) * vg.v[k];
                gb.v[k] = fma_t(c.ab, va.v[k], c.b) * vg.v[k];
            }
            if (valid) {
                store_vec<T, VEC>(gx + ia * batch + s, ga);
                store_vec<T, VEC>(gx + ib * batch + s, gb);
            }
        }
        sab = lane_group_sum<T, LPR>(sab);
        sa = lane_group_sum<T, LPR>(sa);
        sb = lane_group_sum<T, LPR>(sb);
        s1 = lane_group_sum<T, LPR>(s1);
        if (l >= LPR - 16) {
            const int i = lane & 15;
            T gi = coef_transpose_row<T>(i, sab, sa, sb, s1);
            if (probs != nullptr) gi = softmax16_backward(gi, probs[j * 16 + i]);   // gradient w.r.t. the logits
            if (valid) gw[j * 16 + i] = gi;
        }
    }
}

template <typename S, int VEC>
__global__ __launch_bounds__(kBlock) void fc_backward_x_kernel(const S *__restrict__ x, const int64_t *__restrict__ a,
                                                             const int64_t *__restrict__ b, const S *__restrict__ w,
                                                             const S *__restrict__ gy,
                                                             const int64_t *__restrict__ csr_start,
                                                             const int64_t *__restrict__ csr_list,
                                                             S *__restrict__ gx, int in_dim, int64_t batch,
                                                             int batch_chunks, int out_dim)
{
    using T = typename ComputeOf<S>::type;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = uniform(threadIdx.x >> 6);
    const int64_t items = (int64_t)in_dim * batch_chunks;
    for (int64_t it = (int64_t)blockIdx.x * kWavesPerBlock + wave; it < items; it += (int64_t)gridDim.x * kWavesPerBlock) {
        const int i = (int)(it / batch_chunks);
        const int64_t s = ((it % batch_chunks) * kWave + lane) * VEC;
        const bool live = s < batch;
        const int64_t beg = clamp_index(csr_start[i], 2 * (int64_t)out_dim + 1), end = clamp_index(csr_start[i + 1], 2 * (int64_t)out_dim + 1);
        // consumers in groups of four, one partial sum per position in the group (as fc_backward_x_folded_kernel,
        // whose results this kernel matches bit for bit)
        Pack<T, VEC> part[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int k = 0; k < VEC; ++k) part[u].v[k] = 0;
        int64_t prev = -1;
        for (int64_t cur = beg; cur < end; cur += 4) {
            int64_t j[4];
            Pack<T, VEC> vo[4], vg[4];
            T c_ab[4], c_lin[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                j[u] = cur + u < end ? clamp_index(csr_list[cur + u], out_dim) : -1;
                if (j[u] >= 0) {
                    const int64_t ia = clamp_index(a[j[u]], in_dim), ib = clamp_index(b[j[u]], in_dim);
                    const Coef<T> c = fold16_stored(w + j[u] * 16);
                    // Input i is operand A of neuron j unless only B matches; a neuron wired to the same
                    // feature twice appears twice in the list and takes the B derivative the second time.
                    const bool as_a = ia == i && !(ib == i && prev == j[u]);
                    c_ab[u] = c.ab;
                    c_lin[u] = as_a ? c.a : c.b;
                    if (live) {
                        vo[u] = load_vec<S, VEC>(x + (as_a ? ib : ia) * batch + s);
                        vg[u] = load_vec<S, VEC>(gy + j[u] * batch + s);
                    }
                }
                prev = j[u];
            }
            if (live) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (j[u] >= 0) {
#pragma unroll
                        for (int k = 0; k < VEC; ++k) part[u].v[k] = fma_t(fma_t(c_ab[u], vo[u].v[k], c_lin[u]), vg[u].v[k], part[u].v[k]);
                    }
                }
            }
        }
        Pack<T, VEC> acc;
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc.v[k] = (part[0].v[k] + part[1].v[k]) + (part[2].v[k] + part[3].v[k]);
        if (live) store_vec<S, VEC>(gx + (int64_t)i * batch + s, acc);
    }
}

// ---- folded-coefficient kernels ----------------------------------------------------------------
// The training path folds every neuron's 16 probabilities to 4 coefficients once per step (fc_fold_kernel)
// instead of once per wavefront that touches the neuron, and lets a wavefront carry several rows when one
// row of `batch` samples does not fill 64 lanes: a row takes LPR = 16, 32 or 64 lanes x VEC samples per pass,
// a wavefront 64/LPR rows.  Wiring indices and coefficients are per-lane loads (one address per row group).

// probs (optional) = softmax(logits) when from_logits, folded = fold16 of the probabilities
template <typename T>
__global__ __launch_bounds__(256) void fc_fold_kernel(const T *__restrict__ w_in, T *__restrict__ probs,
                                                     T *__restrict__ folded, int out_dim, int from_logits)
{
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= out_dim) return;
    T p[16];
    if (from_logits) {
        softmax16(w_in + (int64_t)j * 16, p);
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i] = w_in[(int64_t)j * 16 + i];
    }
    if (probs != nullptr) {
#pragma unroll
        for (int i = 0; i < 16; ++i) probs[(int64_t)j * 16 + i] = p[i];
    }
    const Coef<T> c = fold16(p);
    T *f = folded + (int64_t)j * 4;
    f[0] = c.ab;
    f[1] = c.a;
    f[2] = c.b;
    f[3] = c.one;
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void fc_forward_folded_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                                 const int64_t *__restrict__ b,
                                                                 const T *__restrict__ folded, T *__restrict__ y,
                                                                 int out_dim, int64_t batch, int lpr_log2, int in_dim)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int rows = kWave >> lpr_log2, sub = lane >> lpr_log2, l = lane & ((1 << lpr_log2) - 1);
    const int64_t pass = (int64_t)VEC << lpr_log2;
    for (int64_t j0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * rows; j0 < out_dim;
         j0 += (int64_t)gridDim.x * kWavesPerBlock * rows) {
        const int64_t j = j0 + sub;
        if (j >= out_dim) continue;
        const Coef<T> c = load_coef(folded + j * 4);
        const T *xa = x + clamp_index(a[j], in_dim) * batch;
        const T *xb = x + clamp_index(b[j], in_dim) * batch;
        T *yj = y + j * batch;
        for (int64_t s = (int64_t)l * VEC; s < batch; s += pass) {
            const Pack<T, VEC> va = load_vec<T, VEC>(xa + s), vb = load_vec<T, VEC>(xb + s);
            Pack<T, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = gate(c, va.v[k], vb.v[k]);
            store_vec<T, VEC>(yj + s, r);
        }
    }
}

// Forward from the LOGITS: the 16 lanes of every lane row hold the 16 logits of the row group's neuron, take the
// softmax with DPP reductions (maximum, sum, one reciprocal) and fold it to the 4 coefficients as four 16-lane dot
// products with the integer patterns of fold16; the first row writes probabilities and coefficients out for the
// backward pass.  One launch instead of fold + forward; the reductions ride on a kernel that waits for memory.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void fc_forward_logits_kernel(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                                 const int64_t *__restrict__ b,
                                                                 const T *__restrict__ logits, T *__restrict__ probs,
                                                                 T *__restrict__ folded, T *__restrict__ y, int out_dim,
                                                                 int64_t batch, int lpr_log2, int in_dim)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int rows = kWave >> lpr_log2, sub = lane >> lpr_log2, l = lane & ((1 << lpr_log2) - 1);
    const int q = lane & 15;
    // fold16 as dot products with integer patterns; c_1 = sum of gates 8..15
    constexpr int kAb[16] = {0, 1, -1, 0, -1, 0, -2, -1, 1, 2, 0, 1, 0, 1, -1, 0};
    constexpr int kA[16] = {0, 0, 1, 1, 0, 0, 1, 1, -1, -1, 0, 0, -1, -1, 0, 0};
    constexpr int kB[16] = {0, 0, 0, 0, 1, 1, 1, 1, -1, -1, -1, -1, 0, 0, 0, 0};
    int ab = 0, aa = 0, bb = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {                                    // selects, not a table in memory
        ab = q == i ? kAb[i] : ab;
        aa = q == i ? kA[i] : aa;
        bb = q == i ? kB[i] : bb;
    }
    const T w_ab = (T)ab, w_a = (T)aa, w_b = (T)bb, w_1 = q >= 8 ? T(1) : T(0);
    const int64_t pass = (int64_t)VEC << lpr_log2;
    for (int64_t j0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * rows; j0 < out_dim;
         j0 += (int64_t)gridDim.x * kWavesPerBlock * rows) {
        const bool valid = j0 + sub < out_dim;
        const int64_t j = valid ? j0 + sub : out_dim - 1;            // every lane takes part in the reductions
        const T lg = logits[j * 16 + q];
        const T e = exp(lg - row16_max(lg));
        const T p = e * (T(1) / row16_sum(e));
        Coef<T> c;
        c.ab = row16_sum(p * w_ab);
        c.a = row16_sum(p * w_a);
        c.b = row16_sum(p * w_b);
        c.one = row16_sum(p * w_1);
        if (valid && l < 16) {
            probs[j * 16 + q] = p;
            if (q < 4) folded[j * 4 + q] = q == 0 ? c.ab : (q == 1 ? c.a : (q == 2 ? c.b : c.one));
        }
        if (!valid) continue;
        const T *xa = x + clamp_index(a[j], in_dim) * batch;
        const T *xb = x + clamp_index(b[j], in_dim) * batch;
        T *yj = y + j * batch;
        for (int64_t s = (int64_t)l * VEC; s < batch; s += pass) {
            const Pack<T, VEC> va = load_vec<T, VEC>(xa + s), vb = load_vec<T, VEC>(xb + s);
            Pack<T, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = gate(c, va.v[k], vb.v[k]);
            store_vec<T, VEC>(yj + s, r);
        }
    }
}

// The walk of input i over its consumers, shared by the kernels below: returns the input gradient of the lane's VEC
// samples from s on, sum over the consumers j of gy[j] * d gate_j / d x_i, taken in groups of four with one partial
// sum per position in the group and added as (0 + 1) + (2 + 3).  Input i is operand A of neuron j unless only B
// matches; a neuron wired to the same feature twice appears twice in the list and takes the B derivative the second
// time.  With LPR != 0 (a row of the batch = LPR lanes x VEC samples, xi = the lane's samples of x[i]) the visit that
// reaches a neuron through its first operand also writes the neuron's 16 gate gradients.
template <typename T, int VEC, int LPR>
__device__ __forceinline__ Pack<T, VEC> fc_walk_consumers(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                          const int64_t *__restrict__ b, const T *__restrict__ folded,
                                                          const T *__restrict__ gy, const int64_t *__restrict__ csr_list,
                                                          T *__restrict__ gw, const T *__restrict__ probs, int in_dim, int out_dim,
                                                          int64_t batch, int64_t i, int64_t beg, int64_t end, int64_t s, bool live,
                                                          const Pack<T, VEC> &xi, int lane)
{
    Pack<T, VEC> part[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < VEC; ++k) part[u].v[k] = 0;
    // A group of four consumers needs three dependent fetches (list entry -> wiring, coefficients, probabilities -> rows).
    // They are staggered over the groups: while the rows of group g are fetched and used, the wiring of group g + 1 and
    // the list entries of group g + 2 are already on their way, so a group waits for ONE fetch, not three.  Every load
    // is issued unconditionally from a clamped, always valid address and its value discarded afterwards where it does
    // not count: a load under a per-lane condition makes the compiler wait for ALL outstanding loads at the end of its
    // branch, which turned the 4 x 3 fetches of a group into twelve round trips in a row.
    struct Meta {
        int32_t j[4], io[4];                                         // consumer (-1: none), row of its other operand
        T c_ab[4], c_lin[4], pr[4];
        bool first[4];
    };
    const int64_t list_last = 2 * (int64_t)out_dim - 1;
    auto list_entries = [&](int64_t cur, int32_t (&j)[4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t at = cur + u;
            const int32_t v = (int32_t)clamp_index(csr_list[at < list_last ? at : list_last], out_dim);
            j[u] = at < end ? v : -1;
        }
    };
    const int q16 = lane & 15;
    auto wiring = [&](const int32_t (&j)[4], int32_t prev_j, Meta &m) {
        int64_t ia[4], ib[4];
        Coef<T> c[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int32_t jj = j[u] < 0 ? 0 : j[u];
            ia[u] = a[jj];
            ib[u] = b[jj];
            c[u] = load_coef(folded + (int64_t)jj * 4);
            m.pr[u] = T(0);
        }
        if (probs != nullptr) {                                      // uniform over the launch
#pragma unroll
            for (int u = 0; u < 4; ++u) m.pr[u] = probs[(int64_t)(j[u] < 0 ? 0 : j[u]) * 16 + q16];
        }
        int32_t prev = prev_j;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t ja = clamp_index(ia[u], in_dim), jb = clamp_index(ib[u], in_dim);
            const bool have = j[u] >= 0;
            const bool as_a = ja == i && !(jb == i && prev == j[u]);
            m.j[u] = j[u];
            m.first[u] = have && as_a;
            m.io[u] = (int32_t)(as_a ? jb : ja);
            m.c_ab[u] = have ? c[u].ab : T(0);
            m.c_lin[u] = have ? (as_a ? c[u].a : c[u].b) : T(0);
            prev = j[u];
        }
    };
    int32_t j_next[4] = {-1, -1, -1, -1}, j_after[4] = {-1, -1, -1, -1};
    Meta cur_m, next_m;
    list_entries(beg, j_next);
    wiring(j_next, -1, cur_m);
    // With one row per wavefront the tests below are scalar branches and a list of up to four consumers fetches nothing
    // ahead; with several rows they would diverge, and fetching ahead regardless is the faster code.
    constexpr bool kAlwaysAhead = LPR != 0 && LPR != kWave;
    if (kAlwaysAhead || beg + 4 < end) list_entries(beg + 4, j_next);
    const int64_t s_at = live ? s : 0;                               // lanes beyond the batch read the row's start and drop it
    for (int64_t cur = beg; cur < end; cur += 4) {                   // the lanes of a row group leave the loop together
        Pack<T, VEC> vo[4], vg[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            vo[u] = load_vec<T, VEC>(x + (int64_t)cur_m.io[u] * batch + s_at);
            vg[u] = load_vec<T, VEC>(gy + (int64_t)(cur_m.j[u] < 0 ? 0 : cur_m.j[u]) * batch + s_at);
        }
        if (kAlwaysAhead || cur + 4 < end) {
            wiring(j_next, cur_m.j[3], next_m);
            if (kAlwaysAhead || cur + 8 < end) list_entries(cur + 8, j_after);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool use = cur_m.j[u] >= 0 && live;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                vo[u].v[k] = use ? vo[u].v[k] : T(0);
                vg[u].v[k] = use ? vg[u].v[k] : T(0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (cur_m.j[u] < 0) continue;
#pragma unroll
            for (int k = 0; k < VEC; ++k) part[u].v[k] = fma_t(fma_t(cur_m.c_ab[u], vo[u].v[k], cur_m.c_lin[u]), vg[u].v[k], part[u].v[k]);
            if constexpr (LPR != 0) if (cur_m.first[u]) {                    // uniform over the row group
                T sab = 0, sa = 0, sb = 0, s1 = 0;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    sab = fma_t(vg[u].v[k], xi.v[k] * vo[u].v[k], sab);
                    sa = fma_t(vg[u].v[k], xi.v[k], sa);
                    sb = fma_t(vg[u].v[k], vo[u].v[k], sb);
                    s1 += vg[u].v[k];
                }
                sab = lane_group_sum<T, LPR>(sab);
                sa = lane_group_sum<T, LPR>(sa);
                sb = lane_group_sum<T, LPR>(sb);
                s1 = lane_group_sum<T, LPR>(s1);
                if (lane % LPR >= LPR - 16) {
                    T gi = coef_transpose_row<T>(q16, sab, sa, sb, s1);
                    if (probs != nullptr) gi = softmax16_backward(gi, cur_m.pr[u]);
                    gw[(int64_t)cur_m.j[u] * 16 + q16] = gi;
                }
            }
        }
        cur_m = next_m;
#pragma unroll
        for (int u = 0; u < 4; ++u) j_next[u] = j_after[u];
    }
    Pack<T, VEC> acc;
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc.v[k] = (part[0].v[k] + part[1].v[k]) + (part[2].v[k] + part[3].v[k]);
    return acc;
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void fc_backward_x_folded_kernel(
    const T *__restrict__ x, const int64_t *__restrict__ a, const int64_t *__restrict__ b, const T *__restrict__ folded,
    const T *__restrict__ gy, const int64_t *__restrict__ csr_start, const int64_t *__restrict__ csr_list,
    T *__restrict__ gx, int in_dim, int64_t batch, int batch_chunks, int lpr_log2, int out_dim)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int rows = kWave >> lpr_log2, sub = lane >> lpr_log2, l = lane & ((1 << lpr_log2) - 1);
    const int64_t items = (int64_t)((in_dim + rows - 1) >> (6 - lpr_log2)) * batch_chunks;
    for (int64_t it = (int64_t)blockIdx.x * kWavesPerBlock + wave; it < items; it += (int64_t)gridDim.x * kWavesPerBlock) {
        const int64_t i = (it / batch_chunks) * rows + sub;
        const int64_t s = (((it % batch_chunks) << lpr_log2) + l) * VEC;
        if (i >= in_dim || s >= batch) continue;
        const int64_t beg = clamp_index(csr_start[i], 2 * (int64_t)out_dim + 1), end = clamp_index(csr_start[i + 1], 2 * (int64_t)out_dim + 1);
        const Pack<T, VEC> none{};
        const Pack<T, VEC> acc = fc_walk_consumers<T, VEC, 0>(x, a, b, folded, gy, csr_list, (T *)nullptr, (const T *)nullptr, in_dim, out_dim,
                                                              batch, i, beg, end, s, true, none, lane);
        store_vec<T, VEC>(gx + i * batch + s, acc);
    }
}

// Both gradients in one pass for any wiring, as long as one pass of LPR lanes x VEC samples covers the batch: the
// wavefront that owns input i walks its consumers (fc_walk_consumers) and, on the visit that reaches a
// consumer through its FIRST operand -- which happens exactly once per neuron, and has the neuron's gy row, its first
// operand row (x[i]) and its second operand row in registers -- also forms the four sums of the weight gradient
// (as fc_backward_w_kernel: same lanes, same order, same reduction) and writes the neuron's 16 gate gradients.
// Saves the second pass over gy and the operand rows that a separate weight-gradient kernel makes.
template <typename T, int VEC, int LPR>
__device__ __forceinline__ bool fc_backward_fused_item(const T *__restrict__ x, const int64_t *__restrict__ a,
                                                       const int64_t *__restrict__ b, const T *__restrict__ folded,
                                                       const T *__restrict__ gy, const int64_t *__restrict__ csr_start,
                                                       const int64_t *__restrict__ csr_list, T *__restrict__ gw, int in_dim,
                                                       int64_t batch, const T *__restrict__ probs, int64_t it, int lane,
                                                       Pack<T, VEC> &acc, int64_t &i, int out_dim)
{
    const int sub = lane / LPR, l = lane % LPR;
    constexpr int ROWS = kWave / LPR;
    const int64_t s = (int64_t)l * VEC;
    const bool row_ok = it * ROWS + sub < in_dim;
    i = row_ok ? it * ROWS + sub : in_dim - 1;
    const bool live = row_ok && s < batch;                           // lanes beyond the batch add zeros to the sums
    const int64_t beg = clamp_index(csr_start[i], 2 * (int64_t)out_dim + 1), end = row_ok ? clamp_index(csr_start[i + 1], 2 * (int64_t)out_dim + 1) : beg;
    Pack<T, VEC> xi;
#pragma unroll
    for (int k = 0; k < VEC; ++k) xi.v[k] = 0;
    if (live) xi = load_vec<T, VEC>(x + i * batch + s);
    acc = fc_walk_consumers<T, VEC, LPR>(x, a, b, folded, gy, csr_list, gw, probs, in_dim, out_dim, batch, i, beg, end, s, live, xi, lane);
    return live;
}

template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void fc_backward_fused_kernel(
    const T *__restrict__ x, const int64_t *__restrict__ a, const int64_t *__restrict__ b, const T *__restrict__ folded,
    const T *__restrict__ gy, const int64_t *__restrict__ csr_start, const int64_t *__restrict__ csr_list,
    T *__restrict__ gx, T *__restrict__ gw, int in_dim, int64_t batch, const T *__restrict__ probs, int out_dim)
{
    constexpr int ROWS = kWave / LPR;
    const int lane = threadIdx.x & (kWave - 1), wave = uniform(threadIdx.x >> 6);   // with one row per wavefront the whole index walk is scalar
    const int64_t groups = (in_dim + ROWS - 1) / ROWS;
    const int64_t s = (int64_t)(lane % LPR) * VEC;
    for (int64_t it = (int64_t)blockIdx.x * kWavesPerBlock + wave; it < groups; it += (int64_t)gridDim.x * kWavesPerBlock) {
        Pack<T, VEC> acc;
        int64_t i;
        if (fc_backward_fused_item<T, VEC, LPR>(x, a, b, folded, gy, csr_start, csr_list, gw, in_dim, batch, probs, it, lane, acc, i, out_dim))
            store_vec<T, VEC>(gx + i * batch + s, acc);
    }
}

// The same pass with the input gradient written sample-major, gx [batch, in_dim]: the wavefronts of a workgroup own
// F = waves * 64/LPR consecutive inputs, park their rows in an LDS tile [F][bp] and the workgroup writes the tile out
// transposed, F consecutive elements per sample.  Same sums in the same order as fc_backward_fused_kernel.
// 16 wavefronts when a wavefront owns one input (F = 16), 8 when it owns two or four (F = 16 or 32): the walk of several
// rows at once needs more than the 128 registers a workgroup of 1024 lanes leaves a lane.
template <int LPR> constexpr int smout_waves() { return LPR == kWave ? 16 : 8; }
static inline int64_t smout_row_pitch(int64_t batch) { return ((batch + 31) & ~31ll) + 4; }   // pitch % 32 == 4: the transposed reads spread over the banks
template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(smout_waves<LPR>() * kWave) void fc_backward_fused_smout_kernel(
    const T *__restrict__ x, const int64_t *__restrict__ a, const int64_t *__restrict__ b, const T *__restrict__ folded,
    const T *__restrict__ gy, const int64_t *__restrict__ csr_start, const int64_t *__restrict__ csr_list,
    T *__restrict__ gx, T *__restrict__ gw, int in_dim, int batch, int bp, const T *__restrict__ probs, int out_dim)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *tile = reinterpret_cast<T *>(smem);
    constexpr int kSmOutWaves = smout_waves<LPR>(), ROWS = kWave / LPR, F = kSmOutWaves * ROWS;
    const int lane = threadIdx.x & (kWave - 1), wave = uniform(threadIdx.x >> 6);   // with one row per wavefront the whole index walk is scalar
    const int64_t groups = (in_dim + ROWS - 1) / ROWS;
    const int64_t it = (int64_t)blockIdx.x * kSmOutWaves + wave;
    if (it < groups) {
        Pack<T, VEC> acc;
        int64_t i;
        if (fc_backward_fused_item<T, VEC, LPR>(x, a, b, folded, gy, csr_start, csr_list, gw, in_dim, batch, probs, it, lane, acc, i, out_dim)) {
            T *row = tile + (size_t)(wave * ROWS + lane / LPR) * bp + (lane % LPR) * VEC;
            store_vec<T, VEC>(row, acc);                             // one wide LDS store (bp is a multiple of 4 elements)
        }
    }
    __syncthreads();
    const int64_t i0 = (int64_t)blockIdx.x * F;
    for (int e = threadIdx.x; e < F * batch; e += kSmOutWaves * kWave) {
        const int f = e % F, s = e / F;
        if (i0 + f < in_dim) gx[(int64_t)s * in_dim + i0 + f] = tile[(size_t)f * bp + s];
    }
}

// ---- 2-D transpose through a padded LDS tile -------------------------------------------------
// TILE x TILE elements per workgroup of 256 threads; the 32 x 32 tile gives small matrices four times as many workgroups.
template <typename T, int TILE>
__global__ __launch_bounds__(256) void transpose_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t rows,
                                                      int64_t cols)
{
    __shared__ T tile[TILE][TILE + 1];
    constexpr int RPP = 256 / TILE;                                  // tile rows covered per pass
    const int tx = threadIdx.x % TILE, ty = threadIdx.x / TILE;
    const int64_t r0 = (int64_t)blockIdx.y * TILE, c0 = (int64_t)blockIdx.x * TILE;
#pragma unroll
    for (int k = 0; k < TILE / RPP; ++k) {
        const int64_t r = r0 + ty + RPP * k, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + RPP * k][tx] = src[r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE / RPP; ++k) {
        const int64_t c = c0 + ty + RPP * k, r = r0 + tx;
        if (r < rows && c < cols) dst[c * rows + r] = tile[tx][ty + RPP * k];
    }
}

// ---- GroupSum on feature-major activations ---------------------------------------------------
// partial[slice][g][b] = sum over the rows f of class g that belong to the slice of x[f][b]; rows are dealt
// to the 4 wavefronts of a workgroup and combined in LDS in a fixed order, slices by a second kernel, so
// the sums are reproducible.
template <typename T>
__global__ __launch_bounds__(256) void group_sum_fm_kernel(const T *__restrict__ x, T *__restrict__ partial, int64_t class_rows,
                                                         int64_t batch, int k, int slices)
{
    __shared__ T meet[4][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int g = blockIdx.y, slice = blockIdx.z;
    const int64_t b = (int64_t)blockIdx.x * kWave + lane;
    const int64_t r0 = class_rows * slice / slices, r1 = class_rows * (slice + 1) / slices;
    T acc = 0;
    if (b < batch) {
        const T *p = x + ((int64_t)g * class_rows + r0 + wave) * batch + b;
        int64_t r = r0 + wave;
        for (; r + 12 < r1; r += 16) {                               // four rows of this wavefront in flight
            const T v0 = p[0], v1 = p[4 * batch], v2 = p[8 * batch], v3 = p[12 * batch];
            acc += (v0 + v1) + (v2 + v3);
            p += 16 * batch;
        }
        for (; r < r1; r += 4) {
            acc += *p;
            p += 4 * batch;
        }
    }
    meet[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && b < batch)
        partial[((int64_t)slice * k + g) * batch + b] = (meet[0][lane] + meet[1][lane]) + (meet[2][lane] + meet[3][lane]);
}
// out[b][g] = sum over slices of partial[slice][g][b]
template <typename T>
__global__ __launch_bounds__(256) void group_sum_finish_kernel(const T *__restrict__ partial, T *__restrict__ out, int64_t batch,
                                                             int k, int slices, T inv_tau)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;       // sample fastest: the loads of a wavefront are contiguous
    if (i >= batch * k) return;
    const int g = (int)(i / batch);
    const int64_t b = i - (int64_t)g * batch;
    const T *p = partial + (int64_t)g * batch + b;
    const int64_t step = (int64_t)k * batch;
    T acc = 0;
    int s = 0;
    for (; s + 8 <= slices; s += 8) {                                // eight loads in flight, added in slice order
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[(s + u) * step];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; s < slices; ++s) acc += p[s * step];
    out[b * k + g] = acc * inv_tau;
}
// GroupSum in ONE launch for classes of a few thousand rows: a workgroup of 16 wavefronts owns one class and 32
// samples (a 128-byte line of every row); a lane keeps sample lane % 32 and takes rows 32 t + 2 wave + lane / 32 (sixteen
// loads in flight); the two row phases of a wavefront are added through a lane shuffle, the 16 wavefronts in LDS,
// pairwise -- a fixed order.
constexpr int kGroupSumOnceWaves = 16;
constexpr int kGroupSumOnceSamples = 32;
constexpr int64_t kGroupSumOnceMaxRows = 4096;
template <typename T>
__global__ __launch_bounds__(kGroupSumOnceWaves * kWave) void group_sum_once_kernel(const T *__restrict__ x, T *__restrict__ out,
                                                                                   int64_t class_rows, int64_t batch, int k, T inv_tau)
{
    __shared__ T meet[kGroupSumOnceWaves][kGroupSumOnceSamples];
    constexpr int kStep = 2 * kGroupSumOnceWaves;                     // rows between two loads of a lane
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int g = blockIdx.y;
    const int64_t b = (int64_t)blockIdx.x * kGroupSumOnceSamples + (lane & 31);
    const int64_t b_at = b < batch ? b : batch - 1;                   // lanes past the batch read its last sample and drop it
    const T *base = x + (int64_t)g * class_rows * batch + b_at;
    const int64_t first = (int64_t)wave * 2 + (lane >> 5), last = class_rows - 1;
    T acc = 0;
    for (int64_t r0 = first; r0 < class_rows; r0 += 16 * kStep) {
        T v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int64_t r = r0 + kStep * u;
            v[u] = base[(r < last ? r : last) * batch];              // every load unconditional, from a row of the class
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) acc += r0 + kStep * u < class_rows ? v[u] : T(0);
    }
    acc += __shfl_down(acc, 32);                                      // the two row phases: lanes 0..31 hold the wavefront's sums
    if (lane < 32) meet[wave][lane] = acc;
    __syncthreads();
    if (threadIdx.x < kGroupSumOnceSamples && b < batch) {
        T part[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)                                   // wavefronts 4q .. 4q + 3, then the four quarters
            part[q] = (meet[4 * q][threadIdx.x] + meet[4 * q + 1][threadIdx.x]) + (meet[4 * q + 2][threadIdx.x] + meet[4 * q + 3][threadIdx.x]);
        out[b * k + g] = ((part[0] + part[1]) + (part[2] + part[3])) * inv_tau;
    }
}
// grad_x[f][b] = grad_out[b][class of f] * (1 / tau); a workgroup writes 64 feature rows of one 64-sample column chunk
template <typename T>
__global__ __launch_bounds__(256) void group_sum_backward_fm_kernel(const T *__restrict__ grad_out, T *__restrict__ grad_x,
                                                                  int64_t class_rows, int64_t batch, int k, int64_t bchunks, T inv_tau)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t fb = blockIdx.x / bchunks, bc = blockIdx.x - fb * bchunks;
    const int64_t b = bc * kWave + lane;
    if (b >= batch) return;
    const int64_t f0 = fb * 64, features = class_rows * k;
    const int64_t f_end = f0 + 64 < features ? f0 + 64 : features;
    // the class of a row changes at most a few times along the 64 rows: the value is loaded when it does (wave-uniform)
    int64_t next = 0;
    T v = T(0);
    for (int64_t f = f0 + wave; f < f_end; f += 4) {
        if (f >= next) {
            const int64_t cls = f / class_rows;
            next = (cls + 1) * class_rows;
            v = grad_out[b * k + cls] * inv_tau;
        }
        grad_x[f * batch + b] = v;
    }
}

// gate[r] = index of the first maximum of the 16 logits of row r (a NaN counts as the maximum, as in torch.argmax)
template <typename S>
__global__ __launch_bounds__(256) void gate_argmax_kernel(const S *__restrict__ logits, uint8_t *__restrict__ gate, int64_t rows)
{
    using T = typename ComputeOf<S>::type;
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    T best = load_one(logits + r * 16);
    int at = 0;
#pragma unroll
    for (int i = 1; i < 16; ++i) {
        const T v = load_one(logits + r * 16 + i);
        if (v > best || (v != v && best == best)) {
            best = v;
            at = i;
        }
    }
    gate[r] = (uint8_t)at;
}

int grid_for(int64_t items)
{
    const int64_t blocks = clg_ceil_div(items, kWavesPerBlock);
    return (int)(blocks < 1 ? 1 : (blocks > (1 << 20) ? (1 << 20) : blocks));
}

template <typename T>
constexpr int vec_width() { return 16 / sizeof(T); }

// log2 of the lanes one row of `batch` samples takes at `vec` samples per lane: 16, 32 or 64 lanes
int lanes_per_row_log2(int64_t batch, int vec)
{
    const int64_t lanes = clg_ceil_div(batch, (int64_t)vec);
    return lanes <= 16 ? 4 : (lanes <= 32 ? 5 : 6);
}

int check_fc(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch, const char *name, bool half_ok = false)
{
    if (half_ok)
        CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64 || dtype == CLG_F16, "%s: dtype must be CLG_F32, CLG_F64 or CLG_F16, got %d",
                    name, dtype);
    else
        CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "%s: dtype must be CLG_F32 or CLG_F64, got %d", name, dtype);
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && batch > 0, "%s: in_dim, out_dim and batch must be positive (%lld, %lld, %lld)",
                name, (long long)in_dim, (long long)out_dim, (long long)batch);
    CLG_REQUIRE(in_dim < (1ll << 31) && out_dim < (1ll << 31), "%s: in_dim/out_dim above 2^31-1 are not supported", name);
    return CLG_OK;
}

}  // namespace

extern "C" int clg_gate_argmax(int dtype, const void *logits, uint8_t *gate, int64_t rows, void *stream)
{
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64 || dtype == CLG_F16, "clg_gate_argmax: dtype must be CLG_F32, CLG_F64 or CLG_F16, got %d",
                dtype);
    CLG_REQUIRE(logits && gate, "clg_gate_argmax: null pointer argument");
    CLG_REQUIRE(rows > 0 && rows < (1ll << 39), "clg_gate_argmax: rows must be in 1..2^39-1");
    const dim3 grid((unsigned)clg_ceil_div(rows, 256)), block(256);
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32) hipLaunchKernelGGL(gate_argmax_kernel<float>, grid, block, 0, st, (const float *)logits, gate, rows);
    else if (dtype == CLG_F64) hipLaunchKernelGGL(gate_argmax_kernel<double>, grid, block, 0, st, (const double *)logits, gate, rows);
    else hipLaunchKernelGGL(gate_argmax_kernel<__half>, grid, block, 0, st, (const __half *)logits, gate, rows);
    CLG_CHECK_LAUNCH("clg_gate_argmax");
    return CLG_OK;
}

extern "C" int clg_fc_forward(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *w, void *y,
                              int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_forward", true)) return e;
    CLG_REQUIRE(x && a && b && w && y, "clg_fc_forward: null pointer argument");
    const dim3 grid(grid_for(out_dim)), block(kBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_LAUNCH_F(S, VEC) \
    hipLaunchKernelGGL((fc_forward_kernel<S, VEC>), grid, block, 0, st, (const S *)x, a, b, (const S *)w, (S *)y, (int)out_dim, batch, (int)in_dim)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_F(float, 4);
        else CLG_LAUNCH_F(float, 1);
    } else if (dtype == CLG_F64) {
        if (batch % 2 == 0) CLG_LAUNCH_F(double, 2);
        else CLG_LAUNCH_F(double, 1);
    } else {
        if (batch % 8 == 0) CLG_LAUNCH_F(__half, 8);
        else CLG_LAUNCH_F(__half, 1);
    }
#undef CLG_LAUNCH_F
    CLG_CHECK_LAUNCH("clg_fc_forward");
    return CLG_OK;
}

static int fc_backward_w_impl(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *grad_y, void *grad_w,
                             int64_t in_dim, int64_t out_dim, int64_t batch, void *stream, const void *probs, const char *name)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, name, true)) return e;
    CLG_REQUIRE(x && a && b && grad_y && grad_w, "%s: null pointer argument", name);
    const dim3 block(kBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_LAUNCH_BW(T, VEC, LPR)                                                                                      \
    hipLaunchKernelGGL((fc_backward_w_kernel<T, VEC, LPR>), dim3(grid_for(clg_ceil_div(out_dim, (int64_t)(kWave / LPR)))), \
                       block, 0, st, (const T *)x, a, b, (const T *)grad_y, (T *)grad_w, (int)out_dim, batch,              \
                       (const T *)probs, (int)in_dim)
#define CLG_LAUNCH_BW_ROWS(T, VEC)                                                                                      \
    do {                                                                                                               \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                 \
        if (lg == 4) CLG_LAUNCH_BW(T, VEC, 16);                                                                        \
        else if (lg == 5) CLG_LAUNCH_BW(T, VEC, 32);                                                                   \
        else CLG_LAUNCH_BW(T, VEC, 64);                                                                                \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_BW_ROWS(float, 4);
        else CLG_LAUNCH_BW_ROWS(float, 1);
    } else if (dtype == CLG_F64) {
        if (batch % 2 == 0) CLG_LAUNCH_BW_ROWS(double, 2);
        else CLG_LAUNCH_BW_ROWS(double, 1);
    } else {
        if (batch % 8 == 0) CLG_LAUNCH_BW_ROWS(__half, 8);
        else CLG_LAUNCH_BW_ROWS(__half, 1);
    }
#undef CLG_LAUNCH_BW_ROWS
#undef CLG_LAUNCH_BW
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

extern "C" int clg_fc_backward_w(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *grad_y,
                                 void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    return fc_backward_w_impl(dtype, x, a, b, grad_y, grad_w, in_dim, out_dim, batch, stream, nullptr, "clg_fc_backward_w");
}

extern "C" int clg_fc_backward_logits(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *w,
                                      const void *grad_y, void *grad_logits, int64_t in_dim, int64_t out_dim, int64_t batch,
                                      void *stream)
{
    CLG_REQUIRE(w, "clg_fc_backward_logits: null pointer argument");
    return fc_backward_w_impl(dtype, x, a, b, grad_y, grad_logits, in_dim, out_dim, batch, stream, w, "clg_fc_backward_logits");
}

extern "C" int clg_fc_backward_x(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *w,
                                 const void *grad_y, const int64_t *csr_start, const int64_t *csr_list, void *grad_x,
                                 int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_backward_x", true)) return e;
    CLG_REQUIRE(x && a && b && w && grad_y && csr_start && csr_list && grad_x, "clg_fc_backward_x: null pointer argument");
    hipStream_t st = clg_stream(stream);
    const dim3 block(kBlock);
#define CLG_LAUNCH_BX(T, VEC)                                                                                          \
    do {                                                                                                               \
        const int chunks = (int)clg_ceil_div(batch, (int64_t)kWave * VEC);                                             \
        hipLaunchKernelGGL((fc_backward_x_kernel<T, VEC>), dim3(grid_for(in_dim * chunks)), block, 0, st, (const T *)x, \
                           a, b, (const T *)w, (const T *)grad_y, csr_start, csr_list, (T *)grad_x, (int)in_dim, batch,  \
                           chunks, (int)out_dim);                                                                                 \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_BX(float, 4);
        else CLG_LAUNCH_BX(float, 1);
    } else if (dtype == CLG_F64) {
        if (batch % 2 == 0) CLG_LAUNCH_BX(double, 2);
        else CLG_LAUNCH_BX(double, 1);
    } else {
        if (batch % 8 == 0) CLG_LAUNCH_BX(__half, 8);
        else CLG_LAUNCH_BX(__half, 1);
    }
#undef CLG_LAUNCH_BX
    CLG_CHECK_LAUNCH("clg_fc_backward_x");
    return CLG_OK;
}

extern "C" int clg_fc_fold(int dtype, int from_logits, const void *w_in, void *probs, void *folded, int64_t out_dim,
                           void *stream)
{
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "clg_fc_fold: dtype must be CLG_F32 or CLG_F64, got %d", dtype);
    CLG_REQUIRE(w_in && folded, "clg_fc_fold: null pointer argument");
    CLG_REQUIRE(out_dim > 0 && out_dim < (1ll << 31), "clg_fc_fold: out_dim must be in [1, 2^31-1], got %lld", (long long)out_dim);
    const dim3 grid((unsigned)clg_ceil_div(out_dim, (int64_t)256)), block(256);
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32)
        hipLaunchKernelGGL(fc_fold_kernel<float>, grid, block, 0, st, (const float *)w_in, (float *)probs, (float *)folded,
                           (int)out_dim, from_logits);
    else
        hipLaunchKernelGGL(fc_fold_kernel<double>, grid, block, 0, st, (const double *)w_in, (double *)probs,
                           (double *)folded, (int)out_dim, from_logits);
    CLG_CHECK_LAUNCH("clg_fc_fold");
    return CLG_OK;
}

// softmax + fold of the logits of up to kFoldManyMax tensors [rows_i, 16] in one launch (a network's layers at the
// start of a training step): the arithmetic of fc_fold_kernel and of the set-up launch of the fused block, row by row.
constexpr int kFoldManyMax = 16;
struct FoldMany {
    const void *logits[kFoldManyMax];
    void *probs[kFoldManyMax], *folded[kFoldManyMax];
    int64_t start[kFoldManyMax + 1];                                  // first row of tensor i in the launch's row numbering
    int n;
};
template <typename T>
__global__ __launch_bounds__(256) void fold_many_kernel(FoldMany m)
{
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= m.start[m.n]) return;
    int t = 0;
    while (q >= m.start[t + 1]) ++t;
    const int64_t r = q - m.start[t];
    T p[16];
    softmax16(reinterpret_cast<const T *>(m.logits[t]) + r * 16, p);
    T *pr = reinterpret_cast<T *>(m.probs[t]) + r * 16;
#pragma unroll
    for (int i = 0; i < 16; ++i) pr[i] = p[i];
    const Coef<T> c = fold16(p);
    T *f = reinterpret_cast<T *>(m.folded[t]) + r * 4;
    f[0] = c.ab;
    f[1] = c.a;
    f[2] = c.b;
    f[3] = c.one;
}

extern "C" int clg_fold_many(int dtype, int n, const void *const *logits, void *const *probs, void *const *folded, const int64_t *rows,
                             void *stream)
{
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "clg_fold_many: dtype must be CLG_F32 or CLG_F64, got %d", dtype);
    CLG_REQUIRE(n >= 1 && n <= kFoldManyMax, "clg_fold_many: 1 to %d tensors per call, got %d", kFoldManyMax, n);
    CLG_REQUIRE(logits && probs && folded && rows, "clg_fold_many: null pointer argument");
    FoldMany m = {};
    m.n = n;
    for (int i = 0; i < n; ++i) {
        CLG_REQUIRE(logits[i] && probs[i] && folded[i] && rows[i] > 0, "clg_fold_many: tensor %d: null pointer or no rows", i);
        m.logits[i] = logits[i], m.probs[i] = probs[i], m.folded[i] = folded[i];
        m.start[i + 1] = m.start[i] + rows[i];
    }
    CLG_REQUIRE(m.start[n] < (1ll << 31) * 256, "clg_fold_many: too many rows for one launch");
    const dim3 grid((unsigned)clg_ceil_div(m.start[n], (int64_t)256)), block(256);
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32) hipLaunchKernelGGL(fold_many_kernel<float>, grid, block, 0, st, m);
    else hipLaunchKernelGGL(fold_many_kernel<double>, grid, block, 0, st, m);
    CLG_CHECK_LAUNCH("clg_fold_many");
    return CLG_OK;
}

extern "C" int clg_fc_forward_folded(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                     void *y, int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_forward_folded")) return e;
    CLG_REQUIRE(x && a && b && folded && y, "clg_fc_forward_folded: null pointer argument");
    const dim3 block(kBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_LAUNCH_FF(T, VEC)                                                                                           \
    do {                                                                                                               \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                 \
        hipLaunchKernelGGL((fc_forward_folded_kernel<T, VEC>), dim3(grid_for(clg_ceil_div(out_dim, (int64_t)(kWave >> lg)))), \
                           block, 0, st, (const T *)x, a, b, (const T *)folded, (T *)y, (int)out_dim, batch, lg, (int)in_dim);       \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_FF(float, 4);
        else CLG_LAUNCH_FF(float, 1);
    } else {
        if (batch % 2 == 0) CLG_LAUNCH_FF(double, 2);
        else CLG_LAUNCH_FF(double, 1);
    }
#undef CLG_LAUNCH_FF
    CLG_CHECK_LAUNCH("clg_fc_forward_folded");
    return CLG_OK;
}

extern "C" int clg_transpose_2d(int elem_size, const void *src, void *dst, int64_t rows, int64_t cols, void *stream);

extern "C" int clg_fc_forward_logits_ex(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *logits,
                                        void *probs, void *folded, void *y, int64_t in_dim, int64_t out_dim, int64_t batch,
                                        int flags, void *x_fm, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_forward_logits")) return e;
    CLG_REQUIRE((flags & ~CLG_FC_X_SAMPLE_MAJOR) == 0, "clg_fc_forward_logits: unknown flags 0x%x", flags);
    if ((flags & CLG_FC_X_SAMPLE_MAJOR) == 0)
        return clg_fc_forward_logits(dtype, x, a, b, logits, probs, folded, y, in_dim, out_dim, batch, stream);
    CLG_REQUIRE(x && x_fm, "clg_fc_forward_logits: CLG_FC_X_SAMPLE_MAJOR needs x [batch, in_dim] and room for its copy [in_dim, batch]");
    if (int e = clg_transpose_2d(dtype == CLG_F64 ? 8 : 4, x, x_fm, batch, in_dim, stream)) return e;
    return clg_fc_forward_logits(dtype, x_fm, a, b, logits, probs, folded, y, in_dim, out_dim, batch, stream);
}

extern "C" int clg_fc_forward_logits(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *logits,
                                     void *probs, void *folded, void *y, int64_t in_dim, int64_t out_dim, int64_t batch,
                                     void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_forward_logits")) return e;
    CLG_REQUIRE(x && a && b && logits && probs && folded && y, "clg_fc_forward_logits: null pointer argument");
    const dim3 block(kBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_LAUNCH_FL(T, VEC)                                                                                           \
    do {                                                                                                               \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                 \
        hipLaunchKernelGGL((fc_forward_logits_kernel<T, VEC>), dim3(grid_for(clg_ceil_div(out_dim, (int64_t)(kWave >> lg)))), \
                           block, 0, st, (const T *)x, a, b, (const T *)logits, (T *)probs, (T *)folded, (T *)y,           \
                           (int)out_dim, batch, lg, (int)in_dim);                                                              \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_FL(float, 4);
        else CLG_LAUNCH_FL(float, 1);
    } else {
        if (batch % 2 == 0) CLG_LAUNCH_FL(double, 2);
        else CLG_LAUNCH_FL(double, 1);
    }
#undef CLG_LAUNCH_FL
    CLG_CHECK_LAUNCH("clg_fc_forward_logits");
    return CLG_OK;
}

extern "C" int clg_fc_backward_x_folded(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                        const void *grad_y, const int64_t *csr_start, const int64_t *csr_list, void *grad_x,
                                        int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, "clg_fc_backward_x_folded")) return e;
    CLG_REQUIRE(x && a && b && folded && grad_y && csr_start && csr_list && grad_x,
                "clg_fc_backward_x_folded: null pointer argument");
    hipStream_t st = clg_stream(stream);
    const dim3 block(kBlock);
#define CLG_LAUNCH_BXF(T, VEC)                                                                                          \
    do {                                                                                                               \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                 \
        const int chunks = (int)clg_ceil_div(batch, (int64_t)VEC << lg);                                               \
        const int64_t items = clg_ceil_div(in_dim, (int64_t)(kWave >> lg)) * chunks;                                   \
        hipLaunchKernelGGL((fc_backward_x_folded_kernel<T, VEC>), dim3(grid_for(items)), block, 0, st, (const T *)x, a, b, \
                           (const T *)folded, (const T *)grad_y, csr_start, csr_list, (T *)grad_x, (int)in_dim, batch,     \
                           chunks, lg, (int)out_dim);                                                                        \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_BXF(float, 4);
        else CLG_LAUNCH_BXF(float, 1);
    } else {
        if (batch % 2 == 0) CLG_LAUNCH_BXF(double, 2);
        else CLG_LAUNCH_BXF(double, 1);
    }
#undef CLG_LAUNCH_BXF
    CLG_CHECK_LAUNCH("clg_fc_backward_x_folded");
    return CLG_OK;
}

static int backward_sole_impl(const char *name, int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                              const void *probs, const void *grad_y, void *grad_x, void *grad_w, int64_t in_dim, int64_t out_dim,
                              int64_t batch, int64_t k, double tau, void *stream)
{
    if (int e = check_fc(dtype, in_dim, out_dim, batch, name)) return e;
    CLG_REQUIRE(x && a && b && folded && grad_y && grad_x && grad_w, "%s: null pointer argument", name);
    CLG_REQUIRE(2 * out_dim == in_dim, "%s: needs 2*out_dim == in_dim (every input read exactly once), got %lld, %lld", name,
                (long long)out_dim, (long long)in_dim);
    const bool classes = k > 0;                                      // grad_y is the gradient of a GroupSum's output [batch, k]
    CLG_REQUIRE(!classes || (k <= 65535 && out_dim % k == 0 && tau != 0.0), "%s: k must divide out_dim (%lld) and tau must not be zero", name,
                (long long)out_dim);
    const int64_t class_rows = classes ? out_dim / k : 1;
    const dim3 block(kBlock);
    hipStream_t st = clg_stream(stream);
#define CLG_LAUNCH_BS(T, VEC, LPR)                                                                                         \
    do {                                                                                                                  \
        const dim3 grid(grid_for(clg_ceil_div(out_dim, (int64_t)(kWave / LPR))));                                         \
        if (classes)                                                                                                      \
            hipLaunchKernelGGL((fc_backward_sole_kernel<T, VEC, LPR, true>), grid, block, 0, st, (const T *)x, a, b, (const T *)folded, \
                               (const T *)grad_y, (T *)grad_x, (T *)grad_w, (int)out_dim, batch, (const T *)probs, (int)k, class_rows, \
                               T(1) / (T)tau);                                                                            \
        else                                                                                                              \
            hipLaunchKernelGGL((fc_backward_sole_kernel<T, VEC, LPR, false>), grid, block, 0, st, (const T *)x, a, b, (const T *)folded, \
                               (const T *)grad_y, (T *)grad_x, (T *)grad_w, (int)out_dim, batch, (const T *)probs, 0, (int64_t)1, T(1)); \
    } while (0)
#define CLG_LAUNCH_BS_ROWS(T, VEC)                                                                                         \
    do {                                                                                                                  \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                    \
        if (lg == 4) CLG_LAUNCH_BS(T, VEC, 16);                                                                           \
        else if (lg == 5) CLG_LAUNCH_BS(T, VEC, 32);                                                                      \
        else CLG_LAUNCH_BS(T, VEC, 64);                                                                                   \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_BS_ROWS(float, 4);
        else CLG_LAUNCH_BS_ROWS(float, 1);
    } else {
        if (batch % 2 == 0) CLG_LAUNCH_BS_ROWS(double, 2);
        else CLG_LAUNCH_BS_ROWS(double, 1);
    }
#undef CLG_LAUNCH_BS_ROWS
#undef CLG_LAUNCH_BS
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

extern "C" int clg_fc_backward_sole(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                    const void *probs, const void *grad_y, void *grad_x, void *grad_w, int64_t in_dim,
                                    int64_t out_dim, int64_t batch, void *stream)
{
    return backward_sole_impl("clg_fc_backward_sole", dtype, x, a, b, folded, probs, grad_y, grad_x, grad_w, in_dim, out_dim, batch, 0, 1.0,
                              stream);
}

extern "C" int clg_fc_backward_sole_classes(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                            const void *probs, const void *grad_out, void *grad_x, void *grad_w, int64_t in_dim,
                                            int64_t out_dim, int64_t batch, int64_t k, double tau, void *stream)
{
    CLG_REQUIRE(k > 0, "clg_fc_backward_sole_classes: k must be positive");
    return backward_sole_impl("clg_fc_backward_sole_classes", dtype, x, a, b, folded, probs, grad_out, grad_x, grad_w, in_dim, out_dim, batch, k,
                              tau, stream);
}

// largest batch one pass of a wavefront row covers: 64 lanes x VEC samples
static int64_t fused_batch_limit(int dtype, int64_t batch)
{
    const int vec = dtype == CLG_F32 ? (batch % 4 == 0 ? 4 : 1) : (batch % 2 == 0 ? 2 : 1);
    return (int64_t)kWave * vec;
}

extern "C" int clg_fc_backward_fused_fits(int dtype, int64_t batch)
{
    return (dtype == CLG_F32 || dtype == CLG_F64) && batch > 0 && batch <= fused_batch_limit(dtype, batch) ? 1 : 0;
}

extern "C" int clg_fc_backward_fused_ex(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                        const void *probs, const void *grad_y, const int64_t *csr_start, const int64_t *csr_list,
                                        void *grad_x, void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, int flags,
                                        void *scratch, void *stream)
{
    const char *name = "clg_fc_backward_fused";
    if (int e = check_fc(dtype, in_dim, out_dim, batch, name)) return e;
    CLG_REQUIRE(x && a && b && folded && grad_y && csr_start && csr_list && grad_x && grad_w, "%s: null pointer argument", name);
    CLG_REQUIRE((flags & ~(CLG_FC_GX_SAMPLE_MAJOR | CLG_FC_GY_SAMPLE_MAJOR)) == 0, "%s: unknown flags 0x%x", name, flags);
    if (flags & CLG_FC_GY_SAMPLE_MAJOR) {                            // grad_y [batch, out_dim]: its feature-major copy goes to scratch
        CLG_REQUIRE(scratch, "%s: CLG_FC_GY_SAMPLE_MAJOR needs scratch for out_dim * batch elements", name);
        CLG_REQUIRE(batch <= fused_batch_limit(dtype, batch), "%s: batch %lld exceeds what one pass covers (%lld)", name, (long long)batch,
                    (long long)fused_batch_limit(dtype, batch));
        if (int e = clg_transpose_2d(dtype == CLG_F64 ? 8 : 4, grad_y, scratch, batch, out_dim, stream)) return e;
        grad_y = scratch;
    }
    CLG_REQUIRE(batch <= fused_batch_limit(dtype, batch),
                "%s: batch %lld exceeds what one pass covers (%lld); use clg_fc_backward_x_folded and clg_fc_backward_logits", name,
                (long long)batch, (long long)fused_batch_limit(dtype, batch));
    hipStream_t st = clg_stream(stream);
    const bool sm_out = (flags & CLG_FC_GX_SAMPLE_MAJOR) != 0;
    const int bp = (int)smout_row_pitch(batch);
#define CLG_LAUNCH_BF(T, VEC, LPR)                                                                                           \
    do {                                                                                                                    \
        if (sm_out) {                                                                                                       \
            constexpr int kSmOutWaves = smout_waves<LPR>(), F = kSmOutWaves * (kWave / LPR);                                \
            hipLaunchKernelGGL((fc_backward_fused_smout_kernel<T, VEC, LPR>), dim3((unsigned)clg_ceil_div(in_dim, (int64_t)F)), \
                               dim3(kSmOutWaves * kWave), (size_t)F * bp * sizeof(T), st, (const T *)x, a, b, (const T *)folded, \
                               (const T *)grad_y, csr_start, csr_list, (T *)grad_x, (T *)grad_w, (int)in_dim, (int)batch, bp, \
                               (const T *)probs, (int)out_dim);                                                                      \
        } else {                                                                                                            \
            hipLaunchKernelGGL((fc_backward_fused_kernel<T, VEC, LPR>),                                                     \
                               dim3(grid_for(clg_ceil_div(in_dim, (int64_t)(kWave / LPR)))), dim3(kBlock), 0, st, (const T *)x, a, b, \
                               (const T *)folded, (const T *)grad_y, csr_start, csr_list, (T *)grad_x, (T *)grad_w, (int)in_dim, \
                               batch, (const T *)probs, (int)out_dim);                                                              \
        }                                                                                                                   \
    } while (0)
#define CLG_LAUNCH_BF_ROWS(T, VEC)                                                                                         \
    do {                                                                                                                  \
        const int lg = lanes_per_row_log2(batch, VEC);                                                                    \
        if (lg == 4) CLG_LAUNCH_BF(T, VEC, 16);                                                                           \
        else if (lg == 5) CLG_LAUNCH_BF(T, VEC, 32);                                                                      \
        else CLG_LAUNCH_BF(T, VEC, 64);                                                                                   \
    } while (0)
    if (dtype == CLG_F32) {
        if (batch % 4 == 0) CLG_LAUNCH_BF_ROWS(float, 4);
        else CLG_LAUNCH_BF_ROWS(float, 1);
    } else {
        if (batch % 2 == 0) CLG_LAUNCH_BF_ROWS(double, 2);
        else CLG_LAUNCH_BF_ROWS(double, 1);
    }
#undef CLG_LAUNCH_BF_ROWS
#undef CLG_LAUNCH_BF
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

extern "C" int clg_fc_backward_fused(int dtype, const void *x, const int64_t *a, const int64_t *b, const void *folded,
                                     const void *probs, const void *grad_y, const int64_t *csr_start, const int64_t *csr_list,
                                     void *grad_x, void *grad_w, int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    return clg_fc_backward_fused_ex(dtype, x, a, b, folded, probs, grad_y, csr_start, csr_list, grad_x, grad_w, in_dim, out_dim, batch, 0,
                                    nullptr, stream);
}

extern "C" int clg_transpose_2d(int elem_size, const void *src, void *dst, int64_t rows, int64_t cols, void *stream)
{
    CLG_REQUIRE(src && dst, "clg_transpose_2d: null pointer argument");
    CLG_REQUIRE(rows > 0 && cols > 0, "clg_transpose_2d: rows and cols must be positive");
    const bool small = clg_ceil_div(cols, 64) * clg_ceil_div(rows, 64) < 2048;     // few 64 x 64 tiles: take 32 x 32 ones
    const int tile = small ? 32 : 64;
    const int64_t gx = clg_ceil_div(cols, tile), gy = clg_ceil_div(rows, tile);
    CLG_REQUIRE(gy <= 65535, "clg_transpose_2d: more than 65535*64 rows are not supported");
    const dim3 grid((unsigned)gx, (unsigned)gy), block(256);
    hipStream_t st = clg_stream(stream);
#define CLG_TRANSPOSE(U)                                                                                                \
    do {                                                                                                               \
        if (small) hipLaunchKernelGGL((transpose_kernel<U, 32>), grid, block, 0, st, (const U *)src, (U *)dst, rows, cols); \
        else hipLaunchKernelGGL((transpose_kernel<U, 64>), grid, block, 0, st, (const U *)src, (U *)dst, rows, cols);   \
    } while (0)
    switch (elem_size) {
    case 1: CLG_TRANSPOSE(uint8_t); break;
    case 2: CLG_TRANSPOSE(uint16_t); break;
    case 4: CLG_TRANSPOSE(uint32_t); break;
    case 8: CLG_TRANSPOSE(uint64_t); break;
    default: CLG_REQUIRE(false, "clg_transpose_2d: elem_size must be 1, 2, 4 or 8, got %d", elem_size);
    }
#undef CLG_TRANSPOSE
    CLG_CHECK_LAUNCH("clg_transpose_2d");
    return CLG_OK;
}

extern "C" int64_t clg_group_sum_scratch_bytes(int dtype, int64_t features, int64_t batch, int64_t k)
{
    if (features <= 0 || batch <= 0 || k <= 0 || features % k != 0) return -1;
    return 64 * k * batch * (dtype == CLG_F64 ? 8 : 4);               // at most 64 row slices
}

static int group_sum_impl(int dtype, const void *x, void *out, void *partial, int64_t partial_bytes, int64_t features,
                          int64_t batch, int64_t k, double tau, void *stream, const char *name)
{
    CLG_REQUIRE(tau != 0.0, "%s: tau must not be zero", name);
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "%s: dtype must be CLG_F32 or CLG_F64, got %d", name, dtype);
    CLG_REQUIRE(x && out && partial, "%s: null pointer argument", name);
    CLG_REQUIRE(features > 0 && batch > 0 && k > 0 && k <= 65535, "%s: features, batch and k must be positive, k <= 65535", name);
    CLG_REQUIRE(features % k == 0, "in_dim (%lld) has to be divisible by k (%lld) but it is not", (long long)features, (long long)k);
    const int64_t class_rows = features / k, bchunks = clg_ceil_div(batch, kWave);
    CLG_REQUIRE(bchunks < (1ll << 31), "%s: batch too large for one launch", name);
    // row slices until about four workgroups per CU, at least 64 rows each
    int64_t slices = clg_ceil_div(1024, bchunks * k);
    if (slices > class_rows / 64) slices = class_rows / 64;
    slices = slices < 1 ? 1 : (slices > 64 ? 64 : slices);
    const int64_t need = slices * k * batch * (dtype == CLG_F64 ? 8 : 4);
    CLG_REQUIRE(partial_bytes < 0 || need <= partial_bytes,
                "%s: k * batch = %lld needs %lld bytes of partial sums, the built-in buffer holds %lld (use clg_group_sum with a "
                "caller-provided scratch buffer for this size)", name, (long long)(k * batch), (long long)need, (long long)partial_bytes);
    hipStream_t st = clg_stream(stream);
    const dim3 grid((unsigned)bchunks, (unsigned)k, (unsigned)slices);
    if (dtype == CLG_F32) {
        hipLaunchKernelGGL(group_sum_fm_kernel<float>, grid, dim3(256), 0, st, (const float *)x, (float *)partial, class_rows, batch, (int)k,
                           (int)slices);
        hipLaunchKernelGGL(group_sum_finish_kernel<float>, dim3((unsigned)clg_ceil_div(batch * k, 256)), dim3(256), 0, st,
                           (const float *)partial, (float *)out, batch, (int)k, (int)slices, 1.0f / (float)tau);
    } else {
        hipLaunchKernelGGL(group_sum_fm_kernel<double>, grid, dim3(256), 0, st, (const double *)x, (double *)partial, class_rows, batch,
                           (int)k, (int)slices);
        hipLaunchKernelGGL(group_sum_finish_kernel<double>, dim3((unsigned)clg_ceil_div(batch * k, 256)), dim3(256), 0, st,
                           (const double *)partial, (double *)out, batch, (int)k, (int)slices, 1.0 / tau);
    }
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

extern "C" int clg_group_sum(int dtype, const void *x, void *out, void *scratch, int64_t features, int64_t batch, int64_t k,
                             double tau, void *stream)
{
    return group_sum_impl(dtype, x, out, scratch, -1, features, batch, k, tau, stream, "clg_group_sum");
}

extern "C" int clg_group_sum_once_fits(int64_t features, int64_t batch, int64_t k)
{
    if (features <= 0 || batch <= 0 || k <= 0 || k > 65535 || features % k != 0) return 0;
    // enough workgroups to be worth a launch of its own kind, and at most 128 rows per lane
    return features / k <= kGroupSumOnceMaxRows && features / k >= 64 && clg_ceil_div(batch, (int64_t)kGroupSumOnceSamples) * k >= 32 &&
                   clg_ceil_div(batch, (int64_t)kGroupSumOnceSamples) < (1ll << 31)
               ? 1
               : 0;
}

extern "C" int clg_group_sum_once(int dtype, const void *x, void *out, int64_t features, int64_t batch, int64_t k, double tau,
                                  void *stream)
{
    const char *name = "clg_group_sum_once";
    CLG_REQUIRE(tau != 0.0, "%s: tau must not be zero", name);
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "%s: dtype must be CLG_F32 or CLG_F64, got %d", name, dtype);
    CLG_REQUIRE(x && out, "%s: null pointer argument", name);
    CLG_REQUIRE(features > 0 && batch > 0 && k > 0 && k <= 65535, "%s: features, batch and k must be positive, k <= 65535", name);
    CLG_REQUIRE(features % k == 0, "in_dim (%lld) has to be divisible by k (%lld) but it is not", (long long)features, (long long)k);
    CLG_REQUIRE(clg_group_sum_once_fits(features, batch, k), "%s: %lld rows per class x %lld samples is not a size for the one-launch "
                "kernel (clg_group_sum_once_fits); use clg_group_sum", name, (long long)(features / k), (long long)batch);
    hipStream_t st = clg_stream(stream);
    const dim3 grid((unsigned)clg_ceil_div(batch, (int64_t)kGroupSumOnceSamples), (unsigned)k), block(kGroupSumOnceWaves * kWave);
    if (dtype == CLG_F32)
        hipLaunchKernelGGL(group_sum_once_kernel<float>, grid, block, 0, st, (const float *)x, (float *)out, features / k, batch, (int)k,
                           1.0f / (float)tau);
    else
        hipLaunchKernelGGL(group_sum_once_kernel<double>, grid, block, 0, st, (const double *)x, (double *)out, features / k, batch, (int)k,
                           1.0 / tau);
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

// ---- GroupSum for callers that cannot allocate ---------------------------------------------------
// The partial sums of clg_group_sum live in a buffer that is part of the library image: every GPU the library runs
// on holds its own copy of the array until the process ends.  In host code the array's name is only a stand-in for
// the symbol; the device address is asked for once per device (with that device current) and kept.
constexpr int64_t kStaticScratchBytes = 1 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static int static_scratch_ptr(void **out, const char *name)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptr_of[kMaxDevices];                                 // device address of `scratch` per device, nullptr = not asked yet
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        clg_set_error("%s: cannot identify the current device (%s)", name, e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return CLG_ELAUNCH;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of[dev] == nullptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            clg_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", name, dev, hipGetErrorString(e));
            return CLG_ELAUNCH;
        }
        ptr_of[dev] = p;
    }
    *out = ptr_of[dev];
    return CLG_OK;
}

extern "C" int64_t clg_group_sum_static_max_bytes(void) { return kStaticScratchBytes; }

// Looks the buffer's device address up for the current device (a runtime query, not a stream operation): callers that
// capture clg_group_sum_static into a HIP graph call this once per device BEFORE the capture starts; after it the entry
// point makes no runtime call besides its two launches.
extern "C" int clg_group_sum_static_init(void)
{
    void *p = nullptr;
    return static_scratch_ptr(&p, "clg_group_sum_static_init");
}

extern "C" int clg_group_sum_static(int dtype, const void *x, void *out, int64_t features, int64_t batch, int64_t k, double tau,
                                    void *stream)
{
    void *partial = nullptr;
    if (int e = static_scratch_ptr(&partial, "clg_group_sum_static")) return e;
    return group_sum_impl(dtype, x, out, partial, kStaticScratchBytes, features, batch, k, tau, stream, "clg_group_sum_static");
}

extern "C" int clg_group_sum_backward(int dtype, const void *grad_out, void *grad_x, int64_t features, int64_t batch, int64_t k,
                                      double tau, void *stream)
{
    CLG_REQUIRE(tau != 0.0, "clg_group_sum_backward: tau must not be zero");
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "clg_group_sum_backward: dtype must be CLG_F32 or CLG_F64, got %d", dtype);
    CLG_REQUIRE(grad_out && grad_x, "clg_group_sum_backward: null pointer argument");
    CLG_REQUIRE(features > 0 && batch > 0 && k > 0 && features % k == 0, "clg_group_sum_backward: features must be a positive multiple of k");
    const int64_t bchunks = clg_ceil_div(batch, kWave), blocks = clg_ceil_div(features, 64) * bchunks;
    CLG_REQUIRE(blocks < (1ll << 31), "clg_group_sum_backward: problem too large for one launch");
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32)
        hipLaunchKernelGGL(group_sum_backward_fm_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, (const float *)grad_out,
                           (float *)grad_x, features / k, batch, (int)k, bchunks, 1.0f / (float)tau);
    else
        hipLaunchKernelGGL(group_sum_backward_fm_kernel<double>, dim3((unsigned)blocks), dim3(256), 0, st, (const double *)grad_out,
                           (double *)grad_x, features / k, batch, (int)k, bchunks, 1.0 / tau);
    CLG_CHECK_LAUNCH("clg_group_sum_backward");
    return CLG_OK;
}
