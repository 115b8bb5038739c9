// Fully connected logic layer on SAMPLE-major tensors, x [batch, in_dim] -> y [batch, out_dim]: the layout the module
// API hands over at the boundary of a LogicLayer stack.  The feature-major kernels (logic_fc.hip) need a transposed copy
// of x on the way in and of grad_y / grad_x on the way back; here a workgroup stages whole sample rows in LDS instead
// (x[s, :] for the forward, x[s, :] and grad_y[s, :] for the input gradient), lanes run along neurons or input features,
// gather from LDS and read / write global memory in contiguous rows.  For layers whose rows fit LDS.  An OPTION
// (clg_fc_sm_preferred): on the GPU the feature-major kernels plus their transposed copies are faster at 8000 -> 8000
// neurons and 256 samples, because summing over samples is a lane reduction there and a second pass with partial sums
// here; these kernels need fewer microseconds of host launch work.
//
// Tables made once per wiring by clg_fc_sm_plan (host):
//   ab32    int32 [out, 2]     the two inputs of every neuron
//   start32 int32 [in + 1]     the reverse map of src/difflogic/difflogic.py:71-87 with 32-bit offsets
//   entry   int32 [2 out, 2]   per reverse-map entry: (neuron | first-operand flag << 31, the neuron's OTHER input)
// and per step by clg_fc_fold_sm (one launch): probs [out, 16], folded [out, 4] and, per reverse-map entry, the two
// coefficients its derivative needs, coef_e [2 out, 2] = (c_ab, c_a or c_b) -- so the input gradient reads everything
// about a consumer with two contiguous loads instead of three random ones.
#include <stdlib.h>

#include <type_traits>

#include "clg_common.h"

int clg_launch_reduce_coef(int dtype, const void *partial, void *out, int64_t rows, int nb, int G, hipStream_t st, const char *name,
                           const void *probs);
int clg_allow_lds(const void *kernel, size_t bytes, const char *name);

namespace {

constexpr int kSmBlock = 1024;   // 16 wavefronts per workgroup and kSmUnroll independent items per lane: the loops below are
constexpr int kSmUnroll = 4;     // chains of L2 round trips, and that is what hides them
constexpr int kSmWNeurons = 2;   // neurons per lane of the weight-gradient kernel
constexpr int kSmLdsBudget = 150 * 1024;    // rows a workgroup may hold
constexpr int kSmMaxParts = 64;             // partial sums per neuron the scratch buffer holds

template <typename T>
__device__ __forceinline__ Coef<T> coef_at(const T *__restrict__ f)
{
    return Coef<T>{f[0], f[1], f[2], f[3]};
}

// n elements of a sample row into LDS; 16-byte loads when the row length allows (rows then start 16-byte aligned
// whenever the tensor does)
template <typename T>
__device__ __forceinline__ void stage_row(T *__restrict__ dst, const T *__restrict__ src, int n)
{
    constexpr int V = 16 / sizeof(T);
    if ((n % V) == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
        using Vec = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
        const Vec *s4 = reinterpret_cast<const Vec *>(src);
        Vec *d4 = reinterpret_cast<Vec *>(dst);
        for (int i = threadIdx.x; i < n / V; i += kSmBlock) d4[i] = s4[i];
    } else {
        for (int i = threadIdx.x; i < n; i += kSmBlock) dst[i] = src[i];
    }
}

// threads [0, out): softmax + fold of neuron t; threads [out, 3 out): coefficients of reverse-map entry t - out
template <typename T>
__global__ __launch_bounds__(256) void fc_fold_sm_kernel(const T *__restrict__ logits, const int32_t *__restrict__ entry,
                                                       T *__restrict__ probs, T *__restrict__ folded, T *__restrict__ coef_e,
                                                       int out_dim)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= 3ll * out_dim) return;
    const bool neuron = t < out_dim;
    const int64_t e = t - out_dim;
    const int32_t en = neuron ? 0 : entry[2 * e];
    const int64_t j = neuron ? t : (int64_t)(en & 0x7fffffff);
    T p[16];
    softmax16(logits + j * 16, p);
    const Coef<T> c = fold16(p);
    if (neuron) {
#pragma unroll
        for (int i = 0; i < 16; ++i) probs[j * 16 + i] = p[i];
        T *f = folded + j * 4;
        f[0] = c.ab, f[1] = c.a, f[2] = c.b, f[3] = c.one;
    } else {
        coef_e[2 * e] = c.ab;
        coef_e[2 * e + 1] = en < 0 ? c.a : c.b;                      // flag: the entry's owner is the neuron's first operand
    }
}

// one sample per workgroup: x[s, :] in LDS, lanes along neurons
template <typename T>
__global__ __launch_bounds__(kSmBlock) void fc_forward_sm_kernel(const T *__restrict__ x, const int32_t *__restrict__ ab32,
                                                               const T *__restrict__ folded, T *__restrict__ y, int in_dim,
                                                               int out_dim)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    const int64_t s = blockIdx.x;
    stage_row(xs, x + s * in_dim, in_dim);
    T *yr = y + s * out_dim;
    bool staged = false;
    for (int j0 = threadIdx.x; j0 < out_dim; j0 += kSmBlock * kSmUnroll) {
        int2 ab[kSmUnroll];
        Coef<T> c[kSmUnroll];
#pragma unroll
        for (int u = 0; u < kSmUnroll; ++u) {                        // wiring and coefficients of kSmUnroll neurons in flight
            const int j = j0 + u * kSmBlock;
            if (j < out_dim) {
                ab[u] = reinterpret_cast<const int2 *>(ab32)[j];
                c[u] = coef_at(folded + (int64_t)j * 4);
            }
        }
        if (!staged) {                                               // (the first loads travel while the row is staged)
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int u = 0; u < kSmUnroll; ++u) {
            const int j = j0 + u * kSmBlock;
            if (j < out_dim) yr[j] = gate(c[u], xs[ab[u].x], xs[ab[u].y]);
        }
    }
}

// one sample per workgroup: x[s, :] and grad_y[s, :] in LDS, lanes along input features, consumers in list order
template <typename T>
__global__ __launch_bounds__(kSmBlock) void fc_backward_x_sm_kernel(const T *__restrict__ x, const T *__restrict__ gy,
                                                                  const int32_t *__restrict__ start32,
                                                                  const int32_t *__restrict__ entry, const T *__restrict__ coef_e,
                                                                  T *__restrict__ gx, int in_dim, int out_dim)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    T *gs = xs + ((in_dim + 3) & ~3);                                 // keeps the second row 16-byte aligned
    const int64_t s = blockIdx.x;
    stage_row(xs, x + s * in_dim, in_dim);
    stage_row(gs, gy + s * out_dim, out_dim);
    T *gxr = gx + s * in_dim;
    bool staged = false;
    for (int i0 = threadIdx.x; i0 < in_dim; i0 += kSmBlock * kSmUnroll) {
        // kSmUnroll features per lane side by side: their list bounds, then their entries, are in flight together
        int beg[kSmUnroll], end[kSmUnroll];
        T acc[kSmUnroll];
        int longest = 0;
#pragma unroll
        for (int u = 0; u < kSmUnroll; ++u) {
            const int i = i0 + u * kSmBlock;
            beg[u] = end[u] = 0;
            acc[u] = T(0);
            if (i < in_dim) {
                beg[u] = start32[i];
                end[u] = start32[i + 1];
            }
            longest = max(longest, end[u] - beg[u]);
        }
        if (!staged) {
            __syncthreads();
            staged = true;
        }
        for (int k = 0; k < longest; ++k) {                          // consumers in list order: a fixed order of additions
            int2 en[kSmUnroll];
            T c_ab[kSmUnroll], c_lin[kSmUnroll];
#pragma unroll
            for (int u = 0; u < kSmUnroll; ++u) {
                const int e = beg[u] + k;
                if (e < end[u]) {
                    en[u] = reinterpret_cast<const int2 *>(entry)[e];
                    c_ab[u] = coef_e[2 * (int64_t)e];
                    c_lin[u] = coef_e[2 * (int64_t)e + 1];
                }
            }
#pragma unroll
            for (int u = 0; u < kSmUnroll; ++u)
                if (beg[u] + k < end[u]) acc[u] = fma_t(fma_t(c_ab[u], xs[en[u].y], c_lin[u]), gs[en[u].x & 0x7fffffff], acc[u]);
        }
#pragma unroll
        for (int u = 0; u < kSmUnroll; ++u) {
            const int i = i0 + u * kSmBlock;
            if (i < in_dim) gxr[i] = acc[u];
        }
    }
}

// Up to 4 samples x one slice of the neurons per pass of a workgroup: x rows in LDS, lanes along neurons (kSmWNeurons
// per lane, sums in registers), grad_y read in rows.  Workgroup (grp, slice) takes the sample chunks grp, grp + groups, ...
// in order; partial [out][groups][4] (the layout reduce_coef_partials_kernel adds up in order)
template <typename T>
__global__ __launch_bounds__(kSmBlock) void fc_backward_w_sm_kernel(const T *__restrict__ x, const T *__restrict__ gy,
                                                                  const int32_t *__restrict__ ab32, T *__restrict__ partial,
                                                                  int in_dim, int out_dim, int batch, int sw, int groups)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);
    const int grp = blockIdx.x;
    const int per = (out_dim + gridDim.y - 1) / gridDim.y;           // <= kSmWNeurons * kSmBlock (host)
    const int j_lo = blockIdx.y * per, j_hi = min(out_dim, j_lo + per);
    int j[kSmWNeurons];
    int2 ab[kSmWNeurons];
    T acc[kSmWNeurons][4];
#pragma unroll
    for (int u = 0; u < kSmWNeurons; ++u) {
        j[u] = j_lo + threadIdx.x + u * kSmBlock;
        ab[u] = j[u] < j_hi ? reinterpret_cast<const int2 *>(ab32)[j[u]] : make_int2(0, 0);
        acc[u][0] = acc[u][1] = acc[u][2] = acc[u][3] = T(0);
    }
    const int chunks = (batch + sw - 1) / sw;
    for (int chunk = grp; chunk < chunks; chunk += groups) {
        const int s0 = chunk * sw, s_cur = min(sw, batch - s0);
        if (chunk != grp) __syncthreads();                           // every lane is done with the previous rows
        stage_row(xs, x + (int64_t)s0 * in_dim, s_cur * in_dim);     // consecutive samples: one contiguous run
        T g[kSmWNeurons][4];                                         // sw <= 4: grad_y of all samples in flight while the rows land
#pragma unroll
        for (int u = 0; u < kSmWNeurons; ++u)
#pragma unroll
            for (int s = 0; s < 4; ++s) g[u][s] = s < s_cur && j[u] < j_hi ? gy[(int64_t)(s0 + s) * out_dim + j[u]] : T(0);
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kSmWNeurons; ++u) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if (s < s_cur) {
                    const T a = xs[s * in_dim + ab[u].x], b = xs[s * in_dim + ab[u].y];
                    acc[u][0] = fma_t(g[u][s], a * b, acc[u][0]);
                    acc[u][1] = fma_t(g[u][s], a, acc[u][1]);
                    acc[u][2] = fma_t(g[u][s], b, acc[u][2]);
                    acc[u][3] += g[u][s];
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kSmWNeurons; ++u) {
        if (j[u] >= j_hi) continue;
        T *p = partial + ((int64_t)j[u] * groups + grp) * 4;
        if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<float4 *>(p) = make_float4(acc[u][0], acc[u][1], acc[u][2], acc[u][3]);
        } else {
            p[0] = acc[u][0], p[1] = acc[u][1], p[2] = acc[u][2], p[3] = acc[u][3];
        }
    }
}

int elem_of(int dtype) { return dtype == CLG_F64 ? 8 : 4; }

// Launch shape of the weight gradient: sw samples per pass (up to 4 rows within the LDS budget), `groups` workgroups
// along the samples (one partial sum per neuron each), `slices` along the neurons: at most kSmWNeurons per lane, and
// enough workgroups for the GPU.
struct WShape {
    int sw, groups, slices;
};
WShape w_shape(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch)
{
    int64_t sw = kSmLdsBudget / (in_dim * elem_of(dtype));
    sw = sw > 4 ? 4 : sw < 1 ? 1 : sw;
    if (sw > batch) sw = batch;
    int64_t groups = clg_ceil_div(batch, sw);
    if (groups > kSmMaxParts) groups = kSmMaxParts;
    const int64_t least = clg_ceil_div(out_dim, (int64_t)kSmWNeurons * kSmBlock), most = clg_ceil_div(out_dim, kSmBlock);
    int64_t slices = clg_ceil_div(256, groups);
    slices = slices < least ? least : slices > most ? most : slices;
    return WShape{(int)sw, (int)groups, (int)slices};
}

int check_sm(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch, const char *name)
{
    CLG_REQUIRE(dtype == CLG_F32 || dtype == CLG_F64, "%s: dtype must be CLG_F32 or CLG_F64, got %d", name, dtype);
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && batch > 0, "%s: in_dim, out_dim and batch must be positive", name);
    CLG_REQUIRE(out_dim < (1ll << 30) && in_dim < (1ll << 30) && batch < (1ll << 31), "%s: dimensions too large", name);
    return CLG_OK;
}

}  // namespace

extern "C" int clg_fc_sm_fits(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch)
{
    if ((dtype != CLG_F32 && dtype != CLG_F64) || in_dim <= 0 || out_dim <= 0 || batch <= 0) return 0;
    if (out_dim >= (1ll << 30) || in_dim >= (1ll << 30)) return 0;
    const int64_t e = elem_of(dtype);
    if ((((in_dim + 3) & ~3ll) + out_dim) * e > kSmLdsBudget) return 0;   // x[s, :] and grad_y[s, :] of the input gradient
    return in_dim * e <= kSmLdsBudget && clg_ceil_div(out_dim, (int64_t)kSmWNeurons * kSmBlock) <= 65535 ? 1 : 0;
}

// What the module asks: these kernels only when CLG_FC_SAMPLE_MAJOR=1 says so.  At 8000 -> 8000 neurons and 256 samples
// they lose to the feature-major kernels with their transposed copies once launch cost is out of the picture (the
// weight gradient needs a second pass over the rows plus a reduction of partial sums, where the feature-major kernel
// sums along the lanes), so they are an option, not the default.
extern "C" int clg_fc_sm_preferred(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch)
{
    const char *e = clg_knob(K_FC_SAMPLE_MAJOR);
    return e != nullptr && atoi(e) != 0 && clg_fc_sm_fits(dtype, in_dim, out_dim, batch);
}

// HOST function: tables of the sample-major kernels from the wiring and its reverse map
extern "C" int clg_fc_sm_plan(const int64_t *a, const int64_t *b, const int64_t *csr_start, const int64_t *csr_list, int64_t in_dim,
                              int64_t out_dim, int32_t *ab32, int32_t *start32, int32_t *entry)
{
    CLG_REQUIRE(a && b && csr_start && csr_list && ab32 && start32 && entry, "clg_fc_sm_plan: null pointer argument");
    CLG_REQUIRE(in_dim > 0 && out_dim > 0 && out_dim < (1ll << 30) && in_dim < (1ll << 30), "clg_fc_sm_plan: dimensions out of range");
    for (int64_t j = 0; j < out_dim; ++j) {
        CLG_REQUIRE(a[j] >= 0 && a[j] < in_dim && b[j] >= 0 && b[j] < in_dim, "clg_fc_sm_plan: neuron %lld is wired to a feature outside 0..%lld",
                    (long long)j, (long long)in_dim - 1);
        ab32[2 * j] = (int32_t)a[j];
        ab32[2 * j + 1] = (int32_t)b[j];
    }
    CLG_REQUIRE(csr_start[0] == 0 && csr_start[in_dim] == 2 * out_dim, "clg_fc_sm_plan: the reverse map does not hold 2*out_dim entries");
    for (int64_t i = 0; i < in_dim; ++i) {
        const int64_t beg = csr_start[i], end = csr_start[i + 1];
        CLG_REQUIRE(beg <= end && end <= 2 * out_dim, "clg_fc_sm_plan: the reverse map offsets are not increasing");
        start32[i] = (int32_t)beg;
        int64_t prev = -1;
        for (int64_t e = beg; e < end; ++e) {
            const int64_t j = csr_list[e];
            CLG_REQUIRE(j >= 0 && j < out_dim && (a[j] == i || b[j] == i), "clg_fc_sm_plan: reverse-map entry %lld does not name a consumer of "
                        "feature %lld", (long long)e, (long long)i);
            // Input i is operand A of neuron j unless only B matches; a neuron wired to the same feature twice appears
            // twice in the list and takes the B derivative the second time (the rule of the feature-major kernels).
            const bool as_a = a[j] == i && !(b[j] == i && prev == j);
            entry[2 * e] = (int32_t)j | (as_a ? (int32_t)0x80000000 : 0);
            entry[2 * e + 1] = (int32_t)(as_a ? b[j] : a[j]);
            prev = j;
        }
    }
    start32[in_dim] = (int32_t)(2 * out_dim);
    return CLG_OK;
}

extern "C" int clg_fc_fold_sm(int dtype, const void *logits, const int32_t *entry, void *probs, void *folded, void *coef_e,
                              int64_t out_dim, void *stream)
{
    if (int e = check_sm(dtype, 1, out_dim, 1, "clg_fc_fold_sm")) return e;
    CLG_REQUIRE(logits && entry && probs && folded && coef_e, "clg_fc_fold_sm: null pointer argument");
    const dim3 grid((unsigned)clg_ceil_div(3 * out_dim, 256)), block(256);
    hipStream_t st = clg_stream(stream);
    if (dtype == CLG_F32)
        hipLaunchKernelGGL(fc_fold_sm_kernel<float>, grid, block, 0, st, (const float *)logits, entry, (float *)probs, (float *)folded,
                           (float *)coef_e, (int)out_dim);
    else
        hipLaunchKernelGGL(fc_fold_sm_kernel<double>, grid, block, 0, st, (const double *)logits, entry, (double *)probs, (double *)folded,
                           (double *)coef_e, (int)out_dim);
    CLG_CHECK_LAUNCH("clg_fc_fold_sm");
    return CLG_OK;
}

extern "C" int clg_fc_forward_sm(int dtype, const void *x, const int32_t *ab32, const void *folded, void *y, int64_t in_dim,
                                 int64_t out_dim, int64_t batch, void *stream)
{
    const char *name = "clg_fc_forward_sm";
    if (int e = check_sm(dtype, in_dim, out_dim, batch, name)) return e;
    CLG_REQUIRE(x && ab32 && folded && y, "%s: null pointer argument", name);
    const size_t lds = (size_t)in_dim * elem_of(dtype);
    CLG_REQUIRE(lds <= (size_t)kSmLdsBudget, "%s: a row of %lld features does not fit LDS (clg_fc_sm_fits)", name, (long long)in_dim);
    hipStream_t st = clg_stream(stream);
    const dim3 grid((unsigned)batch), block(kSmBlock);
    if (dtype == CLG_F32) {
        if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_forward_sm_kernel<float>), lds, name)) return e;
        hipLaunchKernelGGL(fc_forward_sm_kernel<float>, grid, block, lds, st, (const float *)x, ab32, (const float *)folded, (float *)y,
                           (int)in_dim, (int)out_dim);
    } else {
        if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_forward_sm_kernel<double>), lds, name)) return e;
        hipLaunchKernelGGL(fc_forward_sm_kernel<double>, grid, block, lds, st, (const double *)x, ab32, (const double *)folded, (double *)y,
                           (int)in_dim, (int)out_dim);
    }
    CLG_CHECK_LAUNCH(name);
    return CLG_OK;
}

extern "C" int64_t clg_fc_backward_sm_scratch_bytes(int dtype, int64_t in_dim, int64_t out_dim, int64_t batch)
{
    if (!clg_fc_sm_fits(dtype, in_dim, out_dim, batch)) return -1;
    return out_dim * w_shape(dtype, in_dim, out_dim, batch).groups * 4 * elem_of(dtype);
}

extern "C" int clg_fc_backward_sm(int dtype, const void *x, const void *grad_y, const int32_t *ab32, const int32_t *start32,
                                  const int32_t *entry, const void *coef_e, const void *probs, void *grad_x, void *grad_w,
                                  void *scratch, int64_t in_dim, int64_t out_dim, int64_t batch, void *stream)
{
    const char *name = "clg_fc_backward_sm";
    if (int e = check_sm(dtype, in_dim, out_dim, batch, name)) return e;
    CLG_REQUIRE(x && grad_y && ab32 && start32 && entry && coef_e, "%s: null pointer argument", name);
    CLG_REQUIRE(grad_x || grad_w, "%s: neither gradient asked for", name);
    CLG_REQUIRE(!grad_w || scratch, "%s: the weight gradient needs scratch (clg_fc_backward_sm_scratch_bytes)", name);
    CLG_REQUIRE(clg_fc_sm_fits(dtype, in_dim, out_dim, batch), "%s: rows of %lld + %lld elements do not fit LDS (clg_fc_sm_fits)", name,
                (long long)in_dim, (long long)out_dim);
    hipStream_t st = clg_stream(stream);
    const int e_sz = elem_of(dtype);
    if (grad_x != nullptr) {
        const size_t lds = (size_t)(((in_dim + 3) & ~3ll) + out_dim) * e_sz;
        const dim3 grid((unsigned)batch), block(kSmBlock);
        if (dtype == CLG_F32) {
            if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_backward_x_sm_kernel<float>), lds, name)) return e;
            hipLaunchKernelGGL(fc_backward_x_sm_kernel<float>, grid, block, lds, st, (const float *)x, (const float *)grad_y, start32, entry,
                               (const float *)coef_e, (float *)grad_x, (int)in_dim, (int)out_dim);
        } else {
            if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_backward_x_sm_kernel<double>), lds, name)) return e;
            hipLaunchKernelGGL(fc_backward_x_sm_kernel<double>, grid, block, lds, st, (const double *)x, (const double *)grad_y, start32, entry,
                               (const double *)coef_e, (double *)grad_x, (int)in_dim, (int)out_dim);
        }
        CLG_CHECK_LAUNCH(name);
    }
    if (grad_w == nullptr) return CLG_OK;
    const WShape ws = w_shape(dtype, in_dim, out_dim, batch);
    const int sw = ws.sw, groups = ws.groups, slices = ws.slices;
    const size_t lds = (size_t)sw * in_dim * e_sz;
    const dim3 grid((unsigned)groups, (unsigned)slices), block(kSmBlock);
    if (dtype == CLG_F32) {
        if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_backward_w_sm_kernel<float>), lds, name)) return e;
        hipLaunchKernelGGL(fc_backward_w_sm_kernel<float>, grid, block, lds, st, (const float *)x, (const float *)grad_y, ab32, (float *)scratch,
                           (int)in_dim, (int)out_dim, (int)batch, sw, groups);
    } else {
        if (int e = clg_allow_lds(reinterpret_cast<const void *>(fc_backward_w_sm_kernel<double>), lds, name)) return e;
        hipLaunchKernelGGL(fc_backward_w_sm_kernel<double>, grid, block, lds, st, (const double *)x, (const double *)grad_y, ab32,
                           (double *)scratch, (int)in_dim, (int)out_dim, (int)batch, sw, groups);
    }
    CLG_CHECK_LAUNCH(name);
    return clg_launch_reduce_coef(dtype, scratch, grad_w, out_dim, groups, 1, st, name, probs);
}
