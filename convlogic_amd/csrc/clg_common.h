// Shared host/device helpers of the gfx950 logic-layer kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "convlogic_amd.h"

// ---- host side: error reporting ------------------------------------------------------------
void clg_set_error(const char *fmt, ...);

#define CLG_REQUIRE(cond, ...)       \
    do {                             \
        if (!(cond)) {               \
            clg_set_error(__VA_ARGS__); \
            return CLG_EINVAL;       \
        }                            \
    } while (0)

// Checks the launch that was just enqueued (launch-configuration errors only; no sync).
#define CLG_CHECK_LAUNCH(name)                                                      \
    do {                                                                            \
        hipError_t e_ = hipGetLastError();                                          \
        if (e_ != hipSuccess) {                                                     \
            clg_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));    \
            return CLG_ELAUNCH;                                                     \
        }                                                                           \
    } while (0)

// ---- host side: tuning knobs ---------------------------------------------------------------
// Environment variables CLG_<name>, for measurement and for forcing a code path in tests (unset = the measured
// optimum).  They are read ONCE per process, on the first lookup, so a launch costs no getenv(); clg_reload_knobs()
// (C ABI) reads them again after the environment was changed.
#define CLG_KNOBS(X)                                                                                                   \
    X(BWDW_CELLS) X(BWDW_PADDED) X(BWDX_BANDS) X(BWDX_CSR) X(BWDX_DIRECT) X(BWDX_HSW) X(BWDX_SPLIT) X(BWD_4X4)         \
    X(EVAL_CHUNK_BYTES) X(EVAL_NPW) X(EVAL_WALK_R) X(EVAL_WALK_SEG) X(FWD_4X4) X(FWD_CT) X(FWD_DIRECT) X(FWD_NW)       \
    X(FWD_ONE_ROW) X(FWD_S) X(FWD_SOFTMAX_IN_KERNEL) X(FWD_SUBSET) X(GSUM_SLICES) X(PACKED_4X4_HALVES) X(PACK_TILE)    \
    X(BWDW_LDS) X(BIN_CT) X(BIN_S) X(BIN_NW) X(BIN_HSW) X(BIN_PARTS) X(BIN_PIECE) X(BIN_HL) X(FWD_KPL)
enum ClgKnob {
#define CLG_KNOB_ENUM(name) K_##name,
    CLG_KNOBS(CLG_KNOB_ENUM)
#undef CLG_KNOB_ENUM
    K_COUNT
};
// value of the variable as read at the last (re)load, or nullptr when it was not set
const char *clg_knob(ClgKnob k);

static inline int64_t clg_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline hipStream_t clg_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;  // CDNA wavefront

// ---- device side ---------------------------------------------------------------------------
#if defined(__HIPCC__)

template <typename T>
struct Coef {  // y = ab*a*b + a_*a + b_*b + one
    T ab, a, b, one;
};

// Folds 16 gate probabilities into the 4 coefficients of the multilinear form.  Gate i has the
// truth table bits i = f00*8 + f01*4 + f10*2 + f11 and op_i(a,b) = f00 + (f10-f00) a + (f01-f00) b
// + (f00-f01-f10+f11) ab; the sums below are those columns written out (fixed order, so forward
// and backward kernels see bit-identical coefficients).
template <typename T>
__device__ __forceinline__ Coef<T> fold16(const T *__restrict__ w)
{
    Coef<T> c;
    c.ab = ((w[1] - w[2]) - w[4]) - T(2) * w[6] - w[7] + w[8] + T(2) * w[9] + w[11] + w[13] - w[14];
    c.a = (w[2] + w[3]) + (w[6] + w[7]) - (w[8] + w[9]) - (w[12] + w[13]);
    c.b = (w[4] + w[5]) + (w[6] + w[7]) - (w[8] + w[9]) - (w[10] + w[11]);
    c.one = ((w[8] + w[9]) + (w[10] + w[11])) + ((w[12] + w[13]) + (w[14] + w[15]));
    return c;
}

// softmax of 16 logits (maximum subtracted, one reciprocal), as clg_fc_fold computes it
template <typename T>
__device__ __forceinline__ void softmax16(const T *__restrict__ logits, T (&p)[16])
{
    T m = logits[0];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = logits[i];
        m = p[i] > m ? p[i] : m;
    }
    T sum = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = exp(p[i] - m);
        sum += p[i];
    }
    const T inv = T(1) / sum;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] *= inv;
        // the probability as it is stored: a fold of p in the same kernel must not contract this product into its sums, or
        // its coefficients would differ in the last bit from kernel to kernel and from a fold of the stored values
        asm volatile("" : "+v"(p[i]));
    }
}

template <typename T>
__device__ __forceinline__ T fma_t(T a, T b, T c);
template <>
__device__ __forceinline__ float fma_t<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <>
__device__ __forceinline__ double fma_t<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Gate value in the folded form, as three FMAs: a*(c_a + c_ab*b) + (c_b*b + c_1).  Always this
// instruction sequence, so equal inputs give equal bits wherever it is evaluated (the pool argmax
// depends on that).  With one-hot weights and binary inputs every intermediate is a small integer.
template <typename T>
__device__ __forceinline__ T gate(const Coef<T> &c, T a, T b)
{
    return fma_t(a, fma_t(c.ab, b, c.a), fma_t(c.b, b, c.one));
}
template <typename T>
__device__ __forceinline__ T gate_da(const Coef<T> &c, T b) { return fma_t(c.ab, b, c.a); }
template <typename T>
__device__ __forceinline__ T gate_db(const Coef<T> &c, T a) { return fma_t(c.ab, a, c.b); }

// grad_w[i] = sum_k COEF[k][i] * s[k] for the partial sums s = (sum g*ab, sum g*a, sum g*b, sum g).
template <typename T>
__device__ __forceinline__ T coef_transpose_row(int i, T sab, T sa, T sb, T s1)
{
    const int f00 = (i >> 3) & 1, f01 = (i >> 2) & 1, f10 = (i >> 1) & 1, f11 = i & 1;
    return T(f00 - f01 - f10 + f11) * sab + T(f10 - f00) * sa + T(f01 - f00) * sb + T(f00) * s1;
}

// ---- wave64 reductions with DPP (no LDS) ---------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_zero(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_zero(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_zero(double v)
{
    const uint64_t u = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)u, CTRL, ROW_MASK, 0xF, false);
    const uint32_t hi = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(u >> 32), CTRL, ROW_MASK, 0xF, false);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

// Sum over the 64 lanes in a fixed tree; the total is valid in lane 63 (returned broadcast).
template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
    v += dpp_zero<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v += dpp_zero<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v += dpp_zero<0x141, 0xF>(v);  // row_half_mirror
    v += dpp_zero<0x140, 0xF>(v);  // row_mirror
    v += dpp_zero<0x142, 0xA>(v);  // row_bcast15 into rows 1,3
    v += dpp_zero<0x143, 0xC>(v);  // row_bcast31 into rows 2,3
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)u, 63);
        const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(u >> 32), 63);
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    }
}

// Sum over each row of 16 lanes, valid in all of its lanes (the first four steps of wave_sum).
template <typename T>
__device__ __forceinline__ T row16_sum(T v)
{
    v += dpp_zero<0xB1, 0xF>(v);
    v += dpp_zero<0x4E, 0xF>(v);
    v += dpp_zero<0x141, 0xF>(v);
    v += dpp_zero<0x140, 0xF>(v);
    return v;
}
// Maximum over each row of 16 lanes, valid in all of its lanes.
template <typename T>
__device__ __forceinline__ T row16_max(T v)
{
    T o = dpp_zero<0xB1, 0xF>(v);
    v = o > v ? o : v;
    o = dpp_zero<0x4E, 0xF>(v);
    v = o > v ? o : v;
    o = dpp_zero<0x141, 0xF>(v);
    v = o > v ? o : v;
    o = dpp_zero<0x140, 0xF>(v);
    return o > v ? o : v;
}
// Gradient w.r.t. the logit of a 16-way softmax from the gradient g w.r.t. its probability p, the 16 gates
// of one node sitting in the 16 lanes of a row: p_i (g_i - sum_j p_j g_j).
template <typename T>
__device__ __forceinline__ T softmax16_backward(T g, T p) { return p * (g - row16_sum(p * g)); }

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// A wiring / reverse-map entry as the kernels use it: forced into 0..n-1, so that a corrupted index buffer (the host checks
// are cached and a write through `.data` goes past them) reads a wrong row instead of faulting the GPU.
__device__ __forceinline__ int64_t clamp_index(int64_t i, int64_t n) { return i < 0 ? 0 : (i < n ? i : n - 1); }

// selection tap: ch << 16 | row << 8 | col
struct Tap {
    int ch, ry, rx;
};
// Decoded and forced into the layer's ranges (channel < cin, row < kh, column < kw): the kernels turn taps into addresses
// without bounds checks, so a selection buffer that was corrupted behind the cached host check must not reach them raw.
struct TapLimit {
    int cin, kh, kw;
};
__device__ __forceinline__ int tap_channel(int32_t s, int cin) { return min((s >> 16) & 0xFFFF, cin - 1); }
__device__ __forceinline__ Tap unpack_tap(int32_t s, const TapLimit &lim)
{
    return Tap{tap_channel(s, lim.cin), min((s >> 8) & 0xFF, lim.kh - 1), min(s & 0xFF, lim.kw - 1)};
}

// ---- bitwise gates on packed samples ---------------------------------------------------------
struct Masks {
    uint32_t f00, f01, f10, f11;  // all-ones / all-zeros per truth-table entry
};
__device__ __forceinline__ Masks gate_masks(int id)
{
    return Masks{0u - ((id >> 3) & 1u), 0u - ((id >> 2) & 1u), 0u - ((id >> 1) & 1u), 0u - (id & 1u)};
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// 2:1 multiplexers on bits: b selects inside each half, a selects the half.  V is uint32_t or a
// vector of them (the masks are splat).
template <typename V>
__device__ __forceinline__ V gate_vec(const Masks &m, V a, V b)
{
    const V t1 = (b & (V)m.f11) | (~b & (V)m.f10);
    const V t0 = (b & (V)m.f01) | (~b & (V)m.f00);
    return (a & t1) | (~a & t0);
}
__device__ __forceinline__ uint32_t gate_bits(const Masks &m, uint32_t a, uint32_t b) { return gate_vec<uint32_t>(m, a, b); }

#endif  // __HIPCC__
