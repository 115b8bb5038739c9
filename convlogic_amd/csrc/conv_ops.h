// Element policies of the fused conv-logic block forward: relaxed gates on float / double with a 2x2 max pool and its
// arg-max code, or bitwise gates on 64 packed samples per uint64 word with an OR pool.
#pragma once

#include "conv_tile.h"

#if defined(__HIPCC__)
namespace {

// ---- element policies ------------------------------------------------------------------------
template <typename T>
struct FloatOps {
    using Elem = T;
    static constexpr int kParams = 28;                               // LDS elements per kernel: 7 gates x (ab, a, b, one)
    struct Params {
        Tree<T> tr;
    };
    // params = gate probabilities [c_out, 7, 16]
    static __device__ __forceinline__ void stage_params(Elem *__restrict__ dst, const void *__restrict__ params, int c0, int ct_cur,
                                                        int tid, int nthreads)
    {
        const T *w = reinterpret_cast<const T *>(params);
        for (int q = tid; q < ct_cur * 7; q += nthreads) {
            const Coef<T> cf = fold16(w + ((int64_t)c0 * 7 + q) * 16);
            dst[q * 4 + 0] = cf.ab;
            dst[q * 4 + 1] = cf.a;
            dst[q * 4 + 2] = cf.b;
            dst[q * 4 + 3] = cf.one;
        }
    }
    static __device__ __forceinline__ Params load(const Elem *__restrict__ src, int lc)
    {
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            pr.tr.g[k].ab = to_sgpr(src[(lc * 7 + k) * 4 + 0]);
            pr.tr.g[k].a = to_sgpr(src[(lc * 7 + k) * 4 + 1]);
            pr.tr.g[k].b = to_sgpr(src[(lc * 7 + k) * 4 + 2]);
            pr.tr.g[k].one = to_sgpr(src[(lc * 7 + k) * 4 + 3]);
        }
        return pr;
    }
    // folded = [c_out][7][4] coefficients written by convblock_w_prepare_kernel
    static __device__ __forceinline__ Params load_global(const void *__restrict__ folded, int c)
    {
        const T *fc = reinterpret_cast<const T *>(folded) + (int64_t)c * 28;
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) pr.tr.g[k] = Coef<T>{fc[4 * k], fc[4 * k + 1], fc[4 * k + 2], fc[4 * k + 3]};
        return pr;
    }
    static __device__ __forceinline__ Elem root(const Params &pr, const Elem (&v)[8]) { return eval_tree(pr.tr, v).root; }
    // strict > in window order (0,0),(0,1),(1,0),(1,1): the first maximum wins
    static __device__ __forceinline__ void pool_store(Elem r0, Elem r0o, Elem r1, Elem r1o, Elem *__restrict__ yb,
                                                      uint8_t *__restrict__ ab, int idx)
    {
        Elem best = r0;
        int code = 0;
        if (r0o > best) { best = r0o; code = 1; }
        if (r1 > best) { best = r1; code = 2; }
        if (r1o > best) { best = r1o; code = 3; }
        yb[idx] = best;
        ab[idx] = (uint8_t)code;
    }
    // the same rule on the four values of a window in a register array
    static __device__ __forceinline__ Elem pool4(const Elem (&r)[4], int &code)
    {
        Elem best = r[0];
        code = 0;
#pragma unroll
        for (int q = 1; q < 4; ++q) {
            if (r[q] > best) {
                best = r[q];
                code = q;
            }
        }
        return best;
    }
};

struct BitOps {
    using Elem = uint64_t;
    static constexpr int kParams = 1;                                // 7 gate ids, 4 bits each
    struct Params {
        Masks m[7];
    };
    // params = gate ids uint8 [c_out, 7]
    static __device__ __forceinline__ void stage_params(Elem *__restrict__ dst, const void *__restrict__ params, int c0, int ct_cur,
                                                        int tid, int nthreads)
    {
        const uint8_t *gid = reinterpret_cast<const uint8_t *>(params);
        for (int q = tid; q < ct_cur; q += nthreads) {
            uint64_t pk = 0;
            for (int k = 0; k < 7; ++k) pk |= (uint64_t)(gid[((int64_t)c0 + q) * 7 + k] & 15) << (4 * k);
            dst[q] = pk;
        }
    }
    static __device__ __forceinline__ Params load(const Elem *__restrict__ src, int lc)
    {
        const uint32_t pk = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src[lc]);
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) pr.m[k] = gate_masks((pk >> (4 * k)) & 15);
        return pr;
    }
    static __device__ __forceinline__ Params load_global(const void *__restrict__ gates, int c)
    {
        const uint8_t *gid = reinterpret_cast<const uint8_t *>(gates) + (int64_t)c * 7;
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) pr.m[k] = gate_masks(gid[k] & 15);
        return pr;
    }
    static __device__ __forceinline__ Elem gate64(const Masks &m, Elem a, Elem b)
    {
        const uint32_t lo = gate_bits(m, (uint32_t)a, (uint32_t)b), hi = gate_bits(m, (uint32_t)(a >> 32), (uint32_t)(b >> 32));
        return ((uint64_t)hi << 32) | lo;
    }
    static __device__ __forceinline__ Elem root(const Params &pr, const Elem (&v)[8])
    {
        Elem leaf[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) leaf[q] = gate64(pr.m[q], v[2 * q], v[2 * q + 1]);
        return gate64(pr.m[6], gate64(pr.m[4], leaf[0], leaf[1]), gate64(pr.m[5], leaf[2], leaf[3]));
    }
    static __device__ __forceinline__ void pool_store(Elem r0, Elem r0o, Elem r1, Elem r1o, Elem *__restrict__ yb,
                                                      uint8_t *__restrict__, int idx)
    {
        yb[idx] = (r0 | r0o) | (r1 | r1o);
    }
    static __device__ __forceinline__ Elem pool4(const Elem (&r)[4], int &code)
    {
        code = 0;
        return (r[0] | r[1]) | (r[2] | r[3]);
    }
};

}  // namespace
#endif
