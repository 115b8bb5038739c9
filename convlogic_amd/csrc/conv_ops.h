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
    static constexpr bool kOrPool = false;
    struct Params {
        Tree<T> tr;
    };
    // params = gate probabilities [c_out, 7, 16], or the logits (from_logits): then the softmax is taken here and, where
    // probs_out is given, written out for the backward pass
    static __device__ __forceinline__ void stage_params(Elem *__restrict__ dst, const void *__restrict__ params, int c0, int ct_cur,
                                                        int tid, int nthreads, bool from_logits = false, void *probs_out = nullptr)
    {
        const T *w = reinterpret_cast<const T *>(params);
        for (int q = tid; q < ct_cur * 7; q += nthreads) {
            const T *row = w + ((int64_t)c0 * 7 + q) * 16;
            T pr[16];
            if (from_logits) {
                softmax16(row, pr);
                if (probs_out != nullptr) {
                    T *po = reinterpret_cast<T *>(probs_out) + ((int64_t)c0 * 7 + q) * 16;
#pragma unroll
                    for (int i = 0; i < 16; ++i) po[i] = pr[i];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = row[i];
            }
            const Coef<T> cf = fold16(pr);
            dst[q * 4 + 0] = cf.ab;
            dst[q * 4 + 1] = cf.a;
            dst[q * 4 + 2] = cf.b;
            dst[q * 4 + 3] = cf.one;
        }
    }
    // the same with the coefficients left in vector registers (every lane reads the same LDS words): for loops that
    // meet a kernel once, where 28 moves to scalar registers cost more than they save
    static __device__ __forceinline__ Params load_once(const Elem *__restrict__ src, int lc)
    {
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            pr.tr.g[k].ab = src[(lc * 7 + k) * 4 + 0];
            pr.tr.g[k].a = src[(lc * 7 + k) * 4 + 1];
            pr.tr.g[k].b = src[(lc * 7 + k) * 4 + 2];
            pr.tr.g[k].one = src[(lc * 7 + k) * 4 + 3];
        }
        return pr;
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
    static __device__ __forceinline__ Elem pool4(const Params &, const Elem (&r)[4], int &code)
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

// Packed samples, gates as three bitwise multiplexers with the truth table as all-ones / all-zeros masks: two of the
// four masks of a gate have to sit in vector registers (one scalar operand per instruction), which pays when a
// wavefront evaluates a kernel at many positions.
struct BitOps {
    using Elem = uint64_t;
    static constexpr int kParams = 1;                                // 7 gate ids, 4 bits each
    static constexpr bool kOrPool = true;                            // the pool is an OR: any order, no arg-max
    struct Params {
        Masks m[7];
    };
    // params = gate ids uint8 [c_out, 7]
    static __device__ __forceinline__ void stage_params(Elem *__restrict__ dst, const void *__restrict__ params, int c0, int ct_cur,
                                                        int tid, int nthreads, bool = false, void * = nullptr)
    {
        const uint8_t *gid = reinterpret_cast<const uint8_t *>(params);
        for (int q = tid; q < ct_cur; q += nthreads) {
            uint64_t pk = 0;
            for (int k = 0; k < 7; ++k) pk |= (uint64_t)(gid[((int64_t)c0 + q) * 7 + k] & 15) << (4 * k);
            dst[q] = pk;
        }
    }
    static __device__ __forceinline__ Params load_once(const Elem *__restrict__ src, int lc) { return load(src, lc); }
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
    // the same tree on 32 samples
    static __device__ __forceinline__ uint32_t root32(const Params &pr, const uint32_t (&v)[8])
    {
        uint32_t leaf[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) leaf[q] = gate_bits(pr.m[q], v[2 * q], v[2 * q + 1]);
        return gate_bits(pr.m[6], gate_bits(pr.m[4], leaf[0], leaf[1]), gate_bits(pr.m[5], leaf[2], leaf[3]));
    }
    static __device__ __forceinline__ Elem root_true(const Params &pr, const Elem (&v)[8]) { return root(pr, v); }
    static __device__ __forceinline__ Elem join(const Params &, Elem a, Elem b) { return a | b; }
    static __device__ __forceinline__ Elem join_last(const Params &, Elem a, Elem b) { return a | b; }
    static __device__ __forceinline__ Elem pool4(const Params &, const Elem (&r)[4], int &code)
    {
        code = 0;
        return (r[0] | r[1]) | (r[2] | r[3]);
    }
};

// The same for kernels that a wavefront evaluates at ONE position before it moves on (no room to amortise vector
// masks): a gate is its algebraic normal form  y = c0 ^ (c1 & a) ^ (c2 & b) ^ (c3 & a & b)  with the constant
// c0 moved into the truth table of the gate that consumes y (an input that arrives inverted permutes the table), so a
// gate costs three 3-input bit operations with one scalar mask each; the root's c0 is applied once at the end.
// tree_code(): the 7 gate ids of a kernel -> bits 3k..3k+2 = (c1, c2, c3) of gate k, bit 21 = c0 of the root.
__host__ __device__ inline uint32_t tree_code(const uint8_t *gid)
{
    uint32_t code = 0;
    int inv[7];                                                      // gate k delivers its true output xor inv[k]
#pragma unroll
    for (int k = 0; k < 7; ++k) {
        const int id = gid[k] & 15;
        const int pa = k < 4 ? 0 : inv[2 * (k - 4)], pb = k < 4 ? 0 : inv[2 * (k - 4) + 1];
        // truth table entry for (a, b) = bit 3 - 2a - b of the gate id
        const int f00 = (id >> (3 - 2 * pa - pb)) & 1, f01 = (id >> (3 - 2 * pa - (pb ^ 1))) & 1;
        const int f10 = (id >> (3 - 2 * (pa ^ 1) - pb)) & 1, f11 = (id >> (3 - 2 * (pa ^ 1) - (pb ^ 1))) & 1;
        inv[k] = f00;
        code |= (uint32_t)((f00 ^ f10) | ((f00 ^ f01) << 1) | ((f00 ^ f01 ^ f10 ^ f11) << 2)) << (3 * k);
    }
    return code | ((uint32_t)inv[6] << 21);
}

struct BitOpsAnf {
    using Elem = uint64_t;
    static constexpr int kParams = 1;                                // tree_code of the kernel
    static constexpr bool kOrPool = true;                            // the pool is an OR: any order, no arg-max
    struct Params {
        uint32_t c1[7], c2[7], c3[7], inv;                           // all-ones / all-zeros
    };
    static __device__ __forceinline__ Params unpack(uint32_t code)
    {
        Params pr;
#pragma unroll
        for (int k = 0; k < 7; ++k) {
            pr.c1[k] = 0u - ((code >> (3 * k)) & 1u);
            pr.c2[k] = 0u - ((code >> (3 * k + 1)) & 1u);
            pr.c3[k] = 0u - ((code >> (3 * k + 2)) & 1u);
        }
        pr.inv = 0u - ((code >> 21) & 1u);
        return pr;
    }
    // params = gate ids uint8 [c_out, 7]
    static __device__ __forceinline__ void stage_params(Elem *__restrict__ dst, const void *__restrict__ params, int c0, int ct_cur,
                                                        int tid, int nthreads, bool = false, void * = nullptr)
    {
        const uint8_t *gid = reinterpret_cast<const uint8_t *>(params);
        for (int q = tid; q < ct_cur; q += nthreads) dst[q] = tree_code(gid + ((int64_t)c0 + q) * 7);
    }
    static __device__ __forceinline__ Params load(const Elem *__restrict__ src, int lc)
    {
        return unpack((uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)src[lc]));
    }
    static __device__ __forceinline__ Params load_once(const Elem *__restrict__ src, int lc) { return load(src, lc); }
    static __device__ __forceinline__ Params load_global(const void *__restrict__ gates, int c)
    {
        return unpack(tree_code(reinterpret_cast<const uint8_t *>(gates) + (int64_t)c * 7));
    }
    static __device__ __forceinline__ uint32_t gate32(const Params &pr, int k, uint32_t a, uint32_t b)
    {
        // v_bitop3_b32 with the table spelled out (0xF0 = first, 0xCC = second, 0xAA = third operand), so that every
        // instruction carries exactly one scalar mask
        const uint32_t t = __builtin_amdgcn_bitop3_b32(a, b, pr.c3[k], 0xF0 & 0xCC & 0xAA);
        const uint32_t u = __builtin_amdgcn_bitop3_b32(t, a, pr.c1[k], 0xF0 ^ (0xCC & 0xAA));
        return __builtin_amdgcn_bitop3_b32(u, b, pr.c2[k], 0xF0 ^ (0xCC & 0xAA));
    }
    static __device__ __forceinline__ uint32_t root32(const Params &pr, const Elem (&v)[8], int shift)
    {
        uint32_t leaf[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) leaf[q] = gate32(pr, q, (uint32_t)(v[2 * q] >> shift), (uint32_t)(v[2 * q + 1] >> shift));
        return gate32(pr, 6, gate32(pr, 4, leaf[0], leaf[1]), gate32(pr, 5, leaf[2], leaf[3]));
    }
    // The root WITHOUT its constant: the true value is root(...) ^ pr.inv.  The 2x2 OR pool takes the constant along:
    // join() of raw values stays raw (OR of the true values = AND of the raw ones when they are inverted), join_last()
    // delivers the true pooled value -- one bit operation each, where the plain form needs an XOR per position.
    static __device__ __forceinline__ Elem root(const Params &pr, const Elem (&v)[8])
    {
        return ((uint64_t)root32(pr, v, 32) << 32) | root32(pr, v, 0);
    }
    static __device__ __forceinline__ Elem root_true(const Params &pr, const Elem (&v)[8])
    {
        return root(pr, v) ^ (((uint64_t)pr.inv << 32) | pr.inv);
    }
    template <int TABLE>
    static __device__ __forceinline__ Elem join_as(const Params &pr, Elem a, Elem b)
    {
        const uint32_t lo = __builtin_amdgcn_bitop3_b32((uint32_t)a, (uint32_t)b, pr.inv, TABLE);
        const uint32_t hi = __builtin_amdgcn_bitop3_b32((uint32_t)(a >> 32), (uint32_t)(b >> 32), pr.inv, TABLE);
        return ((uint64_t)hi << 32) | lo;
    }
    // inv ? a & b : a | b      (0xF0 = a, 0xCC = b, 0xAA = inv)
    static __device__ __forceinline__ Elem join(const Params &pr, Elem a, Elem b) { return join_as<0xD4>(pr, a, b); }
    // inv ? ~(a & b) : a | b
    static __device__ __forceinline__ Elem join_last(const Params &pr, Elem a, Elem b) { return join_as<0x7E>(pr, a, b); }
    static __device__ __forceinline__ Elem pool4(const Params &pr, const Elem (&r)[4], int &code)
    {
        code = 0;
        return join_last(pr, join(pr, r[0], r[1]), join(pr, r[2], r[3]));
    }
};

}  // namespace
#endif
