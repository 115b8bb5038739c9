/* CPU oracle for the packed-bit inference path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the three reference kernels that have no python twin:
 *   pack      src/difflogic/cuda/difflogic_kernel.cu:334-413
 *   eval      src/difflogic/cuda/difflogic_kernel.cu:271-293 with the gate switch of
 *             src/common/cuda_utils.cuh:162-199
 *   groupsum  src/difflogic/cuda/difflogic_kernel.cu:417-482
 * Words are handled as unsigned 64-bit lanes or as bytes; every gate is bitwise,
 * so the word width only fixes how samples map to bits (sample s = bit s%bits of
 * word s/bits, LSB first).
 *
 * Used by tests/ (against the numpy restatement in convlogic_oracle.py) and by
 * bench.py's cpu_baseline leg.  Nothing in the product links or loads it.
 * The reference has no tests for this path ("parity unpinned by the reference");
 * both restatements are pinned by the closed forms listed in convlogic_oracle.py.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static inline uint64_t gate64(uint64_t a, uint64_t b, int op)
{
    switch (op) {
    case 0: return 0;
    case 1: return a & b;
    case 2: return a & ~b;
    case 3: return a;
    case 4: return b & ~a;
    case 5: return b;
    case 6: return a ^ b;
    case 7: return a | b;
    case 8: return ~(a | b);
    case 9: return ~(a ^ b);
    case 10: return ~b;
    case 11: return ~b | a;
    case 12: return ~a;
    case 13: return ~a | b;
    case 14: return ~(a & b);
    default: return ~(uint64_t)0;
    }
}

/* x [in_dim, row_bytes] -> y [out_dim, row_bytes]; row_bytes = words * word_size. */
void oracle_eval_packed(const uint8_t *x, const int64_t *a, const int64_t *b, const uint8_t *gate,
                        uint8_t *y, int64_t out_dim, int64_t row_bytes)
{
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < out_dim; ++j) {
        const uint8_t *pa = x + a[j] * row_bytes, *pb = x + b[j] * row_bytes;
        uint8_t *py = y + j * row_bytes;
        const int op = gate[j];
        int64_t i = 0;
        for (; i + 8 <= row_bytes; i += 8) {
            uint64_t va, vb, vy;
            memcpy(&va, pa + i, 8);
            memcpy(&vb, pb + i, 8);
            vy = gate64(va, vb, op);
            memcpy(py + i, &vy, 8);
        }
        for (; i < row_bytes; ++i)
            py[i] = (uint8_t)gate64(pa[i], pb[i], op);
    }
}

/* t bool bytes [F, B] -> words [F, ceil(B/bits)] as little-endian byte rows. */
void oracle_pack_bits(const uint8_t *t, uint8_t *words, int64_t F, int64_t B, int bits)
{
    const int64_t W = (B + bits - 1) / bits, row_bytes = W * (bits / 8);
#pragma omp parallel for schedule(static)
    for (int64_t f = 0; f < F; ++f) {
        uint8_t *row = words + f * row_bytes;
        memset(row, 0, (size_t)row_bytes);
        for (int64_t s = 0; s < B; ++s)
            if (t[f * B + s])
                row[s >> 3] |= (uint8_t)(1u << (s & 7));
    }
}

/* words [F, row_bytes] -> out int32 [S, k], S = row_bytes*8 - pad_len. */
void oracle_group_bit_sum(const uint8_t *words, int32_t *out, int64_t F, int64_t row_bytes, int64_t pad_len,
                          int64_t k)
{
    const int64_t S = row_bytes * 8 - pad_len, cs = F / k;
#pragma omp parallel for schedule(static)
    for (int64_t s = 0; s < S; ++s)
        for (int64_t g = 0; g < k; ++g) {
            int32_t acc = 0;
            for (int64_t i = 0; i < cs; ++i)
                acc += (words[(g * cs + i) * row_bytes + (s >> 3)] >> (s & 7)) & 1;
            out[s * k + g] = acc;
        }
}
