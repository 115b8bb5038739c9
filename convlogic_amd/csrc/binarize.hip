// Input binarisation in front of the logic layers: every pixel is compared with L thresholds and the
// results become L times as many {0,1} channels, threshold-major (channel l * c0 + c), either as floats
// for training or directly as packed words for inference (64 samples per word, group-major images --
// the layout the packed conv-logic block reads).
#include "clg_common.h"

namespace {

constexpr int kLevelsPerPass = 4;

// thread = one element of the [c0, h*w] plane set, blockIdx.y = group of 64 samples, blockIdx.z = pass over
// four thresholds: lanes read consecutive pixels of one sample (coalesced), 64 samples fill a word.
__global__ __launch_bounds__(256) void threshold_pack_kernel(const float *__restrict__ x, const float *__restrict__ thr,
                                                           uint64_t *__restrict__ words, int64_t n, int64_t plane_elems, int levels)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= plane_elems) return;
    const int64_t g = blockIdx.y;
    const int l0 = blockIdx.z * kLevelsPerPass;
    float t[kLevelsPerPass];
#pragma unroll
    for (int l = 0; l < kLevelsPerPass; ++l) t[l] = l0 + l < levels ? thr[l0 + l] : 0.0f;
    uint64_t w[kLevelsPerPass] = {0, 0, 0, 0};
    const int64_t s0 = g * 64;
    const int count = n - s0 < 64 ? (int)(n - s0) : 64;
    const float *src = x + s0 * plane_elems + e;
    for (int s = 0; s < count; s += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = s + j < count ? src[(int64_t)(s + j) * plane_elems] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
#pragma unroll
            for (int l = 0; l < kLevelsPerPass; ++l) w[l] |= (uint64_t)(s + j < count && v[j] > t[l]) << (s + j);
        }
    }
#pragma unroll
    for (int l = 0; l < kLevelsPerPass; ++l)
        if (l0 + l < levels) __builtin_nontemporal_store(w[l], &words[(g * levels + l0 + l) * plane_elems + e]);
}

__global__ __launch_bounds__(256) void threshold_float_kernel(const float *__restrict__ x, const float *__restrict__ thr,
                                                            float *__restrict__ out, int64_t n, int64_t plane_elems, int levels)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * plane_elems) return;
    const int64_t s = i / plane_elems, e = i - s * plane_elems;
    const float v = x[i];
    for (int l = 0; l < levels; ++l) out[(s * levels + l) * plane_elems + e] = v > thr[l] ? 1.0f : 0.0f;
}

int check_threshold_args(const void *x, const void *thr, const void *out, int64_t n, int64_t c0, int64_t hw, int64_t levels,
                         const char *name)
{
    CLG_REQUIRE(x && thr && out, "%s: null pointer argument", name);
    CLG_REQUIRE(n > 0 && c0 > 0 && hw > 0 && levels > 0, "%s: n, channels, pixels and levels must be positive", name);
    CLG_REQUIRE(levels <= 4096 && c0 * hw < (1ll << 31), "%s: at most 4096 levels and 2^31-1 elements per sample", name);
    return CLG_OK;
}

}  // namespace

extern "C" int clg_threshold_pack_images(const float *x, const float *thresholds, uint64_t *words, int64_t n, int64_t c0,
                                         int64_t hw, int64_t levels, void *stream)
{
    if (int e = check_threshold_args(x, thresholds, words, n, c0, hw, levels, "clg_threshold_pack_images")) return e;
    const int64_t groups = clg_ceil_div(n, 64), passes = clg_ceil_div(levels, kLevelsPerPass);
    CLG_REQUIRE(groups <= 65535 * 64ll, "clg_threshold_pack_images: batch too large for one launch");
    const int64_t plane_elems = c0 * hw;
    // the grid's y extent is limited to 65535: larger batches go in slabs of 65535 groups
    for (int64_t g0 = 0; g0 < groups; g0 += 65535) {
        const int64_t gs = groups - g0 < 65535 ? groups - g0 : 65535;
        hipLaunchKernelGGL(threshold_pack_kernel, dim3((unsigned)clg_ceil_div(plane_elems, 256), (unsigned)gs, (unsigned)passes),
                           dim3(256), 0, clg_stream(stream), x + g0 * 64 * plane_elems, thresholds,
                           words + g0 * levels * plane_elems, n - g0 * 64, plane_elems, (int)levels);
        CLG_CHECK_LAUNCH("clg_threshold_pack_images");
    }
    return CLG_OK;
}

extern "C" int clg_threshold_images(const float *x, const float *thresholds, float *out, int64_t n, int64_t c0, int64_t hw,
                                    int64_t levels, void *stream)
{
    if (int e = check_threshold_args(x, thresholds, out, n, c0, hw, levels, "clg_threshold_images")) return e;
    const int64_t total = n * c0 * hw;
    CLG_REQUIRE(clg_ceil_div(total, 256) < (1ll << 31), "clg_threshold_images: batch too large for one launch");
    hipLaunchKernelGGL(threshold_float_kernel, dim3((unsigned)clg_ceil_div(total, 256)), dim3(256), 0, clg_stream(stream), x,
                       thresholds, out, n, c0 * hw, (int)levels);
    CLG_CHECK_LAUNCH("clg_threshold_images");
    return CLG_OK;
}
