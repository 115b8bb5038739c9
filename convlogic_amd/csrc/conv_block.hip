// Fused conv-logic block: entry points and shape dispatch.
#include "conv_common.h"

int clg_convblock_check(const clg_conv_geom *gg, Geom *g, int dtype, const char *name);
int clg_convblock_forward_generic(int dtype, const Geom &g, const void *x, const void *w, const int32_t *selection, void *y,
                                  uint8_t *argmax, hipStream_t st);
int clg_convblock_backward_x_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_x, hipStream_t st);
int clg_convblock_backward_w_generic(int dtype, const Geom &g, const void *grad_y, const void *x, const void *w,
                                     const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                                     hipStream_t st);
int clg_convblock_partial_blocks(const Geom &g);

extern "C" int clg_convblock_forward(int dtype, const clg_conv_geom *gg, const void *x, const void *w, const int32_t *selection,
                                     void *y, uint8_t *argmax, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_forward")) return e;
    CLG_REQUIRE(x && w && selection && y && argmax, "clg_convblock_forward: null pointer argument");
    return clg_convblock_forward_generic(dtype, g, x, w, selection, y, argmax, clg_stream(stream));
}

extern "C" int clg_convblock_backward_x(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                        const int32_t *selection, const uint8_t *argmax, void *grad_x, void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_x")) return e;
    CLG_REQUIRE(grad_y && x && w && selection && argmax && grad_x, "clg_convblock_backward_x: null pointer argument");
    return clg_convblock_backward_x_generic(dtype, g, grad_y, x, w, selection, argmax, grad_x, clg_stream(stream));
}

extern "C" int64_t clg_convblock_backward_w_scratch_bytes(int dtype, const clg_conv_geom *gg)
{
    Geom g;
    if (clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_w_scratch_bytes")) return -1;
    return (int64_t)g.c * clg_convblock_partial_blocks(g) * 28 * (dtype == CLG_F64 ? 8 : 4);
}

extern "C" int clg_convblock_backward_w(int dtype, const clg_conv_geom *gg, const void *grad_y, const void *x, const void *w,
                                        const int32_t *selection, const uint8_t *argmax, void *grad_w, void *scratch,
                                        void *stream)
{
    Geom g;
    if (int e = clg_convblock_check(gg, &g, dtype, "clg_convblock_backward_w")) return e;
    CLG_REQUIRE(grad_y && x && w && selection && argmax && grad_w && scratch, "clg_convblock_backward_w: null pointer argument");
    return clg_convblock_backward_w_generic(dtype, g, grad_y, x, w, selection, argmax, grad_w, scratch, clg_stream(stream));
}
