/* C ABI of the glue between two levels of a coarse-to-fine hierarchy of inpainting layers
 * (libinpaint_hip.so): what sits between the solution of level l and the inputs of level l+1.
 *
 * The reference describes the hierarchy (README.md:64-71: one layer instance, with its own id, per
 * level) but ships no code for the step between levels; this interface is the build's own.  Same
 * conventions as tvinpaint.h: device pointers, contiguous NCHW float32, `stream` a hipStream_t passed
 * as void*, return 0 = ok, INPAINT_ERR_* codes, hierarchy_last_error() for the message.  The calls
 * only enqueue work and allocate nothing.
 */
#ifndef HIERARCHY_H_
#define HIERARCHY_H_

#include "tvinpaint.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One launch that prepares level l+1 from level l:
 *   sol : (n,c,h,w) solution of the coarse level
 *   up  : (n,c,2h,2w) = scale * bilinear x2 upsampling of sol (half-pixel centres, border clamped: the
 *         definition torch.nn.functional.interpolate(mode="bilinear", align_corners=False) uses).  It is
 *         both the right-hand side b and the starting point of the fine level; flow vectors are in pixels,
 *         hence scale = 2.
 *   img : (n,1,2h,2w) guidance image of the fine level, or NULL
 *   wx, wy : (n,1,2h,2w) edge weights exp(-alpha |I(y,x+1) - I(y,x)|), exp(-alpha |I(y+1,x) - I(y,x)|),
 *         1 in the last column / row -- the dx, dy inputs of tvinpaint_forward.  Untouched when img is NULL.
 */
int hierarchy_next_level_forward(const float* sol, const float* img, float* up, float* wx, float* wy, int n, int c,
                                 int h, int w, float scale, float alpha, void* stream);

/* Adjoint of the upsampling: g_sol (n,c,h,w) = scale * up2^T (g_b + g_init), where g_b and g_init are the
 * fine level's gradients wrt its right-hand side and its starting point (tvinpaint_backward's gb and gi),
 * both (n,c,2h,2w); g_init may be NULL.  The edge weights have no gradient here: the guidance image is data.
 */
int hierarchy_next_level_backward(const float* g_b, const float* g_init, float* g_sol, int n, int c, int h, int w,
                                  float scale, void* stream);

const char* hierarchy_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* HIERARCHY_H_ */
