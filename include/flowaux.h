/* C ABI of the two small flow layers that feed the inpainting layer (libinpaint_hip.so): the
 * quadratic sub-pixel fit of a matching cost and the median of a per-pixel displacement histogram.
 *
 * Same conventions as tvinpaint.h: plain pointers and sizes, device pointers on the current HIP
 * device, contiguous float32 tensors, `stream` a hipStream_t passed as void* (NULL = the default
 * stream).  Return value 0 = ok; the error codes are the INPAINT_ERR_* values of tvinpaint.h and
 * flowaux_last_error() describes the failure.  The calls only enqueue work; they keep no state and
 * allocate nothing (the one scratch buffer is the caller's).
 */
#ifndef FLOWAUX_H_
#define FLOWAUX_H_

#include "tvinpaint.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces FlowQuadFitting::forward (cudaQuadFit/cudaCode/quadFit.h:22-23,
 * cudaQuadFit/cudaCode/quadFit.cu:14-139,308-331), bound by cudaQuadFit/QuadFit_cuda.cpp:41-75.
 *   im0, im1 : (n,ic,ih,iw) feature maps of the first / second image
 *   flow     : (n,flow_channels,ih,iw), flow_channels >= 2; channel 0 = x, channel 1 = y displacement.
 *              (The reference kernel indexes a 2-channel tensor, quadFit.cu:314, while its Python module
 *              hands over 3 channels, cudaQuadFit/QuadFitting.py:53; the channel count is explicit here.)
 *   out      : (n,3,ih,iw) = (offset in x, offset in y, fitted score); all three are zero where
 *              the displaced pixel leaves the image (a NaN displacement counts as leaving it; the reference
 *              would index with an undefined integer).  The callee writes 3 channels as the reference
 *              kernel does (quadFit.cu:137,315; the reference binding allocates only 2, QuadFit_cuda.cpp:60).
 */
int quadfit_forward(const float* im0, const float* im1, const float* flow, float* out, int n, int ic, int ih,
                    int iw, int flow_channels, void* stream);

/* Replaces FlowQuadFitting::backward (quadFit.h:30-32, quadFit.cu:145-300,338-369), bound by
 * QuadFit_cuda.cpp:83-114.
 *   gin    : (n,3,ih,iw) upstream gradient wrt `out`
 *   g0, g1 : (n,ic,ih,iw) gradients wrt im0 / im1 (overwritten).  There is no gradient wrt the flow
 *            (quadFit.h:11-12).
 *   workspace, workspace_bytes : device scratch of at least quadfit_backward_workspace_bytes(n,ih,iw)
 *            bytes, 16-byte aligned, contents irrelevant on entry.  With it g1 is GATHERED through a
 *            per-call inverse map (no float atomics unless more than 4 pixels land on one position).
 *            workspace == NULL selects the reference's scatter with float atomics (quadFit.cu:279-283,
 *            296), which this GPU executes far below memory speed.  Either way the sums that form g1 are
 *            order dependent at the rounding level, as they are in the reference.
 */
long long quadfit_backward_workspace_bytes(int n, int ih, int iw);
int quadfit_backward(const float* im0, const float* im1, const float* flow, const float* gin, float* g0,
                     float* g1, int n, int ic, int ih, int iw, int flow_channels, void* workspace,
                     long long workspace_bytes, void* stream);

/* Replaces MediMax::forward (cudaMedian/cudaCode/medimax.h:13, cudaMedian/cudaCode/medimax.cu:17-44,
 * 131-168), bound by cudaMedian/median_cuda.cpp:36-70.
 *   vol : (n,ih,iw,num_disp) histogram over num_disp displacement bins, bins innermost
 *   out : (n,2,ih,iw) = (position of the median in bins, mass of the bin that holds it); zero where the
 *         running sum never reaches one half.
 * All n samples are processed (the reference kernel derives the pixel from an index into the 2-channel
 * output, medimax.cu:23, which is right for n == 1 only).
 */
int medimax_forward(const float* vol, float* out, int n, int ih, int iw, int num_disp, void* stream);

/* Replaces MediMax::backward (medimax.h:14, medimax.cu:46-93,170-190), bound by median_cuda.cpp:72-105.
 *   gin  : (n,2,ih,iw) upstream gradient wrt `out`       gvol : (n,ih,iw,num_disp) (overwritten)
 */
int medimax_backward(const float* vol, const float* gin, float* gvol, int n, int ih, int iw, int num_disp,
                     void* stream);

/* Measurement hooks, as tvinpaint_profile / tvinpaint_profile_read: with profiling on, every backward
 * call brackets one kernel with a HIP event pair on the caller's stream; _read waits for them and returns their
 * total.  enable = 1: the per-source pass of the quadratic fit, the whole-histogram kernel of the median;
 * enable = 2: the gather pass of the quadratic fit (the median as for 1); 0 switches the events off. */
int flowaux_profile(int enable);
int flowaux_profile_read(double* total_ms, int* launches);

const char* flowaux_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* FLOWAUX_H_ */
