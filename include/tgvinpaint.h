/* C ABI of the MI355X TGV inpainting layer (libinpaint_hip.so).
 *
 * Same conventions as tvinpaint.h: plain pointers and sizes, device pointers on the current HIP
 * device unless the parameter says "host", contiguous NCHW float32 tensors, `stream` a hipStream_t
 * passed as void* (NULL = the default stream).  Return value 0 = ok; the error codes are the
 * INPAINT_ERR_* values of tvinpaint.h and tgvinpaint_last_error() describes the failure.
 *
 * Tensor layout: the layer's state is (u, v1, v2) per flow channel.  `init`, `out`, `gin`, `gi` are
 * (n, 3*ic, ih, iw) in variable-major order (all u channels, all v1 channels, all v2 channels) -- for
 * ic == 1 exactly the reference's 3-channel tensor.  `dx`, `dy` are (n, 2, ih, iw): channel 0 the
 * edge weight in [0,1], channel 1 the weight beta >= 0 of the auxiliary variables' regulariser.
 */
#ifndef TGVINPAINT_H_
#define TGVINPAINT_H_

#include "tvinpaint.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces FistaTGVHuberB2_id::forward (cudaTGV/cudaCode/TGVInpaintFista.h:70-71,
 * cudaTGV/cudaCode/TGVInpaintFistaBetas.cu:2475-2618), bound by cudaTGV/TGVInpaintFista_cuda.cpp:47-106.
 *   dx, dy : (n,2,ih,iw) read only (never scaled in place)     c : (n,1,ih,iw)     b : (n,ic,ih,iw)
 *   init   : (n,3*ic,ih,iw) starting point                    out : (n,3*ic,ih,iw) x after 2*floor(its/2) iterations
 * The Lipschitz constant (FistaInpaintB2_findLipshitz, TGVInpaintFistaBetas.cu:101-148,2513-2527) is
 * computed per sample on the device.  n > 1 runs n independent problems (the reference accepts 1). */
int tgvinpaint_forward(const float* dx, const float* dy, const float* c, const float* b, const float* init,
                       float* out, int n, int ic, int ih, int iw, int its, int id, void* stream);

/* Replaces FistaTGVHuberB2_id::backward (TGVInpaintFista.h:81-84, TGVInpaintFistaBetas.cu:2621-3063),
 * bound by TGVInpaintFista_cuda.cpp:117-172.
 *   gin     : (n,3*ic,ih,iw) upstream gradient.  If it holds any non-finite entry, or is zero
 *             everywhere, those entries are zeroed IN PLACE, all five outputs are zero and the id's
 *             run counter is left alone (TGVInpaintFistaBetas.cu:2686-2703).  This check is the call's
 *             one host wait.
 *   gx, gy  : (n,2,ih,iw)   gc : (n,1,ih,iw)   gb : (n,ic,ih,iw)   gi : (n,3*ic,ih,iw)   (overwritten)
 * Must follow a tgvinpaint_forward with the same shape, its and id. */
int tgvinpaint_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin,
                        float* gx, float* gy, float* gc, float* gb, float* gi, int n, int ic, int ih,
                        int iw, int its, int id, void* stream);

/* Per-id state (idStructBs, TGVInpaintFista.h:7-50); separate from the TV layer's ids.
 * state6 (host) = {run, av_GC, av_GX, av_GY, av_GB, av_GI}. */
int tgvinpaint_get_state(int id, double* state6);
int tgvinpaint_set_state(int id, const double* state6);
int tgvinpaint_reset_id(int id);

/* Which gradient the next backwards on `id` return.  0 (default): the reference's, bit for bit.  1: the corrected
 * gradient -- the adjoint is linearised at the y the forward pass really used (the reference rebuilds u with a
 * simplified prox and the auxiliary variables without their momentum, TGVInpaintFistaBetas.cu:1478-1541, and uses the
 * checkpoint y_k0 for y_k0+1 at every segment start, 2914-2917), the upper-triangle v2 block multiplies by hub^2 like
 * its siblings (355), iteration 0 is back-propagated too (2851-2933, 3047), and the multipliers (87-93) are 1.  The
 * clamp of the adjoint iterates (562-583), the upstream check and the output guard stay.  With them inactive the
 * result is the gradient of the forward pass (tests compare it with the float64 oracle that automatic differentiation
 * pins).  Any channel count; two adjoint steps per launch with two channels (5% slower than the default), one
 * otherwise.  Set it before the forward pass whose backward it is meant for, as tvinpaint_gradient_mode. */
int tgvinpaint_gradient_mode(int id, int mode);

/* Which intermediate iterates (the x05 rows of TGVInpaintFista.cu:2775-2814) the next forwards on `id` keep for
 * the backward pass.  0: none -- the backward recomputes every segment from its checkpoint, the reference's order
 * of work and its memory footprint.  1: those of the last segment.  2 (default): all of them -- its states
 * (3 fields each) of memory, no recompute, and the fastest backward.  The gradients are the same bits in every
 * mode.  A forward whose gradients are never asked for is fastest with 0.  Mode 2 falls back to 1 when the rows
 * would need more than INPAINT_KEEP_GB (default 32) GiB or the device cannot allocate them; INPAINT_KEEP=0|1|2 overrides this call.
 * No counterpart in the reference, which always recomputes. */
int tgvinpaint_keep_iterates(int id, int mode);

/* Statistics of the last backward's output guard (check_gradUpdate, TGVInpaintFistaHelp.cu:155-177):
 * 5 tensors (C, X, Y, B, I) x {mean |g|, max |g|, count above 5e6, count non-finite, action}.  The
 * guard on I looks at the u block only (TGVInpaintFistaBetas.cu:3014-3021). */
int tgvinpaint_guard_stats(int id, double* stats25);

long long tgvinpaint_slot_bytes(int id);

/* Who owns the TGV slots' device memory: as tvinpaint_set_allocator (the reference's per-forward calloc / free of the
 * checkpoints: TGVInpaintFistaBetas.cu:2534-2546, TGVInpaintFista.h:18-37). */
int tgvinpaint_set_allocator(inpaint_alloc_fn alloc, inpaint_release_fn release, void* user);

/* The per-sample step scale L = 1 / (max(32, max_p s_p) + 0.01) the last call on this id used
 * (host array of n doubles).  Waits for the slot's stream. */
int tgvinpaint_lipschitz(int id, double* L_host, int n);

/* Host-only: the guard's decision rule with this layer's constants (update_correct_av_step_host,
 * TGVInpaintFistaHelp.cu:119-151). */
int tgvinpaint_guard_decide(int run, double av_gc, double av_running, double* mult_out, double* av_out);

/* Text of the last error on the calling thread ("" if none; the same text as tvinpaint_last_error). */
const char* tgvinpaint_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* TGVINPAINT_H_ */
