/* C ABI of the MI355X TV inpainting layer (libinpaint_hip.so).
 *
 * Plain pointers and sizes only; every pointer is a device pointer on the current HIP device unless
 * the parameter says "host".  All tensors are contiguous NCHW float32.  `stream` is a hipStream_t
 * passed as void* (NULL = the default stream); the calls enqueue work and return without waiting.
 * Return value 0 = ok; anything else is an error and tvinpaint_last_error() describes it.
 */
#ifndef TVINPAINT_H_
#define TVINPAINT_H_

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes shared by the TV and TGV entry points. */
#define INPAINT_OK 0
#define INPAINT_ERR_ID 1        /* id outside [0, 10)            (reference: returns 1, TV.cu:1468-1472) */
#define INPAINT_ERR_ARG 2       /* null pointer / non-positive size / its out of range                   */
#define INPAINT_ERR_ITS 3       /* its needs more than 100 checkpoints (reference: TV.h:9-15 overflows)  */
#define INPAINT_ERR_PAIRING 4   /* backward does not match the forward that filled this id's state       */
#define INPAINT_ERR_HIP 5       /* a HIP runtime call failed                                             */

/* Replaces TVInpaintFista::forward (cudaTV/cudaCode/TVInpaintFista.h:71-72,
 * cudaTV/cudaCode/TVInpaintFista.cu:1463-1559), bound by cudaTV/TVInpaintFista_cuda.cpp:47-88.
 *   dx, dy, c : (n,1,ih,iw) edge weights along W / along H and confidence, read only
 *   b, init   : (n,ic,ih,iw) right-hand side and starting point, read only
 *   out       : (n,ic,ih,iw) x after 2*floor(its/2) FISTA iterations
 *   id        : state slot in [0,10); the matching backward consumes the checkpoints stored here.
 * n > 1 runs n independent problems (the reference accepts n == 1 only). */
int tvinpaint_forward(const float* dx, const float* dy, const float* c, const float* b, const float* init,
                      float* out, int n, int ic, int ih, int iw, int its, int id, void* stream);

/* Replaces TVInpaintFista::backward (TVInpaintFista.h:82-85, TVInpaintFista.cu:1570-1831), bound by
 * TVInpaintFista_cuda.cpp:99-143.
 *   gin            : (n,ic,ih,iw) upstream gradient; non-finite entries are zeroed IN PLACE
 *                    (TVInpaintFista.cu:1609-1623)
 *   gx, gy, gc     : (n,1,ih,iw) gradients wrt dx, dy, c   (overwritten)
 *   gb, gi         : (n,ic,ih,iw) gradients wrt b and init (overwritten)
 * Must follow a tvinpaint_forward with the same shape, its and id.
 * Range: the gradients are those of the reference's arithmetic bit for bit while they stay normal floats (tested for
 * upstream gradients from 1e-30 to 1e30 times N(0,1)); results that fall into the denormal range (upstream around
 * 1e-36 and below) agree to their last bits only.  The same holds for tgvinpaint_backward. */
int tvinpaint_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin,
                       float* gx, float* gy, float* gc, float* gb, float* gi, int n, int ic, int ih,
                       int iw, int its, int id, void* stream);

/* The forward pass of tvinpaint_forward for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same arguments, kernels and result (bit for bit) as tvinpaint_forward, without an id: nothing is kept for a
 * backward pass, so there is no matching backward.  The iterate ping-pongs live in a fixed device array inside
 * the library (64 MiB per GPU, held until the process ends), so the call makes no hipMalloc / hipFree; it returns
 * INPAINT_ERR_ARG when n*ic*ih*iw exceeds tvinpaint_forward_noalloc_max_floats() (4,194,304 floats = one field of
 * 16 x 2 x 256 x 512).  All calls on one GPU share that array: calls that overlap on one GPU (two streams, two
 * threads) race; calls ordered on one stream do not.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make that call outside a graph capture. */
int tvinpaint_forward_noalloc(const float* dx, const float* dy, const float* c, const float* b, const float* init,
                              float* out, int n, int ic, int ih, int iw, int its, void* stream);
long long tvinpaint_forward_noalloc_max_floats(void);

/* Per-id state (idStruct, TVInpaintFista.h:7-50).  state6 (host) = {run, av_GC, av_GX, av_GY, av_GB,
 * av_GI}.  get waits for the slot's stream; reset frees the slot's device buffers as well. */
int tvinpaint_get_state(int id, double* state6);
int tvinpaint_set_state(int id, const double* state6);
int tvinpaint_reset_id(int id);

/* Statistics of the last backward's output guard (check_gradUpdate, TVInpaintFista.cu:158-175), host
 * array of 5 tensors (C, X, Y, B, I) x {mean |g|, max |g|, count above 1e7, count non-finite,
 * action (0 plain, 1 rescaled, 2 killed)}.  Waits for the slot's stream. */
int tvinpaint_guard_stats(int id, double* stats25);

/* Which gradient the next backwards on `id` return.  0 (default): the reference's, bit for bit, with everything
 * its hand-derived backward does differently from the chain rule.  1: the corrected gradient -- the adjoint is
 * linearised at the y the forward pass really used (the reference rebuilds y from the half-step iterates with a
 * simplified prox, TVInpaintFista.cu:1130-1189, and uses the checkpoint y_k0 for y_k0+1 at every segment start,
 * 1724-1727), iteration 0 is back-propagated too (the reference stops before it and returns g_x[1] as the gradient
 * wrt the start, 1696-1729, 1816), and the multipliers 0.1 / 0.1 / 1.0 and the global 0.1 (63-69) are 1.  The
 * clamp of the adjoint iterates (797-799), the upstream scrub and the output guard stay.  With them inactive the
 * result is the gradient of the forward pass (tests compare it with automatic differentiation).  Any channel
 * count; same speed as the default.  Set it before the forward pass whose backward it is meant for: the forward pass
 * latches the id's mode (with every x05 row kept it stores, at each checkpoint, only the half that mode's backward
 * reads), and a backward pass under another mode returns INPAINT_ERR_PAIRING, whatever the keep mode. */
int tvinpaint_gradient_mode(int id, int mode);

/* Which intermediate iterates (the x05 rows of TVInpaintFista.cu:1678-1687) the next forwards on `id` keep for
 * the backward pass.  0: none -- the backward recomputes every segment from its checkpoint, the reference's order
 * of work and its memory footprint (2 sqrt(its) + sqrt(its) fields).  1: those of the last segment.  2 (default):
 * all of them -- its fields of memory, no recompute, and the fastest backward.  The gradients are the same bits
 * in every mode.  A forward whose gradients are never asked for is fastest with 0.  Mode 2 falls back to 1 when
 * the rows would need more than INPAINT_KEEP_GB GiB (when the variable is not set: more than 32 GiB, or more than a
 * quarter of the device's free memory at the moment the slot has to grow) or the device cannot allocate them;
 * INPAINT_KEEP=0|1|2 overrides this call.
 * No counterpart in the reference, which always recomputes. */
int tvinpaint_keep_iterates(int id, int mode);

/* Bytes of device memory the slot currently owns (0 if none). */
long long tvinpaint_slot_bytes(int id);

/* Who owns the slots' device memory.  The reference callocs and frees its checkpoints on the host in every forward
 * (TVInpaintFista.cu:1510-1521, TVInpaintFista.h:18-37); here each id holds ONE device block per shape, and by default
 * the library takes it from hipMalloc.  A host program that runs its own pool (PyTorch's caching allocator) hands over
 * two callbacks instead, so that the block comes out of, and goes back to, the pool it can see and reuse:
 *   alloc(bytes, device, stream, user) -> device pointer aligned to 256 bytes, or NULL when it cannot (the call then
 *                                         fails with INPAINT_ERR_HIP, or falls back from keep mode 2 to 1)
 *   release(ptr, user)                    called once per block: when the id's shape changes, by tvinpaint_reset_id,
 *                                         never while work on the block is still in flight (the id's stream is
 *                                         synchronised first)
 * Both NULL restores hipMalloc / hipFree.  A block is always released by the callback pair that made it, so the
 * allocator may be changed while ids hold memory.  Not thread safe against concurrent forwards. */
typedef void* (*inpaint_alloc_fn)(unsigned long long bytes, int device, void* stream, void* user);
typedef void (*inpaint_release_fn)(void* ptr, void* user);
int tvinpaint_set_allocator(inpaint_alloc_fn alloc, inpaint_release_fn release, void* user);

/* Host-only: checkpoint schedule and FISTA extrapolation factors the layer uses for `its`
 * (TVInpaintFista.cu:1499-1508,1523 and 1525-1532).  iterations_out holds floor(sqrt(its)) ints. */
int tvinpaint_schedule(int its, int* iterations_out, int* max_inter_its);
void tvinpaint_step_sizes(int its, float* out);

/* Host-only: the guard's decision rule for one tensor (update_correct_av_step_host,
 * TVInpaintFista.cu:128-155).  Returns the action and writes the multiplier and the new running mean. */
int tvinpaint_guard_decide(int run, double av_gc, double av_running, double* mult_out, double* av_out);

/* The INPAINT_* environment variables (testing and tuning switches: kernel selection, strip heights, keep-mode
 * override and budget) are read once per process, on the first call that needs one, and again by every *_reset_id()
 * and by this call; changing one in a running process has no effect until then. */
void inpaint_reload_env(void);
/* The keep mode INPAINT_KEEP / INPAINT_KEEP_LAST currently force on every id (-1: none), as last read. */
int inpaint_keep_override(void);

/* Text of the last error on the calling thread ("" if none). */
const char* tvinpaint_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* TVINPAINT_H_ */
