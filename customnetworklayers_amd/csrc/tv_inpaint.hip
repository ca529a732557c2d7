// Huber-TV FISTA inpainting layer for MI355X (gfx950): kernels, per-id state and the C ABI.
//
// What the layer computes is fixed by the reference's kernels
// (cudaTV/cudaCode/TVInpaintFista.cu, cited per function below as TV.cu).  How it is computed is not:
//   * samples are a grid dimension (n >= 1), weights are scaled by L = 1/8 and masked at the image
//     border when they are loaded (no scaled copies, no textures);
//   * checkpoints, the x05 history, the adjoint iterates, the per-segment fp32 accumulators and
//     their fp64 totals all live in one device arena per id, sized once per shape;
//   * the y rebuild (get_yk) is fused into the adjoint kernels: y_{k+1} is rebuilt in registers and
//     never written to HBM;
//   * the output guard runs on the device (two reductions, a one-thread decision, a finalize
//     pass), so a backward call enqueues work and returns without a host synchronisation.
//
// Arithmetic contract: every value that can reach a Huber / prox switch (the iterates y, x, x05,
// the rebuilt y, the triangle norms) is computed with the operation order of the reference source,
// IEEE division and square root and no fused multiply-add (build with -ffp-contract=off).  At 100
// iterations a one-ulp deviation there flips a few hundred switches and moves the gradients by
// ~5e-3 of their maximum, above the layer's 1e-3 tolerance.
#include "inpaint_common.h"
#include "tv_strip_kernels.h"

#include <cstddef>
#include <cstdlib>

namespace {

using namespace inpaint;

// TV.cu:44,52,63-69,84-90
constexpr float kDelta = 0.1f;
constexpr float kLocalGCMult = 0.1f;
constexpr float kLocalGBMult = 1.0f;
constexpr float kGlobalGMult = 0.1f;
constexpr float kL = 0.125f;  // 1/Lipschitz, TV.cu:1478 (a power of two: scaling is exact)
const GuardParams kGuard = {10000000., 0., 50., 10., 0.975};

// Prox adjoint + confidence / rhs gradient: TV.cu:806-828 (and 240-255 for the first step).
// Only g05 continues down the chain; none of these values reaches a switch.
template <bool FIRST, bool TRUE_ADJ = false>
__device__ __forceinline__ void prox_adjoint(float df_dxk, float bb, float x05v, float conf, float& g05,
                                             float& gc, float& gb) {
  constexpr float kGC = TRUE_ADJ ? 1.f : kLocalGCMult, kGB = TRUE_ADJ ? 1.f : kLocalGBMult;
  const float diff = bb - x05v;
  const float sign = (diff < 0) ? -1.f : 1.f;
  if (1. + (double)conf >= (double)(sign * diff)) {
    gc += df_dxk * (bb / (1.f + conf) - (conf * bb + x05v) / ((1.f + conf) * (1.f + conf))) * kGC;
    g05 = df_dxk / (1.f + conf);
    gb += df_dxk * conf / (1.f + conf) * kGB;
  } else if (FIRST) {
    g05 = df_dxk;
    gc += sign * df_dxk * kGC;
    gb = 0.f;  // TV.cu:254
  } else if (conf >= sign * diff) {  // TV.cu:818-822, unreachable for conf >= 0
    g05 = 0.f;
    gb += df_dxk * kGB;
  } else {
    g05 = df_dxk;
    gc += sign * df_dxk * kGC;
  }
}

// First adjoint step: TV.cu:222-287.  TRUE_ADJ: multipliers 1 (the corrected gradient).
template <bool TRUE_ADJ>
__global__ __launch_bounds__(256) void tv_adjoint_first(const float* __restrict__ cf, const float* __restrict__ b,
                                                        const float* __restrict__ x05, float* __restrict__ gc,
                                                        float* __restrict__ gb, float* __restrict__ g05,
                                                        const float* __restrict__ gin, int C, long long HW,
                                                        long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // over n*HW pixels
  if (i >= total) return;
  const long long s = i / HW, p = i - s * HW;
  const float conf = cf[i];
  float gcv = gc[i];
  for (int ch = 0; ch < C; ch++) {
    const long long q = (s * C + ch) * HW + p;
    float g05v, gbv = gb[q];
    prox_adjoint<true, TRUE_ADJ>(gin[q], b[q], x05[q], conf, g05v, gcv, gbv);
    g05[q] = g05v;
    gb[q] = gbv;
  }
  gc[i] = gcv;
}

// Corrected gradient only: the gradient step of iteration 0, which the reference never back-propagates
// (TV.cu:1696-1729 ends after producing g05[0]; TV.cu:1816 returns g_x[1] as the gradient wrt the start).
// gi = J^T(y_0) g05[0] + g_x[0] with the transposed Jacobian of TV.cu:651-771 at the starting point y_0, and
// the weight gradients of iteration 0 (multiplier 1) are added to the fp64 totals.  One thread per pixel; each
// of the three triangles a pixel belongs to is evaluated here, as the reference's kernels do.
__global__ __launch_bounds__(256) void tv_adjoint_iter0(const float* __restrict__ wx_, const float* __restrict__ wy_,
                                                        const float* __restrict__ y0, const float* __restrict__ g05,
                                                        const float* __restrict__ gx0, float* __restrict__ gi,
                                                        double* __restrict__ tot_gx, double* __restrict__ tot_gy, int C,
                                                        int H, int W, long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // over n*HW pixels
  if (i >= total) return;
  const long long HW = (long long)H * W;
  const long long smp = i / HW, p = i - smp * HW;
  const int h = (int)(p / W), w = (int)(p - (long long)h * W);
  const float* wx = wx_ + smp * HW;
  const float* wy = wy_ + smp * HW;
  const float wx_0 = (w > 0) ? kL * wx[p - 1] : 0.f;
  const float wx_1 = (w < W - 1) ? kL * wx[p] : 0.f;
  const float wy_0 = (h > 0) ? kL * wy[p - W] : 0.f;
  const float wy_1 = (h < H - 1) ? kL * wy[p] : 0.f;
  const float wx_2 = (h > 0 && w < W - 1) ? kL * wx[p - W] : 0.f;
  const float wy_2 = (w > 0 && h < H - 1) ? kL * wy[p - 1] : 0.f;
  float gwx = 0.f, gwy = 0.f;
  for (int ch = 0; ch < C; ch++) {
    const long long q = (smp * C + ch) * HW;
    const float* y = y0 + q;
    const float* g = g05 + q;
    auto at = [&](const float* f, int hh, int ww) {
      return (hh >= 0 && hh < H && ww >= 0 && ww < W) ? f[(long long)hh * W + ww] : 0.f;
    };
    const float yk = y[p], df_dy = g[p];
    float t = df_dy;
    if (h > 0) {  // triangle owned by the pixel above, TV.cu:655-686
      const float yu = at(y, h - 1, w), yur = at(y, h - 1, w + 1), gu = at(g, h - 1, w), gur = at(g, h - 1, w + 1);
      const float a_y = (yk - yu) * (yk - yu) * wy_0;
      const float a_x = (yu - yur) * (yu - yur) * wx_2;
      const float hub = sqrtf(a_x + a_y);
      if (hub > kDelta) {
        const float nom = kDelta / hub;
        const float denom = nom / (2.f * hub * hub);
        t -= (df_dy - gu) * (wy_0 * nom);
        const float temp = -denom * 2.f * (yk - yu) * wy_0;
        t -= (df_dy - gu) * wy_0 * (yk - yu) * temp;
        t -= (gur - gu) * wx_2 * (yur - yu) * temp;
      } else {
        t -= (df_dy - gu) * wy_0;
      }
    }
    if (w > 0) {  // triangle owned by the pixel to the left, TV.cu:687-720
      const float yl = at(y, h, w - 1), yld = at(y, h + 1, w - 1), gl = at(g, h, w - 1), gld = at(g, h + 1, w - 1);
      const float a_x = (yk - yl) * (yk - yl) * wx_0;
      const float a_y = (yl - yld) * (yl - yld) * wy_2;
      const float hub = sqrtf(a_x + a_y);
      if (hub > kDelta) {
        const float nom = kDelta / hub;
        const float denom = nom / (2.f * hub * hub);
        t -= (df_dy - gl) * (wx_0 * nom);
        const float temp = -denom * 2.f * (yk - yl) * wx_0;
        t -= (df_dy - gl) * wx_0 * (yk - yl) * temp;
        t -= (gld - gl) * wy_2 * (yld - yl) * temp;
      } else {
        t -= (df_dy - gl) * wx_0;
      }
    }
    {  // the pixel's own triangle, TV.cu:722-771
      const float yr = at(y, h, w + 1), yd = at(y, h + 1, w), gr = at(g, h, w + 1), gd = at(g, h + 1, w);
      const float a_x = (yk - yr) * (yk - yr) * wx_1;
      const float a_y = (yk - yd) * (yk - yd) * wy_1;
      const float hub = sqrtf(a_x + a_y);
      if (hub > kDelta) {
        const float nom = kDelta / hub;
        const float denom = nom / (2.f * hub * hub);
        t -= (df_dy - gd) * (wy_1 * nom);
        t -= (df_dy - gr) * (wx_1 * nom);
        const float temp = denom * 2.f * ((yd - yk) * wy_1 + (yr - yk) * wx_1);
        t -= (df_dy - gd) * wy_1 * (yk - yd) * temp;
        t -= (df_dy - gr) * wx_1 * (yk - yr) * temp;
        if (w < W - 1)
          gwx = gwx - (yk - yr) * ((df_dy - gr) * (nom - a_x * denom) - (df_dy - gd) * (yk - yr) * (yk - yd) * denom * wy_1);
        if (h < H - 1)
          gwy = gwy - (yk - yd) * ((df_dy - gd) * (nom - a_y * denom) - (df_dy - gr) * (yk - yd) * (yk - yr) * denom * wx_1);
      } else {
        t -= (df_dy - gd) * wy_1;
        t -= (df_dy - gr) * wx_1;
        if (w < W - 1) gwx = gwx - (yk - yr) * (df_dy - gr);
        if (h < H - 1) gwy = gwy - (yk - yd) * (df_dy - gd);
      }
    }
    gi[q + p] = t + gx0[q + p];
  }
  tot_gx[i] += (double)gwx;
  tot_gy[i] += (double)gwy;
}

// -------------------------------------------------------------------------------------------------
// per-id state (idStruct, TVInpaintFista.h:7-50)
// -------------------------------------------------------------------------------------------------
struct Slot {
  int run = 0;
  int n = 0, ic = 0, ih = 0, iw = 0, its = -1;
  bool forward_done = false;
  // Which x05 rows the forward pass keeps for the backward pass (tvinpaint_keep_iterates): 0 none (every segment is
  // recomputed from its checkpoint, the reference's order of work), 1 those of the last segment, 2 all of them (no
  // recompute at all; the ring then has one row per iteration).
  int keep_mode = 2;
  // Which half of a checkpoint behind the first the last forward stored: -1 both; 0 only y (what the reference's backward
  // reads at a segment start); 1 only x (what the corrected gradient reads).  A forward that keeps every x05 row stores
  // the half its id's gradient mode needs, since no segment is ever recomputed from the checkpoint.
  int ckpt_half = -1;
  int fwd_grad_mode = 0;  // the mode the last forward pass ran under: its backward passes must ask for the same one
  int grad_mode = 0;    // 0: the reference's backward, bit for bit; 1: the corrected gradient (tvinpaint_gradient_mode)
  int ring_rows = 0;    // rows of the x05 ring the arena was laid out for
  // shape and its whose every-row ring (keep mode 2) the device refused: later forwards of that shape go straight
  // to keep mode 1 instead of freeing the arena and asking again on every call; cleared by reset_id
  long long refused[5] = {0, 0, 0, 0, 0};
  int x05_mode = 0;     // how the last forward laid its rows out: 2 row = iteration, else row = iteration - first kept
  int x05_from = 0;     // first iteration whose x05 row the last forward kept
  bool x05_valid = false;
  std::vector<int> iterations;
  std::vector<float> steps;
  int max_inter_its = 0;
  hipStream_t stream = nullptr;
  Arena arena;
  // buffers (field = n*ic*ih*iw floats, plane = n*ih*iw)
  float *ypp[2] = {nullptr, nullptr}, *xpp[2] = {nullptr, nullptr}, *ckpt_y = nullptr, *ckpt_x = nullptr, *x05 = nullptr;
  float *g05[2] = {nullptr, nullptr}, *gxk[2] = {nullptr, nullptr}, *gx_final = nullptr;
  // per-segment fp32 accumulators, double-buffered: every adjoint step reads one set and writes the other
  float *acc_gc[2] = {nullptr, nullptr}, *acc_gx[2] = {nullptr, nullptr}, *acc_gy[2] = {nullptr, nullptr},
        *acc_gb[2] = {nullptr, nullptr};
  int acc_cur = 0;   // set of the shared accumulators (gc, gx, gy) the next adjoint launch reads
  bool acc_fresh = false;  // the next pair launch starts a segment: its accumulators are zero, read from `zeros` (the pair that ended the segment before wrote none)
  int accb_cur = 0;  // set of the per-channel accumulator (gb) the next adjoint step reads
  double *tot_gc = nullptr, *tot_gx = nullptr, *tot_gy = nullptr, *tot_gb = nullptr;
  // strip path: one fp32 record per segment and tensor, added into the totals after the last segment
  float *seg_gc = nullptr, *seg_gx = nullptr, *seg_gy = nullptr, *seg_gb = nullptr;
  float* zeros = nullptr;  // one field of zeros, never written after the slot is made: the accumulators a segment's first pair starts from
  int seg_cur = 0;  // segment the backward pass is in
  GuardState* guard = nullptr;      // device
  double pending_av[5] = {0, 0, 0, 0, 0};  // running means to upload when the arena is (re)made
  bool have_guard_state = false;
};

Slot g_slots[kUniqueIds];
Allocator g_allocator;  // tvinpaint_set_allocator

KernelTimer g_timer;

size_t field_count(const Slot& s) { return (size_t)s.n * s.ic * s.ih * s.iw; }
size_t plane_count(const Slot& s) { return (size_t)s.n * s.ih * s.iw; }

int fetch_running_means(Slot& s) {
  if (s.guard) {
    GuardState host;
    INPAINT_HIP(hipStreamSynchronize(s.stream));
    INPAINT_HIP(hipMemcpy(&host, s.guard, kGuardHeaderBytes, hipMemcpyDeviceToHost));
    for (int k = 0; k < 5; k++) s.pending_av[k] = host.av[k];
  }
  return 0;
}

int prepare_slot(Slot& s, int n, int ic, int ih, int iw, int its, int keep_mode, hipStream_t stream) {
  int dev = -1;
  INPAINT_HIP(hipGetDevice(&dev));
  std::vector<int> iterations;
  int max_inter_its = 0;
  make_schedule(its, iterations, max_inter_its);
  const int ring_rows = keep_mode == 2 ? std::max(its, 1) : std::max(max_inter_its, 1);
  const bool same = s.arena.base && s.arena.device == dev && s.n == n && s.ic == ic && s.ih == ih &&
                    s.iw == iw && s.its == its && s.ring_rows >= ring_rows;  // the ring only grows
  s.stream = stream;
  if (same) return 0;
  int rc = fetch_running_means(s);  // the running means survive a change of shape
  if (rc) return rc;
  s.guard = nullptr;  // the arena is about to be released; the means live in pending_av until the new one exists
  s.n = n; s.ic = ic; s.ih = ih; s.iw = iw; s.its = its;
  make_schedule(its, s.iterations, s.max_inter_its);
  make_step_sizes(its, s.steps);
  const size_t F = field_count(s), P = plane_count(s);
  s.ring_rows = ring_rows;
  const size_t nck = std::max<size_t>(s.iterations.size(), 1), ring = (size_t)ring_rows;
  size_t need = 0;
  need += Arena::padded(F, 4) * (2 + 2 + 2 * nck + ring + 2 + 2 + 1 + 2 + 1);
  need += Arena::padded(P, 4) * 6;
  need += Arena::padded(P, 8) * 3 + Arena::padded(F, 8);
  need += Arena::padded(P * nck, 4) * 3 + Arena::padded(F * nck, 4);
  need += Arena::padded(1, sizeof(GuardState));
  rc = s.arena.reserve(need, g_allocator, stream);
  if (rc) return rc;
  Arena& a = s.arena;
  s.ypp[0] = a.take<float>(F); s.ypp[1] = a.take<float>(F);
  s.xpp[0] = a.take<float>(F); s.xpp[1] = a.take<float>(F);
  s.ckpt_y = a.take<float>(F * nck); s.ckpt_x = a.take<float>(F * nck);
  s.x05 = a.take<float>(F * ring);
  s.g05[0] = a.take<float>(F); s.g05[1] = a.take<float>(F);
  s.gxk[0] = a.take<float>(F); s.gxk[1] = a.take<float>(F); s.gx_final = a.take<float>(F);
  for (int i = 0; i < 2; i++) {
    s.acc_gb[i] = a.take<float>(F);
    s.acc_gc[i] = a.take<float>(P); s.acc_gx[i] = a.take<float>(P); s.acc_gy[i] = a.take<float>(P);
  }
  s.tot_gc = a.take<double>(P); s.tot_gx = a.take<double>(P); s.tot_gy = a.take<double>(P);
  s.tot_gb = a.take<double>(F);
  s.seg_gc = a.take<float>(P * nck); s.seg_gx = a.take<float>(P * nck); s.seg_gy = a.take<float>(P * nck);
  s.seg_gb = a.take<float>(F * nck);
  s.zeros = a.take<float>(F);
  s.guard = a.take<GuardState>(1);
  if (!s.guard) return fail(INPAINT_ERR_HIP, "arena layout overflow");
  hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)F)), dim3(256), 0, stream, s.zeros, (long long)F);
  GuardState init;
  memset(&init, 0, sizeof(init));
  for (int k = 0; k < 5; k++) { init.av[k] = s.pending_av[k]; init.scale[k] = 1.0; }
  INPAINT_HIP(hipMemcpyAsync(s.guard, &init, sizeof(init), hipMemcpyHostToDevice, stream));
  INPAINT_HIP(hipStreamSynchronize(stream));  // `init` is a stack object
  return 0;
}

int check_common(const void* const* ptrs, int nptrs, int n, int ic, int ih, int iw, int its, int id) {
  if (id < 0 || id >= kUniqueIds)
    return fail(INPAINT_ERR_ID, "Cannot use an id that is negative or larger/equal than the maximal one: %d/%d", id,
                kUniqueIds);
  for (int i = 0; i < nptrs; i++)
    if (!ptrs[i]) return fail(INPAINT_ERR_ARG, "null pointer argument (position %d)", i);
  if (n < 1 || ic < 1 || ih < 1 || iw < 1 || its < 0)
    return fail(INPAINT_ERR_ARG, "bad sizes n=%d ic=%d ih=%d iw=%d its=%d", n, ic, ih, iw, its);
  if (n > 65535) return fail(INPAINT_ERR_ARG, "n=%d exceeds the launch grid", n);
  // the strip kernels address up to four planes of a tensor with one 32-bit byte offset from a common base pointer
  if ((long long)ih * iw * std::min(std::max(ic, 2), 4) >= (1ll << 30))
    return fail(INPAINT_ERR_ARG, "ih*iw = %lld pixels per plane exceed 2^29 (2^28 with more than 3 channels)", (long long)ih * iw);
  if ((int)std::floor(std::sqrt((double)its)) > kMaxCheckpoints)
    return fail(INPAINT_ERR_ITS, "its=%d needs more than %d checkpoints", its, kMaxCheckpoints);
  return 0;
}

// -------------------------------------------------------------------------------------------------
// kernel selection: the wave-strip kernels (more than 4 channels: in channel groups).  INPAINT_TV_PATH=tile used to
// select the LDS-tile kernels written first; they are no longer built, and the setting is refused.
// -------------------------------------------------------------------------------------------------
int refuse_removed_path() {
  if (knobs().tv_tile_path)
    return fail(INPAINT_ERR_ARG, "INPAINT_TV_PATH=tile names the LDS-tile kernels, which this library no longer contains; unset it (INPAINT_TV_FUSE=0 selects the one-iteration strip kernels)");
  return 0;
}
// The x05 rows the forward pass keeps.  INPAINT_KEEP=0|1|2 overrides the id's setting (INPAINT_KEEP_LAST=0 is the
// older spelling of INPAINT_KEEP=0); keeping all rows needs its * field bytes, at most INPAINT_KEEP_GB (default 32).
int resolve_keep_mode(const Slot& s, int n, int ic, int ih, int iw, int its) {
  int mode = knobs().keep >= 0 ? knobs().keep : s.keep_mode;
  if (mode == 2) {
    const double bytes = 4.0 * n * ic * (double)ih * iw * its;
    if (bytes > knobs().keep_gb * 1073741824.0) mode = 1;
  }
  return mode;
}
int strip_rows(int n, int ih, int iw, int cols, int forced_rows, int lag) {
  // Rows per wavefront: taller strips amortise the start-up latency and the one-row overlap
  // between strips, but the launch should still put about two wavefronts on each of the 1024 SIMDs
  // (measured on the 4 x 2 x 384 x 1248 workload: 16 rows beat 8 and 24).
  if (forced_rows > 0) return forced_rows;
  const long long sx = (iw + cols - 1) / cols;
  return choose_strip_rows(sx * n, ih, 4, lag);
}

// Channel groups: the strip kernels are instantiated for 1..4 channels (the adjoint pair for 1..2).  More channels
// run as consecutive launches over groups of up to kGroup channels, each launch getting the per-channel tensors
// already moved to its first channel and the tensor's channel count as the plane stride.  Forward channels never
// couple.  The adjoint couples them through gc, gwx, gwy only, and those are summed in channel order step by step:
// one-step launches issued group after group reproduce that order exactly.
constexpr int kGroup = 4;
inline const float* at_channel(const Slot& s, const float* p, int ch0) { return p ? p + (size_t)ch0 * s.ih * s.iw : nullptr; }
inline float* at_channel(const Slot& s, float* p, int ch0) { return p ? p + (size_t)ch0 * s.ih * s.iw : nullptr; }

template <int C>
void launch_forward_strip(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                          const float* b, const float* xin, float* xout, const float* yin, float* yout, float* x05,
                          float t) {
  auto kern = x05 ? tvstrip::tv_forward_strip<C, true> : tvstrip::tv_forward_strip<C, false>;
  const int R = strip_rows(s.n, s.ih, s.iw, tvstrip::kFwdCols, knobs().tv_fwd_rows, 6);
  const int sx = (s.iw + tvstrip::kFwdCols - 1) / tvstrip::kFwdCols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);  // a multiple of 8: one share per XCD
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xin, xout, yin, yout, x05, s.n, s.ih, s.iw, t, R, sx, sy, s.ic);
}

// Two forward iterations in one launch (strip path only): (xin, yin) = iterate k, (xout, yout) = iterate k+2;
// x05a / x05b receive the pre-prox values of iterations k and k+1 when given.
// groups: the launch covers that many consecutive channel groups of C channels (one wavefront per strip and group)
template <int C>
void launch_forward_pair_strip(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                               const float* b, const float* xin, float* xout, const float* yin, float* yout,
                               float* x05a, float* x05b, float tA, float tB, bool ring, float tP, int groups = 1,
                               float* keep_x = nullptr, float* keep_y = nullptr) {
  auto kern = tvstrip::tv_forward_strip2<C, false>;
  if (x05a && ring) kern = (xout || yout) ? tvstrip::tv_forward_strip2<C, true, true> : tvstrip::tv_forward_strip2<C, true, true, false>;
  else if (x05a) kern = tvstrip::tv_forward_strip2<C, true>;
  const int R = strip_rows(s.n * groups, s.ih, s.iw, tvstrip::kFwd2Cols, knobs().tv_fwd_rows, 8);
  const int sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n * groups;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xin, xout, yin, yout, x05a, x05b, s.n, s.ih, s.iw, tA, tB,
                     (x05a && ring) ? tP : 0.f, R, sx, sy, s.ic, groups, keep_x, keep_y);
}

// A launch that cannot give every SIMD of the chip a wavefront lasts as long as one wavefront needs for its strip, and
// that time is proportional to the channels the wavefront carries: such launches run one channel per wavefront.
bool forward_split_channels(const Slot& s) {
  if (s.ic < 2 || s.ic > kGroup) return false;
  if (knobs().tv_fwd_split >= 0) return knobs().tv_fwd_split == 1;
  const long long sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols;
  // (measured, two channels, 50 iterations: 2 x 112 x 256 0.187 -> 0.162 ms per forward pass, 2 x 224 x 512 0.221 -> 0.197 ms,
  // 2 x 448 x 1024 no difference)
  return sx * ((s.ih + 1) / 2) * s.n <= 8ll * compute_unit_count();  // strips of two rows: at most two wavefronts per SIMD
}

bool forward_pairs(const Slot& s) {
  return knobs().tv_fuse;
}

// ring: xin / yin are the x05 rows of the two iterations before this pair and the iterate is rebuilt from them
// (tP: extrapolation factor of the iteration that made it); such a launch writes x05 rows only
void launch_forward_pair(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                         const float* b, const float* xin, float* xout, const float* yin, float* yout, float* x05a,
                         float* x05b, float tA, float tB, bool ring = false, float tP = 0.f, float* keep_x = nullptr,
                         float* keep_y = nullptr) {
  // keep_x / keep_y: where the launch leaves a copy of its input iterate (checkpoint 0 = the starting point)
  if (forward_split_channels(s)) {
    launch_forward_pair_strip<1>(s, stream, dx, dy, c, b, xin, xout, yin, yout, x05a, x05b, tA, tB, ring, tP, s.ic, keep_x, keep_y);
    return;
  }
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    const float *gb = at_channel(s, b, ch0), *gxi = at_channel(s, xin, ch0), *gyi = at_channel(s, yin, ch0);
    float *gxo = at_channel(s, xout, ch0), *gyo = at_channel(s, yout, ch0), *ga = at_channel(s, x05a, ch0), *gbb = at_channel(s, x05b, ch0);
    float *kx = at_channel(s, keep_x, ch0), *ky = at_channel(s, keep_y, ch0);
    switch (std::min(kGroup, s.ic - ch0)) {
      case 1: launch_forward_pair_strip<1>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, ga, gbb, tA, tB, ring, tP, 1, kx, ky); break;
      case 2: launch_forward_pair_strip<2>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, ga, gbb, tA, tB, ring, tP, 1, kx, ky); break;
      case 3: launch_forward_pair_strip<3>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, ga, gbb, tA, tB, ring, tP, 1, kx, ky); break;
      default: launch_forward_pair_strip<4>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, ga, gbb, tA, tB, ring, tP, 1, kx, ky); break;
    }
  }
}

void launch_forward(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                    const float* b, const float* xin, float* xout, const float* yin, float* yout, float* x05,
                    float t) {
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    const float *gb = at_channel(s, b, ch0), *gxi = at_channel(s, xin, ch0), *gyi = at_channel(s, yin, ch0);
    float *gxo = at_channel(s, xout, ch0), *gyo = at_channel(s, yout, ch0), *gh = at_channel(s, x05, ch0);
    switch (std::min(kGroup, s.ic - ch0)) {
      case 1: launch_forward_strip<1>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, gh, t); break;
      case 2: launch_forward_strip<2>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, gh, t); break;
      case 3: launch_forward_strip<3>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, gh, t); break;
      default: launch_forward_strip<4>(s, stream, dx, dy, c, gb, gxi, gxo, gyi, gyo, gh, t); break;
    }
  }
}

// One group of a one-step adjoint launch.  Shared accumulators (gc, gwx, gwy): set acc_cur in, the other out, flipped
// by the caller after every launch; per-channel accumulators (gb): set accb_cur in, the other out, flipped once per
// step.  last_group: this launch completes the step (a segment-start step then flushes the shared accumulators).
template <int C, bool END, bool TRUE_ADJ, bool FIRST = false>
void launch_adjoint_strip(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                          const float* b, const float* xa, const float* xb, const float* yck, const float* g05_in,
                          float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float t, int ch0, bool last_group,
                          const float* x05_last = nullptr) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  auto kern = (gx_final && !FIRST) ? tvstrip::tv_adjoint_strip<C, END, !FIRST, TRUE_ADJ, FIRST>
                                   : tvstrip::tv_adjoint_strip<C, END, false, TRUE_ADJ, FIRST>;
  const int R = strip_rows(s.n, s.ih, s.iw, tvstrip::kAdjCols, knobs().tv_adj_rows, 6);
  const int sx = (s.iw + tvstrip::kAdjCols - 1) / tvstrip::kAdjCols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);  // a multiple of 8: one share per XCD
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, at_channel(s, b, ch0), at_channel(s, xa, ch0), at_channel(s, xb, ch0),
                     at_channel(s, yck, ch0), s.acc_gc[i], s.acc_gc[o], at_channel(s, (const float*)s.acc_gb[ib], ch0),
                     at_channel(s, s.acc_gb[ob], ch0), s.acc_gx[i], s.acc_gx[o], s.acc_gy[i], s.acc_gy[o],
                     at_channel(s, g05_in, ch0), at_channel(s, g05_out, ch0), at_channel(s, gxk, ch0), at_channel(s, gxk_m1, ch0),
                     at_channel(s, gx_final, ch0), s.seg_gc + sP, at_channel(s, s.seg_gb + sF, ch0), s.seg_gx + sP, s.seg_gy + sP,
                     s.n, s.ih, s.iw, t, R, sx, sy, s.ic, last_group ? 1 : 0, at_channel(s, x05_last, ch0));
}

// The first two steps of the reverse sweep in one launch (strip path, at most kGroup channels, the second step not
// a segment's first iteration): step j = len - 2 as launch_adjoint runs it, with the sweep's first step (the upstream
// gradient `gin` through the prox at the last x05 row) done on the way in.  The accumulators start at zero in set
// acc_cur; the launch writes the other set, then the sets flip as after any step.
template <bool TRUE_ADJ>
void launch_adjoint_first_two(Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c, const float* b,
                              const float* x05_last, const float* xa, const float* xb, const float* gin, float* g05_out,
                              const float* gxk, float* gxk_m1, float t) {
  switch (s.ic) {
    case 1: launch_adjoint_strip<1, false, TRUE_ADJ, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, true, x05_last); break;
    case 2: launch_adjoint_strip<2, false, TRUE_ADJ, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, true, x05_last); break;
    case 3: launch_adjoint_strip<3, false, TRUE_ADJ, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, true, x05_last); break;
    default: launch_adjoint_strip<4, false, TRUE_ADJ, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, true, x05_last); break;
  }
  s.acc_cur = 1 - s.acc_cur;
  s.accb_cur = 1 - s.accb_cur;
}

// One adjoint step: reads accumulator set acc_cur, writes the other one, then flips acc_cur.
// TRUE_ADJ (strip path only, the caller checks): the corrected gradient; with END, yck is the checkpointed x.
template <bool END, bool TRUE_ADJ = false>
bool launch_adjoint(Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                  const float* b, const float* xa, const float* xb, const float* yck, const float* g05_in,
                  float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float t) {
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    const bool last = ch0 + kGroup >= s.ic;
    switch (std::min(kGroup, s.ic - ch0)) {
      case 1: launch_adjoint_strip<1, END, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0, last); break;
      case 2: launch_adjoint_strip<2, END, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0, last); break;
      case 3: launch_adjoint_strip<3, END, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0, last); break;
      default: launch_adjoint_strip<4, END, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0, last); break;
    }
    s.acc_cur = 1 - s.acc_cur;
  }
  s.accb_cur = 1 - s.accb_cur;
  return true;
}

// Two adjoint steps in one launch (strip path): A = local iteration j (x05 slots xa = j, xb = j-1), B = j-1
// (third y source xc = slot j-2, or the checkpoint y when B is the segment's first iteration).
template <int C, bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_strip(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                               const float* b, const float* xa, const float* xb, const float* xc, const float* g05_in,
                               float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  auto kern = gx_final ? tvstrip::tv_adjoint_strip2<C, BEND, true, TRUE_ADJ> : tvstrip::tv_adjoint_strip2<C, BEND, false, TRUE_ADJ>;
  const int R = strip_rows(s.n, s.ih, s.iw, tvstrip::kFwd2Cols, knobs().tv_adj_rows, 8);
  const int sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib], s.acc_gb[ob],
                     zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final, s.seg_gc + sP,
                     s.seg_gb + sF, s.seg_gx + sP, s.seg_gy + sP, s.n, s.ih, s.iw, tA, tB, R, sx, sy, s.ic);
}

// Rows per strip of the two-wavefront pair kernel.  Its workgroups (one strip each) are resident four per CU, so a
// launch runs in ceil(workgroups / (4 * CUs)) rounds of (R + pipeline rows + start-up) row steps each; the strip
// height that minimises rounds x steps is taken.
int pair_split_rows(int n, int ih, int iw) {
  if (knobs().tv_adj_rows > 0) return knobs().tv_adj_rows;
  const long long cap = 4ll * compute_unit_count();
  const long long sx = (iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols;
  int best = 16;
  long long best_cost = -1;
  for (int R = 8; R <= 64; R++) {
    const long long wg = sx * ((ih + R - 1) / R) * n;
    const long long cost = ((wg + cap - 1) / cap) * (R + 7);
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = R;
    }
  }
  return best;
}

// 3 and 4 channels: the two steps of a pair in two wavefronts of a workgroup (one strip per 128-thread workgroup)
template <int C, bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_split(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                               const float* b, const float* xa, const float* xb, const float* xc, const float* g05_in,
                               float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  auto kern = gx_final ? tvstrip::tv_adjoint_strip2w<C, BEND, true, TRUE_ADJ> : tvstrip::tv_adjoint_strip2w<C, BEND, false, TRUE_ADJ>;
  const int R = pair_split_rows(s.n, s.ih, s.iw);
  const int sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols, sy = (s.ih + R - 1) / R;
  const long long strips = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)((strips + 7) / 8 * 8)), block(128);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib], s.acc_gb[ob],
                     zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final, s.seg_gc + sP,
                     s.seg_gb + sF, s.seg_gx + sP, s.seg_gy + sP, s.n, s.ih, s.iw, tA, tB, R, sx, sy, s.ic);
}

// 5 to 8 channels: two channel groups, step A and step B of each in a wavefront of its own (one strip per 256-thread
// workgroup, two workgroups resident per CU)
int pair_quad_rows(int n, int ih, int iw) {
  if (knobs().tv_adj_rows > 0) return knobs().tv_adj_rows;
  const long long cap = 2ll * compute_unit_count();
  const long long sx = (iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols;
  int best = 16;
  long long best_cost = -1;
  for (int R = 8; R <= 96; R++) {
    const long long wg = sx * ((ih + R - 1) / R) * n;
    const long long cost = ((wg + cap - 1) / cap) * (R + 12);  // 3 rows of start-up and two intervals of three rows behind
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = R;
    }
  }
  return best;
}

template <int CM, int C1, bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_quad(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                              const float* b, const float* xa, const float* xb, const float* xc, const float* g05_in,
                              float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  auto kern = gx_final ? tvstrip::tv_adjoint_strip4w<CM, C1, BEND, true, TRUE_ADJ> : tvstrip::tv_adjoint_strip4w<CM, C1, BEND, false, TRUE_ADJ>;
  const int R = pair_quad_rows(s.n, s.ih, s.iw);
  const int sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols, sy = (s.ih + R - 1) / R;
  const long long strips = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)((strips + 7) / 8 * 8)), block(256);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib], s.acc_gb[ob],
                     zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final, s.seg_gc + sP,
                     s.seg_gb + sF, s.seg_gx + sP, s.seg_gy + sP, s.n, s.ih, s.iw, tA, tB, R, sx, sy, s.ic);
}

// Two channels, one per wavefront (one strip per 128-thread workgroup), for launches that cannot fill the chip
bool adjoint_split_channels(const Slot& s) {
  if (s.ic != 2) return false;
  if (knobs().tv_adj_split >= 0) return knobs().tv_adj_split == 1;
  // Split while strips of 16 rows, one wavefront for both channels, would leave the chip short of wavefronts: the
  // unsplit kernel then has to take low strips, and walks 8 halo rows for each.  Measured, 50 iterations, backward pass
  // unsplit -> split (16-row strips per CU in brackets): 1 x 384 x 1248 0.571 -> 0.523 ms (2.0), 2 x 384 x 1248
  // 0.869 -> 0.855 (3.9), 2 x 448 x 1024 0.856 -> 0.850 (3.9), 4 x 300 x 900 0.959 -> 0.946 (4.5), 3 x 384 x 1248
  // 1.191 -> 1.196 (5.9), 4 x 384 x 1248 slower (7.9).
  const long long sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols;
  return sx * ((s.ih + 15) / 16) * s.n <= 5ll * compute_unit_count();
}

template <bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_channels(const Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c,
                                  const float* b, const float* xa, const float* xb, const float* xc, const float* g05_in,
                                  float* g05_out, const float* gxk, float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  auto kern = gx_final ? tvstrip::tv_adjoint_strip2c<BEND, true, TRUE_ADJ> : tvstrip::tv_adjoint_strip2c<BEND, false, TRUE_ADJ>;
  const int R = strip_rows(2 * s.n, s.ih, s.iw, tvstrip::kFwd2Cols, knobs().tv_adj_rows, 9);
  const int sx = (s.iw + tvstrip::kFwd2Cols - 1) / tvstrip::kFwd2Cols, sy = (s.ih + R - 1) / R;
  const long long strips = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)((strips + 7) / 8 * 8)), block(128);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, dx, dy, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib], s.acc_gb[ob],
                     zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final, s.seg_gc + sP,
                     s.seg_gb + sF, s.seg_gx + sP, s.seg_gy + sP, s.n, s.ih, s.iw, tA, tB, R, sx, sy, s.ic);
}

constexpr int kPairChannels = 8;  // the most channels a pair launch holds (two groups of four)

// (a pair adds step A's and step B's terms of its channels in the reference's order of summation only when the
// launch holds every channel)
template <bool BEND, bool TRUE_ADJ = false>
void launch_adjoint_pair(Slot& s, hipStream_t stream, const float* dx, const float* dy, const float* c, const float* b,
                         const float* xa, const float* xb, const float* xc, const float* g05_in, float* g05_out,
                         const float* gxk, float* gxk_m1, float* gx_final, float tA, float tB) {
  if (s.ic == 1)
    launch_adjoint_pair_strip<1, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 2 && adjoint_split_channels(s))
    launch_adjoint_pair_channels<BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 2)
    launch_adjoint_pair_strip<2, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 3)
    launch_adjoint_pair_split<3, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 4)
    launch_adjoint_pair_split<4, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 5)
    launch_adjoint_pair_quad<3, 2, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 6)
    launch_adjoint_pair_quad<3, 3, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 7)
    launch_adjoint_pair_quad<4, 3, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else
    launch_adjoint_pair_quad<4, 4, BEND, TRUE_ADJ>(s, stream, dx, dy, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  s.acc_cur = 1 - s.acc_cur;
  s.accb_cur = 1 - s.accb_cur;
}

bool adjoint_pairs(const Slot& s) {
  if (!knobs().tv_fuse_adj) return false;
  // the launch must hold every channel (pairs over launches of channel groups would sum the shared accumulators in
  // another order): one wavefront for 1 or 2 channels, two for 3 or 4, four (two channel groups) for 5 to 8; more
  // channels take the one-step kernel, group after group
  return forward_pairs(s) && s.ic <= kPairChannels;
}

// -------------------------------------------------------------------------------------------------
// Fixed scratch of tvinpaint_forward_noalloc: the y and x ping-pongs of a forward pass (4 fields) in a
// device array that is part of the code object, so that the call allocates nothing.  Every GPU the
// library is loaded on holds its own copy (64 MiB) at its own address until the process ends; the
// name `scratch` is only a host-side handle of it, the address comes from hipGetSymbolAddress, once
// per device.
// -------------------------------------------------------------------------------------------------
constexpr size_t kNoAllocMaxField = size_t(1) << 22;  // floats per field (n*ic*ih*iw), 16 MiB
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) float scratch[4 * kNoAllocMaxField];
float* g_scratch_ptr[kNoAllocMaxDevices] = {nullptr};

int scratch_of_current_device(float** out) {
  int dev = -1;
  INPAINT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kNoAllocMaxDevices) return fail(INPAINT_ERR_ARG, "device index %d is beyond %d", dev, kNoAllocMaxDevices);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    INPAINT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(INPAINT_ERR_HIP, "hipGetSymbolAddress returned no address for the scratch array");
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

extern "C" {

int tvinpaint_forward(const float* dx, const float* dy, const float* c, const float* b, const float* init,
                      float* out, int n, int ic, int ih, int iw, int its, int id, void* stream_) {
  const void* ptrs[] = {dx, dy, c, b, init, out};
  int rc = check_common(ptrs, 6, n, ic, ih, iw, its, id);
  if (rc) return rc;
  rc = refuse_removed_path();
  if (rc) return rc;
  hipStream_t stream = (hipStream_t)stream_;
  Slot& s = g_slots[id];
  s.forward_done = false;
  s.x05_valid = false;
  s.ckpt_half = -1;
  s.fwd_grad_mode = s.grad_mode;
  int keep = resolve_keep_mode(s, n, ic, ih, iw, its);
  const long long shape[5] = {n, ic, ih, iw, its};
  if (keep == 2 && std::equal(shape, shape + 5, s.refused)) keep = 1;
  if (keep == 2 && !(s.arena.base && s.n == n && s.ic == ic && s.ih == ih && s.iw == iw && s.its == its && s.ring_rows >= its) &&
      rows_exceed_free_memory(4.0 * n * ic * (double)ih * iw * its))
    keep = 1;  // (the slot would have to grow by more than a quarter of the free device memory)
  rc = prepare_slot(s, n, ic, ih, iw, its, keep, stream);
  if (rc && keep == 2) {  // no room for every x05 row: keep the last segment's instead and recompute the others
    (void)hipGetLastError();
    keep = 1;
    rc = prepare_slot(s, n, ic, ih, iw, its, keep, stream);
    if (!rc) std::copy(shape, shape + 5, s.refused);
  }
  if (rc) return rc;
  const size_t F = field_count(s), FB = F * sizeof(float);
  const int K = 2 * (its / 2);
  // iterate k reads (Y(k), X(k)) and writes (Y(k+1), X(k+1)); a checkpointed iterate lives in its
  // checkpoint buffer, so no copies are made (the reference copies to the host, TV.cu:1541-1546)
  auto ck_index = [&](int k) {
    for (size_t i = 0; i < s.iterations.size(); i++)
      if (s.iterations[i] == k) return (int)i;
    return -1;
  };
  auto Ybuf = [&](int k) { int i = ck_index(k); return (i >= 0 && k < K) ? s.ckpt_y + (size_t)i * F : s.ypp[k & 1]; };
  auto Xbuf = [&](int k) {
    if (k == K) return out;
    int i = ck_index(k);
    return i >= 0 ? s.ckpt_x + (size_t)i * F : s.xpp[k & 1];
  };
  if (K == 0) {
    INPAINT_HIP(hipMemcpyAsync(out, init, FB, hipMemcpyDeviceToDevice, stream));
    if (!s.iterations.empty()) {  // its == 1: the reference leaves calloc'ed (zero) checkpoints
      hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)F)), dim3(256), 0, stream, s.ckpt_y, (long long)F);
      hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)F)), dim3(256), 0, stream, s.ckpt_x, (long long)F);
    }
  } else {
    // checkpoint 0 = the starting point: the first pair launch reads `init` itself and leaves the two copies as it
    // goes; one-iteration launches get them from a copy kernel
    // a forward that keeps every x05 row never recomputes from a checkpoint: it stores only the half of a checkpoint
    // the backward pass of this id's gradient mode reads at a segment start (y: the reference's; x: the corrected one,
    // which also reads checkpoint 0's y when it back-propagates iteration 0)
    const bool want_x = s.grad_mode == 1, want_y = !want_x;
    s.ckpt_half = (keep == 2 && forward_pairs(s)) ? (want_x ? 1 : 0) : -1;
    const bool copy_in_pair = forward_pairs(s) && out != init;  // (a caller that iterates in place keeps the copy launch)
    if (!copy_in_pair)
      hipLaunchKernelGGL(copy_twice_f32, dim3(grid_stride((long long)F)), dim3(256), 0, stream, init, s.ckpt_y, s.ckpt_x,
                         (long long)F);
    // first iteration whose x05 row is kept, and the ring row of iteration k
    const int kl = s.iterations.empty() ? K : (keep == 2 ? 0 : (keep == 1 ? s.iterations.back() : K));
    auto ring_row = [&](int k) { return s.x05 + (size_t)(keep == 2 ? k : k - kl) * F; };
    if (forward_pairs(s)) {
      // two iterations per launch; K is even and so is every checkpoint index.  The intermediate
      // iterate k+1 stays in registers, so the ping-pong alternates per pair.
      auto Yp = [&](int k) { int i = ck_index(k); return (i >= 0 && k < K) ? s.ckpt_y + (size_t)i * F : s.ypp[(k >> 1) & 1]; };
      auto Xp = [&](int k) {
        if (k == K) return out;
        int i = ck_index(k);
        return i >= 0 ? s.ckpt_x + (size_t)i * F : s.xpp[(k >> 1) & 1];
      };
      // kept iterations also store their x05 rows: the backward pass would otherwise recompute exactly these values
      // from the checkpoints (TV.cu:1678-1687)
      for (int k = 0; k < K; k += 2) {
        float* h0 = k >= kl ? ring_row(k) : nullptr;
        if (keep == 2 && k >= 2) {
          // With every x05 row kept the iterate need not travel through memory either: the pair rebuilds it from the
          // two rows before it, as the recompute launches of the backward pass do, and stores it only where somebody
          // reads it -- at a checkpoint and at the end.
          // At the end that is x alone (the result); at a checkpoint the half the backward pass will read.
          const bool last = k + 2 == K, ck = !last && ck_index(k + 2) >= 0;
          launch_forward_pair(s, stream, dx, dy, c, b, ring_row(k - 2), (last || (ck && want_x)) ? Xp(k + 2) : nullptr,
                              ring_row(k - 1), (ck && want_y) ? Yp(k + 2) : nullptr, h0, h0 + F, s.steps[k], s.steps[k + 1], true,
                              s.steps[k - 1]);
        } else if (k == 0 && copy_in_pair) {
          // (with every x05 row kept the next pair rebuilds its input from those rows: the iterate is stored only where
          // somebody reads it)
          const bool last = 2 == K, ck = !last && ck_index(2) >= 0;
          const bool sx = keep != 2 || last || (ck && want_x), sy = keep != 2 || (ck && want_y);
          launch_forward_pair(s, stream, dx, dy, c, b, init, sx ? Xp(2) : nullptr, init, sy ? Yp(2) : nullptr, h0,
                              h0 ? h0 + F : nullptr, s.steps[0], s.steps[1], false, 0.f, (keep != 2 || want_x) ? s.ckpt_x : nullptr, s.ckpt_y);
        }
        else
          launch_forward_pair(s, stream, dx, dy, c, b, Xp(k), Xp(k + 2), Yp(k), Yp(k + 2), h0, h0 ? h0 + F : nullptr,
                              s.steps[k], s.steps[k + 1]);
      }
    } else {
      for (int k = 0; k < K; k++)
        launch_forward(s, stream, dx, dy, c, b, Xbuf(k), Xbuf(k + 1), Ybuf(k), Ybuf(k + 1),
                       k >= kl ? ring_row(k) : nullptr, s.steps[k]);
    }
    s.x05_valid = kl < K;
    s.x05_from = kl;
    s.x05_mode = keep;
  }
  INPAINT_HIP(hipGetLastError());
  s.forward_done = true;
  return 0;
}

// The forward pass of tvinpaint_forward for callers that cannot allocate (code under graph capture, serving loops):
// same kernels and launch order, no id, no checkpoints and no x05 rows (nothing is kept for a backward pass), the
// two iterate ping-pongs in the library's fixed scratch.  Calls no hipMalloc / hipFree.  Nothing in the scratch has
// to start at zero: every launch writes all pixels of the buffers the next one reads.  Calls that overlap on one
// GPU (two streams, two threads) share the scratch and race.
int tvinpaint_forward_noalloc(const float* dx, const float* dy, const float* c, const float* b, const float* init,
                              float* out, int n, int ic, int ih, int iw, int its, void* stream_) {
  const void* ptrs[] = {dx, dy, c, b, init, out};
  int rc = check_common(ptrs, 6, n, ic, ih, iw, its, 0);
  if (rc) return rc;
  const unsigned long long F64 = (unsigned long long)n * ic * (unsigned long long)ih * iw;
  if (F64 > kNoAllocMaxField)
    return fail(INPAINT_ERR_ARG, "tvinpaint_forward_noalloc: n*ic*ih*iw = %llu floats exceeds the fixed scratch (%zu per field)",
                F64, kNoAllocMaxField);
  float* base = nullptr;
  rc = scratch_of_current_device(&base);
  if (rc) return rc;
  hipStream_t stream = (hipStream_t)stream_;
  Slot s;  // shape only: the launch helpers read n, ic, ih, iw
  s.n = n; s.ic = ic; s.ih = ih; s.iw = iw; s.its = its;
  const size_t F = (size_t)F64;
  float* ypp[2] = {base, base + kNoAllocMaxField};
  float* xpp[2] = {base + 2 * kNoAllocMaxField, base + 3 * kNoAllocMaxField};
  const int K = 2 * (its / 2);
  if (K == 0) {
    if (out != init) INPAINT_HIP(hipMemcpyAsync(out, init, F * sizeof(float), hipMemcpyDeviceToDevice, stream));
    return 0;
  }
  // In place (out == init) a launch that both reads the starting point and stores the result would have strips read
  // halo pixels that their neighbours have already overwritten: that is the single pair launch of its = 2 or 3.  It
  // then reads a copy of the starting point in the scratch (one copy kernel more, as tvinpaint_forward does in place).
  const float *x0 = init, *y0 = init;
  if (out == init && K == 2 && forward_pairs(s)) {
    hipLaunchKernelGGL(copy_twice_f32, dim3(grid_stride((long long)F)), dim3(256), 0, stream, init, xpp[0], ypp[0], (long long)F);
    x0 = xpp[0];
    y0 = ypp[0];
  }
  // extrapolation factors as make_step_sizes produces them (TV.cu:1525-1532), one at a time
  double t = 1, t_prev = 1;
  auto next_step = [&]() {
    t_prev = t;
    t = (1. + std::sqrt(1. + 4. * t * t)) / 2.;
    return (float)std::max(0.0, (t_prev - 1.) / t);
  };
  if (forward_pairs(s)) {
    for (int k = 0; k < K; k += 2) {
      const float tA = next_step(), tB = next_step();
      const int i = (k >> 1) & 1;
      launch_forward_pair(s, stream, dx, dy, c, b, k == 0 ? x0 : xpp[i], k + 2 == K ? out : xpp[1 - i],
                          k == 0 ? y0 : ypp[i], ypp[1 - i], nullptr, nullptr, tA, tB);
    }
  } else {
    for (int k = 0; k < K; k++) {
      const int i = k & 1;
      launch_forward(s, stream, dx, dy, c, b, k == 0 ? init : xpp[i], k + 1 == K ? out : xpp[1 - i],
                     k == 0 ? init : ypp[i], ypp[1 - i], nullptr, next_step());
    }
  }
  INPAINT_HIP(hipGetLastError());
  return 0;
}

long long tvinpaint_forward_noalloc_max_floats(void) { return (long long)kNoAllocMaxField; }

int tvinpaint_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin, float* gx,
                       float* gy, float* gc, float* gb, float* gi, int n, int ic, int ih, int iw, int its, int id,
                       void* stream_) {
  const void* ptrs[] = {dx, dy, c, b, gin, gx, gy, gc, gb, gi};
  int rc = check_common(ptrs, 10, n, ic, ih, iw, its, id);
  if (rc) return rc;
  hipStream_t stream = (hipStream_t)stream_;
  Slot& s = g_slots[id];
  if (!s.forward_done || !s.arena.base || s.n != n || s.ic != ic || s.ih != ih || s.iw != iw || s.its != its)
    return fail(INPAINT_ERR_PAIRING, "backward(id=%d) does not match the last forward on this id", id);
  const bool corr = s.grad_mode == 1;
  // One rule in every keep mode (a forward that keeps every x05 row stores only the checkpoint halves its mode reads,
  // so there the other mode could not be served at all):
  if (s.grad_mode != s.fwd_grad_mode)
    return fail(INPAINT_ERR_PAIRING, "the gradient mode of id %d was changed after its forward pass: set it before the forward pass, or run the forward pass again", id);
  s.stream = stream;
  const size_t F = field_count(s), P = plane_count(s);
  const int gF = grid_stride((long long)F);

  s.acc_cur = 0;
  s.accb_cur = 0;
  // The strip kernels keep one fp32 record of the accumulators per segment; the records are added into the fp64
  // totals after the last segment, in the reference's order (TV.cu:1730 flushes after every segment: same bits,
  // but the totals are not read and rewritten ten times).
  SegmentJobs sj;
  {
    float* segs[4] = {s.seg_gc, s.seg_gx, s.seg_gy, s.seg_gb};
    double* tots_[4] = {s.tot_gc, s.tot_gx, s.tot_gy, s.tot_gb};
    for (int k = 0; k < 4; k++) {
      sj.acc[k] = nullptr;
      sj.seg[k] = segs[k];
      sj.total[k] = tots_[k];
      sj.n[k] = k < 3 ? (long long)P : (long long)F;
    }
  }
  // The sweep's first step rides on its second when the last segment has at least four iterations (that second step
  // is then an inner step) and one launch holds every channel.  That launch starts from zero accumulators without
  // reading them, and every launch after it reads only what its predecessor wrote in full: nothing to clear.
  const int nseg = (int)s.iterations.size();
  const bool first_two = adjoint_pairs(s) && s.ic <= kGroup && knobs().tv_fuse_first && nseg > 0 &&
                         2 * ((its - s.iterations[nseg - 1]) / 2) >= 4;
  {
    ZeroList z;
    int k = 0;
    if (!first_two) {
      for (float* p : {s.g05[0], s.g05[1], s.gxk[0], s.gxk[1], s.gx_final, s.acc_gb[0]}) { z.ptr[k] = p; z.bytes[k++] = (long long)F * 4; }
      for (float* p : {s.acc_gc[0], s.acc_gx[0], s.acc_gy[0]}) { z.ptr[k] = p; z.bytes[k++] = (long long)P * 4; }
    }
    // (the totals need no clearing: every one of them is written when the segment records are added up)
    // one launch: these buffers zeroed, the upstream gradient scrubbed (TV.cu:1609-1623), the guard's statistics cleared
    hipLaunchKernelGGL(backward_prologue_many, dim3(gF, k + 2), dim3(256), 0, stream, z, k, gin, (long long)F, s.guard);
  }

  // buffer roles of TV.cu:1638-1641: g05[0]/g05[1] and gxk[0]/gxk[1] ping-pong with the parity of
  // the local iteration index.  A step reads the partial g_x[k+1] from one gxk buffer and writes the
  // partial g_x[k] to the other; the completed g_x[k+1] itself is only ever read after the very last
  // step (TV.cu:800 calls its store a debugging aid), so only that step stores it, into gx_final.
  int lastIt = its;
  int pp_src = 1;  // g05 / g_x buffer the next adjoint launch reads (pair path)
  for (int outer = nseg - 1; outer >= 0; outer--) {
    const int k0 = s.iterations[outer];
    const int len = 2 * ((lastIt - k0) / 2);
    bool flushed = false;
    s.seg_cur = outer;
    const float* cky = s.ckpt_y + (size_t)outer * F;
    const float* ckx = s.ckpt_x + (size_t)outer * F;
    // recompute the segment, keeping x05 (TV.cu:1678-1687) -- unless it is the last segment and the forward pass
    // left its x05 rows in the ring
    const bool have_x05 = s.x05_valid && k0 >= s.x05_from;
    // rows of this segment: one per iteration of the whole run when all were kept, else the segment's own ring
    float* const ring = s.x05 + (s.x05_valid && s.x05_mode == 2 ? (size_t)k0 * F : 0);
    if (!have_x05 || s.x05_mode != 2) s.x05_valid = false;  // a recomputed (or a shared) ring is overwritten below
    if (have_x05) {
    } else if (forward_pairs(s)) {
      // Only the x05 rows are kept.  The first pair starts from the checkpoint; every later pair rebuilds its input
      // iterate from the two x05 rows before it (x_j = prox(x05[j-1]), y_j = x_j + s_{j-1} (x_j - prox(x05[j-2])),
      // the forward pass's own expressions), so no iterate travels through memory.
      for (int j = 0; j < len; j += 2) {  // segments have even length
        if (j == 0)
          launch_forward_pair(s, stream, dx, dy, c, b, ckx, nullptr, cky, nullptr, ring, ring + F, s.steps[k0],
                              s.steps[k0 + 1]);
        else
          launch_forward_pair(s, stream, dx, dy, c, b, ring + (size_t)(j - 2) * F, nullptr, ring + (size_t)(j - 1) * F,
                              nullptr, ring + (size_t)j * F, ring + (size_t)(j + 1) * F, s.steps[k0 + j],
                              s.steps[k0 + j + 1], true, s.steps[k0 + j - 1]);
      }
    } else {
      for (int j = 0; j < len; j++) {
        const float* yin = (j == 0) ? cky : s.ypp[j & 1];
        const float* xin = (j == 0) ? ckx : s.xpp[j & 1];
        launch_forward(s, stream, dx, dy, c, b, xin, s.xpp[(j + 1) & 1], yin, s.ypp[(j + 1) & 1],
                       ring + (size_t)j * F, s.steps[k0 + j]);
      }
    }
    // reverse sweep (TV.cu:1696-1729)
    int timed_run = 0;
    if (adjoint_pairs(s)) {
      // The g05 / g_x ping-pong flips once per launch: `src` holds what the next launch reads.  The
      // first step of the whole backward writes g05[1]; a segment's last launch leaves its result
      // where the next segment picks it up.
      int j = len - 1;
      if (outer == nseg - 1 && first_two) {
        // the sweep's first step rides on its second
        const float *x_last = ring + (size_t)j * F, *xa = ring + (size_t)(j - 1) * F, *xb = ring + (size_t)(j - 2) * F;
        if (corr) launch_adjoint_first_two<true>(s, stream, dx, dy, c, b, x_last, xa, xb, gin, s.g05[0], s.gxk[1], s.gxk[0], s.steps[k0 + j - 1]);
        else launch_adjoint_first_two<false>(s, stream, dx, dy, c, b, x_last, xa, xb, gin, s.g05[0], s.gxk[1], s.gxk[0], s.steps[k0 + j - 1]);
        pp_src = 0;
        j -= 2;
      } else if (outer == nseg - 1 && j >= 0) {  // (its < 2: no iterations, nothing to back-propagate)
        if (corr)
          hipLaunchKernelGGL(tv_adjoint_first<true>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b,
                             ring + (size_t)j * F, s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic,
                             (long long)ih * iw, (long long)P);
        else
          hipLaunchKernelGGL(tv_adjoint_first<false>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b,
                             ring + (size_t)j * F, s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic,
                             (long long)ih * iw, (long long)P);
        pp_src = 1;
        j--;
      }
      // corrected gradient: the same launches with the TRUE_ADJ kernels; a segment's first iteration takes the
      // checkpointed x (to rebuild the true y_{k0+1}) where the reference's takes the checkpoint y
      const float* ck = corr ? ckx : cky;
      if (j >= 0 && ((j + 1) & 1)) {  // an odd number of steps is left: one single step, then pairs
        const float* xa = ring + (size_t)j * F;
        float *g_in = s.g05[pp_src], *g_out = s.g05[1 - pp_src], *x_in = s.gxk[pp_src], *x_out = s.gxk[1 - pp_src];
        if (j > 0) {
          const float* xb = ring + (size_t)(j - 1) * F;
          if (corr) launch_adjoint<false, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j]);
          else launch_adjoint<false>(s, stream, dx, dy, c, b, xa, xb, nullptr, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j]);
        } else {
          float* gf = outer == 0 ? s.gx_final : nullptr;
          if (corr) flushed = launch_adjoint<true, true>(s, stream, dx, dy, c, b, xa, xa, ck, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j]);
          else flushed = launch_adjoint<true>(s, stream, dx, dy, c, b, xa, xa, ck, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j]);
        }
        pp_src = 1 - pp_src;
        j--;
      }
      for (; j >= 1; j -= 2) {
        const float* xa = ring + (size_t)j * F;
        const float* xb = ring + (size_t)(j - 1) * F;
        float *g_in = s.g05[pp_src], *g_out = s.g05[1 - pp_src], *x_in = s.gxk[pp_src], *x_out = s.gxk[1 - pp_src];
        // A pair that ends a segment stores the segment's sums as a record; it does not write the zeros the next segment
        // starts from: a segment's first pair reads zeros from the slot's field of zeros instead, which stays in the
        // cache (and the next backward pass clears the accumulators itself, or starts with a launch that does not read them).
        s.acc_fresh = outer < nseg - 1 && j == len - 1;
        if (j - 1 > 0) {
          const float* xc = ring + (size_t)(j - 2) * F;
          if (timed_run == 0) g_timer.begin(stream);
          if (corr) launch_adjoint_pair<false, true>(s, stream, dx, dy, c, b, xa, xb, xc, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j], s.steps[k0 + j - 1]);
          else launch_adjoint_pair<false>(s, stream, dx, dy, c, b, xa, xb, xc, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j], s.steps[k0 + j - 1]);
          timed_run++;
          if (j - 2 <= 1) g_timer.end(stream, timed_run);  // one event pair around the sweep's run of launches
        } else {
          // B is the segment's first iteration; the very last one's g_x is the gradient wrt the start
          float* gf = outer == 0 ? s.gx_final : nullptr;
          if (corr) launch_adjoint_pair<true, true>(s, stream, dx, dy, c, b, xa, xb, ck, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j], s.steps[k0 + j - 1]);
          else launch_adjoint_pair<true>(s, stream, dx, dy, c, b, xa, xb, ck, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j], s.steps[k0 + j - 1]);
          flushed = true;
        }
        pp_src = 1 - pp_src;
      }
      s.acc_fresh = false;
    } else
    for (int j = len - 1; j >= 0; j--) {
      const float t = s.steps[k0 + j];
      const float* xa = ring + (size_t)j * F;
      const int odd = j & 1;
      if (outer == nseg - 1 && j == len - 1) {
        if (corr)
          hipLaunchKernelGGL(tv_adjoint_first<true>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b, xa,
                             s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic, (long long)ih * iw, (long long)P);
        else
          hipLaunchKernelGGL(tv_adjoint_first<false>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b, xa,
                             s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic, (long long)ih * iw, (long long)P);
      } else if (j > 0) {
        const float* xb = ring + (size_t)(j - 1) * F;
        if (timed_run == 0) g_timer.begin(stream);
        if (corr)
          launch_adjoint<false, true>(s, stream, dx, dy, c, b, xa, xb, nullptr, s.g05[odd ? 0 : 1], s.g05[odd ? 1 : 0],
                                      s.gxk[odd ? 0 : 1], s.gxk[odd ? 1 : 0], nullptr, t);
        else
          launch_adjoint<false>(s, stream, dx, dy, c, b, xa, xb, nullptr, s.g05[odd ? 0 : 1], s.g05[odd ? 1 : 0],
                                s.gxk[odd ? 0 : 1], s.gxk[odd ? 1 : 0], nullptr, t);
        timed_run++;
        if (j == 1) g_timer.end(stream, timed_run);  // one event pair around the sweep's run of launches
      } else if (corr) {
        // corrected gradient: linearise at the true y_{k0+1}, rebuilt from x05[k0] and the checkpointed x_{k0}
        flushed = launch_adjoint<true, true>(s, stream, dx, dy, c, b, xa, xa, ckx, s.g05[1], s.g05[0], s.gxk[1],
                                             s.gxk[0], outer == 0 ? s.gx_final : nullptr, t);
      } else {
        // the very last step's g_x[k+1] is the gradient wrt the starting point (TV.cu:1785,1816)
        flushed = launch_adjoint<true>(s, stream, dx, dy, c, b, xa, xa, cky, s.g05[1], s.g05[0], s.gxk[1], s.gxk[0],
                                       outer == 0 ? s.gx_final : nullptr, t);
      }
    }
    // fp32 segment sums into the fp64 totals (TV.cu:1730); the strip kernel of the segment's first
    // iteration has already done it
    if (!flushed) {
      SegmentJobs st = sj;
      float* accs[4] = {s.acc_gc[s.acc_cur], s.acc_gx[s.acc_cur], s.acc_gy[s.acc_cur], s.acc_gb[s.accb_cur]};
      for (int k = 0; k < 4; k++) {
        st.acc[k] = accs[k];
        st.seg[k] = sj.seg[k] + (size_t)outer * sj.n[k];
      }
      hipLaunchKernelGGL(segment_store_many, dim3(gF, 4), dim3(256), 0, stream, st);
    }
    lastIt = k0;
  }

  hipLaunchKernelGGL(combine_segments_many, dim3(gF, 4), dim3(256), 0, stream, sj, nseg);
  if (corr && 2 * (its / 2) > 0) {
    // corrected gradient: back-propagate through iteration 0 as well (the reference stops before it); the last
    // step above left g05[0] and the partial g_x[0] in the halves of the ping-pongs it wrote, checkpoint 0 is y_0
    const int last = adjoint_pairs(s) ? pp_src : 0;
    hipLaunchKernelGGL(tv_adjoint_iter0, dim3(grid1d((long long)P)), dim3(256), 0, stream, dx, dy, s.ckpt_y, s.g05[last],
                       s.gxk[last], s.gx_final, s.tot_gx, s.tot_gy, ic, ih, iw, (long long)P);
  }
  // output guard on the device (TV.cu:1760-1791), then scale and store (TV.cu:1795-1818)
  const double* tots[4] = {s.tot_gc, s.tot_gx, s.tot_gy, s.tot_gb};
  const long long cnts[5] = {(long long)P, (long long)P, (long long)P, (long long)F, (long long)F};
  GuardJobs jobs;
  long long longest = 0;
  for (int k = 0; k < 5; k++) {
    jobs.ptr[k] = k < 4 ? (const void*)tots[k] : (const void*)s.gx_final;
    jobs.n[k] = cnts[k];
    jobs.is_f32[k] = k == 4;
    longest = std::max(longest, cnts[k]);
  }
  hipLaunchKernelGGL(guard_reduce_many, dim3(kGuardBlocks, 5), dim3(256), 0, stream, jobs, s.guard, kGuard.max_tolerance, false);
  hipLaunchKernelGGL(guard_tail_decide_many, dim3(guard_grid(longest), 5), dim3(256), 0, stream, jobs, s.guard, s.run, kGuard, false);
  FinalizeJobs fin;
  float* outs[4] = {gc, gx, gy, gb};
  for (int k = 0; k < 4; k++) {
    fin.total[k] = tots[k];
    fin.out[k] = outs[k];
    fin.n[k] = cnts[k];
    fin.chain_const[k] = (k == 1 || k == 2) ? (double)kL : 1.0;  // gx, gy carry the weight scaling (TV.cu:1797-1818)
    fin.chain_per_sample[k] = nullptr;
    fin.per_sample[k] = 1;
  }
  fin.f32_src = s.gx_final;  // the gradient wrt the starting point, guarded as a float tensor (TV.cu:1784-1791,1816)
  fin.f32_out = gi;
  fin.f32_n = (long long)F;
  fin.f32_scale = 4;
  hipLaunchKernelGGL(finalize_many, dim3(gF, 5), dim3(256), 0, stream, fin, s.guard, kGuard, corr ? 1.f : kGlobalGMult);
  INPAINT_HIP(hipGetLastError());
  if (knobs().stats_every > 0 && s.run % knobs().stats_every == 1 % knobs().stats_every) {  // TV.cu:1766: run % 75 == 1
    rc = print_guard_report(s.guard, stream, id, false);
    if (rc) return rc;
  }
  s.run++;  // TV.cu:1829
  return 0;
}

int tvinpaint_selftest_guard(const void* values, long long n, int is_f32, int run, double running_mean, float* out,
                            double* result7) {
  return guard_selftest(values, n, is_f32 != 0, run, running_mean, kGuard, false, out, result7);
}

int tvinpaint_get_state(int id, double* state6) {
  if (id < 0 || id >= kUniqueIds || !state6) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  int rc = fetch_running_means(s);
  if (rc) return rc;
  state6[0] = s.run;
  for (int k = 0; k < 5; k++) state6[1 + k] = s.pending_av[k];
  return 0;
}

int tvinpaint_set_state(int id, const double* state6) {
  if (id < 0 || id >= kUniqueIds || !state6) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  s.run = (int)state6[0];
  for (int k = 0; k < 5; k++) s.pending_av[k] = state6[1 + k];
  if (s.guard) {
    INPAINT_HIP(hipStreamSynchronize(s.stream));
    INPAINT_HIP(hipMemcpy(reinterpret_cast<char*>(s.guard) + offsetof(GuardState, av), s.pending_av, 5 * sizeof(double),
                         hipMemcpyHostToDevice));
  }
  return 0;
}

int tvinpaint_reset_id(int id) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  reload_knobs();
  Slot& s = g_slots[id];
  if (s.arena.base) (void)hipStreamSynchronize(s.stream);
  int rc = s.arena.release();
  s = Slot();
  return rc;
}

int tvinpaint_guard_stats(int id, double* stats25) {
  if (id < 0 || id >= kUniqueIds || !stats25) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  if (!s.guard) return fail(INPAINT_ERR_PAIRING, "id %d holds no state", id);
  GuardState host;
  INPAINT_HIP(hipStreamSynchronize(s.stream));
  INPAINT_HIP(hipMemcpy(&host, s.guard, kGuardHeaderBytes, hipMemcpyDeviceToHost));
  memcpy(stats25, host.report, sizeof(host.report));
  return 0;
}

int tvinpaint_gradient_mode(int id, int mode) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  if (mode < 0 || mode > 1) return fail(INPAINT_ERR_ARG, "gradient mode %d is not 0 or 1", mode);
  g_slots[id].grad_mode = mode;
  return 0;
}

int tvinpaint_keep_iterates(int id, int mode) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  if (mode < 0 || mode > 2) return fail(INPAINT_ERR_ARG, "keep mode %d is not 0, 1 or 2", mode);
  g_slots[id].keep_mode = mode;
  return 0;
}

int tvinpaint_set_allocator(inpaint_alloc_fn alloc, inpaint_release_fn release, void* user) {
  if ((alloc == nullptr) != (release == nullptr)) return fail(INPAINT_ERR_ARG, "tvinpaint_set_allocator: give both callbacks or neither");
  g_allocator.alloc = alloc;
  g_allocator.release = release;
  g_allocator.user = alloc ? user : nullptr;
  return 0;
}

long long tvinpaint_slot_bytes(int id) {
  if (id < 0 || id >= kUniqueIds) return 0;
  return (long long)g_slots[id].arena.bytes;
}

int tvinpaint_schedule(int its, int* iterations_out, int* max_inter_its) {
  std::vector<int> it;
  int m = 0;
  make_schedule(its, it, m);
  for (size_t i = 0; i < it.size(); i++) iterations_out[i] = it[i];
  if (max_inter_its) *max_inter_its = m;
  return (int)it.size();
}

void tvinpaint_step_sizes(int its, float* out) {
  std::vector<float> s;
  make_step_sizes(its, s);
  for (size_t i = 0; i < s.size(); i++) out[i] = s[i];
}

int tvinpaint_guard_decide(int run, double av_gc, double av_running, double* mult_out, double* av_out) {
  double mult = 1.0, av = av_running;
  int action = guard_decide_rule(run, av_gc, av, mult, kGuard);
  if (mult_out) *mult_out = mult;
  if (av_out) *av_out = av;
  return action;
}

void inpaint_reload_env(void) { reload_knobs(); }

int inpaint_keep_override(void) { return knobs().keep; }

int tvinpaint_profile(int enable) {
  g_timer.enabled = enable != 0;
  g_timer.reset();
  return 0;
}

int tvinpaint_profile_read(double* total_ms, int* launches) { return g_timer.read(total_ms, launches); }

const char* tvinpaint_last_error(void) { return error_buffer(); }

}  // extern "C"
