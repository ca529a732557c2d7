// Quadratic sub-pixel fit of a matching cost and median of a per-pixel displacement histogram for
// MI355X (gfx950): the two small layers upstream of the inpainting layer.  C ABI in
// include/flowaux.h; reference: cudaQuadFit/cudaCode/quadFit.cu (QF.cu below) and
// cudaMedian/cudaCode/medimax.cu (MM.cu).
//
// Arithmetic: every expression keeps the reference's operation order and types (its double
// literals promote the surrounding sub-expression), no contraction, IEEE division -- the per-pixel
// results are bit-equal to a plain C++ evaluation of the reference source.  The one exception is the
// gradient wrt the second feature map, a scatter with float atomics whose order is not defined
// (here or in the reference).
//
// Layout of the work:
//  * quadratic fit: one pixel per lane, lanes along the image row, a loop over the feature
//    channels.  Per channel a wavefront reads one 256-byte row segment of the first map and three
//    (shifted, overlapping) row segments of the second map around the displaced position; the
//    overlaps are served by the vector L1.  HBM sees every feature once: (2C+5) floats per pixel
//    forward, (5C+5) backward (the scatter reads and writes its target).
//  * median: the histogram bins are innermost in memory, so a lane that walked its own pixel's bins
//    would touch a new cache line per step.  Instead a wavefront stages 64 pixels x 32 bins through
//    LDS with full-line loads (32 lanes x 4 B = one 128-byte line of one pixel), and each lane then
//    walks its pixel's bins from LDS in the reference's sequential order (row pitch 33 words: no
//    bank conflicts).  The forward pass stops at the chunk in which the last pixel of the block
//    found its median.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdlib>

#include "../../include/flowaux.h"
#include "inpaint_common.h"

namespace {

using inpaint::fail;

// optional timing of the dominant kernel of each backward pass (the bench switches it on)
inpaint::KernelTimer g_timer;
int g_timed_pass = 1;  // quadratic fit, backward: 1 = the per-source pass, 2 = the gather pass

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Pixels that are close in
// the image read the same lines of the second feature map (the rows above and below, the shifted
// segments), so the blocks are renumbered such that every XCD works through one contiguous band of
// the pixel range.  The grid is a multiple of 8 blocks; blocks past the end return.
__device__ __forceinline__ long long banded_pixel_index() {
  const int per_xcd = gridDim.x >> 3;
  const int logical_block = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  return (long long)logical_block * 256 + threadIdx.x;
}
inline dim3 banded_grid(long long pixels) { return dim3((unsigned)(((pixels + 255) / 256 + 7) / 8 * 8)); }

// ---------------------------------------------------------------------------------------------
// quadratic fit
// ---------------------------------------------------------------------------------------------
struct Fit {
  bool inside;
  int validX, validY;
  unsigned o00, o0p, o0m, op0, om0;  // offsets of the five taps inside one channel plane
  int ix, iy;
  float c00, ax, ay, bx, by, fx, fy;
};

// QF.cu:75-104 == QF.cu:198-226: the two parabolas through the five costs, their validity and vertices
__device__ __forceinline__ void finish_fit(Fit& f, float cost00, float cost0p, float costp0, float cost0m, float costm0,
                                           int iidx, int iidy, int H, int W) {
  f.c00 = cost00;
  f.ax = 0.5 * (cost0p + cost0m - 2. * cost00);  // QF.cu:75-78
  f.ay = 0.5 * (costp0 + costm0 - 2. * cost00);
  f.bx = 0.5 * (cost0p - cost0m);
  f.by = 0.5 * (costp0 - costm0);
  f.validX = (f.ax < 0 && f.ax * f.ax >= 0.25 * f.bx * f.bx);  // QF.cu:83-89
  f.validY = (f.ay < 0 && f.ay * f.ay >= 0.25 * f.by * f.by);
  if (!(iidx < W - 1 && iidx > 0)) f.validX = 0;
  if (!(iidy < H - 1 && iidy > 0)) f.validY = 0;
  f.fx = f.fy = 0.f;
  if (f.validX) f.fx = -0.5 * f.bx / f.ax;  // QF.cu:92-104
  if (f.validY) f.fy = -0.5 * f.by / f.ay;
}

// QF.cu:22-104 (forward) == QF.cu:149-226 (backward): displaced position, the five matching
// costs, the two parabolas and their validity.
__device__ __forceinline__ Fit fit_pixel(const float* __restrict__ a, const float* __restrict__ q,
                                         const float* __restrict__ fl, int d, int H, int W, size_t HW, int h, int w) {
  Fit f;
  const unsigned p = (unsigned)h * W + w;
  const float idx = w + fl[p];       // QF.cu:31-32
  const float idy = h + fl[HW + p];
  f.inside = idx <= W - 1 && idx >= 0 && idy <= H - 1 && idy >= 0;  // QF.cu:35; a NaN displacement counts as outside
  f.validX = f.validY = 0;
  f.c00 = f.ax = f.ay = f.bx = f.by = f.fx = f.fy = 0.f;
  f.ix = f.iy = 0;
  f.o00 = f.o0p = f.o0m = f.op0 = f.om0 = 0;
  if (!f.inside) return f;
  const int iidx = (int)floor(idx + 0.5);  // QF.cu:47-48
  const int iidy = (int)floor(idy + 0.5);
  const int iidx_m = max(iidx - 1, 0), iidy_m = max(iidy - 1, 0);  // QF.cu:50-53
  const int iidx_p = min(iidx + 1, W - 1), iidy_p = min(iidy + 1, H - 1);
  f.ix = iidx; f.iy = iidy;
  f.o00 = (unsigned)iidy * W + iidx;
  f.o0p = (unsigned)iidy * W + iidx_p;
  f.o0m = (unsigned)iidy * W + iidx_m;
  f.op0 = (unsigned)iidy_p * W + iidx;
  f.om0 = (unsigned)iidy_m * W + iidx;
  float cost00 = 0.f, cost0p = 0.f, costp0 = 0.f, cost0m = 0.f, costm0 = 0.f;
#pragma unroll 4
  for (int cc = 0; cc < d; cc++) {  // QF.cu:63-71
    const float I1 = a[(size_t)cc * HW + p];
    const float* qc = q + (size_t)cc * HW;
    cost00 += I1 * qc[f.o00];
    cost0p += I1 * qc[f.o0p];
    costp0 += I1 * qc[f.op0];
    cost0m += I1 * qc[f.o0m];
    costm0 += I1 * qc[f.om0];
  }
  finish_fit(f, cost00, cost0p, costp0, cost0m, costm0, iidx, iidy, H, W);
  return f;
}

// QF.cu:14-139.  Every pixel writes its three outputs (zero outside the image), so no fill pass.
__global__ __launch_bounds__(256) void quadfit_forward_kernel(const float* __restrict__ im0, const float* __restrict__ im1,
                                                              const float* __restrict__ flow, float* __restrict__ out,
                                                              int N, int d, int H, int W, int fc) {
  const size_t HW = (size_t)H * W;
  const long long t = banded_pixel_index();
  if (t >= (long long)N * HW) return;
  const int n = (int)(t / HW);
  const unsigned p = (unsigned)(t - (long long)n * HW);
  const int h = p / W, w = p - h * W;
  const Fit f = fit_pixel(im0 + (size_t)n * d * HW, im1 + (size_t)n * d * HW, flow + (size_t)n * fc * HW, d, H, W, HW, h, w);
  float* o = out + (size_t)n * 3 * HW + p;
  float score = 0.f;
  if (f.inside)  // QF.cu:136 (fx, fy are zero wherever QF.cu:125-133 would not store them)
    score = f.ax * f.fx * f.fx + f.bx * f.fx + f.c00 + f.ay * f.fy * f.fy + f.by * f.fy;
  o[0] = f.fx;
  o[HW] = f.fy;
  o[2 * HW] = score;
}

// QF.cu:145-300.  g0 is written by its own pixel (zero outside the image); g1 is zero-filled
// before the launch and collects the scatter.
__global__ __launch_bounds__(256) void quadfit_backward_kernel(const float* __restrict__ im0, const float* __restrict__ im1,
                                                               const float* __restrict__ flow, const float* __restrict__ gin,
                                                               float* __restrict__ g0, float* __restrict__ g1, int N,
                                                               int d, int H, int W, int fc) {
  const size_t HW = (size_t)H * W;
  const long long t = banded_pixel_index();
  if (t >= (long long)N * HW) return;
  const int n = (int)(t / HW);
  const unsigned p = (unsigned)(t - (long long)n * HW);
  const int h = p / W, w = p - h * W;
  const float* a = im0 + (size_t)n * d * HW;
  const float* q = im1 + (size_t)n * d * HW;
  float* G0 = g0 + (size_t)n * d * HW;
  float* G1 = g1 + (size_t)n * d * HW;
  const Fit f = fit_pixel(a, q, flow + (size_t)n * fc * HW, d, H, W, HW, h, w);
  if (!f.inside) {
    for (int cc = 0; cc < d; cc++) G0[(size_t)cc * HW + p] = 0.f;
    return;
  }
  const int validX = f.validX, validY = f.validY;
  const float ax = f.ax, ay = f.ay, fx = f.fx, fy = f.fy;
  // QF.cu:244-253
  const float dfx_dbx = validX ? -1. / (2. * ax) : 0.;
  const float dfx_dax = validX ? -fx / ax : 0.;
  const float dfy_dby = validY ? -1. / (2. * ay) : 0.;
  const float dfy_day = validY ? -fy / ay : 0.;
  const float ds_dax = validX ? fx * fx : 0.;
  const float ds_dbx = validX ? fx : 0.;
  const float ds_dc = (validX || validY) ? 1. : 0.;
  const float ds_day = validY ? fy * fy : 0.;
  const float ds_dby = validY ? fy : 0.;
  const float dFdfx = gin[(size_t)n * 3 * HW + p];  // QF.cu:261-263
  const float dFdfy = gin[(size_t)n * 3 * HW + HW + p];
  const float dFds = gin[(size_t)n * 3 * HW + 2 * HW + p];
  // the channel-independent factors of QF.cu:279-290, each in the type the source gives it
  const double k00 = -2. * dFdfx * dfx_dax - 2. * dFdfy * dfy_day - 2. * dFds * ds_dax - 2. * dFds * ds_day + 2. * dFds * ds_dc;
  const float k0p = dFdfx * dfx_dax + dFdfx * dfx_dbx + dFds * ds_dax + dFds * ds_dbx;
  const float k0m = dFdfx * dfx_dax - dFdfx * dfx_dbx + dFds * ds_dax - dFds * ds_dbx;
  const float kp0 = dFdfy * dfy_day + dFdfy * dfy_dby + dFds * ds_day + dFds * ds_dby;
  const float km0 = dFdfy * dfy_day - dFdfy * dfy_dby + dFds * ds_day - dFds * ds_dby;
  if (validX || validY) {
#pragma unroll 2
    for (int cc = 0; cc < d; cc++) {
      const float* qc = q + (size_t)cc * HW;
      float* gc = G1 + (size_t)cc * HW;
      const float I1 = a[(size_t)cc * HW + p];
      const float I2 = qc[f.o00], I2_0p = qc[f.o0p], I2_0m = qc[f.o0m], I2_p0 = qc[f.op0], I2_m0 = qc[f.om0];
      unsafeAtomicAdd(gc + f.o00, (float)(0.5 * I1 * k00));
      unsafeAtomicAdd(gc + f.o0p, (float)(0.5 * I1 * k0p));
      unsafeAtomicAdd(gc + f.o0m, (float)(0.5 * I1 * k0m));
      unsafeAtomicAdd(gc + f.op0, (float)(0.5 * I1 * kp0));
      unsafeAtomicAdd(gc + f.om0, (float)(0.5 * I1 * km0));
      G0[(size_t)cc * HW + p] = 0.5 * (I2 * k00 + I2_0p * k0p + I2_0m * k0m + I2_p0 * kp0 + I2_m0 * km0);
    }
  } else {  // QF.cu:293-297: only the centre cost carries a gradient
#pragma unroll 4
    for (int cc = 0; cc < d; cc++) {
      const float I1 = a[(size_t)cc * HW + p];
      const float I2 = q[(size_t)cc * HW + f.o00];
      G0[(size_t)cc * HW + p] = I2 * dFds;
      unsafeAtomicAdd(G1 + (size_t)cc * HW + f.o00, I1 * dFds);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Quadratic fit, backward without float atomics.  Agent-scope float atomics are executed at the
// memory side on this GPU and run two orders of magnitude below HBM speed, so the scatter into the
// gradient of the second feature map is turned into a gather through a per-call inverse map:
//   pass A (per source pixel)  fit, gradient wrt the first map, the five scatter coefficients of the
//                              pixel (they do not depend on the channel) and one integer atomic that
//                              appends the pixel to the list of its displaced position (kSlots entries
//                              per position; what does not fit goes to an overflow list);
//   pass B (per target pixel)  gathers, per channel, I1 * coefficient from the sources listed at the
//                              target and at its four neighbours (a source centred on the left
//                              neighbour reaches the target with its right tap, and so on);
//   pass C (overflow list)     sources that found their list full scatter with float atomics after
//                              pass B -- rare: it takes more than kSlots pixels landing on one position.
// A tap that the image border clamps back onto the centre carries a zero coefficient (the axis is
// not fitted at the border), so the gather leaves it out.
// Workspace (caller provided): count[P] | overflow count, pad | slots[P*kSlots] | overflow list[P] | coef[5*P].
// ---------------------------------------------------------------------------------------------
constexpr int kSlots = 4;

struct QfWorkspace {
  int* count;      // sources per displaced position
  int* ovf_count;  // one counter
  int* slots;      // [P][kSlots] source pixel (index inside its sample)
  int* ovf;        // global index of the sources that did not fit
  float* coef;     // [5][P]: taps 00, 0p, 0m, p0, m0
};
long long qf_workspace_bytes(long long P) { return (long long)sizeof(int) * (P * (7 + kSlots) + 64 + 4); }
QfWorkspace qf_carve(void* base, long long P) {
  QfWorkspace w;
  int* p = reinterpret_cast<int*>(base);
  w.count = p;
  w.ovf_count = p + P;
  w.slots = p + (P + 64 + 3) / 4 * 4;  // 16-byte aligned: a position's kSlots entries are read as one int4
  w.ovf = w.slots + P * kSlots;
  w.coef = reinterpret_cast<float*>(w.ovf + P);
  return w;
}

// the channel-independent factors of QF.cu:244-263,279-297 as multipliers of I1 (scatter) and I2 (g0)
struct Factors {
  bool any_valid;
  double k00;
  float k0p, k0m, kp0, km0, dFds;
};
__device__ __forceinline__ Factors scatter_factors(const Fit& f, const float* __restrict__ gin, size_t n, size_t HW, unsigned p) {
  Factors k;
  const int validX = f.validX, validY = f.validY;
  const float ax = f.ax, ay = f.ay, fx = f.fx, fy = f.fy;
  const float dfx_dbx = validX ? -1. / (2. * ax) : 0.;  // QF.cu:244-253
  const float dfx_dax = validX ? -fx / ax : 0.;
  const float dfy_dby = validY ? -1. / (2. * ay) : 0.;
  const float dfy_day = validY ? -fy / ay : 0.;
  const float ds_dax = validX ? fx * fx : 0.;
  const float ds_dbx = validX ? fx : 0.;
  const float ds_dc = (validX || validY) ? 1. : 0.;
  const float ds_day = validY ? fy * fy : 0.;
  const float ds_dby = validY ? fy : 0.;
  const float dFdfx = gin[n * 3 * HW + p];  // QF.cu:261-263
  const float dFdfy = gin[n * 3 * HW + HW + p];
  const float dFds = gin[n * 3 * HW + 2 * HW + p];
  k.any_valid = validX || validY;
  k.dFds = dFds;
  k.k00 = -2. * dFdfx * dfx_dax - 2. * dFdfy * dfy_day - 2. * dFds * ds_dax - 2. * dFds * ds_day + 2. * dFds * ds_dc;
  k.k0p = dFdfx * dfx_dax + dFdfx * dfx_dbx + dFds * ds_dax + dFds * ds_dbx;
  k.k0m = dFdfx * dfx_dax - dFdfx * dfx_dbx + dFds * ds_dax - dFds * ds_dbx;
  k.kp0 = dFdfy * dfy_day + dFdfy * dfy_dby + dFds * ds_day + dFds * ds_dby;
  k.km0 = dFdfy * dfy_day - dFdfy * dfy_dby + dFds * ds_day - dFds * ds_dby;
  return k;
}

__global__ __launch_bounds__(256) void quadfit_backward_sources(const float* __restrict__ im0, const float* __restrict__ im1,
                                                                const float* __restrict__ flow, const float* __restrict__ gin,
                                                                float* __restrict__ g0, QfWorkspace ws, int N, int d, int H,
                                                                int W, int fc) {
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW;
  const long long t = banded_pixel_index();
  if (t >= P) return;
  const int n = (int)(t / HW);
  const unsigned p = (unsigned)(t - (long long)n * HW);
  const int h = p / W, w = p - h * W;
  const float* a = im0 + (size_t)n * d * HW;
  const float* q = im1 + (size_t)n * d * HW;
  float* G0 = g0 + (size_t)n * d * HW;
  const Fit f = fit_pixel(a, q, flow + (size_t)n * fc * HW, d, H, W, HW, h, w);
  if (!f.inside) {
    for (int cc = 0; cc < d; cc++) G0[(size_t)cc * HW + p] = 0.f;
    return;
  }
  const Factors k = scatter_factors(f, gin, n, HW, p);
  // scatter coefficients: contribution to g1 at a tap = I1 * coefficient (QF.cu:279-283,296)
  ws.coef[0 * P + t] = k.any_valid ? (float)(0.5 * k.k00) : k.dFds;
  ws.coef[1 * P + t] = k.any_valid ? 0.5f * k.k0p : 0.f;
  ws.coef[2 * P + t] = k.any_valid ? 0.5f * k.k0m : 0.f;
  ws.coef[3 * P + t] = k.any_valid ? 0.5f * k.kp0 : 0.f;
  ws.coef[4 * P + t] = k.any_valid ? 0.5f * k.km0 : 0.f;
  const long long centre = (long long)n * HW + f.o00;
  const int pos = atomicAdd(ws.count + centre, 1);
  if (pos < kSlots) ws.slots[centre * kSlots + pos] = (int)p;
  else ws.ovf[atomicAdd(ws.ovf_count, 1)] = (int)t;
  if (k.any_valid) {
#pragma unroll 4
    for (int cc = 0; cc < d; cc++) {  // QF.cu:286-290
      const float* qc = q + (size_t)cc * HW;
      const float I2 = qc[f.o00], I2_0p = qc[f.o0p], I2_0m = qc[f.o0m], I2_p0 = qc[f.op0], I2_m0 = qc[f.om0];
      G0[(size_t)cc * HW + p] = 0.5 * (I2 * k.k00 + I2_0p * k.k0p + I2_0m * k.k0m + I2_p0 * k.kp0 + I2_m0 * k.km0);
    }
  } else {
#pragma unroll 4
    for (int cc = 0; cc < d; cc++) G0[(size_t)cc * HW + p] = q[(size_t)cc * HW + f.o00] * k.dFds;  // QF.cu:295
  }
}

__global__ __launch_bounds__(256) void quadfit_backward_gather(const float* __restrict__ im0, float* __restrict__ g1,
                                                               QfWorkspace ws, int N, int d, int H, int W) {
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW;
  const long long t = banded_pixel_index();
  if (t >= P) return;
  const int n = (int)(t / HW);
  const unsigned p = (unsigned)(t - (long long)n * HW);
  const int h = p / W, w = p - h * W;
  const long long base = (long long)n * HW;
  const float* a = im0 + (size_t)n * d * HW;
  float* G1 = g1 + (size_t)n * d * HW + p;
  // (position whose sources reach this pixel, tap they reach it with); -1: outside the image
  long long ctr[5];
  ctr[0] = base + p;
  ctr[1] = w > 0 ? base + p - 1 : -1;      // right tap of the left neighbour
  ctr[2] = w < W - 1 ? base + p + 1 : -1;  // left tap of the right neighbour
  ctr[3] = h > 0 ? base + p - W : -1;      // lower tap of the upper neighbour
  ctr[4] = h < H - 1 ? base + p + W : -1;  // upper tap of the lower neighbour
  // compact list of the (source, coefficient) pairs that reach this pixel, in registers
  constexpr int kPairs = 8;
  unsigned src[kPairs];
  float cf[kPairs];
#pragma unroll
  for (int j = 0; j < kPairs; j++) {
    src[j] = p;
    cf[j] = 0.f;
  }
  int cnt[5];
  int np = 0;
#pragma unroll
  for (int k = 0; k < 5; k++) {
    cnt[k] = ctr[k] >= 0 ? min(ws.count[ctr[k]], kSlots) : 0;
#pragma unroll
    for (int i = 0; i < kSlots; i++) {
      if (i < cnt[k]) {
        const unsigned sidx = (unsigned)ws.slots[ctr[k] * kSlots + i];
        const float c = ws.coef[(long long)k * P + base + sidx];
#pragma unroll
        for (int j = 0; j < kPairs; j++)
          if (np == j) {
            src[j] = sidx;
            cf[j] = c;
          }
        np++;
      }
    }
  }
  // longest list among the wavefront's active lanes: the unrolled gathers beyond it are skipped by a uniform branch
  unsigned need = 0;
#pragma unroll
  for (int j = 0; j < kPairs; j++)
    if (__ballot(np > j) != 0) need |= 1u << j;
  if (np <= kPairs) {
    for (int cc = 0; cc < d; cc++) {
      const float* ac = a + (size_t)cc * HW;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < kPairs; j++)
        if (need & (1u << j)) acc += ac[src[j]] * cf[j];
      G1[(size_t)cc * HW] = acc;
    }
    return;
  }
  for (int cc = 0; cc < d; cc++) {  // more pairs than registers: walk the lists per channel
    const float* ac = a + (size_t)cc * HW;
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < 5; k++)
      for (int i = 0; i < cnt[k]; i++) {
        const unsigned sidx = (unsigned)ws.slots[ctr[k] * kSlots + i];
        acc += ac[sidx] * ws.coef[(long long)k * P + base + sidx];
      }
    G1[(size_t)cc * HW] = acc;
  }
}

// sources whose list was full: float atomics, after the gather has written g1
__global__ __launch_bounds__(256) void quadfit_backward_overflow(const float* __restrict__ im0, const float* __restrict__ flow,
                                                                 float* __restrict__ g1, QfWorkspace ws, int N, int d, int H,
                                                                 int W, int fc) {
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW;
  const long long total = (long long)*ws.ovf_count * d;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    const int e = (int)(i / d), cc = (int)(i - (long long)e * d);  // one lane per (source, channel)
    const long long t = ws.ovf[e];
    const int n = (int)(t / HW);
    const unsigned p = (unsigned)(t - (long long)n * HW);
    const int h = p / W, w = p - h * W;
    const float* fl = flow + (size_t)n * fc * HW;
    const float idx = w + fl[p], idy = h + fl[HW + p];  // QF.cu:31-32,47-53 (the pixel is inside the image)
    const int iidx = (int)floor(idx + 0.5), iidy = (int)floor(idy + 0.5);
    const unsigned o[5] = {(unsigned)iidy * W + iidx, (unsigned)iidy * W + min(iidx + 1, W - 1),
                           (unsigned)iidy * W + max(iidx - 1, 0), (unsigned)min(iidy + 1, H - 1) * W + iidx,
                           (unsigned)max(iidy - 1, 0) * W + iidx};
    const float I1 = im0[((size_t)n * d + cc) * HW + p];
    float* gc = g1 + ((size_t)n * d + cc) * HW;
#pragma unroll
    for (int k = 0; k < 5; k++) {
      const float cf = ws.coef[(long long)k * P + t];
      if (cf != 0.f) unsafeAtomicAdd(gc + o[k], I1 * cf);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Tiled kernels.  A lane that reads its five taps straight from memory issues gathers whose
// addresses follow the (jittery) flow; the vector L1 then handles them almost lane by lane and
// becomes the bound.  Here a block owns a 64 x 16 tile of pixels (4 rows per lane), finds the
// bounding box of all taps of the tile, and per channel stages that window of the second feature
// map in LDS with row-wise coalesced loads (double buffered: the next channel's window is in flight
// while the taps of the current one are read from LDS).  A pixel whose taps do not fit the window's
// capacity reads them from memory as before.
// ---------------------------------------------------------------------------------------------
constexpr int kTW = 64;  // tile width: one pixel column per lane
constexpr int kMaxWinW = 128;  // widest window
template <int PX>              // PX pixels per lane (rows PX * wave + i): tile height, window capacity in floats
struct TileCfg {
  static constexpr int TH = 4 * PX, ELEMS = (96 * (4 * PX + 16) + 255) / 256 * 256;
};
constexpr int kPxForward = 2, kPxSources = 2;

struct Box {
  int x0, y0, w, h;
};
struct TilePx {
  bool inside, far;
  int ix, iy, xm, xp, ym, yp;
  unsigned p;     // the pixel's offset inside a channel plane
  unsigned o[5];  // taps 00, 0p, 0m, p0, m0: offsets into the window, or into the plane when far
};

// QF.cu:31-53: displaced position and tap coordinates of pixel (x, y); widens the tile's bounding box
__device__ __forceinline__ void locate(TilePx& s, const float* __restrict__ fl, size_t HW, int H, int W, int x, int y,
                                       bool valid, int& minx, int& maxx, int& miny, int& maxy) {
  s.inside = s.far = false;
  s.ix = s.iy = s.xm = s.xp = s.ym = s.yp = 0;
  s.p = valid ? (unsigned)y * W + x : 0u;
  if (!valid) return;
  const float idx = x + fl[s.p];
  const float idy = y + fl[HW + s.p];
  if (!(idx <= W - 1 && idx >= 0 && idy <= H - 1 && idy >= 0)) return;  // QF.cu:35; NaN counts as outside
  s.inside = true;
  s.ix = (int)floor(idx + 0.5);
  s.iy = (int)floor(idy + 0.5);
  s.xm = max(s.ix - 1, 0); s.ym = max(s.iy - 1, 0);
  s.xp = min(s.ix + 1, W - 1); s.yp = min(s.iy + 1, H - 1);
  minx = min(minx, s.xm); maxx = max(maxx, s.xp);
  miny = min(miny, s.ym); maxy = max(maxy, s.yp);
}

__device__ __forceinline__ Box block_box(int minx, int maxx, int miny, int maxy, int* red, int capacity) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    minx = min(minx, __shfl_xor(minx, o));
    maxx = max(maxx, __shfl_xor(maxx, o));
    miny = min(miny, __shfl_xor(miny, o));
    maxy = max(maxy, __shfl_xor(maxy, o));
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    red[wave * 4 + 0] = minx; red[wave * 4 + 1] = maxx; red[wave * 4 + 2] = miny; red[wave * 4 + 3] = maxy;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; k++) {
    minx = min(minx, red[k * 4 + 0]); maxx = max(maxx, red[k * 4 + 1]);
    miny = min(miny, red[k * 4 + 2]); maxy = max(maxy, red[k * 4 + 3]);
  }
  Box b{0, 0, 0, 0};
  if (maxx >= minx) {
    b.x0 = minx; b.y0 = miny;
    b.w = min(maxx - minx + 1, kMaxWinW);
    b.h = min(maxy - miny + 1, capacity / b.w);
  }
  return b;
}

__device__ __forceinline__ void place(TilePx& s, const Box& b, int W) {
  if (!s.inside) return;
  s.far = !(s.xp - b.x0 < b.w && s.yp - b.y0 < b.h);
  if (s.far) {
    s.o[0] = (unsigned)s.iy * W + s.ix; s.o[1] = (unsigned)s.iy * W + s.xp; s.o[2] = (unsigned)s.iy * W + s.xm;
    s.o[3] = (unsigned)s.yp * W + s.ix; s.o[4] = (unsigned)s.ym * W + s.ix;
  } else {
    const int cx = s.ix - b.x0, cy = s.iy - b.y0;
    s.o[0] = cy * b.w + cx; s.o[1] = cy * b.w + (s.xp - b.x0); s.o[2] = cy * b.w + (s.xm - b.x0);
    s.o[3] = (s.yp - b.y0) * b.w + cx; s.o[4] = (s.ym - b.y0) * b.w + cx;
  }
}

// Streams the windows of planes q[0 .. d) through a double buffer in LDS and calls
// consume(cc, window, plane, extra, live) for each.  Two channels are in flight per thread: while channel c is consumed
// from LDS, channel c+1 waits in registers (loaded one step earlier) and channel c+2 is being loaded.  extra = pre(cc) is
// loaded together with the window of channel cc (values of another plane that the consumer needs).  Every load and
// every LDS store of the loop is unconditional -- elements past the window's end re-read its first element, channels
// past the last one re-read the last one -- so that the compiler can wait for exactly the loads a step needs instead of
// for all loads in flight; `live` is false for the surplus step of an odd channel count (the same for the whole block):
// the consumer must neither store nor accumulate then.
template <int PX, typename Pre, typename Consume>
__device__ __forceinline__ void window_pass(const float* __restrict__ q, int d, size_t HW, int W, const Box& box,
                                            float (*win)[TileCfg<PX>::ELEMS], Pre pre, Consume consume) {
  constexpr int kElems = TileCfg<PX>::ELEMS, kPer = kElems / 256;
  static_assert(kElems % 256 == 0, "every thread stores the same number of window elements");
  const int count = box.w * box.h;
  // window elements of this thread: e = threadIdx.x + 256 k, row e / w, column e % w (exact in float for these sizes)
  unsigned goff[kPer];
  const float inv_w = 1.0f / (float)max(box.w, 1);
#pragma unroll
  for (int k = 0; k < kPer; k++) {
    const int e = threadIdx.x + 256 * k;
    const int r = (int)(((float)e + 0.5f) * inv_w);
    goff[k] = e < count ? (unsigned)(r * W + (e - r * box.w)) : 0u;
  }
  const float* corner = q + (size_t)box.y0 * W + box.x0;
  auto fetch = [&](int c, float (&r)[kPer]) {
    const float* src = corner + (size_t)c * HW;
#pragma unroll
    for (int k = 0; k < kPer; k++) r[k] = src[goff[k]];
  };
  auto stash = [&](const float (&r)[kPer], float* buf) {
#pragma unroll
    for (int k = 0; k < kPer; k++) buf[threadIdx.x + 256 * k] = r[k];
  };
  const int last = d - 1;
  float ra[kPer], rb[kPer];
  fetch(0, ra);
  auto ea = pre(0);
  fetch(min(1, last), rb);
  auto eb = pre(min(1, last));
  stash(ra, win[0]);
  __syncthreads();
  for (int c0 = 0; c0 < d; c0 += 2) {
    {  // channel c0 is in win[0], c0 + 1 on its way into rb
      const auto e = ea;
      fetch(min(c0 + 2, last), ra);
      ea = pre(min(c0 + 2, last));
      consume(c0, win[0], q + (size_t)c0 * HW, e, true);
      stash(rb, win[1]);
      __syncthreads();
    }
    {  // channel c0 + 1 is in win[1], c0 + 2 on its way into ra
      const auto e = eb;
      const int c = min(c0 + 1, last);
      fetch(min(c0 + 3, last), rb);
      eb = pre(min(c0 + 3, last));
      consume(c, win[1], q + (size_t)c * HW, e, c0 + 1 < d);
      stash(ra, win[0]);
      __syncthreads();
    }
  }
}

// The same stream with the windows loaded from memory straight into LDS (global_load_lds: no staging registers) through a
// ring of kDmaStages buffers: while channel c is consumed, channels c+1 and c+2 are on their way and channel c+3 is asked
// for as soon as c has been consumed -- three channels in flight per wavefront instead of two, one barrier per channel.
// Loads return in order, so "at most two channels' worth of loads outstanding" means channel c has arrived (a wavefront's
// stores in between make the wait a little longer, never shorter); the barrier then makes every wavefront's part of the
// window visible.  A buffer is overwritten two barriers after its last reader has passed the barrier that follows its
// consumption.  No `pre` values: for consumers that need the window only.
// The four buffers are four separate __shared__ arrays, not one: the compiler waits, before a read of LDS, for every load
// into LDS that may alias it, and it can tell loads into different variables apart, not into parts of one.
template <int PX, typename Consume>
__device__ __forceinline__ void window_pass_dma(const float* __restrict__ q, int d, size_t HW, int W, const Box& box,
                                                float* w0, float* w1, float* w2, float* w3, Consume consume) {
  constexpr int kElems = TileCfg<PX>::ELEMS, kPer = kElems / 256;
  static_assert(kElems % 256 == 0, "every thread loads the same number of window elements");
  typedef const __attribute__((address_space(1))) void* GlobalPtr;
  typedef __attribute__((address_space(3))) void* LdsPtr;
  const int count = box.w * box.h;
  unsigned goff[kPer];
  const float inv_w = 1.0f / (float)max(box.w, 1);
#pragma unroll
  for (int k = 0; k < kPer; k++) {
    const int e = threadIdx.x + 256 * k;
    const int r = (int)(((float)e + 0.5f) * inv_w);
    goff[k] = e < count ? (unsigned)(r * W + (e - r * box.w)) : 0u;
  }
  const float* corner = q + (size_t)box.y0 * W + box.x0;
  const int wave_first = __builtin_amdgcn_readfirstlane((int)(threadIdx.x & ~63u));  // lane l of the wavefront writes element wave_first + l
  auto fetch = [&](int c, float* buf) {
    const float* src = corner + (size_t)c * HW;
#pragma unroll
    for (int k = 0; k < kPer; k++)
      __builtin_amdgcn_global_load_lds((GlobalPtr)(src + goff[k]), (LdsPtr)(buf + 256 * k + wave_first), 4, 0, 0);
  };
  const int last = d - 1;
  auto phase = [&](int c, float* buf, float* refill) {
    // channel c's loads have landed when at most the two younger channels' loads are outstanding
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * kPer) : "memory");
    const int cc = min(c, last);
    consume(cc, buf, q + (size_t)cc * HW, 0, c < d);
    fetch(min(c + 3, last), refill);
  };
  fetch(0, w0);
  fetch(min(1, last), w1);
  fetch(min(2, last), w2);
  for (int c0 = 0; c0 < d; c0 += 4) {
    phase(c0, w0, w3);
    phase(c0 + 1, w1, w0);
    phase(c0 + 2, w2, w1);
    phase(c0 + 3, w3, w2);
  }
  // (the loads still in flight at the end target LDS: they must have landed before the workgroup's LDS is handed on)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// the five taps of every inside pixel of the lane, from the window or (far pixels) from the plane
template <int PX, typename Body>
__device__ __forceinline__ void each_pixel_taps(const TilePx (&px)[PX], const float* buf, const float* plane, Body body) {
#pragma unroll
  for (int i = 0; i < PX; i++) {
    if (px[i].inside) {
      float t[5];
      if (!px[i].far) {
#pragma unroll
        for (int k = 0; k < 5; k++) t[k] = buf[px[i].o[k]];
      } else {
#pragma unroll
        for (int k = 0; k < 5; k++) t[k] = plane[px[i].o[k]];
      }
      body(i, t);
    }
  }
}

// decode the block's tile (XCD-banded numbering); false: the block has no tile
__device__ __forceinline__ bool tile_of_block(int N, int tiles_x, int tiles_y, int& n, int& tx, int& ty) {
  const int per_xcd = gridDim.x >> 3;
  const int lb = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int tiles = tiles_x * tiles_y;
  if (lb >= N * tiles) return false;
  n = lb / tiles;
  const int r = lb - n * tiles;
  ty = r / tiles_x;
  tx = r - ty * tiles_x;
  return true;
}

// MODE 0: the forward pass (QF.cu:14-139).  MODE 1: pass A of the backward pass (fit, g0, coefficients, lists).
template <int MODE, int PX>
__global__ __launch_bounds__(256) void quadfit_tiles(const float* __restrict__ im0, const float* __restrict__ im1,
                                                     const float* __restrict__ flow, const float* __restrict__ gin,
                                                     float* __restrict__ res, QfWorkspace ws, int N, int d, int H, int W,
                                                     int fc, int tiles_x, int tiles_y) {
  constexpr int kPX = PX, kTH = TileCfg<PX>::TH;
  __shared__ float win[2][TileCfg<PX>::ELEMS];
  __shared__ int red[16];
  int n, tx, ty;
  if (!tile_of_block(N, tiles_x, tiles_y, n, tx, ty)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW;
  const float* a = im0 + (size_t)n * d * HW;
  const float* q = im1 + (size_t)n * d * HW;
  const float* fl = flow + (size_t)n * fc * HW;
  const int x = tx * kTW + lane;
  TilePx px[kPX];
  bool valid[kPX];
  int minx = INT_MAX, maxx = INT_MIN, miny = INT_MAX, maxy = INT_MIN;
#pragma unroll
  for (int i = 0; i < kPX; i++) {
    const int y = ty * kTH + wave * kPX + i;
    valid[i] = x < W && y < H;
    locate(px[i], fl, HW, H, W, x, y, valid[i], minx, maxx, miny, maxy);
  }
  const Box box = block_box(minx, maxx, miny, maxy, red, TileCfg<PX>::ELEMS);
#pragma unroll
  for (int i = 0; i < kPX; i++) place(px[i], box, W);

  float cost[kPX][5];
#pragma unroll
  for (int i = 0; i < kPX; i++)
#pragma unroll
    for (int k = 0; k < 5; k++) cost[i][k] = 0.f;
  struct FirstMap {
    float v[kPX];
  };
  auto first_map = [&](int cc) {  // the lane's pixels of the first feature map (offset 0 for a pixel outside the image)
    FirstMap m;
#pragma unroll
    for (int i = 0; i < kPX; i++) m.v[i] = a[(size_t)cc * HW + px[i].p];
    return m;
  };
  window_pass<PX>(q, d, HW, W, box, win, first_map, [&](int cc, const float* buf, const float* plane, const FirstMap& m, bool live) {
    each_pixel_taps<PX>(px, buf, plane, [&](int i, const float (&t)[5]) {  // QF.cu:63-71
      if (live) {
#pragma unroll
        for (int k = 0; k < 5; k++) cost[i][k] += m.v[i] * t[k];
      }
    });
  });

  Fit f[kPX];
#pragma unroll
  for (int i = 0; i < kPX; i++) {
    f[i].inside = px[i].inside;
    f[i].validX = f[i].validY = 0;
    f[i].c00 = f[i].ax = f[i].ay = f[i].bx = f[i].by = f[i].fx = f[i].fy = 0.f;
    if (px[i].inside) finish_fit(f[i], cost[i][0], cost[i][1], cost[i][3], cost[i][2], cost[i][4], px[i].ix, px[i].iy, H, W);
  }
  if (MODE == 0) {
#pragma unroll
    for (int i = 0; i < kPX; i++) {
      if (!valid[i]) continue;
      float* o = res + (size_t)n * 3 * HW + px[i].p;
      float score = 0.f;
      if (f[i].inside)  // QF.cu:136
        score = f[i].ax * f[i].fx * f[i].fx + f[i].bx * f[i].fx + f[i].c00 + f[i].ay * f[i].fy * f[i].fy + f[i].by * f[i].fy;
      o[0] = f[i].fx;
      o[HW] = f[i].fy;
      o[2 * HW] = score;
    }
    return;
  }
  float* G0 = res + (size_t)n * d * HW;
  Factors k[kPX];
#pragma unroll
  for (int i = 0; i < kPX; i++) {
    k[i].any_valid = false;
    k[i].k00 = 0.;
    k[i].k0p = k[i].k0m = k[i].kp0 = k[i].km0 = k[i].dFds = 0.f;
    if (valid[i] && !px[i].inside)
      for (int cc = 0; cc < d; cc++) G0[(size_t)cc * HW + px[i].p] = 0.f;
    if (!px[i].inside) continue;
    k[i] = scatter_factors(f[i], gin, n, HW, px[i].p);
    const long long t = (long long)n * HW + px[i].p;
    ws.coef[0 * P + t] = k[i].any_valid ? (float)(0.5 * k[i].k00) : k[i].dFds;  // QF.cu:279-283,296
    ws.coef[1 * P + t] = k[i].any_valid ? 0.5f * k[i].k0p : 0.f;
    ws.coef[2 * P + t] = k[i].any_valid ? 0.5f * k[i].k0m : 0.f;
    ws.coef[3 * P + t] = k[i].any_valid ? 0.5f * k[i].kp0 : 0.f;
    ws.coef[4 * P + t] = k[i].any_valid ? 0.5f * k[i].km0 : 0.f;
    const long long centre = (long long)n * HW + (long long)px[i].iy * W + px[i].ix;
    const int pos = atomicAdd(ws.count + centre, 1);
    if (pos < kSlots) ws.slots[centre * kSlots + pos] = (int)px[i].p;
    else ws.ovf[atomicAdd(ws.ovf_count, 1)] = (int)t;
  }
  auto nothing = [](int) { return 0; };
  window_pass<PX>(q, d, HW, W, box, win, nothing, [&](int cc, const float* buf, const float* plane, int, bool live) {
    each_pixel_taps<PX>(px, buf, plane, [&](int i, const float (&t)[5]) {
      float g;
      if (k[i].any_valid)  // QF.cu:286-290
        g = 0.5 * (t[0] * k[i].k00 + t[1] * k[i].k0p + t[2] * k[i].k0m + t[3] * k[i].kp0 + t[4] * k[i].km0);
      else  // QF.cu:295
        g = t[0] * k[i].dFds;
      if (live) __builtin_nontemporal_store(g, &G0[(size_t)cc * HW + px[i].p]);
    });
  });
}

// Pass A of the backward pass with one read of the second feature map.  The gradient wrt the first map needs
// the finished fit (all channels) and then the five taps of every channel again.  Here a lane owns ONE pixel and
// keeps its taps of up to DMAX channels in registers (5 * DMAX floats) while the windows stream through LDS, so
// the second sweep over the channels is arithmetic and stores only.  Same sums in the same order as MODE 1 of
// quadfit_tiles (QF.cu:63-71 for the costs, QF.cu:279-297 for the gradient).
constexpr int kResidentChannels = 32;
constexpr int kResidentRows = 4;      // tile height: one row per wavefront
constexpr int kResidentElems = 1024;  // window capacity in floats (a 64 x 4 tile with +-3 pixels of spread needs ~800)
constexpr int kResidentDepth = 4;
constexpr int kResidentBand = 16;     // tile rows per band of the block order     // channels in flight per thread

template <int DMAX, bool FULL>  // FULL: exactly DMAX channels
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void quadfit_sources_resident(const float* __restrict__ im0, const float* __restrict__ im1,
                                                                const float* __restrict__ flow, const float* __restrict__ gin,
                                                                float* __restrict__ res, QfWorkspace ws, int N, int d, int H,
                                                                int W, int fc, int tiles_x, int tiles_y) {
  constexpr int kTH = kResidentRows, kElems = kResidentElems, kPer = (kElems + 255) / 256, D = kResidentDepth;
  __shared__ float win[2][kElems];
  __shared__ int red[16];
  int n, tx, ty;
  if (!tile_of_block(N, tiles_x, tiles_y, n, tx, ty)) return;
  {  // consecutive blocks walk DOWN a band of kResidentBand tile rows, then move one tile to the right: the blocks
     // in flight on one XCD cover a patch about as tall as wide, and the window rows that vertically adjacent
     // tiles share are read from memory once
    const int r = ty * tiles_x + tx;
    const int per_band = kResidentBand * tiles_x;
    const int band = r / per_band, rem = r - band * per_band;
    const int bh = min(kResidentBand, tiles_y - band * kResidentBand);
    tx = rem / bh;
    ty = band * kResidentBand + (rem - tx * bh);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW;
  const float* a = im0 + (size_t)n * d * HW;
  const float* q = im1 + (size_t)n * d * HW;
  const float* fl = flow + (size_t)n * fc * HW;
  const int x = tx * kTW + lane, y = ty * kTH + wave;
  const bool valid = x < W && y < H;
  TilePx px;
  int minx = INT_MAX, maxx = INT_MIN, miny = INT_MAX, maxy = INT_MIN;
  locate(px, fl, HW, H, W, x, y, valid, minx, maxx, miny, maxy);
  const Box box = block_box(minx, maxx, miny, maxy, red, kElems);
  place(px, box, W);

  // window elements of this thread: e = threadIdx.x + 256 k, row e / w, column e % w (exact in float for these sizes).
  // Elements past the window's end re-read its first element: every load and LDS access of the channel loop is
  // unconditional, so the loads of D channels stay in flight (no branch between a load and its use).
  const int count = box.w * box.h;
  unsigned goff[kPer];
  const float inv_w = 1.0f / (float)max(box.w, 1);
#pragma unroll
  for (int k = 0; k < kPer; k++) {
    const int e = threadIdx.x + 256 * k;
    const int r = (int)(((float)e + 0.5f) * inv_w);
    goff[k] = e < count ? (unsigned)(r * W + (e - r * box.w)) : 0u;
  }
  const bool near = px.inside && !px.far;
  unsigned lo[5];  // LDS offsets of the taps (0 for a pixel that does not read the window)
#pragma unroll
  for (int k = 0; k < 5; k++) lo[k] = near ? px.o[k] : 0u;
  const float* corner = q + (size_t)box.y0 * W + box.x0;
  // D channels in flight per thread: window elements in regs, the pixel's value of the first map in av
  float regs[D][kPer], av[D];
  auto fetch = [&](int c, float (&r)[kPer], float& first) {
    const float* src = corner + (size_t)c * HW;
#pragma unroll
    for (int k = 0; k < kPer; k++) r[k] = src[goff[k]];
    first = a[(size_t)c * HW + px.p];
  };
  auto stash = [&](const float (&r)[kPer], float* buf) {
#pragma unroll
    for (int k = 0; k < kPer; k++) buf[threadIdx.x + 256 * k] = r[k];
  };

  float tap[DMAX][5];
  float cost[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
  // No load sits behind a condition that the compiler cannot resolve (it would have to wait for every load in flight
  // at each join): past the last channel the loads re-read the last channel and the stores rewrite the idle buffer.
#pragma unroll
  for (int j = 0; j < D; j++) fetch(FULL ? j : min(j, d - 1), regs[j], av[j]);
  stash(regs[0], win[0]);
  __syncthreads();
#pragma unroll
  for (int c = 0; c < DMAX; c++) {
    if (FULL || c < d) {  // the same for the whole block
      const float a_cur = av[c % D];
      if (!FULL || c + D < DMAX)  // this set of registers went to LDS one channel ago
        fetch(FULL ? c + D : min(c + D, d - 1), regs[c % D], av[c % D]);
#pragma unroll
      for (int k = 0; k < 5; k++) tap[c][k] = win[c & 1][lo[k]];
#pragma unroll
      for (int k = 0; k < 5; k++) cost[k] += a_cur * tap[c][k];  // QF.cu:63-71
      if (!FULL || c + 1 < DMAX) stash(regs[(c + 1) % D], win[(c + 1) & 1]);
      __syncthreads();
    }
  }
  if (px.inside && px.far) {  // taps outside the window's capacity: the same sums from memory
    const int xm = max(px.ix - 1, 0), ym = max(px.iy - 1, 0), xp = min(px.ix + 1, W - 1), yp = min(px.iy + 1, H - 1);
    const unsigned fo[5] = {(unsigned)px.iy * W + px.ix, (unsigned)px.iy * W + xp, (unsigned)px.iy * W + xm,
                            (unsigned)yp * W + px.ix, (unsigned)ym * W + px.ix};  // taps 00, 0p, 0m, p0, m0
#pragma unroll
    for (int k = 0; k < 5; k++) cost[k] = 0.f;
#pragma unroll
    for (int c = 0; c < DMAX; c++) {
      if (c < d) {
        const float a_cur = a[(size_t)c * HW + px.p];
#pragma unroll
        for (int k = 0; k < 5; k++) tap[c][k] = q[(size_t)c * HW + fo[k]];
#pragma unroll
        for (int k = 0; k < 5; k++) cost[k] += a_cur * tap[c][k];
      }
    }
  }

  float* G0 = res + (size_t)n * d * HW;
  if (!px.inside) {
    if (valid)
      for (int cc = 0; cc < d; cc++) G0[(size_t)cc * HW + px.p] = 0.f;
    return;
  }
  Fit f;
  f.inside = true;
  f.validX = f.validY = 0;
  f.c00 = f.ax = f.ay = f.bx = f.by = f.fx = f.fy = 0.f;
  finish_fit(f, cost[0], cost[1], cost[3], cost[2], cost[4], px.ix, px.iy, H, W);
  const Factors kf = scatter_factors(f, gin, n, HW, px.p);
  const long long t = (long long)n * HW + px.p;
  ws.coef[0 * P + t] = kf.any_valid ? (float)(0.5 * kf.k00) : kf.dFds;  // QF.cu:279-283,296
  ws.coef[1 * P + t] = kf.any_valid ? 0.5f * kf.k0p : 0.f;
  ws.coef[2 * P + t] = kf.any_valid ? 0.5f * kf.k0m : 0.f;
  ws.coef[3 * P + t] = kf.any_valid ? 0.5f * kf.kp0 : 0.f;
  ws.coef[4 * P + t] = kf.any_valid ? 0.5f * kf.km0 : 0.f;
  const long long centre = (long long)n * HW + (long long)px.iy * W + px.ix;
  const int pos = atomicAdd(ws.count + centre, 1);
  if (pos < kSlots) ws.slots[centre * kSlots + pos] = (int)px.p;
  else ws.ovf[atomicAdd(ws.ovf_count, 1)] = (int)t;
#pragma unroll
  for (int c = 0; c < DMAX; c++) {
    if (c < d) {
      float g;
      if (kf.any_valid)  // QF.cu:286-290
        g = 0.5 * (tap[c][0] * kf.k00 + tap[c][1] * kf.k0p + tap[c][2] * kf.k0m + tap[c][3] * kf.kp0 + tap[c][4] * kf.km0);
      else  // QF.cu:295
        g = tap[c][0] * kf.dFds;
      __builtin_nontemporal_store(g, &G0[(size_t)c * HW + px.p]);  // (the caller reads it, later: kept out of the caches, it leaves them to the windows)
    }
  }
}

// Pass B of the backward pass on tiles of target pixels: the (source, coefficient) pairs of every pixel are
// collected once; per channel the window of the FIRST feature map that covers the tile's sources is
// staged in LDS and the pairs are summed from it.
constexpr int kPairs = 12;
constexpr int kPxGather = 2;

// Twelve reads of one LDS buffer at per-lane element offsets, issued together and waited for once, as one block the
// compiler does not look into: before an LDS read that it sees, it waits for the loads into LDS that may alias it, and
// with four buffers in a ring it takes that to be all of them -- the whole prefetch queue.  The caller has waited for the
// buffer's own loads (window_pass_dma).
static_assert(kPairs == 12, "lds_gather12 reads twelve elements");
__device__ __forceinline__ void lds_gather12(const float* buf, const unsigned (&off)[kPairs], float (&v)[kPairs]) {
  const unsigned b = (unsigned)(size_t)(const __attribute__((address_space(3))) float*)buf;
  unsigned a[kPairs];
#pragma unroll
  for (int j = 0; j < kPairs; j++) a[j] = b + 4u * off[j];
  asm volatile(
      "ds_read_b32 %0, %12\n\tds_read_b32 %1, %13\n\tds_read_b32 %2, %14\n\tds_read_b32 %3, %15\n\t"
      "ds_read_b32 %4, %16\n\tds_read_b32 %5, %17\n\tds_read_b32 %6, %18\n\tds_read_b32 %7, %19\n\t"
      "ds_read_b32 %8, %20\n\tds_read_b32 %9, %21\n\tds_read_b32 %10, %22\n\tds_read_b32 %11, %23\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]), "=&v"(v[8]),
        "=&v"(v[9]), "=&v"(v[10]), "=&v"(v[11])
      : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]), "v"(a[8]), "v"(a[9]), "v"(a[10]),
        "v"(a[11])
      : "memory");
}

template <int PX>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void quadfit_gather_tiles(const float* __restrict__ im0, float* __restrict__ g1, QfWorkspace ws,
                                                            int N, int d, int H, int W, int tiles_x, int tiles_y) {
  constexpr int kTH = TileCfg<PX>::TH;
  __shared__ float win0[TileCfg<PX>::ELEMS], win1[TileCfg<PX>::ELEMS], win2[TileCfg<PX>::ELEMS], win3[TileCfg<PX>::ELEMS];
  __shared__ int red[16];
  int n, tx, ty;
  if (!tile_of_block(N, tiles_x, tiles_y, n, tx, ty)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t HW = (size_t)H * W;
  const long long P = (long long)N * HW, base = (long long)n * HW;
  const float* a = im0 + (size_t)n * d * HW;
  float* G1 = g1 + (size_t)n * d * HW;
  const int x = tx * kTW + lane;
  const float inv_w = 1.0f / (float)W;
  bool valid[PX];
  unsigned pix[PX];
  int np[PX];
  unsigned off[PX][kPairs];  // packed (y << 16 | x) of the source, then its offset in the window
  float cf[PX][kPairs];
  int minx = INT_MAX, maxx = INT_MIN, miny = INT_MAX, maxy = INT_MIN;
  // (position whose sources reach a pixel, tap they reach it with), as an offset in the plane; a neighbour outside the
  // image has no list.  Three reads stand behind every pair -- list length, list, coefficient.  They are issued
  // unconditionally and in batches (an absent list reads the pixel's own, an unused entry coefficient 0 of the sample):
  // lengths and lists of all pixels of the lane together, then the coefficients of one pixel at a time -- three round
  // trips to memory; behind `if (cnt > 0)` / `if (s < cnt)` each read waits for the one before it, some fifty in a row.
  int cnt[PX][5];
  int4 sl[PX][5];
#pragma unroll
  for (int i = 0; i < PX; i++) {
    const int y = ty * kTH + wave * PX + i;
    valid[i] = x < W && y < H;
    pix[i] = valid[i] ? (unsigned)y * W + x : 0u;
    np[i] = 0;
#pragma unroll
    for (int j = 0; j < kPairs; j++) {
      off[i][j] = 0u;
      cf[i][j] = 0.f;
    }
    const bool has[5] = {valid[i], valid[i] && x > 0, valid[i] && x < W - 1, valid[i] && y > 0, valid[i] && y < H - 1};
    const int step[5] = {0, -1, 1, -W, W};
#pragma unroll
    for (int k = 0; k < 5; k++) {
      const long long ctr = base + (long long)pix[i] + (has[k] ? step[k] : 0);
      cnt[i][k] = ws.count[ctr];
      sl[i][k] = *reinterpret_cast<const int4*>(ws.slots + ctr * kSlots);
    }
  }
#pragma unroll
  for (int i = 0; i < PX; i++) {
    const int y = ty * kTH + wave * PX + i;
    const bool has[5] = {valid[i], valid[i] && x > 0, valid[i] && x < W - 1, valid[i] && y > 0, valid[i] && y < H - 1};
    float cv[5][kSlots];
    unsigned spv[5][kSlots];
#pragma unroll
    for (int k = 0; k < 5; k++) {
      cnt[i][k] = has[k] ? min(cnt[i][k], kSlots) : 0;
      const int sv[4] = {sl[i][k].x, sl[i][k].y, sl[i][k].z, sl[i][k].w};
#pragma unroll
      for (int s = 0; s < kSlots; s++) {
        spv[k][s] = s < cnt[i][k] ? (unsigned)sv[s] : 0u;  // source pixel, offset in its plane
        cv[k][s] = ws.coef[(long long)k * P + base + spv[k][s]];
      }
    }
    // (the values are pinned here, all of them: left alone, the optimizer moves each read back behind the branch that
    // uses it)
#pragma unroll
    for (int k = 0; k < 5; k++)
#pragma unroll
      for (int s = 0; s < kSlots; s++) asm volatile("" : "+v"(cv[k][s]));
#pragma unroll
    for (int k = 0; k < 5; k++) {
#pragma unroll
      for (int s = 0; s < kSlots; s++) {
        if (s < cnt[i][k]) {
          const unsigned sp = spv[k][s];  // (below 2^24: the float quotient is off by one at most)
          int sy = (int)((float)sp * inv_w), sx = (int)sp - sy * W;
          if (sx < 0) { sy--; sx += W; }
          if (sx >= W) { sy++; sx -= W; }
          const float c = cv[k][s];
#pragma unroll
          for (int j = 0; j < kPairs; j++)
            if (np[i] == j) {
              off[i][j] = ((unsigned)sy << 16) | (unsigned)sx;
              cf[i][j] = c;
            }
          if (np[i] < kPairs) {
            minx = min(minx, sx); maxx = max(maxx, sx);
            miny = min(miny, sy); maxy = max(maxy, sy);
          }
          np[i]++;
        }
      }
    }
  }
  const Box box = block_box(minx, maxx, miny, maxy, red, TileCfg<PX>::ELEMS);
  // a pixel with more pairs than registers, or with a source outside the window, walks its lists from memory instead
  bool slow[PX];
  unsigned need = 0;
#pragma unroll
  for (int i = 0; i < PX; i++) {
    slow[i] = np[i] > kPairs;
#pragma unroll
    for (int j = 0; j < kPairs; j++) {
      const int sx = off[i][j] & 0xffff, sy = off[i][j] >> 16;
      const bool used = j < np[i];
      if (used && !(sx - box.x0 < box.w && sy - box.y0 < box.h)) slow[i] = true;
      off[i][j] = used ? (unsigned)((sy - box.y0) * box.w + (sx - box.x0)) : 0u;
    }
#pragma unroll
    for (int j = 0; j < kPairs; j++) {
      if (slow[i]) {
        off[i][j] = 0u;
        cf[i][j] = 0.f;
      }
      if (__ballot(!slow[i] && j < np[i]) != 0) need |= 1u << j;  // pairs nobody in the wavefront has are skipped by a uniform branch
    }
  }
  window_pass_dma<PX>(a, d, HW, W, box, win0, win1, win2, win3, [&](int cc, const float* buf, const float* plane, int, bool live) {
    // all window reads of a pixel are issued before the first product: a read inside the branch that skips an unused pair
    // is waited for on the spot, one LDS round trip after the other (an unused pair reads element 0, a broadcast)
#pragma unroll
    for (int i = 0; i < PX; i++) {
      float v[kPairs];
      lds_gather12(buf, off[i], v);
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < kPairs; j++)
        if (need & (1u << j)) acc = __builtin_fmaf(v[j], cf[i][j], acc);
      if (live && valid[i] && !slow[i]) __builtin_nontemporal_store(acc, &G1[(size_t)cc * HW + pix[i]]);
    }
  });
#pragma unroll
  for (int i = 0; i < PX; i++) {
    if (!valid[i] || !slow[i]) continue;
    const int y = ty * kTH + wave * PX + i;
    long long ctr[5];
    ctr[0] = base + pix[i];
    ctr[1] = x > 0 ? base + pix[i] - 1 : -1;
    ctr[2] = x < W - 1 ? base + pix[i] + 1 : -1;
    ctr[3] = y > 0 ? base + pix[i] - W : -1;
    ctr[4] = y < H - 1 ? base + pix[i] + W : -1;
    for (int cc = 0; cc < d; cc++) {
      const float* ac = a + (size_t)cc * HW;
      float acc = 0.f;
      for (int k = 0; k < 5; k++) {
        const int cnt = ctr[k] >= 0 ? min(ws.count[ctr[k]], kSlots) : 0;
        for (int s = 0; s < cnt; s++) {
          const unsigned sp = (unsigned)ws.slots[ctr[k] * kSlots + s];
          acc += ac[sp] * ws.coef[(long long)k * P + base + sp];
        }
      }
      G1[(size_t)cc * HW + pix[i]] = acc;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// median
// ---------------------------------------------------------------------------------------------
constexpr int kBins = 32;  // bins per staged chunk
constexpr int kPitch = kBins + 1;

// 64 pixels x nb bins between HBM and the wavefront's LDS tile; lane -> (pixel 2i + lane/32, bin lane%32)
__device__ __forceinline__ void stage_in(const float* __restrict__ vol, float (*tile)[kPitch], long long p0, long long P,
                                         int D, int c0, int nb, int lane) {
  const int b = lane & 31, half = lane >> 5;
#pragma unroll 8
  for (int i = 0; i < 32; i++) {
    const int px = 2 * i + half;
    const long long qpx = p0 + px;
    float v = 0.f;
    if (qpx < P && b < nb) v = vol[qpx * D + c0 + b];
    tile[px][b] = v;
  }
}
__device__ __forceinline__ void stage_out(float* __restrict__ gvol, float (*tile)[kPitch], long long p0, long long P, int D,
                                          int c0, int nb, int lane) {
  const int b = lane & 31, half = lane >> 5;
#pragma unroll 8
  for (int i = 0; i < 32; i++) {
    const int px = 2 * i + half;
    const long long qpx = p0 + px;
    if (qpx < P && b < nb) gvol[qpx * D + c0 + b] = tile[px][b];
  }
}

struct Crossing {
  bool found;
  int c;
  float score, pmid, alpha;
};
// the walk of MM.cu:26-43 == MM.cu:59-75 over one staged chunk
__device__ __forceinline__ void walk(Crossing& s, const float* row, int c0, int nb) {
  if (s.found) return;
  for (int j = 0; j < nb; j++) {
    const float cScore = row[j];
    if (s.score < 0.5 && s.score + cScore >= 0.5) {
      s.alpha = (1. - 2. * s.score - cScore) / (2. * cScore);  // MM.cu:34
      s.pmid = cScore;
      s.c = c0 + j;
      s.found = true;
      return;
    }
    s.score = s.score + cScore;
  }
}

// MM.cu:17-44.  P = n*h*w pixels; out (n,2,h,w).
__global__ __launch_bounds__(256) void median_forward_kernel(const float* __restrict__ vol, float* __restrict__ out,
                                                             long long P, long long HW, int D) {
  __shared__ float tiles[4][64][kPitch];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long long p0 = ((long long)blockIdx.x * 4 + wave) * 64;
  const long long p = p0 + lane;
  Crossing s{false, 0, 0.f, 1.f, 0.f};
  for (int c0 = 0; c0 < D; c0 += kBins) {
    const int nb = min(kBins, D - c0);
    stage_in(vol, tiles[wave], p0, P, D, c0, nb, lane);
    __syncthreads();
    walk(s, tiles[wave][lane], c0, nb);
    if (__syncthreads_and(s.found || p >= P)) break;
  }
  if (p < P) {
    const long long n = p / HW, q = p - n * HW;
    float med = 0.f, mass = 0.f;
    if (s.found) {
      med = (float)s.c - 0.f + s.alpha;  // MM.cu:35
      mass = s.pmid;
    }
    out[n * 2 * HW + q] = med;
    out[n * 2 * HW + HW + q] = mass;
  }
}

// MM.cu:46-93.  Pass 1 finds each pixel's crossing, pass 2 writes every bin's gradient.
__global__ __launch_bounds__(256) void median_backward_kernel(const float* __restrict__ vol, const float* __restrict__ gin,
                                                              float* __restrict__ gvol, long long P, long long HW, int D) {
  __shared__ float tiles[4][64][kPitch];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long long p0 = ((long long)blockIdx.x * 4 + wave) * 64;
  const long long p = p0 + lane;
  Crossing s{false, 0, 0.f, 1.f, 0.f};
  for (int c0 = 0; c0 < D; c0 += kBins) {
    const int nb = min(kBins, D - c0);
    stage_in(vol, tiles[wave], p0, P, D, c0, nb, lane);
    __syncthreads();
    walk(s, tiles[wave][lane], c0, nb);
    if (__syncthreads_and(s.found || p >= P)) break;
  }
  float g0v = 0.f, g1v = 0.f;
  if (p < P) {
    const long long n = p / HW, q = p - n * HW;
    g0v = gin[n * 2 * HW + q];
    g1v = gin[n * 2 * HW + HW + q];
  }
  const float cross = g0v * s.alpha / (-s.pmid) + g1v;  // MM.cu:69
  const float neg = -g0v / (2. * s.pmid);               // MM.cu:85
  const float pos = +g0v / (2. * s.pmid);               // MM.cu:88
  float score = 0.f;
  for (int c0 = 0; c0 < D; c0 += kBins) {
    const int nb = min(kBins, D - c0);
    __syncthreads();
    stage_in(vol, tiles[wave], p0, P, D, c0, nb, lane);
    __syncthreads();
    float* row = tiles[wave][lane];
    for (int j = 0; j < nb; j++) {  // MM.cu:77-92; the crossing bin keeps the value of MM.cu:69
      const float cScore = row[j];
      float g = (s.found && c0 + j == s.c) ? cross : 0.f;
      if (score + cScore < 0.5) g = neg;
      else if (score >= 0.5) g = pos;
      row[j] = g;
      score = score + cScore;
    }
    __syncthreads();
    stage_out(gvol, tiles[wave], p0, P, D, c0, nb, lane);
  }
}

// ---------------------------------------------------------------------------------------------
// Median, whole histograms in LDS (up to 255 bins): the histograms of 64 consecutive pixels are one
// contiguous run of 64*D floats, staged with 16-byte loads into rows of odd pitch; each lane walks its
// row; the backward pass writes the gradients over the row and the run goes back out the same way.
// HBM sees the histogram once per pass.
// ---------------------------------------------------------------------------------------------
constexpr int kMaxRowBins = 255;

// In: kBatch loads per lane are issued before the first of them is stored to LDS (a loop that stores each value right
// after its load waits for memory once per element: 9 round trips per wavefront at 33 bins where one or two suffice).
template <int VEC, bool OUT>
__device__ __forceinline__ void stage_rows(const float* __restrict__ src, float* __restrict__ dst, float* tile, int total,
                                           int D, int Dp, int lane) {
  constexpr int kStep = 64 * VEC;
  constexpr int kBatch = OUT ? 1 : 8;
  if (VEC == 4 && Dp == D) {  // odd bin counts need no padding: the tile is a plain copy of the run, 16 bytes per lane and step
    const int full = total & ~3;
    if (OUT) {
      for (int i = lane * 4; i < full; i += kStep) *reinterpret_cast<float4*>(dst + i) = *reinterpret_cast<const float4*>(tile + i);
      for (int i = full + lane; i < total; i += 64) dst[i] = tile[i];
    } else {
      for (int i = lane * 4; i < full; i += kStep * 8) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = *reinterpret_cast<const float4*>(src + (i + u * kStep < full ? i + u * kStep : 0));
#pragma unroll
        for (int u = 0; u < 8; u++)
          if (i + u * kStep < full) *reinterpret_cast<float4*>(tile + i + u * kStep) = v[u];
      }
      for (int i = full + lane; i < total; i += 64) tile[i] = src[i];
    }
    return;
  }
  const int qs = kStep / D, rs = kStep - qs * D;
  int i = lane * VEC;
  int px = i / D, b = i - px * D;
  for (; i < total; i += kStep * kBatch) {
    float4 v4[kBatch];
    float v1[kBatch];
    if (!OUT) {  // unconditional loads (an index past the end re-reads the wavefront's first elements)
#pragma unroll
      for (int u = 0; u < kBatch; u++) {
        const int iu = i + u * kStep;
        if (VEC == 4) v4[u] = *reinterpret_cast<const float4*>(src + (iu + 3 < total ? iu : 0));
        else v1[u] = src[iu < total ? iu : 0];
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; u++) {
      const int iu = i + u * kStep;
      if (iu < total) {
        if (VEC == 4 && iu + 3 < total) {
          float* e[4];
          int pe = px, be = b;
#pragma unroll
          for (int k = 0; k < 4; k++) {
            e[k] = tile + pe * Dp + be;
            if (++be >= D) { be = 0; pe++; }
          }
          if (OUT) {
            float4 v;
            v.x = *e[0]; v.y = *e[1]; v.z = *e[2]; v.w = *e[3];
            *reinterpret_cast<float4*>(dst + iu) = v;
          } else {
            *e[0] = v4[u].x; *e[1] = v4[u].y; *e[2] = v4[u].z; *e[3] = v4[u].w;
          }
        } else {  // the run's last, partial vector (or VEC == 1)
          int pe = px, be = b;
          for (int k = 0; k < VEC && iu + k < total; k++) {
            if (OUT) dst[iu + k] = tile[pe * Dp + be];
            else tile[pe * Dp + be] = VEC == 4 ? src[iu + k] : v1[u];
            if (++be >= D) { be = 0; pe++; }
          }
        }
      }
      b += rs;
      px += qs;
      if (b >= D) { b -= D; px++; }
    }
  }
}

template <int VEC, bool BACKWARD>
__global__ __launch_bounds__(64) void median_rows_kernel(const float* __restrict__ vol, const float* __restrict__ gin,
                                                         float* __restrict__ res, long long P, long long HW, int D, int Dp,
                                                         long long first_tile) {
  extern __shared__ __align__(16) float tile[];  // 64 rows of pitch Dp
  const int lane = threadIdx.x;
  const long long p0 = (first_tile + blockIdx.x) * 64;
  const int npx = (int)min((long long)64, P - p0);
  const int total = npx * D;
  stage_rows<VEC, false>(vol + p0 * D, nullptr, tile, total, D, Dp, lane);
  __syncthreads();
  float* row = tile + lane * Dp;
  // the walk of MM.cu:26-43 == MM.cu:59-75, without the early exit (the bins past the crossing are skipped by `found`)
  // The crossing bin's interpolation (a double division) is formed once, after the walk: inside the loop it would run in
  // every iteration in which ANY lane of the wavefront crosses.  The comparisons against 0.5 are the reference's
  // (a float promoted to double compares as the float does).
  bool found = false;
  int cidx = 0;
  float score = 0.f, pmid = 1.f, alpha = 0.f;
  if (lane < npx) {
#pragma unroll 4
    for (int c = 0; c < D; c++) {
      const float cScore = row[c];
      const float sum = score + cScore;
      const bool hit = !found && score < 0.5f && sum >= 0.5f;
      pmid = hit ? cScore : pmid;
      cidx = hit ? c : cidx;
      found = found || hit;
      score = found ? score : sum;  // (the running sum stops in front of the crossing bin)
    }
    if (found) alpha = (1. - 2. * score - pmid) / (2. * pmid);  // MM.cu:34
  }
  const long long p = p0 + lane;
  const long long n = p / HW, q = p - n * HW;
  if (!BACKWARD) {
    if (lane < npx) {
      res[n * 2 * HW + q] = found ? (float)cidx - 0.f + alpha : 0.f;  // MM.cu:35
      res[n * 2 * HW + HW + q] = found ? pmid : 0.f;
    }
    return;
  }
  if (lane < npx) {
    const float g0v = gin[n * 2 * HW + q], g1v = gin[n * 2 * HW + HW + q];
    const float cross = g0v * alpha / (-pmid) + g1v;  // MM.cu:69
    const float neg = -g0v / (2. * pmid);             // MM.cu:85
    const float pos = +g0v / (2. * pmid);             // MM.cu:88
    score = 0.f;
#pragma unroll 4
    for (int c = 0; c < D; c++) {  // MM.cu:77-92; the crossing bin keeps the value of MM.cu:69
      const float cScore = row[c];
      const float sum = score + cScore;
      float g = (found && c == cidx) ? cross : 0.f;
      g = (sum < 0.5f) ? neg : ((score >= 0.5f) ? pos : g);
      row[c] = g;
      score = sum;
    }
  }
  __syncthreads();
  stage_rows<VEC, true>(nullptr, res + p0 * D, tile, total, D, Dp, lane);
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight.
__device__ __forceinline__ void lds_only_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The same pass over FULL tiles of 64 pixels for odd bin counts up to 4 * NV - 1 (no padding: the tile in LDS is a plain
// copy of the run), as a loop: a wavefront keeps the next tile's run in flight (NV 16-byte loads per lane, held in registers)
// while it walks the current one.  With one tile per wavefront only a quarter of the resident wavefronts have loads in
// flight at any time (the rest walk, store or are being launched), and the pass runs at half the rate memory allows.
template <int NV, bool BACKWARD>
__global__ __launch_bounds__(64) void median_stream_kernel(const float* __restrict__ vol, const float* __restrict__ gin,
                                                           float* __restrict__ res, long long tiles, long long HW, int D) {
  extern __shared__ __align__(16) float tile[];  // 64 rows of D floats
  const int lane = threadIdx.x;
  const int per = 16 * D;  // 16-byte elements of a tile
  typedef float vec4 __attribute__((ext_vector_type(4)));  // (an array of HIP's float4 structs ends up in scratch memory)
  vec4* tile4 = reinterpret_cast<vec4*>(tile);
  vec4 v[NV];
  float gn0 = 0.f, gn1 = 0.f;
  // every load unconditional: an element past the run re-reads the lane's first one, and so does every element of the
  // surplus fetch behind a wavefront's last tile (live = false)
  auto fetch = [&](long long t, bool live) {
    const vec4* src = reinterpret_cast<const vec4*>(vol) + t * per;
    const int last = live ? per : 0;
#pragma unroll
    for (int u = 0; u < NV; u++) v[u] = __builtin_nontemporal_load(src + (lane + 64 * u < last ? lane + 64 * u : lane));  // read once
    if (BACKWARD) {
      const long long p = t * 64 + lane, n = p / HW, q = p - n * HW;
      gn0 = gin[n * 2 * HW + q];
      gn1 = gin[n * 2 * HW + HW + q];
    }
  };
  long long t = blockIdx.x;
  if (t >= tiles) return;
  fetch(t, true);
  const float* row = tile + lane * D;
  for (; t < tiles; t += gridDim.x) {
#pragma unroll
    for (int u = 0; u < NV; u++)
      if (lane + 64 * u < per) tile4[lane + 64 * u] = v[u];
    const float g0v = gn0, g1v = gn1;
    const long long tn = t + gridDim.x;
    fetch(tn < tiles ? tn : t, tn < tiles);
    lds_only_barrier();  // (a full barrier would also wait for the loads just issued)
    bool found = false;
    int cidx = 0;
    float score = 0.f, pmid = 1.f, alpha = 0.f;
#pragma unroll 4
    for (int c = 0; c < D; c++) {  // the walk of median_rows_kernel
      const float cScore = row[c];
      const float sum = score + cScore;
      const bool hit = !found && score < 0.5f && sum >= 0.5f;
      pmid = hit ? cScore : pmid;
      cidx = hit ? c : cidx;
      found = found || hit;
      score = found ? score : sum;
    }
    if (found) alpha = (1. - 2. * score - pmid) / (2. * pmid);  // MM.cu:34
    if (!BACKWARD) {
      const long long p = t * 64 + lane, n = p / HW, q = p - n * HW;
      res[n * 2 * HW + q] = found ? (float)cidx - 0.f + alpha : 0.f;  // MM.cu:35
      res[n * 2 * HW + HW + q] = found ? pmid : 0.f;
    } else {
      const float cross = g0v * alpha / (-pmid) + g1v;  // MM.cu:69
      const float neg = -g0v / (2. * pmid);             // MM.cu:85
      const float pos = +g0v / (2. * pmid);             // MM.cu:88
      float* wrow = tile + lane * D;
      score = 0.f;
#pragma unroll 4
      for (int c = 0; c < D; c++) {  // MM.cu:77-92; the crossing bin keeps the value of MM.cu:69
        const float cScore = wrow[c];
        const float sum = score + cScore;
        float g = (found && c == cidx) ? cross : 0.f;
        g = (sum < 0.5f) ? neg : ((score >= 0.5f) ? pos : g);
        wrow[c] = g;
        score = sum;
      }
      lds_only_barrier();
      vec4* dst = reinterpret_cast<vec4*>(res) + t * per;
#pragma unroll
      for (int u = 0; u < NV; u++)
        if (lane + 64 * u < per) dst[lane + 64 * u] = tile4[lane + 64 * u];  // (plain stores: the non-temporal hint costs this pass 7%)
    }
    lds_only_barrier();  // the next tile overwrites the rows
  }
}

template <bool BACKWARD>
void launch_median_rows(const float* vol, const float* gin, float* res, long long P, long long HW, int D, bool aligned,
                        hipStream_t stream) {
  const int Dp = D | 1;
  constexpr int kStreamNV = 10;
  if (aligned && (D & 1) && D >= 5 && D < 4 * kStreamNV && P >= 64 && !inpaint::knobs().median_tile_per_wave) {
    // full tiles in the streaming loop, the last partial tile (if any) below
    const long long tiles = P / 64;
    const long long waves = std::min<long long>(tiles, 16ll * inpaint::compute_unit_count());
    hipLaunchKernelGGL((median_stream_kernel<kStreamNV, BACKWARD>), dim3((unsigned)waves), dim3(64), (size_t)64 * D * sizeof(float), stream,
                       vol, gin, res, tiles, HW, D);
    if (P % 64 == 0) return;
    // (the kernel below takes its pixels from P and blockIdx: give it the last tile only)
    hipLaunchKernelGGL((median_rows_kernel<4, BACKWARD>), dim3(1), dim3(64), (size_t)64 * Dp * sizeof(float), stream, vol, gin, res, P, HW, D,
                       Dp, tiles);
    return;
  }
  const dim3 grid((unsigned)((P + 63) / 64)), block(64);
  const size_t lds = (size_t)64 * Dp * sizeof(float);
  if (aligned && D >= 4)
    hipLaunchKernelGGL((median_rows_kernel<4, BACKWARD>), grid, block, lds, stream, vol, gin, res, P, HW, D, Dp, 0ll);
  else
    hipLaunchKernelGGL((median_rows_kernel<1, BACKWARD>), grid, block, lds, stream, vol, gin, res, P, HW, D, Dp, 0ll);
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

extern "C" {

const char* flowaux_last_error(void) { return inpaint::error_buffer(); }

int flowaux_profile(int enable) {
  g_timer.enabled = enable != 0;
  g_timed_pass = enable == 2 ? 2 : 1;
  g_timer.reset();
  return 0;
}

int flowaux_profile_read(double* total_ms, int* launches) { return g_timer.read(total_ms, launches); }

int quadfit_forward(const float* im0, const float* im1, const float* flow, float* out, int n, int ic, int ih, int iw,
                    int flow_channels, void* stream) {
  if (!im0 || !im1 || !flow || !out) return fail(INPAINT_ERR_ARG, "quadfit_forward: null pointer");
  if (n < 1 || ic < 1 || ih < 1 || iw < 1) return fail(INPAINT_ERR_ARG, "quadfit_forward: bad shape %dx%dx%dx%d", n, ic, ih, iw);
  if (flow_channels < 2) return fail(INPAINT_ERR_ARG, "quadfit_forward: the flow needs at least 2 channels, got %d", flow_channels);
  if ((long long)ih * iw >= (1ll << 31)) return fail(INPAINT_ERR_ARG, "quadfit_forward: image too large");
  const long long P = (long long)n * ih * iw;
  const int tiles_x = (iw + kTW - 1) / kTW, tiles_y = (ih + TileCfg<kPxForward>::TH - 1) / TileCfg<kPxForward>::TH;
  const long long tiles = (long long)n * tiles_x * tiles_y;
  if (tiles >= (1ll << 31) - 8) return fail(INPAINT_ERR_ARG, "quadfit_forward: too many tiles");
  if (inpaint::knobs().quadfit_px_path)
    hipLaunchKernelGGL(quadfit_forward_kernel, banded_grid(P), dim3(256), 0, (hipStream_t)stream, im0, im1, flow, out, n,
                       ic, ih, iw, flow_channels);
  else
    hipLaunchKernelGGL((quadfit_tiles<0, kPxForward>), dim3((unsigned)((tiles + 7) / 8 * 8)), dim3(256), 0, (hipStream_t)stream, im0, im1,
                       flow, nullptr, out, QfWorkspace{}, n, ic, ih, iw, flow_channels, tiles_x, tiles_y);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

long long quadfit_backward_workspace_bytes(int n, int ih, int iw) {
  if (n < 1 || ih < 1 || iw < 1) return 0;
  return qf_workspace_bytes((long long)n * ih * iw);
}

int quadfit_backward(const float* im0, const float* im1, const float* flow, const float* gin, float* g0, float* g1, int n,
                     int ic, int ih, int iw, int flow_channels, void* workspace, long long workspace_bytes, void* stream) {
  if (!im0 || !im1 || !flow || !gin || !g0 || !g1) return fail(INPAINT_ERR_ARG, "quadfit_backward: null pointer");
  if (n < 1 || ic < 1 || ih < 1 || iw < 1) return fail(INPAINT_ERR_ARG, "quadfit_backward: bad shape %dx%dx%dx%d", n, ic, ih, iw);
  if (flow_channels < 2) return fail(INPAINT_ERR_ARG, "quadfit_backward: the flow needs at least 2 channels, got %d", flow_channels);
  if ((long long)ih * iw >= (1ll << 31)) return fail(INPAINT_ERR_ARG, "quadfit_backward: image too large");
  const long long P = (long long)n * ih * iw, total = P * ic;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid = banded_grid(P), block(256);
  if (!workspace) {  // no workspace: scatter with float atomics
    hipLaunchKernelGGL(inpaint::fill_zero_f32, dim3(inpaint::grid_stride(total)), dim3(256), 0, st, g1, total);
    hipLaunchKernelGGL(quadfit_backward_kernel, grid, block, 0, st, im0, im1, flow, gin, g0, g1, n, ic, ih, iw, flow_channels);
    INPAINT_HIP(hipGetLastError());
    return 0;
  }
  if (workspace_bytes < qf_workspace_bytes(P))
    return fail(INPAINT_ERR_ARG, "quadfit_backward: workspace of %lld bytes, %lld needed", workspace_bytes, qf_workspace_bytes(P));
  if (((uintptr_t)workspace & 15) != 0) return fail(INPAINT_ERR_ARG, "quadfit_backward: workspace must be 16-byte aligned");
  if (P >= (1ll << 31)) return fail(INPAINT_ERR_ARG, "quadfit_backward: too many pixels for the inverse map");
  const QfWorkspace ws = qf_carve(workspace, P);
  // the counters start at zero (a fill kernel, so that the call can be captured into a graph)
  hipLaunchKernelGGL(inpaint::fill_zero_f32, dim3(inpaint::grid_stride(P + 64)), dim3(256), 0, st,
                     reinterpret_cast<float*>(ws.count), P + 64);
  const int tiles_x = (iw + kTW - 1) / kTW, tiles_y = (ih + TileCfg<kPxSources>::TH - 1) / TileCfg<kPxSources>::TH;
  const long long tiles = (long long)n * tiles_x * tiles_y;
  const bool px_path = inpaint::knobs().quadfit_px_path;
  if (px_path)
    hipLaunchKernelGGL(quadfit_backward_sources, grid, block, 0, st, im0, im1, flow, gin, g0, ws, n, ic, ih, iw, flow_channels);
  else {
    if (g_timed_pass == 1) g_timer.begin(st);
    if (ic <= kResidentChannels && !inpaint::knobs().quadfit_reread) {
      const int ry = (ih + kResidentRows - 1) / kResidentRows;
      const long long rt = (long long)n * tiles_x * ry;
      const dim3 rgrid((unsigned)((rt + 7) / 8 * 8));
      if (ic == kResidentChannels)
        hipLaunchKernelGGL((quadfit_sources_resident<kResidentChannels, true>), rgrid, block, 0, st, im0, im1, flow, gin, g0, ws, n,
                           ic, ih, iw, flow_channels, tiles_x, ry);
      else
        hipLaunchKernelGGL((quadfit_sources_resident<kResidentChannels, false>), rgrid, block, 0, st, im0, im1, flow, gin, g0, ws, n,
                           ic, ih, iw, flow_channels, tiles_x, ry);
    } else {
      hipLaunchKernelGGL((quadfit_tiles<1, kPxSources>), dim3((unsigned)((tiles + 7) / 8 * 8)), block, 0, st, im0, im1, flow, gin, g0,
                         ws, n, ic, ih, iw, flow_channels, tiles_x, tiles_y);
    }
    if (g_timed_pass == 1) g_timer.end(st, 1);
  }
  if (px_path || ih > 65535 || iw > 65535 || (long long)ih * iw >= (1ll << 24)) {
    hipLaunchKernelGGL(quadfit_backward_gather, grid, block, 0, st, im0, g1, ws, n, ic, ih, iw);
  } else {
    const int gy = (ih + TileCfg<kPxGather>::TH - 1) / TileCfg<kPxGather>::TH;
    const long long gt = (long long)n * tiles_x * gy;
    if (g_timed_pass == 2) g_timer.begin(st);
    hipLaunchKernelGGL((quadfit_gather_tiles<kPxGather>), dim3((unsigned)((gt + 7) / 8 * 8)), block, 0, st, im0, g1, ws, n, ic,
                       ih, iw, tiles_x, gy);
    if (g_timed_pass == 2) g_timer.end(st, 1);
  }
  hipLaunchKernelGGL(quadfit_backward_overflow, dim3(64), block, 0, st, im0, flow, g1, ws, n, ic, ih, iw, flow_channels);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

int medimax_forward(const float* vol, float* out, int n, int ih, int iw, int num_disp, void* stream) {
  if (!vol || !out) return fail(INPAINT_ERR_ARG, "medimax_forward: null pointer");
  if (n < 1 || ih < 1 || iw < 1 || num_disp < 1)
    return fail(INPAINT_ERR_ARG, "medimax_forward: bad shape %dx%dx%dx%d", n, ih, iw, num_disp);
  const long long HW = (long long)ih * iw, P = n * HW;
  if (num_disp <= kMaxRowBins)
    launch_median_rows<false>(vol, nullptr, out, P, HW, num_disp, aligned16(vol), (hipStream_t)stream);
  else
    hipLaunchKernelGGL(median_forward_kernel, dim3((unsigned)((P + 255) / 256)), dim3(256), 0, (hipStream_t)stream, vol, out, P,
                     HW, num_disp);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

int medimax_backward(const float* vol, const float* gin, float* gvol, int n, int ih, int iw, int num_disp, void* stream) {
  if (!vol || !gin || !gvol) return fail(INPAINT_ERR_ARG, "medimax_backward: null pointer");
  if (n < 1 || ih < 1 || iw < 1 || num_disp < 1)
    return fail(INPAINT_ERR_ARG, "medimax_backward: bad shape %dx%dx%dx%d", n, ih, iw, num_disp);
  const long long HW = (long long)ih * iw, P = n * HW;
  if (num_disp <= kMaxRowBins) {
    g_timer.begin((hipStream_t)stream);
    launch_median_rows<true>(vol, gin, gvol, P, HW, num_disp, aligned16(vol) && aligned16(gvol), (hipStream_t)stream);
    g_timer.end((hipStream_t)stream, 1);
  } else
    hipLaunchKernelGGL(median_backward_kernel, dim3((unsigned)((P + 255) / 256)), dim3(256), 0, (hipStream_t)stream, vol, gin,
                     gvol, P, HW, num_disp);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
