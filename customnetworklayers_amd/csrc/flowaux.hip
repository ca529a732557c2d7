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

#include "../../include/flowaux.h"
#include "inpaint_common.h"

namespace {

using inpaint::fail;

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

// QF.cu:22-104 (forward) == QF.cu:149-226 (backward): displaced position, the five matching
// costs, the two parabolas and their validity.
__device__ __forceinline__ Fit fit_pixel(const float* __restrict__ a, const float* __restrict__ q,
                                         const float* __restrict__ fl, int d, int H, int W, size_t HW, int h, int w) {
  Fit f;
  const unsigned p = (unsigned)h * W + w;
  const float idx = w + fl[p];       // QF.cu:31-32
  const float idy = h + fl[HW + p];
  f.inside = !(idx > W - 1 || idx < 0 || idy > H - 1 || idy < 0);  // QF.cu:35
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
  f.c00 = cost00;
  f.ax = 0.5 * (cost0p + cost0m - 2. * cost00);  // QF.cu:75-78
  f.ay = 0.5 * (costp0 + costm0 - 2. * cost00);
  f.bx = 0.5 * (cost0p - cost0m);
  f.by = 0.5 * (costp0 - costm0);
  f.validX = (f.ax < 0 && f.ax * f.ax >= 0.25 * f.bx * f.bx);  // QF.cu:83-89
  f.validY = (f.ay < 0 && f.ay * f.ay >= 0.25 * f.by * f.by);
  if (!(iidx < W - 1 && iidx > 0)) f.validX = 0;
  if (!(iidy < H - 1 && iidy > 0)) f.validY = 0;
  if (f.validX) f.fx = -0.5 * f.bx / f.ax;  // QF.cu:92-104
  if (f.validY) f.fy = -0.5 * f.by / f.ay;
  return f;
}

// QF.cu:14-139.  Every pixel writes its three outputs (zero outside the image), so no fill pass.
__global__ __launch_bounds__(256) void quadfit_forward_kernel(const float* __restrict__ im0, const float* __restrict__ im1,
                                                              const float* __restrict__ flow, float* __restrict__ out,
                                                              int N, int d, int H, int W, int fc) {
  const size_t HW = (size_t)H * W;
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
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
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
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

}  // namespace

extern "C" {

const char* flowaux_last_error(void) { return inpaint::error_buffer(); }

int quadfit_forward(const float* im0, const float* im1, const float* flow, float* out, int n, int ic, int ih, int iw,
                    int flow_channels, void* stream) {
  if (!im0 || !im1 || !flow || !out) return fail(INPAINT_ERR_ARG, "quadfit_forward: null pointer");
  if (n < 1 || ic < 1 || ih < 1 || iw < 1) return fail(INPAINT_ERR_ARG, "quadfit_forward: bad shape %dx%dx%dx%d", n, ic, ih, iw);
  if (flow_channels < 2) return fail(INPAINT_ERR_ARG, "quadfit_forward: the flow needs at least 2 channels, got %d", flow_channels);
  if ((long long)ih * iw >= (1ll << 31)) return fail(INPAINT_ERR_ARG, "quadfit_forward: image too large");
  const long long P = (long long)n * ih * iw;
  hipLaunchKernelGGL(quadfit_forward_kernel, dim3((unsigned)((P + 255) / 256)), dim3(256), 0, (hipStream_t)stream, im0, im1,
                     flow, out, n, ic, ih, iw, flow_channels);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

int quadfit_backward(const float* im0, const float* im1, const float* flow, const float* gin, float* g0, float* g1, int n,
                     int ic, int ih, int iw, int flow_channels, void* stream) {
  if (!im0 || !im1 || !flow || !gin || !g0 || !g1) return fail(INPAINT_ERR_ARG, "quadfit_backward: null pointer");
  if (n < 1 || ic < 1 || ih < 1 || iw < 1) return fail(INPAINT_ERR_ARG, "quadfit_backward: bad shape %dx%dx%dx%d", n, ic, ih, iw);
  if (flow_channels < 2) return fail(INPAINT_ERR_ARG, "quadfit_backward: the flow needs at least 2 channels, got %d", flow_channels);
  if ((long long)ih * iw >= (1ll << 31)) return fail(INPAINT_ERR_ARG, "quadfit_backward: image too large");
  const long long P = (long long)n * ih * iw, total = P * ic;
  hipLaunchKernelGGL(inpaint::fill_zero_f32, dim3(inpaint::grid_stride(total)), dim3(256), 0, (hipStream_t)stream, g1, total);
  hipLaunchKernelGGL(quadfit_backward_kernel, dim3((unsigned)((P + 255) / 256)), dim3(256), 0, (hipStream_t)stream, im0, im1,
                     flow, gin, g0, g1, n, ic, ih, iw, flow_channels);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

int medimax_forward(const float* vol, float* out, int n, int ih, int iw, int num_disp, void* stream) {
  if (!vol || !out) return fail(INPAINT_ERR_ARG, "medimax_forward: null pointer");
  if (n < 1 || ih < 1 || iw < 1 || num_disp < 1)
    return fail(INPAINT_ERR_ARG, "medimax_forward: bad shape %dx%dx%dx%d", n, ih, iw, num_disp);
  const long long HW = (long long)ih * iw, P = n * HW;
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
  hipLaunchKernelGGL(median_backward_kernel, dim3((unsigned)((P + 255) / 256)), dim3(256), 0, (hipStream_t)stream, vol, gin,
                     gvol, P, HW, num_disp);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
