// Huber-TGV FISTA inpainting layer for MI355X (gfx950): kernels, per-id state and the C ABI.
//
// What the layer computes is fixed by the reference's kernels
// (cudaTGV/cudaCode/TGVInpaintFistaBetas.cu, cited per function below as TGV.cu; helpers in
// cudaTGV/cudaCode/TGVInpaintFistaHelp.cu, TGVH.cu).  How it is computed is not:
//   * samples are a grid dimension (n >= 1), each with its own Lipschitz constant, which is
//     reduced and applied on the device (no host round trip, no textures);
//   * state tensors are (n, 3*C, H, W): variable-major (u, v1, v2) inside a sample, as the
//     reference's (3, C, H, W) tensors are for n == 1;
//   * checkpoints, the x05 history, the adjoint iterates, the per-segment fp32 accumulators and
//     their fp64 totals live in one device arena per id;
//   * the output guard runs on the device.
//
// Arithmetic contract: as for the TV layer, every value that can reach a Huber / prox switch is
// computed with the operation order of the reference source, IEEE division and square root and no
// fused multiply-add (build with -ffp-contract=off).  CUDA's rsqrtf (2 ulp, bits not recoverable
// from the sources) is taken as 1.0f / sqrtf(x), both correctly rounded.
#include "inpaint_common.h"
#include "tgv_strip_kernels.h"
#include "../../include/tgvinpaint.h"

#include <cstddef>
#include <cstdlib>

namespace {

using namespace inpaint;

// TGV.cu:58-60,70,78,87-93; TGVH.cu:24-41
constexpr float kD0 = 0.2f, kD1 = 0.2f, kD2 = 0.2f;
constexpr float kBeta = 4.0f;
constexpr float kLocalGCMult = 0.1f;
constexpr float kLocalGBMult = 1.0f;
constexpr float kGlobalGMult = 0.1f;
const GuardParams kGuard = {5000000., 5000000., 35., 10., 0.95};

constexpr int BX = 64, BY = 4;  // one pixel per thread, a wavefront per image row segment

// -------------------------------------------------------------------------------------------------
// device helpers
// -------------------------------------------------------------------------------------------------
struct Plane {  // zero outside the image, like the reference's haloed shared-memory tiles (TGV.cu:1581-1597)
  const float* f;
  int H, W;
  __device__ __forceinline__ float at(int h, int w) const {
    return (h >= 0 && h < H && w >= 0 && w < W) ? f[(size_t)h * W + w] : 0.f;
  }
};

__device__ __forceinline__ float rsq(float x) { return 1.0f / sqrtf(x); }
__device__ __forceinline__ float clampT(const float* f, int h, int w, int H, int W) {
  h = min(max(h, 0), H - 1);
  w = min(max(w, 0), W - 1);
  return f[(size_t)h * W + w];
}

// -------------------------------------------------------------------------------------------------
// Lipschitz bound: TGV.cu:101-148 per pixel, TGV.cu:2516-2527 for the reduction.
// maxbits[s] must hold the bit pattern of 32.0f (= float(max(12, 8*beta) + 0.000001)) on entry.
// -------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(BX* BY) void tgv_lipschitz_kernel(const float* __restrict__ dx_, const float* __restrict__ dy_,
                                                               int H, int W, unsigned int* __restrict__ maxbits) {
  const int w = blockIdx.x * BX + threadIdx.x, h = blockIdx.y * BY + threadIdx.y;
  const size_t HW = (size_t)H * W;
  const float* dx = dx_ + (size_t)blockIdx.z * 2 * HW;
  const float* dy = dy_ + (size_t)blockIdx.z * 2 * HW;
  const float* betaX = dx + HW;
  const float* betaY = dy + HW;
  float v = 0.f;
  if (w < W && h < H) {
    const float wx_0 = (w > 0) ? clampT(dx, h, w - 1, H, W) : 0.f;
    const float wx_1 = (w < W - 1) ? clampT(dx, h, w, H, W) : 0.f;
    const float wy_0 = (h > 0) ? clampT(dy, h - 1, w, H, W) : 0.f;
    const float wy_1 = (h < H - 1) ? clampT(dy, h, w, H, W) : 0.f;
    const float betaTX_1y = (h < H - 1) ? clampT(betaX, h, w, H, W) : 0.f;
    const float betaTX_1x = (w < W - 1) ? clampT(betaX, h, w, H, W) : 0.f;
    const float betaTX_0x = (w > 0) ? clampT(betaX, h - 1, w, H, W) : 0.f;  // sic: (w, h-1) under w > 0 (TGV.cu:116)
    const float betaTX_0y = (h > 0) ? clampT(betaX, h, w - 1, H, W) : 0.f;  // sic: (w-1, h) under h > 0 (TGV.cu:117)
    const float betaTY_1y = (h < H - 1) ? clampT(betaY, h, w, H, W) : 0.f;
    const float betaTY_1x = (w < W - 1) ? clampT(betaY, h, w, H, W) : 0.f;
    const float betaTY_0x = (w > 0) ? clampT(betaY, h - 1, w, H, W) : 0.f;
    const float betaTY_0y = (h > 0) ? clampT(betaY, h, w - 1, H, W) : 0.f;
    float weightx = 0.f, weighty1 = 0.f, weighty2 = 0.f;
    if (h > 0) {
      weightx += 3 * wy_0;
      weighty1 += 2 * betaTX_0y;
      weighty2 += 2 * betaTY_0y;
    }
    if (w > 0) {
      weightx += 3 * wx_0;
      weighty1 += 2 * betaTX_0x;
      weighty2 += 2 * betaTY_0x;
    }
    weightx += 3 * (wy_1 + wx_1);
    weighty1 += 2 * betaTX_1x + 2 * betaTX_1y + 3 * wx_1;
    weighty2 += 2 * betaTY_1x + 2 * betaTY_1y + 3 * wy_1;
    v = fmaxf(weightx, fmaxf(weighty1, weighty2));
  }
  // non-negative floats order like their bit patterns; anything else (negative, NaN) never wins
  // against the 32.0f start value in the reference's std::max either
  unsigned int bits = (v > 0.f) ? __float_as_uint(v) : 0u;
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned int o = __shfl_down(bits, off, 64);
    bits = o > bits ? o : bits;
  }
  if (threadIdx.x == 0 && bits > __float_as_uint(32.0f)) atomicMax(&maxbits[blockIdx.z], bits);
}

// (`counts`, when given: the two words of the upstream check that follows, cleared here)
static __global__ void tgv_lipschitz_init(unsigned int* maxbits, int n, unsigned int* counts) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) maxbits[i] = __float_as_uint((float)(fmax(12., 8. * (double)kBeta) + 0.000001));
  if (counts && i < 2) counts[i] = 0u;
}

__device__ __forceinline__ double lipschitz_from_bits(unsigned int bits) {
  float oneL = __uint_as_float(bits);
  oneL = (float)(1. / (double)(oneL + 0.01f));  // TGV.cu:2526
  return (double)oneL;                           // TGV.cu:2527: double L = oneL
}

// L-scaled private copies of the four weight fields (TGV.cu:2495-2499,2528-2531): (n,H,W) each.
__global__ __launch_bounds__(256) void tgv_scale_kernel(const float* __restrict__ dx, const float* __restrict__ dy,
                                                        const unsigned int* __restrict__ maxbits, float* __restrict__ wx,
                                                        float* __restrict__ wy, float* __restrict__ bx,
                                                        float* __restrict__ by, double* __restrict__ Ls, long long HW,
                                                        long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long s = i / HW, p = i - s * HW;
  const double L = lipschitz_from_bits(maxbits[s]);
  if (p == 0) Ls[s] = L;
  wx[i] = (float)(L * (double)dx[s * 2 * HW + p]);
  wy[i] = (float)(L * (double)dy[s * 2 * HW + p]);
  bx[i] = (float)(L * (double)dx[s * 2 * HW + HW + p]);
  by[i] = (float)(L * (double)dy[s * 2 * HW + HW + p]);
}

// Prox adjoint + confidence / rhs gradient: TGV.cu:592-612, 1418-1442 (and 166-182 for the first step).
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
    gb = 0.f;  // TGV.cu:181
  } else if (conf >= sign * diff) {
    g05 = 0.f;
    gb += df_dxk * kGB;
  } else {
    g05 = df_dxk;
    gc += sign * df_dxk * kGC;
  }
}

// First adjoint step: TGV.cu:151-218.  TRUE_ADJ: multipliers 1 (the corrected gradient).
template <bool TRUE_ADJ>
__global__ __launch_bounds__(256) void tgv_adjoint_first(const float* __restrict__ cf, const float* __restrict__ b,
                                                         const float* __restrict__ x05, float* __restrict__ gc,
                                                         float* __restrict__ gb, float* __restrict__ g05,
                                                         const float* __restrict__ gin, int C, long long HW,
                                                         long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long s = i / HW, p = i - s * HW;
  const long long CHW = HW * C;
  const float conf = cf[i];
  float gcv = gc[i];
  for (int ch = 0; ch < C; ch++) {
    const long long q = s * 3 * CHW + ch * HW + p;
    const long long qb = s * CHW + ch * HW + p;
    float g05v, gbv = gb[qb];
    prox_adjoint<true, TRUE_ADJ>(gin[q], b[qb], x05[q], conf, g05v, gcv, gbv);
    g05[q] = g05v;
    gb[qb] = gbv;
    g05[q + CHW] = gin[q + CHW];          // TGV.cu:215
    g05[q + 2 * CHW] = gin[q + 2 * CHW];  // TGV.cu:216
  }
  gc[i] = gcv;
}

// Corrected gradient only: the gradient step of iteration 0, which the reference never back-propagates
// (TGV.cu:2851-2933 ends after producing g05[0]; TGV.cu:3047 returns g_x[1]).  One thread per pixel applies the
// transposed Jacobian of the step at the starting point y_0 -- the main adjoint kernel's form (TGV.cu:304-507), every
// Huber weight derivative as weight x rsqrt^2, multipliers 1 -- to g05[0] and adds the partial g_x[0]:
// gi = J^T g05[0] + g_x[0] is the gradient wrt the starting point; the weight gradients of iteration 0 are added to the
// fp32 accumulators gwx / gwy (two planes each: edge weight, beta), which the caller flushes into the totals.
__global__ __launch_bounds__(BX* BY) void tgv_adjoint_iter0(
    const float* __restrict__ wx_, const float* __restrict__ wy_, const float* __restrict__ bx_,
    const float* __restrict__ by_, const float* __restrict__ y_, const float* __restrict__ g05_in_,
    const float* __restrict__ gx0_, float* __restrict__ gi_, float* __restrict__ gwx_, float* __restrict__ gwy_,
    int C, int H, int W) {
  const int w = blockIdx.x * BX + threadIdx.x, h = blockIdx.y * BY + threadIdx.y;
  if (w >= W || h >= H) return;
  const size_t HW = (size_t)H * W, CHW = HW * C, S = 3 * CHW;
  const size_t smp = blockIdx.z;
  const float *wx = wx_ + smp * HW, *wy = wy_ + smp * HW, *bx = bx_ + smp * HW, *by = by_ + smp * HW;
  const size_t p = (size_t)h * W + w;
  const float wx_0 = (w > 0) ? wx[p - 1] : 0.f;
  const float wx_1 = (w < W - 1) ? wx[p] : 0.f;
  const float wy_0 = (h > 0) ? wy[p - W] : 0.f;
  const float wy_1 = (h < H - 1) ? wy[p] : 0.f;
  const float wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : 0.f;
  const float wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : 0.f;
  const float b1u = (h > 0) ? bx[p - W] : 0.f, b2u = (h > 0) ? by[p - W] : 0.f;
  const float b1l = (w > 0) ? bx[p - 1] : 0.f, b2l = (w > 0) ? by[p - 1] : 0.f;
  const float b1c = bx[p], b2c = by[p];
  float gwx0 = gwx_[smp * 2 * HW + p], gwx1 = gwx_[smp * 2 * HW + HW + p];
  float gwy0 = gwy_[smp * 2 * HW + p], gwy1 = gwy_[smp * 2 * HW + HW + p];
  for (int ch = 0; ch < C; ch++) {
    const size_t o = smp * S + (size_t)ch * HW;
    const Plane Y{y_ + o, H, W}, Y1{y_ + o + CHW, H, W}, Y2{y_ + o + 2 * CHW, H, W};
    const Plane G{g05_in_ + o, H, W}, G1{g05_in_ + o + CHW, H, W}, G2{g05_in_ + o + 2 * CHW, H, W};
#define QY(F, dh, dw) F.at(h + (dh), w + (dw))
    const float yk = Y.f[p];
    const float g0 = G.f[p], g1 = G1.f[p], g2 = G2.f[p];
    float t0 = g0, t1 = g1, t2 = g2;
    if (h > 0) {  // triangles owned by the pixel above: TGV.cu:304-360 / 1118-1171
      const float beta1 = b1u, beta2 = b2u;
      {
        const float z1 = (w < W - 1) ? ((QY(Y, -1, 1) - QY(Y, -1, 0)) - QY(Y1, -1, 0)) : 0.f;
        const float z2 = ((yk - QY(Y, -1, 0)) - QY(Y2, -1, 0));
        const float A = z2 * z2 * wy_0 + z1 * z1 * wx_2;
        const float hub = rsq(A), hw = fminf(1.f, hub * kD0), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        t0 -= hw * ((g0 - QY(G, -1, 0)) - QY(G2, -1, 0)) * wy_0;
        if (active) {
          const float a2 = z2 * wy_0;
          const float a1 = z1 * wx_2;
          t0 += (dhw * a2) * (a1 * (QY(G, -1, 1) - QY(G, -1, 0) - QY(G1, -1, 0)) +
                                            a2 * (QY(G, 0, 0) - QY(G, -1, 0) - QY(G2, -1, 0)));
        }
      }
      {
        const float u1 = (w < W - 1) ? (QY(Y1, -1, 1) - QY(Y1, -1, 0)) : 0.f;
        const float u2 = (QY(Y1, 0, 0) - QY(Y1, -1, 0));
        const float B = (u1 * u1 + u2 * u2) * beta1;
        const float hub = rsq(B), hw = fminf(1.f, hub * kD1), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        t1 -= beta1 * hw * (g1 - QY(G1, -1, 0));
        if (active)
          t1 += beta1 * (dhw * beta1 * u2) * (u1 * (QY(G1, -1, 1) - QY(G1, -1, 0)) +
                                                                  u2 * (QY(G1, 0, 0) - QY(G1, -1, 0)));
      }
      {
        const float u1 = (w < W - 1) ? (QY(Y2, -1, 1) - QY(Y2, -1, 0)) : 0.f;
        const float u2 = (QY(Y2, 0, 0) - QY(Y2, -1, 0));
        const float B = (u1 * u1 + u2 * u2) * beta2;
        const float hub = rsq(B), hw = fminf(1.f, hub * kD2), dhw = hw * (hub * hub);  // (the reference divides here, TGV.cu:355, where every sibling block multiplies)
        const bool active = hw < 1.0f;
        t2 -= beta2 * hw * (g2 - QY(G2, -1, 0));
        if (active)
          t2 += beta2 * (dhw * beta2 * u2) * (u1 * (QY(G2, -1, 1) - QY(G2, -1, 0)) +
                                                                  u2 * (QY(G2, 0, 0) - QY(G2, -1, 0)));
      }
    }
    if (w > 0) {  // triangles owned by the pixel to the left: TGV.cu:361-418 / 1172-1227
      const float beta1 = b1l, beta2 = b2l;
      {
        const float z1 = (yk - QY(Y, 0, -1) - QY(Y1, 0, -1));
        const float z2 = (h < H - 1) ? (QY(Y, 1, -1) - QY(Y, 0, -1) - QY(Y2, 0, -1)) : 0.f;
        const float A = z2 * z2 * wy_2 + z1 * z1 * wx_0;
        const float hub = rsq(A), hw = fminf(1.f, hub * kD0), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        t0 -= hw * ((g0 - QY(G, 0, -1)) - QY(G1, 0, -1)) * wx_0;
        if (active) {
          const float a1 = z1 * wx_0;
          const float a2 = z2 * wy_2;
          t0 += (dhw * a1) * (a1 * (QY(G, 0, 0) - QY(G, 0, -1) - QY(G1, 0, -1)) +
                                            a2 * (QY(G, 1, -1) - QY(G, 0, -1) - QY(G2, 0, -1)));
        }
      }
      {
        const float u1 = (QY(Y1, 0, 0) - QY(Y1, 0, -1));
        const float u2 = (h < H - 1) ? (QY(Y1, 1, -1) - QY(Y1, 0, -1)) : 0.f;
        const float B = (u1 * u1 + u2 * u2) * beta1;
        const float hub = rsq(B), hw = fminf(1.f, hub * kD1), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        t1 -= beta1 * hw * (g1 - QY(G1, 0, -1));
        if (active)
          t1 += beta1 * (dhw * beta1 * u1) * (u2 * (QY(G1, 1, -1) - QY(G1, 0, -1)) +
                                                                  u1 * (QY(G1, 0, 0) - QY(G1, 0, -1)));
      }
      {
        const float u1 = (QY(Y2, 0, 0) - QY(Y2, 0, -1));
        const float u2 = (h < H - 1) ? (QY(Y2, 1, -1) - QY(Y2, 0, -1)) : 0.f;
        const float B = (u1 * u1 + u2 * u2) * beta2;
        const float hub = rsq(B), hw = fminf(1.f, hub * kD2), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        t2 -= beta2 * hw * (g2 - QY(G2, 0, -1));
        if (active)
          t2 += beta2 * (dhw * beta2 * u1) * (u2 * (QY(G2, 1, -1) - QY(G2, 0, -1)) +
                                                                  u1 * (QY(G2, 0, 0) - QY(G2, 0, -1)));
      }
    }
    {  // the pixel's own triangles: TGV.cu:419-507 / 1228-1333
      const float beta1 = b1c, beta2 = b2c;
      {
        const float z1 = (w < W - 1) ? ((QY(Y, 0, 1) - QY(Y, 0, 0)) - QY(Y1, 0, 0)) : 0.f;
        const float z2 = (h < H - 1) ? ((QY(Y, 1, 0) - QY(Y, 0, 0)) - QY(Y2, 0, 0)) : 0.f;
        const float A = z2 * z2 * wy_1 + z1 * z1 * wx_1;
        const float gr = QY(G, 0, 1), gd = QY(G, 1, 0);
        const float hub = rsq(A), hw = fminf(1.f, hub * kD0), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        const float dz1 = g0 - gr + g1, dz2 = g0 - gd + g2;
        t0 -= hw * (dz2 * wy_1 + dz1 * wx_1);
        t1 -= hw * dz1 * wx_1;
        t2 -= hw * dz2 * wy_1;
        gwx0 = gwx0 + dz1 * (z1 * hw);
        gwy0 = gwy0 + dz2 * (z2 * hw);
        if (active) {
          const float a1 = z1 * wx_1;
          const float a2 = z2 * wy_1;
          const float dot = (dz1 * a1 + dz2 * a2);
          t0 += dot * ((a1 + a2) * dhw);
          t2 += dot * (a2 * dhw);
          t1 += dot * (a1 * dhw);
          // the literal 0.5 makes these two updates double (TGV.cu:452-453)
          gwy0 = (float)((double)gwy0 - (double)((z2 * dhw * z2)) * 0.5 * (double)dot);
          gwx0 = (float)((double)gwx0 - (double)((z1 * dhw * z1)) * 0.5 * (double)dot);
        }
      }
      {
        const float u1 = (w < W - 1) ? (QY(Y1, 0, 1) - QY(Y1, 0, 0)) : 0.f;
        const float u2 = (h < H - 1) ? (QY(Y1, 1, 0) - QY(Y1, 0, 0)) : 0.f;
        const float B = (u1 * u1 + u2 * u2) * beta1;
        const float gr = QY(G1, 0, 1), gd = QY(G1, 1, 0);
        const float hub = rsq(B), hw = fminf(1.f, hub * kD1), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        if (w < W - 1) t1 -= beta1 * hw * (g1 - gr);
        if (h < H - 1) t1 -= beta1 * hw * (g1 - gd);
        gwx1 = gwx1 + ((g1 - gr) * u1 + (g1 - gd) * u2) * hw;
        if (active) {
          const float dot = ((g1 - gr) * u1 * beta1 + (g1 - gd) * u2 * beta1);
          t1 += beta1 * dhw * (u1 + u2) * dot;
          gwx1 = (float)((double)gwx1 -
                         (double)((u2 * dhw * u2 + u1 * dhw * u1)) * 0.5 * (double)dot);
        }
      }
      {
        const float u1 = (w < W - 1) ? (QY(Y2, 0, 1) - QY(Y2, 0, 0)) : 0.f;
        const float u2 = (h < H - 1) ? (QY(Y2, 1, 0) - QY(Y2, 0, 0)) : 0.f;
        const float B = (u1 * u1 + u2 * u2) * beta2;
        const float gr = QY(G2, 0, 1), gd = QY(G2, 1, 0);
        const float hub = rsq(B), hw = fminf(1.f, hub * kD2), dhw = hw * (hub * hub);
        const bool active = hw < 1.0f;
        if (w < W - 1) t2 -= beta2 * hw * (g2 - gr);
        if (h < H - 1) t2 -= beta2 * hw * (g2 - gd);
        gwy1 = gwy1 + ((g2 - gr) * u1 + (g2 - gd) * u2) * hw;
        if (active) {
          const float dot = ((g2 - gr) * u1 * beta2 + (g2 - gd) * u2 * beta2);
          t2 += beta2 * dhw * (u1 + u2) * dot;
          gwy1 = (float)((double)gwy1 -
                         (double)((u2 * dhw * u2 + u1 * dhw * u1)) * 0.5 * (double)dot);
        }
      }
    }
#undef QY
    // J^T g05[0] plus the partial g_x[0]: the gradient wrt the starting point, all three variables
    const size_t q = o + p;
    gi_[q] = t0 + gx0_[q];
    gi_[q + CHW] = t1 + gx0_[q + CHW];
    gi_[q + 2 * CHW] = t2 + gx0_[q + 2 * CHW];
  }
  gwx_[smp * 2 * HW + p] = gwx0;
  gwx_[smp * 2 * HW + HW + p] = gwx1;
  gwy_[smp * 2 * HW + p] = gwy0;
  gwy_[smp * 2 * HW + HW + p] = gwy1;
}

// Upstream check (TGV.cu:2686-2703): counts[0] = non-finite entries, counts[1] != 0 if any finite entry is non-zero.
// One atomic per block and only for non-finite entries; the non-zero flag is a plain store of the same value from
// whichever blocks see one (a counter bumped by every block of the launch would queue up at the memory side).
__global__ __launch_bounds__(256) void tgv_upstream_check(const float* __restrict__ g, long long n,
                                                          unsigned int* __restrict__ counts) {
  typedef float vec4 __attribute__((ext_vector_type(4)));
  unsigned int bad = 0, nz = 0;
  auto look = [&](float v) {
    if (!finite_value(v)) bad++;
    else if (v != 0.f) nz++;
  };
  const long long n4 = ((reinterpret_cast<uintptr_t>(g) & 15) == 0) ? (n >> 2) : 0;  // whole 16-byte groups
  const vec4* __restrict__ g4 = reinterpret_cast<const vec4*>(g);
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (long long)gridDim.x * blockDim.x) {
    const vec4 v = g4[i];
    look(v.x); look(v.y); look(v.z); look(v.w);
  }
  for (long long i = 4 * n4 + (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
    look(g[i]);
  bad = wave_sum_u(bad);
  nz = wave_sum_u(nz);
  __shared__ unsigned int s_bad[4], s_nz[4];
  if ((threadIdx.x & 63) == 0) { s_bad[threadIdx.x >> 6] = bad; s_nz[threadIdx.x >> 6] = nz; }
  __syncthreads();
  if (threadIdx.x == 0) {
    bad = s_bad[0] + s_bad[1] + s_bad[2] + s_bad[3];
    nz = s_nz[0] + s_nz[1] + s_nz[2] + s_nz[3];
    if (bad) atomicAdd(&counts[0], bad);
    if (nz) counts[1] = 1u;
  }
}

// What the upstream check decides (TGV.cu:2698-2703), kept on the device: an upstream gradient with a non-finite entry,
// or zero everywhere, is scrubbed in the caller's tensor; the verdict is latched in the guard's state, where the
// guard's decision and the kernels that store the outputs read it (zeros out, running means and run count untouched).
// The host never learns it and never waits for it.
__global__ __launch_bounds__(256) void tgv_upstream_verdict(float* __restrict__ g, long long n,
                                                            const unsigned int* __restrict__ counts,
                                                            GuardState* __restrict__ gs) {
  const bool bad = counts[0] != 0u || counts[1] == 0u;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    gs->upstream_bad = bad ? 1u : 0u;
    if (bad) gs->skipped += 1u;
  }
  if (!bad) return;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    const float v = g[i];
    if (!finite_value(v)) g[i] = 0.f;
  }
}

// The guard on the gradient wrt the starting point inspects only the u block (TGV.cu:3014-3021):
// gather the u blocks of all samples into one contiguous tensor ...
__global__ __launch_bounds__(256) void tgv_gather_u(const float* __restrict__ src, float* __restrict__ dst,
                                                    long long CHW) {
  // grid (blocks, n): blockIdx.y is the sample
  const float* __restrict__ sp = src + (long long)blockIdx.y * 3 * CHW;
  float* __restrict__ dp = dst + (long long)blockIdx.y * CHW;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < CHW; i += (long long)gridDim.x * blockDim.x)
    dp[i] = sp[i];
}
// ... and apply its verdict to the u blocks only; v1 / v2 gradients pass through (TGV.cu:3047).
__global__ __launch_bounds__(256) void tgv_finalize_init(const float* __restrict__ src, float* __restrict__ out,
                                                         long long CHW, const GuardState* __restrict__ gs, GuardParams p) {
  // grid (blocks, n, 3): blockIdx.y is the sample, blockIdx.z the variable (0 = u)
  const long long base = ((long long)blockIdx.y * 3 + blockIdx.z) * CHW;
  const float* __restrict__ sp = src + base;
  float* __restrict__ op = out + base;
  const bool is_u = blockIdx.z == 0;
  if (gs->upstream_bad) {  // a refused upstream gradient: zeros (TGV.cu:2698-2703)
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < CHW; i += (long long)gridDim.x * blockDim.x) op[i] = 0.f;
    return;
  }
  const double mult = gs->scale[4];
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < CHW; i += (long long)gridDim.x * blockDim.x) {
    float v = sp[i];
    if (is_u) {
      v = guard_limit(v, p);
      if (mult != 1.0) v = (mult == 0.0) ? 0.f : (float)((double)v * mult);
    }
    op[i] = v;
  }
}

// -------------------------------------------------------------------------------------------------
// per-id state (idStructBs, TGVInpaintFista.h:7-50)
// -------------------------------------------------------------------------------------------------
struct Slot {
  // backward passes so far, INCLUDING those whose upstream gradient was refused: the device counts those in
  // GuardState::skipped, and the reference's `run` is the difference (run_count())
  int run = 0;
  int n = 0, ic = 0, ih = 0, iw = 0, its = -1;
  bool forward_done = false;
  // Which x05 rows the forward pass keeps for the backward pass (tgvinpaint_keep_iterates): 0 none (every segment is
  // recomputed from its checkpoint, the reference's order of work), 1 those of the last segment, 2 all of them (no
  // recompute at all; the ring then has one row per iteration).
  int keep_mode = 2;
  // Which half of a checkpoint behind the first the last forward stored: -1 both; 0 only y (what the reference's backward
  // reads at a segment start); 1 only x (what the corrected gradient reads).  A forward that keeps every x05 row stores
  // the half its id's gradient mode needs, since no segment is ever recomputed from the checkpoint.
  int ckpt_half = -1;
  int fwd_grad_mode = 0;  // the mode the last forward pass ran under: its backward passes must ask for the same one
  int grad_mode = 0;    // 0: the reference's backward, bit for bit; 1: the corrected gradient (tgvinpaint_gradient_mode)
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
  // S3 = n*3*ic*ih*iw floats (state), F = n*ic*ih*iw, P = n*ih*iw
  float *wx = nullptr, *wy = nullptr, *bx = nullptr, *by = nullptr;  // L-scaled weights, P each
  double* Ls = nullptr;                                              // per-sample L
  unsigned int* maxbits = nullptr;                                   // per-sample Lipschitz bound (float bits)
  unsigned int* counts = nullptr;                                    // upstream check
  float *ypp[2] = {nullptr, nullptr}, *xpp[2] = {nullptr, nullptr}, *ckpt_y = nullptr, *ckpt_x = nullptr, *x05 = nullptr;
  float *g05[2] = {nullptr, nullptr}, *gxk[2] = {nullptr, nullptr}, *gi_u = nullptr, *gx_final = nullptr;
  // per-segment fp32 accumulators, double-buffered: a strip-kernel step reads one set and writes the other
  float *acc_gc[2] = {nullptr, nullptr}, *acc_gx[2] = {nullptr, nullptr}, *acc_gy[2] = {nullptr, nullptr},
        *acc_gb[2] = {nullptr, nullptr};
  int acc_cur = 0;   // set of the shared accumulators (gc, gx, gy) the next adjoint launch reads
  int accb_cur = 0;  // set of the per-channel accumulator (gb) the next adjoint step reads
  double *tot_gc = nullptr, *tot_gx = nullptr, *tot_gy = nullptr, *tot_gb = nullptr;
  // strip path: one fp32 record per segment and tensor, added into the totals after the last segment
  float *seg_gc = nullptr, *seg_gx = nullptr, *seg_gy = nullptr, *seg_gb = nullptr;
  float* zeros = nullptr;  // a field of zeros (as large as the largest accumulator), never written after the slot is made: the accumulators a segment's first pair starts from
  bool acc_fresh = false;  // the next pair launch starts a segment: its accumulators are zero, read from `zeros` (the pair that ended the segment before wrote none)
  int seg_cur = 0;  // segment the backward pass is in
  GuardState* guard = nullptr;
  double pending_av[5] = {0, 0, 0, 0, 0};
};

Slot g_slots[kUniqueIds];
Allocator g_allocator;  // tgvinpaint_set_allocator
KernelTimer g_timer;

size_t state_count(const Slot& s) { return (size_t)s.n * 3 * s.ic * s.ih * s.iw; }
size_t field_count(const Slot& s) { return (size_t)s.n * s.ic * s.ih * s.iw; }
size_t plane_count(const Slot& s) { return (size_t)s.n * s.ih * s.iw; }

// Reads the guard's running means back (waits for the id's stream); `skipped` = the backward passes the device refused.
int fetch_running_means(Slot& s, unsigned int* skipped = nullptr) {
  if (skipped) *skipped = 0;
  if (s.guard) {
    GuardState host;
    INPAINT_HIP(hipStreamSynchronize(s.stream));
    INPAINT_HIP(hipMemcpy(&host, s.guard, kGuardHeaderBytes, hipMemcpyDeviceToHost));
    for (int k = 0; k < 5; k++) s.pending_av[k] = host.av[k];
    if (skipped) *skipped = host.skipped;
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
  unsigned int skipped = 0;
  int rc = fetch_running_means(s, &skipped);
  if (rc) return rc;
  s.run -= (int)skipped;  // the new guard state starts counting refused passes from zero
  s.guard = nullptr;  // the arena is about to be released; the means live in pending_av until the new one exists
  s.n = n; s.ic = ic; s.ih = ih; s.iw = iw; s.its = its;
  make_schedule(its, s.iterations, s.max_inter_its);
  make_step_sizes(its, s.steps);
  const size_t S3 = state_count(s), F = field_count(s), P = plane_count(s);
  s.ring_rows = ring_rows;
  const size_t nck = std::max<size_t>(s.iterations.size(), 1), ring = (size_t)ring_rows;
  size_t need = 0;
  need += Arena::padded(S3, 4) * (2 + 2 + 2 + 2 + 1) + Arena::padded(S3 * nck, 4) * 2 + Arena::padded(S3 * ring, 4);
  need += Arena::padded(F, 4) * 3 + Arena::padded(F, 8);
  need += Arena::padded(P, 4) * (4 + 2) + Arena::padded(2 * P, 4) * 4;
  need += Arena::padded(P, 8) + Arena::padded(2 * P, 8) * 2;
  need += Arena::padded(P * nck, 4) + Arena::padded(2 * P * nck, 4) * 2 + Arena::padded(F * nck, 4);
  need += Arena::padded((size_t)n, 8) + Arena::padded((size_t)n, 4) + Arena::padded(2, 4);
  need += Arena::padded(std::max(F, 2 * P), 4);  // the field of zeros
  need += Arena::padded(1, sizeof(GuardState));
  rc = s.arena.reserve(need, g_allocator, stream);
  if (rc) return rc;
  Arena& a = s.arena;
  s.wx = a.take<float>(P); s.wy = a.take<float>(P); s.bx = a.take<float>(P); s.by = a.take<float>(P);
  s.Ls = a.take<double>((size_t)n);
  s.maxbits = a.take<unsigned int>((size_t)n);
  s.counts = a.take<unsigned int>(2);
  s.ypp[0] = a.take<float>(S3); s.ypp[1] = a.take<float>(S3);
  s.xpp[0] = a.take<float>(S3); s.xpp[1] = a.take<float>(S3);
  s.ckpt_y = a.take<float>(S3 * nck); s.ckpt_x = a.take<float>(S3 * nck);
  s.x05 = a.take<float>(S3 * ring);
  s.g05[0] = a.take<float>(S3); s.g05[1] = a.take<float>(S3);
  s.gxk[0] = a.take<float>(S3); s.gxk[1] = a.take<float>(S3);
  s.gx_final = a.take<float>(S3);
  s.gi_u = a.take<float>(F);
  for (int i = 0; i < 2; i++) {
    s.acc_gb[i] = a.take<float>(F);
    s.acc_gc[i] = a.take<float>(P); s.acc_gx[i] = a.take<float>(2 * P); s.acc_gy[i] = a.take<float>(2 * P);
  }
  s.tot_gc = a.take<double>(P); s.tot_gx = a.take<double>(2 * P); s.tot_gy = a.take<double>(2 * P);
  s.tot_gb = a.take<double>(F);
  s.seg_gc = a.take<float>(P * nck); s.seg_gx = a.take<float>(2 * P * nck); s.seg_gy = a.take<float>(2 * P * nck);
  s.seg_gb = a.take<float>(F * nck);
  s.zeros = a.take<float>(std::max(F, 2 * P));
  s.guard = a.take<GuardState>(1);
  if (!s.guard) return fail(INPAINT_ERR_HIP, "arena layout overflow");
  hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)std::max(F, 2 * P))), dim3(256), 0, stream, s.zeros, (long long)std::max(F, 2 * P));
  GuardState init;
  memset(&init, 0, sizeof(init));
  for (int k = 0; k < 5; k++) { init.av[k] = s.pending_av[k]; init.scale[k] = 1.0; }
  INPAINT_HIP(hipMemcpyAsync(s.guard, &init, sizeof(init), hipMemcpyHostToDevice, stream));
  INPAINT_HIP(hipStreamSynchronize(stream));
  return 0;
}

// The x05 rows the forward pass keeps.  INPAINT_KEEP=0|1|2 overrides the id's setting (INPAINT_KEEP_LAST=0 is the
// older spelling of INPAINT_KEEP=0); keeping all rows needs its * state bytes, at most INPAINT_KEEP_GB (default 32).
int resolve_keep_mode(const Slot& s, int n, int ic, int ih, int iw, int its) {
  int mode = knobs().keep >= 0 ? knobs().keep : s.keep_mode;
  if (mode == 2) {
    const double bytes = 4.0 * 3 * n * ic * (double)ih * iw * its;
    if (bytes > knobs().keep_gb * 1073741824.0) mode = 1;
  }
  return mode;
}

int check_common(const void* const* ptrs, int nptrs, int n, int ic, int ih, int iw, int its, int id) {
  if (id < 0 || id >= kUniqueIds)
    return fail(INPAINT_ERR_ID, "Cannot use an id that is negative or larger/equal than the maximal one: %d/%d", id,
                kUniqueIds);
  for (int i = 0; i < nptrs; i++)
    if (!ptrs[i]) return fail(INPAINT_ERR_ARG, "null pointer argument (position %d)", i);
  if (n < 1 || ic < 1 || ih < 1 || iw < 1 || its < 0)
    return fail(INPAINT_ERR_ARG, "bad sizes n=%d ic=%d ih=%d iw=%d its=%d", n, ic, ih, iw, its);
  if (n > 65535 || (ih + BY - 1) / BY > 65535)  // (the Lipschitz and iteration-0 kernels put rows / BY and n on the grid)
    return fail(INPAINT_ERR_ARG, "n=%d or ih=%d exceed the launch grid", n, ih);
  if ((long long)ih * iw >= (1ll << 29))  // the strip kernels address two planes of a tensor with one 32-bit byte offset
    return fail(INPAINT_ERR_ARG, "ih*iw = %lld pixels per plane exceed 2^29", (long long)ih * iw);
  if ((int)std::floor(std::sqrt((double)its)) > kMaxCheckpoints)
    return fail(INPAINT_ERR_ITS, "its=%d needs more than %d checkpoints", its, kMaxCheckpoints);
  return 0;
}

// Lipschitz reduction + scaled weight copies for the weights of this call (forward and backward both
// redo it, TGV.cu:2513-2531 and 2667-2679).
void scale_weights(const Slot& s, hipStream_t stream, const float* dx, const float* dy, bool clear_counts = false) {
  const long long P = (long long)plane_count(s), HW = (long long)s.ih * s.iw;
  hipLaunchKernelGGL(tgv_lipschitz_init, dim3((s.n + 255) / 256), dim3(256), 0, stream, s.maxbits, s.n,
                     clear_counts ? s.counts : nullptr);
  hipLaunchKernelGGL(tgv_lipschitz_kernel, dim3((s.iw + BX - 1) / BX, (s.ih + BY - 1) / BY, s.n), dim3(BX, BY), 0, stream,
                     dx, dy, s.ih, s.iw, s.maxbits);
  hipLaunchKernelGGL(tgv_scale_kernel, dim3(grid1d(P)), dim3(256), 0, stream, dx, dy, s.maxbits, s.wx, s.wy, s.bx, s.by,
                     s.Ls, HW, P);
}

// -------------------------------------------------------------------------------------------------
// kernel selection: the wave-strip kernels.  INPAINT_TGV_PATH=px used to select the one-pixel-per-thread kernels
// written first; they are no longer built, and the setting is refused.
// -------------------------------------------------------------------------------------------------
int refuse_removed_path() {
  if (knobs().tgv_px_path)
    return fail(INPAINT_ERR_ARG, "INPAINT_TGV_PATH=px names the per-pixel kernels, which this library no longer contains; unset it (INPAINT_TGV_FUSE=0 selects the one-iteration strip kernels)");
  return 0;
}

// Channel groups: the strip kernels are instantiated for one and two flow channels.  More channels run as consecutive
// launches over groups of two, each getting the per-channel tensors already moved to its first channel and the
// tensor's channel count as the plane stride.  Forward channels never couple; the adjoint couples them through the
// five shared accumulators (gc and the two channels of gwx, gwy) only, summed in channel order step by step, which
// one-step launches issued group after group reproduce exactly.
constexpr int kGroup = 2;
inline const float* at_channel(const Slot& s, const float* p, int ch0) { return p ? p + (size_t)ch0 * s.ih * s.iw : nullptr; }
inline float* at_channel(const Slot& s, float* p, int ch0) { return p ? p + (size_t)ch0 * s.ih * s.iw : nullptr; }
int strip_rows(int n, int ih, int iw, int cols, int forced_rows, int lag) {
  // Rows per wavefront: taller strips amortise the start-up latency and the one-row overlap between
  // strips, but the launch should still keep every SIMD of the chip busy.
  if (forced_rows > 0) return forced_rows;
  const long long sx = (iw + cols - 1) / cols;
  return choose_strip_rows(sx * n, ih, 4, lag);
}

// Rows per strip of the two-wavefront pair kernel.  Its workgroups (one strip each) are resident four per CU, so a
// launch runs in ceil(workgroups / (4 * CUs)) rounds of (R + 3 pipeline rows + start-up) row steps each; the
// strip height that minimises rounds x steps is taken (on 4 x 384 x 1248: 32 rows, 1008 workgroups, one round).
int pair_split_rows(int n, int ih, int iw) {
  if (knobs().tgv_adj_rows > 0) return knobs().tgv_adj_rows;
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
              ? prop.multiProcessorCount
              : 256;
  }
  const long long cap = 4ll * cus;
  const long long sx = (iw + tgvstrip::kCols2 - 1) / tgvstrip::kCols2;
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

template <int C>
void launch_forward_strip(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xin,
                          float* xout, const float* yin, float* yout, float* x05, float t) {
  auto kern = x05 ? tgvstrip::tgv_forward_strip<C, true> : tgvstrip::tgv_forward_strip<C, false>;
  const int R = strip_rows(s.n, s.ih, s.iw, tgvstrip::kCols, knobs().tgv_fwd_rows, 6);
  const int sx = (s.iw + tgvstrip::kCols - 1) / tgvstrip::kCols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);  // a multiple of 8: one share per XCD
  hipLaunchKernelGGL(kern, grid, block, 0, stream, s.wx, s.wy, s.bx, s.by, c, b, xin, xout, yin, yout, x05, s.n, s.ih, s.iw, t,
                     R, sx, sy, s.ic);
}

void launch_forward(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xin, float* xout,
                    const float* yin, float* yout, float* x05, float t) {
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    const float *gb = at_channel(s, b, ch0), *gxi = at_channel(s, xin, ch0), *gyi = at_channel(s, yin, ch0);
    float *gxo = at_channel(s, xout, ch0), *gyo = at_channel(s, yout, ch0), *gh = at_channel(s, x05, ch0);
    if (s.ic - ch0 == 1) launch_forward_strip<1>(s, stream, c, gb, gxi, gxo, gyi, gyo, gh, t);
    else launch_forward_strip<2>(s, stream, c, gb, gxi, gxo, gyi, gyo, gh, t);
  }
}

// Two forward iterations in one launch (strip path): (xin, yin) = iterate k, (xout, yout) = iterate k+2;
// x05a / x05b receive the x05 rows of iterations k and k+1 when given.
template <int C>
void launch_forward_pair_strip(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xin,
                               const float* xin_aux, float* xout, const float* yin, float* yout, float* x05a, float* x05b,
                               bool store_x_aux, float tA, float tB, bool ring, float tP, int groups = 1,
                               float* keep_x = nullptr, float* keep_y = nullptr) {
  auto kern = tgvstrip::tgv_forward_strip2<C, false>;
  if (x05a && ring) kern = (xout || yout) ? tgvstrip::tgv_forward_strip2<C, true, true> : tgvstrip::tgv_forward_strip2<C, true, true, false>;
  else if (x05a) kern = tgvstrip::tgv_forward_strip2<C, true>;
  const int R = strip_rows(s.n * groups, s.ih, s.iw, tgvstrip::kCols2, knobs().tgv_fwd_rows, 8);
  const int sx = (s.iw + tgvstrip::kCols2 - 1) / tgvstrip::kCols2, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n * groups;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, s.wx, s.wy, s.bx, s.by, c, b, xin, xin_aux, xout, yin, yout, x05a, x05b,
                     store_x_aux ? 1 : 0, s.n, s.ih, s.iw, tA, tB, (x05a && ring) ? tP : 0.f, R, sx, sy, s.ic, groups, keep_x, keep_y);
}

// One channel per wavefront, all channels in one launch (the C = 1 instantiation with the channel as a grid dimension;
// forward channels never couple).  Unlike the TV layer this pays at every size: a wavefront with one channel needs 124
// registers instead of 198, so four wavefronts share a SIMD instead of two, which hides more of the kernel's latency
// than the repeated per-pixel work (c, the four weights, masks) costs: 4 x C x 384 x 1248, 100 iterations, forward pass:
// C = 2 3.38 -> 3.33 ms, C = 4 6.93 -> 6.47 ms; 2 x 2 x 224 x 512, 50 iterations: 0.43 -> 0.32 ms.
bool forward_split_channels(const Slot& s) {
  if (s.ic < 2) return false;
  if (knobs().tgv_fwd_split >= 0) return knobs().tgv_fwd_split == 1;
  return true;
}

bool forward_pairs(const Slot& s) {
  return knobs().tgv_fuse;
}

// xin_aux (optional): where v1, v2 of the input iterate are read from instead of xin; store_x_aux: write v1, v2 of xout.
// ring: xin / yin are the x05 rows of the two iterations before this pair and the iterate is rebuilt from them (tP:
// extrapolation factor of the iteration that made it); such a launch writes x05 rows only.
void launch_forward_pair(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xin, float* xout,
                         const float* yin, float* yout, float* x05a, float* x05b, float tA, float tB,
                         const float* xin_aux = nullptr, bool store_x_aux = true, bool ring = false, float tP = 0.f,
                         float* keep_x = nullptr, float* keep_y = nullptr) {
  // keep_x / keep_y: where the launch leaves a copy of its input iterate (checkpoint 0 = the starting point)
  if (forward_split_channels(s)) {
    launch_forward_pair_strip<1>(s, stream, c, b, xin, xin_aux, xout, yin, yout, x05a, x05b, store_x_aux, tA, tB, ring, tP, s.ic,
                                 keep_x, keep_y);
    return;
  }
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    const float *gb = at_channel(s, b, ch0), *gxi = at_channel(s, xin, ch0), *gxa = at_channel(s, xin_aux, ch0), *gyi = at_channel(s, yin, ch0);
    float *gxo = at_channel(s, xout, ch0), *gyo = at_channel(s, yout, ch0), *ga = at_channel(s, x05a, ch0), *gbb = at_channel(s, x05b, ch0);
    float *kx = at_channel(s, keep_x, ch0), *ky = at_channel(s, keep_y, ch0);
    if (s.ic - ch0 == 1)
      launch_forward_pair_strip<1>(s, stream, c, gb, gxi, gxa, gxo, gyi, gyo, ga, gbb, store_x_aux, tA, tB, ring, tP, 1, kx, ky);
    else
      launch_forward_pair_strip<2>(s, stream, c, gb, gxi, gxa, gxo, gyi, gyo, ga, gbb, store_x_aux, tA, tB, ring, tP, 1, kx, ky);
  }
}

// One group of a one-step adjoint launch.  Shared accumulators: set acc_cur in, the other out, flipped by the caller
// after every launch; the per-channel accumulator gb: set accb_cur in, the other out, flipped once per step.
template <int C, bool END, int ADJ, bool FIRST = false>
void launch_adjoint_strip(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xa,
                          const float* xb, const float* yck, const float* g05_in, float* g05_out, const float* gxk,
                          float* gxk_m1, float* gx_final, float t, int ch0, const float* x05_last = nullptr) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  auto kern = (gx_final && !FIRST) ? tgvstrip::tgv_adjoint_strip<C, END, !FIRST, ADJ, FIRST>
                                   : tgvstrip::tgv_adjoint_strip<C, END, false, ADJ, FIRST>;
  const int R = strip_rows(s.n, s.ih, s.iw, tgvstrip::kCols, knobs().tgv_adj_rows, 6);
  const int sx = (s.iw + tgvstrip::kCols - 1) / tgvstrip::kCols, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);
  hipLaunchKernelGGL(kern, grid, block, 0, stream, s.wx, s.wy, s.bx, s.by, c, at_channel(s, b, ch0), at_channel(s, xa, ch0),
                     at_channel(s, xb, ch0), at_channel(s, yck, ch0), s.acc_gc[i], s.acc_gc[o],
                     at_channel(s, (const float*)s.acc_gb[ib], ch0), at_channel(s, s.acc_gb[ob], ch0), s.acc_gx[i], s.acc_gx[o],
                     s.acc_gy[i], s.acc_gy[o], at_channel(s, g05_in, ch0), at_channel(s, g05_out, ch0), at_channel(s, gxk, ch0),
                     at_channel(s, gxk_m1, ch0), at_channel(s, gx_final, ch0), s.n, s.ih, s.iw, t, R, sx, sy, s.ic,
                     at_channel(s, x05_last, ch0));
}

// The first two steps of the reverse sweep in one launch (strip path, at most kGroup channels, the second step not a
// segment's first iteration): step j = len - 2 as launch_adjoint runs it, with the sweep's first step (the upstream
// gradient `gin` through the prox at the last x05 row) done on the way in.  The accumulators start at zero in set
// acc_cur; the launch writes the other set, then the sets flip as after any step.
template <int ADJ>
void launch_adjoint_first_two(Slot& s, hipStream_t stream, const float* c, const float* b, const float* x05_last,
                              const float* xa, const float* xb, const float* gin, float* g05_out, const float* gxk,
                              float* gxk_m1, float t) {
  if (s.ic == 1) launch_adjoint_strip<1, false, ADJ, true>(s, stream, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, x05_last);
  else launch_adjoint_strip<2, false, ADJ, true>(s, stream, c, b, xa, xb, nullptr, gin, g05_out, gxk, gxk_m1, nullptr, t, 0, x05_last);
  s.acc_cur = 1 - s.acc_cur;
  s.accb_cur = 1 - s.accb_cur;
}

// One adjoint step: y is rebuilt inside the kernel from xa = x05[k], xb = x05[k-1] (END: read from the checkpoint yck);
// accumulator set acc_cur is read, the other one written, then acc_cur flips; g_x is stored (to gx_final) only when
// asked.  ADJ > 0: the corrected gradient; ADJ == 2: xb is the checkpointed x.
template <bool END, int ADJ = 0>
void launch_adjoint(Slot& s, hipStream_t stream, const float* c, const float* b, const float* xa, const float* xb,
                    const float* yck, const float* g05_in, float* g05_out, float* gxk, float* gxk_m1, float* gx_final,
                    float t) {
  for (int ch0 = 0; ch0 < s.ic; ch0 += kGroup) {
    if (s.ic - ch0 == 1) launch_adjoint_strip<1, END, ADJ>(s, stream, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0);
    else launch_adjoint_strip<2, END, ADJ>(s, stream, c, b, xa, xb, yck, g05_in, g05_out, gxk, gxk_m1, gx_final, t, ch0);
    s.acc_cur = 1 - s.acc_cur;
  }
  s.accb_cur = 1 - s.accb_cur;
}

// Two adjoint steps in one launch (strip path): A = local iteration j (x05 slots xa = j, xb = j-1), B = j-1
// (xc = slot j-2, or the checkpoint y when B is the segment's first iteration).
// Whether the pair kernel runs its two steps in two wavefronts (the default with two channels).
bool pair_split(int channels) { return knobs().tgv_pair_waves ? knobs().tgv_pair_waves == 2 : channels >= 2; }

// TRUE_ADJ (the corrected gradient) exists for the two-wavefront kernel only; the caller checks pair_split().
template <int C, bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_strip(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xa,
                               const float* xb, const float* xc, const float* g05_in, float* g05_out, const float* gxk,
                               float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  // two channels: the two steps run in two wavefronts of a workgroup (one strip per 128-thread workgroup);
  // one channel: both steps fit one wavefront's registers (four strips per 256-thread workgroup)
  const bool split = pair_split(C);
  auto kern1 = gx_final ? tgvstrip::tgv_adjoint_strip2<C, BEND, true> : tgvstrip::tgv_adjoint_strip2<C, BEND, false>;
  const int R = split ? pair_split_rows(s.n, s.ih, s.iw)
                      : strip_rows(s.n, s.ih, s.iw, tgvstrip::kCols2, knobs().tgv_adj_rows, 8);
  const int sx = (s.iw + tgvstrip::kCols2 - 1) / tgvstrip::kCols2, sy = (s.ih + R - 1) / R;
  const long long waves = (long long)sx * sy * s.n;
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
#define TGV_PAIR_ARGS                                                                                                      \
  s.wx, s.wy, s.bx, s.by, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib], s.acc_gb[ob], zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], \
      zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final, s.seg_gc + sP, s.seg_gb + sF, s.seg_gx + 2 * sP, s.seg_gy + 2 * sP, s.n, s.ih,  \
      s.iw, tA, tB, R, sx, sy, s.ic
  if (split) {
    const dim3 grid((unsigned)((waves + 7) / 8 * 8)), block(128);
    if (gx_final) hipLaunchKernelGGL((tgvstrip::tgv_adjoint_strip2w<C, BEND, true, TRUE_ADJ>), grid, block, 0, stream, TGV_PAIR_ARGS);
    else hipLaunchKernelGGL((tgvstrip::tgv_adjoint_strip2w<C, BEND, false, TRUE_ADJ>), grid, block, 0, stream, TGV_PAIR_ARGS);
  } else {
    const dim3 grid((unsigned)(((waves + 3) / 4 + 7) / 8 * 8)), block(256);
    hipLaunchKernelGGL(kern1, grid, block, 0, stream, TGV_PAIR_ARGS);
  }
#undef TGV_PAIR_ARGS
}

// Rows per strip of the four-wavefront pair kernel (three and four channels).  Its 256-thread workgroups (one strip
// each) are resident two per CU; a strip of R rows takes R + 3 pipeline rows, two intervals of two rows behind and the
// start-up.
int pair_quad_rows(int n, int ih, int iw) {
  if (knobs().tgv_adj_rows > 0) return knobs().tgv_adj_rows;
  const long long cap = 2ll * compute_unit_count();
  const long long sx = (iw + tgvstrip::kCols2 - 1) / tgvstrip::kCols2;
  int best = 16;
  long long best_cost = -1;
  for (int R = 8; R <= 96; R++) {
    const long long wg = sx * ((ih + R - 1) / R) * n;
    const long long cost = ((wg + cap - 1) / cap) * (R + 11);
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = R;
    }
  }
  return best;
}

// 3 and 4 channels: two channel groups, step A and step B of each in a wavefront of its own
template <int CM, int C1, bool BEND, bool TRUE_ADJ>
void launch_adjoint_pair_quad(const Slot& s, hipStream_t stream, const float* c, const float* b, const float* xa,
                              const float* xb, const float* xc, const float* g05_in, float* g05_out, const float* gxk,
                              float* gxk_m1, float* gx_final, float tA, float tB) {
  const int i = s.acc_cur, o = 1 - s.acc_cur, ib = s.accb_cur, ob = 1 - s.accb_cur;
  auto kern = gx_final ? tgvstrip::tgv_adjoint_strip4w<CM, C1, BEND, true, TRUE_ADJ> : tgvstrip::tgv_adjoint_strip4w<CM, C1, BEND, false, TRUE_ADJ>;
  const int R = pair_quad_rows(s.n, s.ih, s.iw);
  const int sx = (s.iw + tgvstrip::kCols2 - 1) / tgvstrip::kCols2, sy = (s.ih + R - 1) / R;
  const long long strips = (long long)sx * sy * s.n;
  const size_t sP = (size_t)s.seg_cur * plane_count(s), sF = (size_t)s.seg_cur * field_count(s);  // this segment's records
  const dim3 grid((unsigned)((strips + 7) / 8 * 8)), block(256);
  const bool zf = s.acc_fresh;  // first pair of a segment: zero accumulators, read from the field of zeros
  hipLaunchKernelGGL(kern, grid, block, 0, stream, s.wx, s.wy, s.bx, s.by, c, b, xa, xb, xc, zf ? s.zeros : s.acc_gc[i], s.acc_gc[o], zf ? s.zeros : s.acc_gb[ib],
                     s.acc_gb[ob], zf ? s.zeros : s.acc_gx[i], s.acc_gx[o], zf ? s.zeros : s.acc_gy[i], s.acc_gy[o], g05_in, g05_out, gxk, gxk_m1, gx_final,
                     s.seg_gc + sP, s.seg_gb + sF, s.seg_gx + 2 * sP, s.seg_gy + 2 * sP, s.n, s.ih, s.iw, tA, tB, R, sx, sy, s.ic);
}

constexpr int kPairChannels = 4;  // the most channels a pair launch holds (two groups of two)

template <bool BEND, bool TRUE_ADJ = false>
void launch_adjoint_pair(Slot& s, hipStream_t stream, const float* c, const float* b, const float* xa, const float* xb,
                         const float* xc, const float* g05_in, float* g05_out, const float* gxk, float* gxk_m1,
                         float* gx_final, float tA, float tB) {
  if (s.ic == 1) launch_adjoint_pair_strip<1, BEND, TRUE_ADJ>(s, stream, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 3) launch_adjoint_pair_quad<2, 1, BEND, TRUE_ADJ>(s, stream, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else if (s.ic == 4) launch_adjoint_pair_quad<2, 2, BEND, TRUE_ADJ>(s, stream, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  else launch_adjoint_pair_strip<2, BEND, TRUE_ADJ>(s, stream, c, b, xa, xb, xc, g05_in, g05_out, gxk, gxk_m1, gx_final, tA, tB);
  s.acc_cur = 1 - s.acc_cur;
  s.accb_cur = 1 - s.accb_cur;
}

bool adjoint_pairs(const Slot& s) {
  if (!knobs().tgv_fuse_adj) return false;
  // a pair adds step A's and step B's terms of its channels back to back, which is the reference's order of summation
  // only when the launch holds every channel: one or two wavefronts for 1 or 2 channels, four (two channel groups) for
  // 3 or 4; more channels take the one-step kernel, group after group
  return forward_pairs(s) && s.ic <= kPairChannels;
}

}  // namespace

extern "C" {

int tgvinpaint_forward(const float* dx, const float* dy, const float* c, const float* b, const float* init,
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
      rows_exceed_free_memory(4.0 * 3 * n * ic * (double)ih * iw * its))
    keep = 1;  // (the slot would have to grow by more than a quarter of the free device memory)
  rc = prepare_slot(s, n, ic, ih, iw, its, keep, stream);
  if (rc && keep == 2) {  // no room for every x05 row: keep the last segment's instead and recompute the others
    (void)hipGetLastError();
    keep = 1;
    rc = prepare_slot(s, n, ic, ih, iw, its, keep, stream);
    if (!rc) std::copy(shape, shape + 5, s.refused);
  }
  if (rc) return rc;
  const size_t S3 = state_count(s), SB = S3 * sizeof(float);
  const int K = 2 * (its / 2);
  auto ck_index = [&](int k) {
    for (size_t i = 0; i < s.iterations.size(); i++)
      if (s.iterations[i] == k) return (int)i;
    return -1;
  };
  auto Ybuf = [&](int k) { int i = ck_index(k); return (i >= 0 && k < K) ? s.ckpt_y + (size_t)i * S3 : s.ypp[k & 1]; };
  auto Xbuf = [&](int k) {
    if (k == K) return out;
    int i = ck_index(k);
    return i >= 0 ? s.ckpt_x + (size_t)i * S3 : s.xpp[k & 1];
  };
  if (K == 0) {
    INPAINT_HIP(hipMemcpyAsync(out, init, SB, hipMemcpyDeviceToDevice, stream));
    if (!s.iterations.empty()) {  // its == 1: the reference leaves calloc'ed (zero) checkpoints
      hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)S3)), dim3(256), 0, stream, s.ckpt_y, (long long)S3);
      hipLaunchKernelGGL(fill_zero_f32, dim3(grid_stride((long long)S3)), dim3(256), 0, stream, s.ckpt_x, (long long)S3);
    }
  } else {
    scale_weights(s, stream, dx, dy);
    // checkpoint 0 = the starting point: the first pair launch reads `init` itself and leaves the two copies as it
    // goes; one-iteration launches (and a caller that iterates in place) get them from a copy kernel
    // a forward that keeps every x05 row never recomputes from a checkpoint: it stores only the half of a checkpoint
    // the backward pass of this id's gradient mode reads at a segment start (y: the reference's; x: the corrected one,
    // which also reads checkpoint 0's y when it back-propagates iteration 0)
    const bool want_x = s.grad_mode == 1, want_y = !want_x;
    s.ckpt_half = (keep == 2 && forward_pairs(s)) ? (want_x ? 1 : 0) : -1;
    const bool copy_in_pair = forward_pairs(s) && out != init;
    if (!copy_in_pair)
      hipLaunchKernelGGL(copy_twice_f32, dim3(grid_stride((long long)S3)), dim3(256), 0, stream, init, s.ckpt_y, s.ckpt_x,
                         (long long)S3);
    // first iteration whose x05 row is kept, and the ring row of iteration k
    const int kl = s.iterations.empty() ? K : (keep == 2 ? 0 : (keep == 1 ? s.iterations.back() : K));
    auto ring_row = [&](int k) { return s.x05 + (size_t)(keep == 2 ? k : k - kl) * S3; };
    if (forward_pairs(s)) {
      // two iterations per launch; K and every checkpoint index are even, the ping-pong alternates per pair
      auto Yp = [&](int k) { int i = ck_index(k); return (i >= 0 && k < K) ? s.ckpt_y + (size_t)i * S3 : s.ypp[(k >> 1) & 1]; };
      auto Xp = [&](int k) {
        if (k == K) return out;
        int i = ck_index(k);
        return i >= 0 ? s.ckpt_x + (size_t)i * S3 : s.xpp[(k >> 1) & 1];
      };
      // kept iterations also store their x05 rows: the backward pass would otherwise recompute exactly these values
      // from the checkpoints (TGV.cu:2775-2814)
      for (int k = 0; k < K; k += 2) {
        float* h0 = k >= kl ? ring_row(k) : nullptr;
        if (keep == 2 && k >= 2) {
          // With every x05 row kept the iterate need not travel through memory either: the pair rebuilds it from the
          // two rows before it, as the recompute launches of the backward pass do, and stores it only where somebody
          // reads it -- at a checkpoint and at the end.
          // At the end that is x alone (the result); at a checkpoint the half the backward pass will read.
          const bool last = k + 2 == K, ck = !last && ck_index(k + 2) >= 0;
          launch_forward_pair(s, stream, c, b, ring_row(k - 2), (last || (ck && want_x)) ? Xp(k + 2) : nullptr, ring_row(k - 1),
                              (ck && want_y) ? Yp(k + 2) : nullptr, h0, h0 + S3, s.steps[k], s.steps[k + 1], nullptr, true, true,
                              s.steps[k - 1]);
        } else if (k == 0 && copy_in_pair) {
          // (with every x05 row kept the next pair rebuilds its input from those rows: the iterate is stored only where
          // somebody reads it)
          const bool last = 2 == K, ck = !last && ck_index(2) >= 0;
          const bool sx = keep != 2 || last || (ck && want_x), sy = keep != 2 || (ck && want_y);
          launch_forward_pair(s, stream, c, b, init, sx ? Xp(2) : nullptr, init, sy ? Yp(2) : nullptr, h0,
                              h0 ? h0 + S3 : nullptr, s.steps[0], s.steps[1], nullptr, true, false, 0.f, (keep != 2 || want_x) ? s.ckpt_x : nullptr, s.ckpt_y);
        }
        else
          launch_forward_pair(s, stream, c, b, Xp(k), Xp(k + 2), Yp(k), Yp(k + 2), h0, h0 ? h0 + S3 : nullptr, s.steps[k],
                              s.steps[k + 1]);
      }
    } else {
      for (int k = 0; k < K; k++)
        launch_forward(s, stream, c, b, Xbuf(k), Xbuf(k + 1), Ybuf(k), Ybuf(k + 1),
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

int tgvinpaint_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin, float* gx,
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
  const size_t S3 = state_count(s), F = field_count(s), P = plane_count(s);
  const int gS = grid_stride((long long)S3), gF = grid_stride((long long)F),
            g2P = grid_stride((long long)(2 * P));

  // (the first of its launches also clears the two words of the upstream check)
  scale_weights(s, stream, dx, dy, true);
  // Upstream check (TGV.cu:2686-2703): any non-finite entry, or an upstream that is zero everywhere, returns
  // all-zero gradients, scrubs the caller's tensor and leaves `run` and the running means alone.  The verdict stays
  // on the device: the sweep below runs either way (on the scrubbed tensor; its kernels address nothing by value),
  // the guard's decision and the kernels that store the outputs read the verdict.  No host wait.
  hipLaunchKernelGGL(tgv_upstream_check, dim3(std::min(grid_stride((long long)S3 / 4 + 1), 2048)), dim3(256), 0, stream, gin, (long long)S3, s.counts);
  hipLaunchKernelGGL(tgv_upstream_verdict, dim3(std::min(gS, 1024)), dim3(256), 0, stream, gin, (long long)S3, s.counts, s.guard);
  // The strip kernels keep one fp32 record of the accumulators per segment; the records are added into the fp64
  // totals after the last segment, in the reference's order (TGV.cu:2944 flushes after every segment: same bits,
  // but the totals are not read and rewritten once per segment).
  SegmentJobs sj;
  {
    float* segs[4] = {s.seg_gc, s.seg_gx, s.seg_gy, s.seg_gb};
    double* tots_[4] = {s.tot_gc, s.tot_gx, s.tot_gy, s.tot_gb};
    const long long ns[4] = {(long long)P, (long long)(2 * P), (long long)(2 * P), (long long)F};
    for (int k = 0; k < 4; k++) {
      sj.acc[k] = nullptr;
      sj.seg[k] = segs[k];
      sj.total[k] = tots_[k];
      sj.n[k] = ns[k];
    }
  }
  // The sweep's first step rides on its second when the last segment has at least four iterations (that second step
  // is then an inner step) and one launch holds every channel.  That launch starts from zero accumulators without
  // reading them, and every launch after it reads only what its predecessor wrote in full: nothing to clear.
  const bool corr_pairs_ok = !corr || pair_split(s.ic);
  const int nseg_all = (int)s.iterations.size();
  const bool first_two = adjoint_pairs(s) && corr_pairs_ok && s.ic <= kGroup && knobs().tgv_fuse_first &&
                         nseg_all > 0 && 2 * ((its - s.iterations[nseg_all - 1]) / 2) >= 4;
  s.acc_cur = 0;
  s.accb_cur = 0;
  if (!first_two) {
    ZeroList z;
    int k = 0;
    for (float* p : {s.g05[0], s.g05[1], s.gxk[0], s.gxk[1], s.gx_final}) { z.ptr[k] = p; z.bytes[k++] = (long long)S3 * 4; }
    z.ptr[k] = s.acc_gb[0]; z.bytes[k++] = (long long)F * 4;
    z.ptr[k] = s.acc_gc[0]; z.bytes[k++] = (long long)P * 4;
    z.ptr[k] = s.acc_gx[0]; z.bytes[k++] = (long long)P * 8;
    z.ptr[k] = s.acc_gy[0]; z.bytes[k++] = (long long)P * 8;
    // (the totals need no clearing: every one of them is written when the segment records are added up)
    hipLaunchKernelGGL(fill_zero_many, dim3(gS, k), dim3(256), 0, stream, z);
  }

  // buffer roles of TGV.cu:2718-2736: g05[0]/g05[1] and gxk[0]/gxk[1] ping-pong with the parity of the
  // local iteration index (the copy of the upstream gradient into gxk[0], TGV.cu:2729, is overwritten
  // before it is read and is not made).
  // The kernels store g_x only at the very last step (into gx_final).
  const float* gi_src = s.gx_final;
  // the corrected gradient has a pair kernel in the two-wavefront form only
  const bool pairs = adjoint_pairs(s) && (!corr || pair_split(s.ic));
  int lastIt = its;
  int pp_src = 1;
  const int nseg = (int)s.iterations.size();
  for (int outer = nseg - 1; outer >= 0; outer--) {
    const int k0 = s.iterations[outer];
    const int len = 2 * ((lastIt - k0) / 2);
    s.seg_cur = outer;
    const float* cky = s.ckpt_y + (size_t)outer * S3;
    const float* ckx = s.ckpt_x + (size_t)outer * S3;
    // recompute the segment, keeping x05 (TGV.cu:2775-2814) -- unless it is the last segment and the forward pass
    // left its x05 rows in the ring
    const bool have_x05 = s.x05_valid && k0 >= s.x05_from;
    // rows of this segment: one per iteration of the whole run when all were kept, else the segment's own ring
    float* const ring = s.x05 + (s.x05_valid && s.x05_mode == 2 ? (size_t)k0 * S3 : 0);
    if (!have_x05 || s.x05_mode != 2) s.x05_valid = false;  // a recomputed (or a shared) ring is overwritten below
    if (have_x05) {
    } else if (forward_pairs(s)) {
      // Only the x05 rows are kept.  The first pair starts from the checkpoint; every later pair rebuilds its input
      // iterate from the two x05 rows before it (the forward pass's own expressions), so no iterate travels
      // through memory.
      for (int j = 0; j < len; j += 2) {  // segments have even length
        if (j == 0)
          launch_forward_pair(s, stream, c, b, ckx, nullptr, cky, nullptr, ring, ring + S3, s.steps[k0], s.steps[k0 + 1]);
        else
          launch_forward_pair(s, stream, c, b, ring + (size_t)(j - 2) * S3, nullptr, ring + (size_t)(j - 1) * S3, nullptr,
                              ring + (size_t)j * S3, ring + (size_t)(j + 1) * S3, s.steps[k0 + j], s.steps[k0 + j + 1],
                              nullptr, false, true, s.steps[k0 + j - 1]);
      }
    } else {
      for (int j = 0; j < len; j++) {
        const float* yin = (j == 0) ? cky : s.ypp[j & 1];
        const float* xin = (j == 0) ? ckx : s.xpp[j & 1];
        launch_forward(s, stream, c, b, xin, s.xpp[(j + 1) & 1], yin, s.ypp[(j + 1) & 1], ring + (size_t)j * S3,
                       s.steps[k0 + j]);
      }
    }
    int timed_run = 0;
    bool flushed = false;  // the pair that ends the segment adds the segment sums to the totals itself
    if (pairs) {  // reverse sweep (TGV.cu:2851-2933), two steps per launch
      // `pp_src` = the g05 / g_x buffer the next launch reads; it flips once per launch
      int j = len - 1;
      if (outer == nseg - 1 && first_two) {
        // the sweep's first step rides on its second
        const float *x_last = ring + (size_t)j * S3, *xa = ring + (size_t)(j - 1) * S3, *xb = ring + (size_t)(j - 2) * S3;
        if (corr) launch_adjoint_first_two<1>(s, stream, c, b, x_last, xa, xb, gin, s.g05[0], s.gxk[1], s.gxk[0], s.steps[k0 + j - 1]);
        else launch_adjoint_first_two<0>(s, stream, c, b, x_last, xa, xb, gin, s.g05[0], s.gxk[1], s.gxk[0], s.steps[k0 + j - 1]);
        pp_src = 0;
        j -= 2;
      } else if (outer == nseg - 1 && j >= 0) {
        if (corr)
          hipLaunchKernelGGL(tgv_adjoint_first<true>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b,
                             ring + (size_t)j * S3, s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic,
                             (long long)ih * iw, (long long)P);
        else
          hipLaunchKernelGGL(tgv_adjoint_first<false>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b,
                             ring + (size_t)j * S3, s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic,
                             (long long)ih * iw, (long long)P);
        pp_src = 1;
        j--;
      }
      if (j >= 0 && ((j + 1) & 1)) {  // an odd number of steps is left: one single step, then pairs
        const float* xa = ring + (size_t)j * S3;
        float *g_in = s.g05[pp_src], *g_out = s.g05[1 - pp_src], *x_in = s.gxk[pp_src], *x_out = s.gxk[1 - pp_src];
        float* gf = outer == 0 ? s.gx_final : nullptr;
        if (j > 0) {
          const float* xb = ring + (size_t)(j - 1) * S3;
          if (corr) launch_adjoint<false, 1>(s, stream, c, b, xa, xb, nullptr, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j]);
          else launch_adjoint<false>(s, stream, c, b, xa, xb, nullptr, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j]);
        } else if (corr) {
          launch_adjoint<false, 2>(s, stream, c, b, xa, ckx, nullptr, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j]);
        } else {
          launch_adjoint<true>(s, stream, c, b, xa, xa, cky, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j]);
        }
        pp_src = 1 - pp_src;
        j--;
      }
      for (; j >= 1; j -= 2) {
        const float* xa = ring + (size_t)j * S3;
        const float* xb = ring + (size_t)(j - 1) * S3;
        float *g_in = s.g05[pp_src], *g_out = s.g05[1 - pp_src], *x_in = s.gxk[pp_src], *x_out = s.gxk[1 - pp_src];
        // A pair that ends a segment stores the segment's sums as a record; it does not write the zeros the next segment
        // starts from (only the sweep's very last launch clears the accumulators): a segment's first pair reads zeros
        // from the slot's field of zeros instead, which stays in the cache.
        s.acc_fresh = outer < nseg - 1 && j == len - 1;
        if (j - 1 > 0) {
          const float* xc = ring + (size_t)(j - 2) * S3;
          if (timed_run == 0) g_timer.begin(stream);
          if (corr) launch_adjoint_pair<false, true>(s, stream, c, b, xa, xb, xc, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j], s.steps[k0 + j - 1]);
          else launch_adjoint_pair<false>(s, stream, c, b, xa, xb, xc, g_in, g_out, x_in, x_out, nullptr, s.steps[k0 + j], s.steps[k0 + j - 1]);
          timed_run++;
          if (j - 2 <= 1) g_timer.end(stream, timed_run);
        } else {
          // B is the segment's first iteration: the checkpoint y (the corrected gradient: the checkpointed x, from
          // which the true y_{k0+1} is rebuilt) stands where x05[j-2] does otherwise
          float* gf = outer == 0 ? s.gx_final : nullptr;
          if (corr) launch_adjoint_pair<true, true>(s, stream, c, b, xa, xb, ckx, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j], s.steps[k0 + j - 1]);
          else launch_adjoint_pair<true>(s, stream, c, b, xa, xb, cky, g_in, g_out, x_in, x_out, gf, s.steps[k0 + j], s.steps[k0 + j - 1]);
          flushed = true;
        }
        pp_src = 1 - pp_src;
      }
      s.acc_fresh = false;
    } else
    for (int j = len - 1; j >= 0; j--) {  // reverse sweep (TGV.cu:2851-2933)
      const float t = s.steps[k0 + j];
      const float* xa = ring + (size_t)j * S3;
      const int odd = j & 1;
      if (outer == nseg - 1 && j == len - 1) {
        if (corr)
          hipLaunchKernelGGL(tgv_adjoint_first<true>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b, xa,
                             s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic, (long long)ih * iw, (long long)P);
        else
          hipLaunchKernelGGL(tgv_adjoint_first<false>, dim3(grid1d((long long)P)), dim3(256), 0, stream, c, b, xa,
                             s.acc_gc[s.acc_cur], s.acc_gb[s.accb_cur], s.g05[1], gin, ic, (long long)ih * iw, (long long)P);
      } else if (j > 0) {
        const float* xb = ring + (size_t)(j - 1) * S3;
        if (timed_run == 0) g_timer.begin(stream);
        if (corr)
          launch_adjoint<false, 1>(s, stream, c, b, xa, xb, nullptr, s.g05[odd ? 0 : 1], s.g05[odd ? 1 : 0],
                                   s.gxk[odd ? 0 : 1], s.gxk[odd ? 1 : 0], nullptr, t);
        else
          launch_adjoint<false>(s, stream, c, b, xa, xb, nullptr, s.g05[odd ? 0 : 1], s.g05[odd ? 1 : 0],
                                s.gxk[odd ? 0 : 1], s.gxk[odd ? 1 : 0], nullptr, t);
        timed_run++;
        if (j == 1) g_timer.end(stream, timed_run);  // one event pair around the sweep's run of launches
      } else if (corr) {
        // corrected gradient: linearise at the true y_{k0+1}, rebuilt from x05[k0] and the checkpointed x_{k0}
        launch_adjoint<false, 2>(s, stream, c, b, xa, ckx, nullptr, s.g05[1], s.g05[0], s.gxk[1], s.gxk[0],
                                 outer == 0 ? s.gx_final : nullptr, t);
      } else {
        // the very last step's g_x is the gradient wrt the starting point (TGV.cu:3047)
        launch_adjoint<true>(s, stream, c, b, xa, xa, cky, s.g05[1], s.g05[0], s.gxk[1], s.gxk[0],
                             outer == 0 ? s.gx_final : nullptr, t);
      }
    }
    // fp32 segment sums into the fp64 totals (TGV.cu:2944)
    if (!flushed) {
      SegmentJobs st = sj;
      const int a = s.acc_cur;
      float* accs[4] = {s.acc_gc[a], s.acc_gx[a], s.acc_gy[a], s.acc_gb[s.accb_cur]};
      for (int k = 0; k < 4; k++) {
        st.acc[k] = accs[k];
        st.seg[k] = sj.seg[k] + (size_t)outer * sj.n[k];
      }
      hipLaunchKernelGGL(segment_store_many, dim3(g2P > gF ? g2P : gF, 4), dim3(256), 0, stream, st);
    }
    lastIt = k0;
  }

  hipLaunchKernelGGL(combine_segments_many, dim3(g2P > gF ? g2P : gF, 4), dim3(256), 0, stream, sj, nseg);
  if (corr && 2 * (its / 2) > 0) {
    // corrected gradient: back-propagate through iteration 0 as well (the reference stops before it).  The last
    // step above left g05[0] and the partial g_x[0] in the halves of the ping-pongs it wrote; checkpoint 0 is y_0; the
    // accumulators are zero after the flush and take iteration 0's weight gradients, which a second flush adds.
    const int a = s.acc_cur;
    const dim3 block(BX, BY), grid((s.iw + BX - 1) / BX, (s.ih + BY - 1) / BY, s.n);
    const int last = pairs ? pp_src : 0;
    hipLaunchKernelGGL(tgv_adjoint_iter0, grid, block, 0, stream, s.wx, s.wy, s.bx, s.by, s.ckpt_y, s.g05[last], s.gxk[last],
                       s.gx_final, s.acc_gx[a], s.acc_gy[a], s.ic, s.ih, s.iw);
    hipLaunchKernelGGL(flush_kernel, dim3(g2P), dim3(256), 0, stream, s.acc_gx[a], s.tot_gx, (long long)(2 * P));
    hipLaunchKernelGGL(flush_kernel, dim3(g2P), dim3(256), 0, stream, s.acc_gy[a], s.tot_gy, (long long)(2 * P));
  }
  // output guard on the device (TGV.cu:2990-3021), then scale and store (TGV.cu:3024-3050)
  hipLaunchKernelGGL(guard_clear_kernel, dim3(1), dim3(64), 0, stream, s.guard);
  {
    const long long CHW = (long long)ic * ih * iw;
    hipLaunchKernelGGL(tgv_gather_u, dim3(std::min(grid_stride(CHW), 1024), n), dim3(256), 0, stream, gi_src, s.gi_u, CHW);
  }
  const double* tots[4] = {s.tot_gc, s.tot_gx, s.tot_gy, s.tot_gb};
  const long long cnts[5] = {(long long)P, (long long)(2 * P), (long long)(2 * P), (long long)F, (long long)F};
  GuardJobs jobs;
  long long longest = 0;
  for (int k = 0; k < 5; k++) {
    jobs.ptr[k] = k < 4 ? (const void*)tots[k] : (const void*)s.gi_u;
    jobs.n[k] = cnts[k];
    jobs.is_f32[k] = k == 4;
    longest = std::max(longest, cnts[k]);
  }
  hipLaunchKernelGGL(guard_reduce_many, dim3(kGuardBlocks, 5), dim3(256), 0, stream, jobs, s.guard, kGuard.max_tolerance, true);
  hipLaunchKernelGGL(guard_tail_decide_many, dim3(guard_grid(longest), 5), dim3(256), 0, stream, jobs, s.guard, s.run, kGuard, true);
  const long long HW2 = 2LL * ih * iw;
  FinalizeJobs fin;
  float* outs[4] = {gc, gx, gy, gb};
  for (int k = 0; k < 4; k++) {
    const bool weights = k == 1 || k == 2;  // gx, gy carry the per-sample weight scaling (TGV.cu:3027-3046)
    fin.total[k] = tots[k];
    fin.out[k] = outs[k];
    fin.n[k] = cnts[k];
    fin.chain_const[k] = weights ? 0.0 : 1.0;
    fin.chain_per_sample[k] = weights ? (const double*)s.Ls : nullptr;
    fin.per_sample[k] = weights ? HW2 : 1;
  }
  hipLaunchKernelGGL(finalize_many, dim3(g2P > gF ? g2P : gF, 4), dim3(256), 0, stream, fin, s.guard, kGuard, corr ? 1.f : kGlobalGMult);
  {
    const long long CHW = (long long)ic * ih * iw;
    hipLaunchKernelGGL(tgv_finalize_init, dim3(std::min(grid_stride(CHW), 1024), n, 3), dim3(256), 0, stream, gi_src, gi, CHW,
                       s.guard, kGuard);
  }
  INPAINT_HIP(hipGetLastError());
  if (knobs().stats_every > 0) {  // TGV.cu:2996: run % 75 == 0, with the run count the reference would hold
    unsigned int skipped = 0;
    INPAINT_HIP(hipStreamSynchronize(stream));
    INPAINT_HIP(hipMemcpy(&skipped, reinterpret_cast<char*>(s.guard) + offsetof(GuardState, skipped), sizeof(skipped), hipMemcpyDeviceToHost));
    if ((s.run - (int)skipped) % knobs().stats_every == 0) {
      rc = print_guard_report(s.guard, stream, id, true);
      if (rc) return rc;
    }
  }
  s.run++;  // TGV.cu:3061 (a refused upstream gradient is counted on the device and taken off again: Slot::run)
  return 0;
}

int tgvinpaint_selftest_guard(const void* values, long long n, int is_f32, int run, double running_mean, float* out,
                            double* result7) {
  return guard_selftest(values, n, is_f32 != 0, run, running_mean, kGuard, true, out, result7);
}

int tgvinpaint_get_state(int id, double* state6) {
  if (id < 0 || id >= kUniqueIds || !state6) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  unsigned int skipped = 0;
  int rc = fetch_running_means(s, &skipped);
  if (rc) return rc;
  state6[0] = s.run - (int)skipped;
  for (int k = 0; k < 5; k++) state6[1 + k] = s.pending_av[k];
  return 0;
}

int tgvinpaint_set_state(int id, const double* state6) {
  if (id < 0 || id >= kUniqueIds || !state6) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  s.run = (int)state6[0];
  for (int k = 0; k < 5; k++) s.pending_av[k] = state6[1 + k];
  if (s.guard) {
    INPAINT_HIP(hipStreamSynchronize(s.stream));
    INPAINT_HIP(hipMemcpy(reinterpret_cast<char*>(s.guard) + offsetof(GuardState, av), s.pending_av, 5 * sizeof(double),
                         hipMemcpyHostToDevice));
    const unsigned int none = 0;
    INPAINT_HIP(hipMemcpy(reinterpret_cast<char*>(s.guard) + offsetof(GuardState, skipped), &none, sizeof(none), hipMemcpyHostToDevice));
  }
  return 0;
}

int tgvinpaint_reset_id(int id) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  reload_knobs();
  Slot& s = g_slots[id];
  if (s.arena.base) (void)hipStreamSynchronize(s.stream);
  int rc = s.arena.release();
  s = Slot();
  return rc;
}

int tgvinpaint_guard_stats(int id, double* stats25) {
  if (id < 0 || id >= kUniqueIds || !stats25) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  if (!s.guard) return fail(INPAINT_ERR_PAIRING, "id %d holds no state", id);
  GuardState host;
  INPAINT_HIP(hipStreamSynchronize(s.stream));
  INPAINT_HIP(hipMemcpy(&host, s.guard, kGuardHeaderBytes, hipMemcpyDeviceToHost));
  memcpy(stats25, host.report, sizeof(host.report));
  return 0;
}

int tgvinpaint_gradient_mode(int id, int mode) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  if (mode < 0 || mode > 1) return fail(INPAINT_ERR_ARG, "gradient mode %d is not 0 or 1", mode);
  g_slots[id].grad_mode = mode;
  return 0;
}

int tgvinpaint_keep_iterates(int id, int mode) {
  if (id < 0 || id >= kUniqueIds) return fail(INPAINT_ERR_ID, "bad id %d", id);
  if (mode < 0 || mode > 2) return fail(INPAINT_ERR_ARG, "keep mode %d is not 0, 1 or 2", mode);
  g_slots[id].keep_mode = mode;
  return 0;
}

int tgvinpaint_set_allocator(inpaint_alloc_fn alloc, inpaint_release_fn release, void* user) {
  if ((alloc == nullptr) != (release == nullptr)) return fail(INPAINT_ERR_ARG, "tgvinpaint_set_allocator: give both callbacks or neither");
  g_allocator.alloc = alloc;
  g_allocator.release = release;
  g_allocator.user = alloc ? user : nullptr;
  return 0;
}

long long tgvinpaint_slot_bytes(int id) {
  if (id < 0 || id >= kUniqueIds) return 0;
  return (long long)g_slots[id].arena.bytes;
}

int tgvinpaint_lipschitz(int id, double* L_host, int n) {
  if (id < 0 || id >= kUniqueIds || !L_host) return fail(INPAINT_ERR_ID, "bad id %d", id);
  Slot& s = g_slots[id];
  if (!s.Ls || n != s.n) return fail(INPAINT_ERR_PAIRING, "id %d holds no state for %d samples", id, n);
  INPAINT_HIP(hipStreamSynchronize(s.stream));
  INPAINT_HIP(hipMemcpy(L_host, s.Ls, sizeof(double) * (size_t)n, hipMemcpyDeviceToHost));
  return 0;
}

int tgvinpaint_guard_decide(int run, double av_gc, double av_running, double* mult_out, double* av_out) {
  double mult = 1.0, av = av_running;
  int action = guard_decide_rule(run, av_gc, av, mult, kGuard);
  if (mult_out) *mult_out = mult;
  if (av_out) *av_out = av;
  return action;
}

int tgvinpaint_profile(int enable) {
  g_timer.enabled = enable != 0;
  g_timer.reset();
  return 0;
}

int tgvinpaint_profile_read(double* total_ms, int* launches) { return g_timer.read(total_ms, launches); }

const char* tgvinpaint_last_error(void) { return error_buffer(); }

}  // extern "C"
