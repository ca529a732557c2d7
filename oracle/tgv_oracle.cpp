// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's Huber-TGV FISTA inpainting layer.
//
// Nothing in the shipped package may import, link or call this file.  It exists so that the
// parity tests, the smoke check and the bench's cpu_baseline leg have something to compare the
// HIP path against.  Every function cites the reference lines it restates (paths relative to the
// reference root; TGV.cu = cudaTGV/cudaCode/TGVInpaintFistaBetas.cu,
// TGVH.cu = cudaTGV/cudaCode/TGVInpaintFistaHelp.cu, TGV.h = cudaTGV/cudaCode/TGVInpaintFista.h).
//
// Arithmetic conventions (the same as the TV restatement):
//   * every floating-point expression is evaluated left to right exactly as written in the
//     reference source, in the type C++ promotion rules give it (a literal such as `1.` or `0.5`
//     makes the surrounding sub-expression double, as it does under nvcc);
//   * no fused multiply-add contraction (build with -ffp-contract=off); division and sqrt are the
//     correctly rounded IEEE ones;
//   * CUDA's rsqrtf (an approximation with a 2 ulp bound whose bits are not recoverable from the
//     sources) is DEFINED here as 1.0f / sqrtf(x), both IEEE: +inf at 0, NaN below 0.  Results
//     agree with a CUDA run only to that bound -- parity unpinned at the ulp level;
//   * `oneL` is passed as 1.0f (TGV.cu:2527,2675), so every product with it is exact; it is kept
//     where the source has it;
//   * texture fetches are point fetches with clamp addressing (only findLipshitz ever leaves the
//     image, TGV.cu:116-122); tensors are (var, channel, h, w) with var in {u, v1, v2}.
//
// Pin status of the functions below:
//   forward iteration, Lipschitz bound, schedule / step sizes .... pinned (energy descent of an
//       independently written TGV energy, closed forms, brute-force Lipschitz on small images)
//   adjoint chain with all quirk toggles OFF ....................... pinned (autograd of an
//       independently written forward, finite differences)
//   what the backward pass does differently from the chain rule -- y rebuilt from the half-step
//   values (aux variables without their extrapolation), the checkpointed y at segment starts, the
//   skipped Jacobian of iteration 0, the division in one v2 block, the clamp -- and the crossed
//   beta reads of the Lipschitz kernel .............................. pinned one at a time
//       (tests/test_tgv_quirk_pins.py: the exact adjoint recursion with autograd Jacobian products
//       and that one deviation; c = 0 and no-rebuild special cases; a sub-run started at x_1;
//       a brute-force bound with explicit [row, col] reads); guard on u only, early return on a
//       bad upstream gradient, multipliers: table / ratio tests in tests/test_tgv_oracle_pins.py.
//   The numeric constants themselves (0.2, 2000, 0.1, 35, 10, 0.95, 5e6, beta = 4) are values
//   read off the reference source; nothing else can fix them.
//
// The batch dimension n is an extension (the reference accepts n == 1 only, TGV.cpp:77-81):
// samples are independent problems, each with its own Lipschitz constant; guard statistics run
// over the whole batch tensor.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr int kUniqueIds = 10;        // TGV.h:5
constexpr int kMaxCheckpoints = 100;  // TGV.h:9-15

// TGV.cu:58-60,70,78,87-93; TGVH.cu:24-41
constexpr float kHDelta2 = 0.2f;
constexpr float kHDeltaY1 = 0.2f;
constexpr float kHDeltaY2 = 0.2f;
constexpr float kBeta = 4.0f;
constexpr float kClipLocalGrad = 2000.0f;
constexpr float kLocalGCMult = 0.1f;
constexpr float kLocalGXMult = 0.1f;
constexpr float kLocalGBMult = 1.0f;
constexpr float kGlobalGMult = 0.1f;
constexpr double kKillT = 35.;
constexpr double kScaleT = 10.;
constexpr double kMemoryT = 0.95;
constexpr double kMaxTolerance = 5000000.;

struct Quirks {
  int end_uses_ckpt_y = 1;     // segment-start adjoint linearises at the checkpoint y (TGV.cu:2914-2917)
  int skip_iter0_adjoint = 1;  // iteration 0's gradient step is never back-propagated (TGV.cu:2851-2925,3047)
  int getyk_rebuild = 1;       // y rebuilt by the get_yk rule, aux y without momentum (TGV.cu:1478-1541); 0: true y
  int scale_factors = 1;       // local/global multipliers (TGV.cu:87-93); 0: all 1
  int clamp = 1;               // clipLocalGrad (TGV.cu:562-583)
  int guard = 1;               // upstream check + output guard (TGV.cu:2686-2703,2990-3021)
  int dw_div = 1;              // `W / hub^2` in the upper-triangle v2 block (TGV.cu:355); 0: `W * hub^2`
};
Quirks g_quirks;

template <class R>
struct IdState {  // TGV.h:7-50
  int run = 0;
  double av_GC = 0, av_GY = 0, av_GX = 0, av_GB = 0, av_GI = 0;
  std::vector<int> iterations;
  std::vector<std::vector<R>> intermediate_x, intermediate_y;
  std::vector<float> stepSizes;
  int maxInterIts = 0;
  int n = 0, ic = 0, ih = 0, iw = 0, its = -1;
};

template <class R>
IdState<R>* states() {
  static IdState<R> s[kUniqueIds];
  return s;
}

// TGVH.cu:42-60
template <typename T>
bool is_valid(const T& value) {
  T max_value = std::numeric_limits<T>::max();
  T min_value = -max_value;
  bool is_inf = !(min_value <= value && value <= max_value);
  bool is_nan = value != value;
  return !is_inf && !is_nan;
}

// TGVH.cu:155-177: values above the tolerance are clamped (not zeroed) and enter the mean clamped.
template <typename S>
void check_gradUpdate(S* tempc, size_t n, double& av_gc, double& is_largest, int& num_above,
                      double av_gc_current, int& invalid) {
  const double maxTolerance = kMaxTolerance;
  is_largest = 0;
  num_above = 0;
  av_gc = 0;
  invalid = 0;
  for (size_t i = 0; i < n; i++)
    if (is_valid(tempc[i])) {
      double tca = std::abs(tempc[i]);
      is_largest = std::max(tca, is_largest);
      if (tca > maxTolerance) {
        if (tempc[i] > 0) tempc[i] = (S)maxTolerance; else tempc[i] = (S)-maxTolerance;
        num_above++;
        tca = maxTolerance;
      }
      double step = double(i) / double(i + 1);
      av_gc = (1. - step) * tca + step * av_gc;
    } else {
      tempc[i] = 0;
      av_gc = av_gc_current * 1000.;
      invalid++;
    }
}

// TGVH.cu:119-151.  Returns 0 = plain running-mean update, 1 = rescaled, 2 = killed.
template <typename S>
int update_correct_av_step_host(int run, double av_gc, double& av_GC, S* tempc, size_t n,
                                double run_step_in) {
  const double run_step = std::min(kMemoryT, run_step_in);
  if (run >= 10 && av_GC * kKillT < av_gc) {
    for (size_t i = 0; i < n; i++) tempc[i] = 0.0;
    av_GC = av_GC * run_step + (1. - run_step) * kScaleT * av_GC;
    return 2;
  }
  const double scale = kScaleT;
  if (run >= 10 && av_GC * scale < av_gc) {
    double mult = scale * av_GC / av_gc;
    for (size_t i = 0; i < n; i++) tempc[i] *= mult;
    av_GC = av_GC * run_step + (1. - run_step) * av_gc * mult;
    return 1;
  } else {
    av_GC = av_GC * run_step + (1. - run_step) * av_gc;
  }
  return 0;
}

// Checkpoint schedule, TGV.cu:2543-2552,2567 (the TV layer's rule).
void make_schedule(int its, std::vector<int>& iterations, int& maxInterIts) {
  iterations.assign((size_t)std::floor(std::sqrt((double)its)), 0);
  maxInterIts = 0;
  for (size_t i = 0; i < iterations.size(); i++) {
    iterations[i] = (int)(std::floor(i * std::sqrt((double)its) * 0.5) * 2);
    if (i > 0) maxInterIts = std::max(maxInterIts, iterations[i] - iterations[i - 1]);
  }
  if (!iterations.empty()) maxInterIts = std::max(maxInterIts, its - iterations.back());
}

// FISTA extrapolation factors, TGV.cu:2569-2576.
void make_step_sizes(int its, std::vector<float>& stepSizes) {
  stepSizes.assign((size_t)std::max(its, 0), 0.f);
  double t(1), t_(1);
  for (size_t i = 0; i < stepSizes.size(); i++) {
    t_ = t;
    t = (1. + std::sqrt(1. + 4. * t * t)) / 2.;
    stepSizes[i] = (float)std::max(0.0, (t_ - 1.) / t);
  }
}

// shared-memory tile read: zero outside the image (TGV.cu:1581-1597)
template <class R>
inline R P(const R* f, int h, int w, int H, int W) {
  return (h >= 0 && h < H && w >= 0 && w < W) ? f[(size_t)h * W + w] : R(0);
}
// clamp-addressed point fetch
template <class R>
inline R T(const R* f, int h, int w, int H, int W) {
  h = std::min(std::max(h, 0), H - 1);
  w = std::min(std::max(w, 0), W - 1);
  return f[(size_t)h * W + w];
}
// the stand-in for CUDA's rsqrtf
template <class R>
inline R rsq(R x) {
  return R(1) / std::sqrt(x);
}

// TGV.cu:101-148 + the host reduction TGV.cu:2516-2527 for one sample: returns L.
// Inputs are the caller's unscaled weight fields.
template <class R>
double lipschitz(const R* dx, const R* dy, const R* betaX, const R* betaY, int H, int W,
                 R* storage_out /* may be null */) {
  R oneL = (R)(float)(std::max(12., 8. * kBeta) + 0.000001);
  std::vector<R> storage((size_t)H * W);
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const R wx_0 = (w > 0) ? T(dx, h, w - 1, H, W) : R(0);
      const R wx_1 = (w < W - 1) ? T(dx, h, w, H, W) : R(0);
      const R wy_0 = (h > 0) ? T(dy, h - 1, w, H, W) : R(0);
      const R wy_1 = (h < H - 1) ? T(dy, h, w, H, W) : R(0);
      const R betaTX_1y = (h < H - 1) ? T(betaX, h, w, H, W) : R(0);
      const R betaTX_1x = (w < W - 1) ? T(betaX, h, w, H, W) : R(0);
      const R betaTX_0x = (w > 0) ? T(betaX, h - 1, w, H, W) : R(0);  // sic: (w, h-1) under w > 0
      const R betaTX_0y = (h > 0) ? T(betaX, h, w - 1, H, W) : R(0);  // sic: (w-1, h) under h > 0
      const R betaTY_1y = (h < H - 1) ? T(betaY, h, w, H, W) : R(0);
      const R betaTY_1x = (w < W - 1) ? T(betaY, h, w, H, W) : R(0);
      const R betaTY_0x = (w > 0) ? T(betaY, h - 1, w, H, W) : R(0);
      const R betaTY_0y = (h > 0) ? T(betaY, h, w - 1, H, W) : R(0);
      R weightx = 0, weighty1 = 0, weighty2 = 0;
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
      storage[(size_t)h * W + w] = std::fmax(weightx, std::fmax(weighty1, weighty2));
    }
  for (size_t i = 0; i < storage.size(); i++) oneL = std::max(oneL, storage[i]);
  if (storage_out) std::copy(storage.begin(), storage.end(), storage_out);
  oneL = (R)(1. / (double)(R)(oneL + R(0.01f)));  // `oneL = 1. / (oneL + 0.01f)` assigned to a float
  return (double)oneL;
}

// L-scaled private copies of the four weight fields of one sample, TGV.cu:2495-2499,2528-2531.
template <class R>
struct Weights {
  std::vector<R> wx, wy, bx, by;
  double L = 0;
  void build(const R* d_x, const R* d_y, int H, int W) {
    const size_t HW = (size_t)H * W;
    L = lipschitz<R>(d_x, d_y, d_x + HW, d_y + HW, H, W, nullptr);
    wx.resize(HW); wy.resize(HW); bx.resize(HW); by.resize(HW);
    for (size_t i = 0; i < HW; i++) {
      wx[i] = (R)(L * (double)d_x[i]);
      wy[i] = (R)(L * (double)d_y[i]);
      bx[i] = (R)(L * (double)d_x[HW + i]);
      by[i] = (R)(L * (double)d_y[HW + i]);
    }
  }
};

// One forward iteration on one sample: TGV.cu:1546-1776 (x05 == nullptr) and 2005-2235 (x05 given;
// the three slots 3*it+{0,1,2} are passed as one (3,C,H,W) block).  x, y, yout: (3,C,H,W).
template <class R>
void forward_iter(const Weights<R>& wt, const R* cf, const R* b, R* x, const R* y, R* yout,
                  R* x05, int C, int H, int W, R t, R oneL) {
  const size_t HW = (size_t)H * W, CHW = HW * C;
  const R *wx = wt.wx.data(), *wy = wt.wy.data(), *bx = wt.bx.data(), *by = wt.by.data();
  const R d0 = R(kHDelta2), d1 = R(kHDeltaY1), d2 = R(kHDeltaY2);
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      const R wx_0 = (w > 0) ? wx[p - 1] : R(0);
      const R wx_1 = (w < W - 1) ? wx[p] : R(0);
      const R wy_0 = (h > 0) ? wy[p - W] : R(0);
      const R wy_1 = (h < H - 1) ? wy[p] : R(0);
      for (int ch = 0; ch < C; ch++) {
        const R* Y0 = y + ch * HW;
        const R* Y1 = y + CHW + ch * HW;
        const R* Y2 = y + 2 * CHW + ch * HW;
        const R x_ = x[ch * HW + p];
        const R bb = b[ch * HW + p];
        R x_loc = bb;
        R yc = Y0[p];
        R yt = yc;
        R y1_new = Y1[p], y2_new = Y2[p];
        const R y1_c = y1_new, y2_c = y2_new;
        if (h > 0) {  // TGV.cu:1613-1640
          const R betaTX = bx[p - W], betaTY = by[p - W];
          const R wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : R(0);
          const R zij_1 = (w < W - 1) ? ((P(Y0, h - 1, w + 1, H, W) - P(Y0, h - 1, w, H, W)) - P(Y1, h - 1, w, H, W)) : R(0);
          const R zij_2 = ((yc - P(Y0, h - 1, w, H, W)) - P(Y2, h - 1, w, H, W));
          const R hub_weight_x = std::fmin(R(1), rsq(zij_2 * zij_2 * wy_0 + zij_1 * zij_1 * wx_2) * d0);
          const R uij1_2 = (y1_c - P(Y1, h - 1, w, H, W));
          const R uij1_1 = (w < W - 1) ? (P(Y1, h - 1, w + 1, H, W) - P(Y1, h - 1, w, H, W)) : R(0);
          const R hub_weight_y1 = std::fmin(R(1), rsq(betaTX * (uij1_2 * uij1_2 + uij1_1 * uij1_1)) * d1);
          const R uij2_1 = (w < W - 1) ? (P(Y2, h - 1, w + 1, H, W) - P(Y2, h - 1, w, H, W)) : R(0);
          const R uij2_2 = (y2_c - P(Y2, h - 1, w, H, W));
          const R hub_weight_y2 = std::fmin(R(1), rsq(betaTY * (uij2_2 * uij2_2 + uij2_1 * uij2_1)) * d2);
          yt -= wy_0 * oneL * (zij_2 * hub_weight_x);
          y1_new -= (betaTX * oneL) * (uij1_2 * hub_weight_y1);
          y2_new -= (betaTY * oneL) * (uij2_2 * hub_weight_y2);
        }
        if (w > 0) {  // TGV.cu:1641-1668
          const R betaTX = bx[p - 1], betaTY = by[p - 1];
          const R wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : R(0);
          const R zij_1 = ((yc - P(Y0, h, w - 1, H, W)) - P(Y1, h, w - 1, H, W));
          const R zij_2 = (h < H - 1) ? ((P(Y0, h + 1, w - 1, H, W) - P(Y0, h, w - 1, H, W)) - P(Y2, h, w - 1, H, W)) : R(0);
          const R hub_weight_x = std::fmin(R(1), rsq(zij_2 * zij_2 * wy_2 + zij_1 * zij_1 * wx_0) * d0);
          const R uij1_1 = (y1_c - P(Y1, h, w - 1, H, W));
          const R uij1_2 = (h < H - 1) ? (P(Y1, h + 1, w - 1, H, W) - P(Y1, h, w - 1, H, W)) : R(0);
          const R hub_weight_y1 = std::fmin(R(1), rsq(betaTX * (uij1_2 * uij1_2 + uij1_1 * uij1_1)) * d1);
          const R uij2_1 = (y2_c - P(Y2, h, w - 1, H, W));
          const R uij2_2 = (h < H - 1) ? (P(Y2, h + 1, w - 1, H, W) - P(Y2, h, w - 1, H, W)) : R(0);
          const R hub_weight_y2 = std::fmin(R(1), rsq(betaTY * (uij2_2 * uij2_2 + uij2_1 * uij2_1)) * d2);
          yt -= wx_0 * oneL * (zij_1 * hub_weight_x);
          y1_new -= (betaTX * oneL) * (uij1_1 * hub_weight_y1);
          y2_new -= (betaTY * oneL) * (uij2_1 * hub_weight_y2);
        }
        {  // TGV.cu:1669-1691
          const R betaTX = bx[p], betaTY = by[p];
          const R zij_1 = (w < W - 1) ? ((yc - P(Y0, h, w + 1, H, W)) + y1_c) : R(0);
          const R zij_2 = (h < H - 1) ? ((yc - P(Y0, h + 1, w, H, W)) + y2_c) : R(0);
          const R hub_weight_x = std::fmin(R(1), rsq(zij_2 * zij_2 * wy_1 + zij_1 * zij_1 * wx_1) * d0);
          const R uij1_1 = (w < W - 1) ? (y1_c - P(Y1, h, w + 1, H, W)) : R(0);
          const R uij1_2 = (h < H - 1) ? (y1_c - P(Y1, h + 1, w, H, W)) : R(0);
          const R hub_weight_y1 = std::fmin(R(1), rsq(betaTX * (uij1_2 * uij1_2 + uij1_1 * uij1_1)) * d1);
          const R uij2_1 = (w < W - 1) ? (y2_c - P(Y2, h, w + 1, H, W)) : R(0);
          const R uij2_2 = (h < H - 1) ? (y2_c - P(Y2, h + 1, w, H, W)) : R(0);
          const R hub_weight_y2 = std::fmin(R(1), rsq(betaTY * (uij2_2 * uij2_2 + uij2_1 * uij2_1)) * d2);
          yt -= wy_1 * oneL * (zij_2 * hub_weight_x);
          y1_new -= (betaTX * oneL) * (uij1_2 * hub_weight_y1);
          y2_new -= (betaTY * oneL) * (uij2_2 * hub_weight_y2) + wy_1 * oneL * (zij_2 * hub_weight_x);
          yt -= wx_1 * oneL * (zij_1 * hub_weight_x);
          y1_new -= (betaTX * oneL) * (uij1_1 * hub_weight_y1) + wx_1 * oneL * (zij_1 * hub_weight_x);
          y2_new -= (betaTY * oneL) * (uij2_1 * hub_weight_y2);
          // aux variables: momentum only, no prox (TGV.cu:1686-1690)
          yout[CHW + ch * HW + p] = y1_new + t * (y1_new - x[CHW + ch * HW + p]);
          yout[2 * CHW + ch * HW + p] = y2_new + t * (y2_new - x[2 * CHW + ch * HW + p]);
          x[CHW + ch * HW + p] = y1_new;
          x[2 * CHW + ch * HW + p] = y2_new;
        }
        if (x05) {  // TGV.cu:2146-2147,2196
          x05[ch * HW + p] = yt;
          x05[CHW + ch * HW + p] = y1_new;
          x05[2 * CHW + ch * HW + p] = y2_new;
        }
        // Huber-1 data prox on u, TGV.cu:1740-1744
        x_loc = (conf * bb + yt) / (R(1) + conf);
        yc = yt - conf;
        yt = yt + conf;
        if (yc > R(1) + bb) x_loc = yc;
        if (yt < bb - R(1)) x_loc = yt;
        yout[ch * HW + p] = x_loc + t * (x_loc - x_);  // TGV.cu:1772-1773
        x[ch * HW + p] = x_loc;
      }
    }
}

// TGV.cu:1478-1541: rebuild y_{k+1}; u as in the TV layer, aux = x05 without momentum.
template <class R>
void get_yk(const R* cf, const R* b, const R* x05_it, const R* x05_itm1, R* yk_out, int C, int H,
            int W, R t) {
  const size_t HW = (size_t)H * W, CHW = HW * C;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      for (int ch = 0; ch < C; ch++) {
        const size_t q = ch * HW + p;
        const R bb = b[q];
        R diff = bb - x05_it[q];
        R sign = (diff < 0) ? R(-1.) : R(1.);
        R yk(0);
        if (1. + (double)conf >= (double)(sign * diff)) {
          const R xk = (conf * bb + x05_it[q]) / (R(1) + conf);
          const R xkm = (conf * bb + x05_itm1[q]) / (R(1) + conf);
          yk = xk + t * (xk - xkm);
        } else {
          const R xk = (conf <= sign * diff) ? bb - diff + sign * conf : bb;
          diff = bb - x05_itm1[q];
          sign = (diff < 0) ? R(-1.) : R(1.);
          yk = xk + t * (xk - ((conf <= sign * diff) ? bb - diff + sign * conf : bb));
        }
        yk_out[q] = yk;
        yk_out[CHW + q] = x05_it[CHW + q];          // TGV.cu:1536
        yk_out[2 * CHW + q] = x05_it[2 * CHW + q];  // TGV.cu:1537
      }
    }
}

struct Mults {
  float gc, gx, gb;
};

// Prox adjoint + confidence / rhs gradient of one u value: TGV.cu:166-182 (init kernel),
// 592-612 (bw_yk), 1418-1442 (end kernel).
template <class R>
inline void prox_adjoint(R df_dxk, R bb, R x05v, R conf, R& g05_out, R& gc_acc, R& gb_acc,
                         const Mults& m, bool init_kernel) {
  const R diff = bb - x05v;
  const R sign = (diff < 0) ? R(-1.) : R(1.);
  if (1. + (double)conf >= (double)(sign * diff)) {
    if (init_kernel) {
      g05_out = df_dxk / (R(1) + conf);
      gc_acc += df_dxk * (bb / (R(1) + conf) - (conf * bb + x05v) / ((R(1) + conf) * (R(1) + conf))) * R(m.gc);
      gb_acc += df_dxk * conf / (R(1) + conf) * R(m.gb);
    } else {
      gc_acc += df_dxk * (bb / (R(1) + conf) - (conf * bb + x05v) / ((R(1) + conf) * (R(1) + conf))) * R(m.gc);
      g05_out = df_dxk / (R(1) + conf);
      gb_acc += df_dxk * conf / (R(1) + conf) * R(m.gb);
    }
  } else {
    if (init_kernel) {
      g05_out = df_dxk;
      gc_acc += sign * df_dxk * R(m.gc);
      gb_acc = 0;
    } else if (conf >= sign * diff) {
      g05_out = 0;
      gb_acc += df_dxk * R(m.gb);
    } else {
      g05_out = df_dxk;
      gc_acc += sign * df_dxk * R(m.gc);
    }
  }
}

// TGV.cu:151-218 on one sample.  gin, g05: (3,C,H,W).
template <class R>
void init_adjoint(const R* cf, const R* b, const R* x05_it, R* gc, R* gb, R* g05, const R* gin,
                  int C, int H, int W, const Mults& m) {
  const size_t HW = (size_t)H * W, CHW = HW * C;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      for (int ch = 0; ch < C; ch++) {
        const size_t q = ch * HW + p;
        prox_adjoint<R>(gin[q], b[q], x05_it[q], conf, g05[q], gc[p], gb[q], m, true);
        g05[CHW + q] = gin[CHW + q];          // TGV.cu:215
        g05[2 * CHW + q] = gin[2 * CHW + q];  // TGV.cu:216
      }
    }
}

// per-pixel accumulators of the weight gradients: channel 0 = edge weight, channel 1 = beta
template <class R>
struct WeightGrads {
  R *gwx0, *gwx1, *gwy0, *gwy1;
};

// Transposed Jacobian of the TGV gradient step at one pixel of one channel plus the pixel's
// own-triangle weight gradients, main adjoint kernel form: TGV.cu:304-558.
template <class R>
inline void jt_main_px(const R* y, const R* y1, const R* y2, const R* g, const R* g1, const R* g2,
                       const Weights<R>& wt, int h, int w, int H, int W, R& gwx0, R& gwx1, R& gwy0,
                       R& gwy1, R gxm, R oneL, bool q7, R& o0, R& o1, R& o2) {
  const size_t p = (size_t)h * W + w;
  const R *wx = wt.wx.data(), *wy = wt.wy.data(), *bx = wt.bx.data(), *by = wt.by.data();
  const R d0 = R(kHDelta2), d1 = R(kHDeltaY1), d2 = R(kHDeltaY2);
  const R wx_0 = (w > 0) ? wx[p - 1] : R(0);
  const R wx_1 = (w < W - 1) ? wx[p] : R(0);
  const R wy_0 = (h > 0) ? wy[p - W] : R(0);
  const R wy_1 = (h < H - 1) ? wy[p] : R(0);
#define Q(f, dh, dw) P(f, h + (dh), w + (dw), H, W)
  const R df_dy = g[p], df_dy1 = g1[p], df_dy2 = g2[p];
  R df_dy_t = df_dy, df_dy1_t = df_dy1, df_dy2_t = df_dy2;
  if (h > 0) {  // TGV.cu:304-360
    const R betaTX = bx[p - W], betaTY = by[p - W];
    const R wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : R(0);
    {
      const R zij_1 = (w < W - 1) ? ((Q(y, -1, 1) - Q(y, -1, 0)) - Q(y1, -1, 0)) : R(0);
      const R zij_2 = ((Q(y, 0, 0) - Q(y, -1, 0)) - Q(y2, -1, 0));
      const R hub_weight_x = rsq(zij_2 * zij_2 * wy_0 + zij_1 * zij_1 * wx_2);
      const R W_TIJ = std::fmin(R(1), hub_weight_x * d0);
      df_dy_t -= oneL * W_TIJ * ((df_dy - Q(g, -1, 0)) - Q(g2, -1, 0)) * wy_0;
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_x * hub_weight_x);
        const R a2 = zij_2 * wy_0;
        const R a1 = zij_1 * wx_2;
        df_dy_t += oneL * (dW_TIJ * a2) * (a1 * (Q(g, -1, 1) - Q(g, -1, 0) - Q(g1, -1, 0)) +
                                          a2 * (Q(g, 0, 0) - Q(g, -1, 0) - Q(g2, -1, 0)));
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y1, -1, 1) - Q(y1, -1, 0)) : R(0);
      const R uij_2 = (Q(y1, 0, 0) - Q(y1, -1, 0));
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_TIJ = std::fmin(R(1), hub_weight_y * d1);
      df_dy1_t -= betaTX * oneL * W_TIJ * (df_dy1 - Q(g1, -1, 0));
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_y * hub_weight_y);
        df_dy1_t += betaTX * oneL * (dW_TIJ * betaTX * uij_2) * (uij_1 * (Q(g1, -1, 1) - Q(g1, -1, 0)) +
                                                                uij_2 * (Q(g1, 0, 0) - Q(g1, -1, 0)));
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y2, -1, 1) - Q(y2, -1, 0)) : R(0);
      const R uij_2 = (Q(y2, 0, 0) - Q(y2, -1, 0));
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_TIJ = std::fmin(R(1), hub_weight_y * d2);
      df_dy2_t -= betaTY * oneL * W_TIJ * (df_dy2 - Q(g2, -1, 0));
      if (W_TIJ < 1.0) {
        // TGV.cu:355: a division where every sibling block multiplies
        const R dW_TIJ = q7 ? W_TIJ / (hub_weight_y * hub_weight_y) : W_TIJ * (hub_weight_y * hub_weight_y);
        df_dy2_t += betaTY * oneL * (dW_TIJ * betaTY * uij_2) * (uij_1 * (Q(g2, -1, 1) - Q(g2, -1, 0)) +
                                                                uij_2 * (Q(g2, 0, 0) - Q(g2, -1, 0)));
      }
    }
  }
  if (w > 0) {  // TGV.cu:361-418
    const R betaTX = bx[p - 1], betaTY = by[p - 1];
    const R wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : R(0);
    {
      const R zij_1 = (Q(y, 0, 0) - Q(y, 0, -1) - Q(y1, 0, -1));
      const R zij_2 = (h < H - 1) ? (Q(y, 1, -1) - Q(y, 0, -1) - Q(y2, 0, -1)) : R(0);
      const R hub_weight_x = rsq(zij_2 * zij_2 * wy_2 + zij_1 * zij_1 * wx_0);
      const R W_TIJ = std::fmin(R(1), hub_weight_x * d0);
      df_dy_t -= oneL * W_TIJ * ((df_dy - Q(g, 0, -1)) - Q(g1, 0, -1)) * wx_0;
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_x * hub_weight_x);
        const R a1 = zij_1 * wx_0;
        const R a2 = zij_2 * wy_2;
        df_dy_t += oneL * (dW_TIJ * a1) * (a1 * (Q(g, 0, 0) - Q(g, 0, -1) - Q(g1, 0, -1)) +
                                          a2 * (Q(g, 1, -1) - Q(g, 0, -1) - Q(g2, 0, -1)));
      }
    }
    {
      const R uij_1 = (Q(y1, 0, 0) - Q(y1, 0, -1));
      const R uij_2 = (h < H - 1) ? (Q(y1, 1, -1) - Q(y1, 0, -1)) : R(0);
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_TIJ = std::fmin(R(1), hub_weight_y * d1);
      df_dy1_t -= betaTX * oneL * W_TIJ * (df_dy1 - Q(g1, 0, -1));
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_y * hub_weight_y);
        df_dy1_t += betaTX * oneL * (dW_TIJ * betaTX * uij_1) * (uij_2 * (Q(g1, 1, -1) - Q(g1, 0, -1)) +
                                                                uij_1 * (Q(g1, 0, 0) - Q(g1, 0, -1)));
      }
    }
    {
      const R uij_1 = (Q(y2, 0, 0) - Q(y2, 0, -1));
      const R uij_2 = (h < H - 1) ? (Q(y2, 1, -1) - Q(y2, 0, -1)) : R(0);
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_TIJ = std::fmin(R(1), hub_weight_y * d2);
      df_dy2_t -= betaTY * oneL * W_TIJ * (df_dy2 - Q(g2, 0, -1));
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_y * hub_weight_y);
        df_dy2_t += betaTY * oneL * (dW_TIJ * betaTY * uij_1) * (uij_2 * (Q(g2, 1, -1) - Q(g2, 0, -1)) +
                                                                uij_1 * (Q(g2, 0, 0) - Q(g2, 0, -1)));
      }
    }
  }
  {  // the pixel's own triangle, TGV.cu:419-507
    const R betaTX = bx[p], betaTY = by[p];
    {
      const R aij_1 = (w < W - 1) ? ((Q(y, 0, 1) - Q(y, 0, 0)) - Q(y1, 0, 0)) : R(0);
      const R aij_2 = (h < H - 1) ? ((Q(y, 1, 0) - Q(y, 0, 0)) - Q(y2, 0, 0)) : R(0);
      const R hub_weight_x = rsq(aij_2 * aij_2 * wy_1 + aij_1 * aij_1 * wx_1);
      const R W_TIJ = std::fmin(R(1), hub_weight_x * d0);
      const R dyij_1 = df_dy - Q(g, 0, 1) + df_dy1;
      const R dyij_2 = df_dy - Q(g, 1, 0) + df_dy2;
      df_dy_t -= oneL * W_TIJ * (dyij_2 * wy_1 + dyij_1 * wx_1);
      df_dy1_t -= oneL * W_TIJ * dyij_1 * wx_1;
      df_dy2_t -= oneL * W_TIJ * dyij_2 * wy_1;
      gwx0 = gwx0 + oneL * gxm * dyij_1 * (aij_1 * W_TIJ);
      gwy0 = gwy0 + oneL * gxm * dyij_2 * (aij_2 * W_TIJ);
      if (W_TIJ < 1.0) {
        const R dW_TIJ = W_TIJ * (hub_weight_x * hub_weight_x);
        const R a1 = aij_1 * wx_1;
        const R a2 = aij_2 * wy_1;
        const R deriv_Tij = (dyij_1 * a1 + dyij_2 * a2) * oneL;
        df_dy_t += deriv_Tij * ((a1 + a2) * dW_TIJ);
        df_dy2_t += deriv_Tij * (a2 * dW_TIJ);
        df_dy1_t += deriv_Tij * (a1 * dW_TIJ);
        gwy0 = (R)((double)gwy0 - (double)(gxm * (aij_2 * dW_TIJ * aij_2)) * 0.5 * (double)deriv_Tij);
        gwx0 = (R)((double)gwx0 - (double)(gxm * (aij_1 * dW_TIJ * aij_1)) * 0.5 * (double)deriv_Tij);
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y1, 0, 1) - Q(y1, 0, 0)) : R(0);
      const R uij_2 = (h < H - 1) ? (Q(y1, 1, 0) - Q(y1, 0, 0)) : R(0);
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_YIJ = std::fmin(R(1), hub_weight_y * d1);
      if (w < W - 1) df_dy1_t -= betaTX * oneL * W_YIJ * (df_dy1 - Q(g1, 0, 1));
      if (h < H - 1) df_dy1_t -= betaTX * oneL * W_YIJ * (df_dy1 - Q(g1, 1, 0));
      gwx1 = gwx1 + oneL * gxm * ((df_dy1 - Q(g1, 0, 1)) * uij_1 + (df_dy1 - Q(g1, 1, 0)) * uij_2) * W_YIJ;
      if (W_YIJ < 1.0) {
        const R dW_YIJ = W_YIJ * (hub_weight_y * hub_weight_y);
        const R deriv_Yij = ((df_dy1 - Q(g1, 0, 1)) * uij_1 * betaTX + (df_dy1 - Q(g1, 1, 0)) * uij_2 * betaTX) * oneL;
        df_dy1_t += betaTX * dW_YIJ * (uij_1 + uij_2) * deriv_Yij;
        gwx1 = (R)((double)gwx1 - (double)(gxm * (uij_2 * dW_YIJ * uij_2 + uij_1 * dW_YIJ * uij_1)) * 0.5 * (double)deriv_Yij);
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y2, 0, 1) - Q(y2, 0, 0)) : R(0);
      const R uij_2 = (h < H - 1) ? (Q(y2, 1, 0) - Q(y2, 0, 0)) : R(0);
      const R hub_weight_y = rsq((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_YIJ = std::fmin(R(1), hub_weight_y * d2);
      if (w < W - 1) df_dy2_t -= betaTY * oneL * W_YIJ * (df_dy2 - Q(g2, 0, 1));
      if (h < H - 1) df_dy2_t -= betaTY * oneL * W_YIJ * (df_dy2 - Q(g2, 1, 0));
      gwy1 = gwy1 + oneL * gxm * ((df_dy2 - Q(g2, 0, 1)) * uij_1 + (df_dy2 - Q(g2, 1, 0)) * uij_2) * W_YIJ;
      if (W_YIJ < 1.0) {
        const R dW_YIJ = W_YIJ * (hub_weight_y * hub_weight_y);
        const R deriv_Yij = ((df_dy2 - Q(g2, 0, 1)) * uij_1 * betaTY + (df_dy2 - Q(g2, 1, 0)) * uij_2 * betaTY) * oneL;
        df_dy2_t += betaTY * dW_YIJ * (uij_1 + uij_2) * deriv_Yij;
        gwy1 = (R)((double)gwy1 - (double)(gxm * (uij_2 * dW_YIJ * uij_2 + uij_1 * dW_YIJ * uij_1)) * 0.5 * (double)deriv_Yij);
      }
    }
  }
  o0 = df_dy_t;
  o1 = df_dy1_t;
  o2 = df_dy2_t;
}

// Same Jacobian in the segment-start kernel's form, TGV.cu:1118-1333: sqrt instead of rsqrt,
// W = 1. / max(1, hub / delta) (a double division), activity test hub > delta, dW = W / hub^2,
// and a different operand order in the own-triangle block.
template <class R>
inline void jt_end_px(const R* y, const R* y1, const R* y2, const R* g, const R* g1, const R* g2,
                      const Weights<R>& wt, int h, int w, int H, int W, R& gwx0, R& gwx1, R& gwy0,
                      R& gwy1, R gxm, R oneL, R& o0, R& o1, R& o2) {
  const size_t p = (size_t)h * W + w;
  const R *wx = wt.wx.data(), *wy = wt.wy.data(), *bx = wt.bx.data(), *by = wt.by.data();
  const R d0 = R(kHDelta2), d1 = R(kHDeltaY1), d2 = R(kHDeltaY2);
  const R wx_0 = (w > 0) ? wx[p - 1] : R(0);
  const R wx_1 = (w < W - 1) ? wx[p] : R(0);
  const R wy_0 = (h > 0) ? wy[p - W] : R(0);
  const R wy_1 = (h < H - 1) ? wy[p] : R(0);
  auto huberW = [](R hub, R delta) { return (R)(1. / (double)std::fmax(R(1), hub / delta)); };
  const R yk = y[p];
  const R df_dy = g[p], df_dy1 = g1[p], df_dy2 = g2[p];
  R df_dy_t = df_dy, df_dy1_t = df_dy1, df_dy2_t = df_dy2;
  if (h > 0) {  // TGV.cu:1118-1171
    const R betaTX = bx[p - W], betaTY = by[p - W];
    const R wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : R(0);
    {
      const R zij_1 = (w < W - 1) ? ((Q(y, -1, 1) - Q(y, -1, 0)) - Q(y1, -1, 0)) : R(0);
      const R zij_2 = ((yk - Q(y, -1, 0)) - Q(y2, -1, 0));
      const R hub_weight_x = std::sqrt(zij_2 * zij_2 * wy_0 + zij_1 * zij_1 * wx_2);
      const R W_TIJ = huberW(hub_weight_x, d0);
      df_dy_t -= oneL * W_TIJ * ((df_dy - Q(g, -1, 0)) - Q(g2, -1, 0)) * wy_0;
      if (hub_weight_x > d0) {
        const R dW_TIJ = W_TIJ / (hub_weight_x * hub_weight_x);
        const R a1 = zij_1 * wx_2;
        const R a2 = zij_2 * wy_0;
        df_dy_t += oneL * (dW_TIJ * a2) * (a1 * (Q(g, -1, 1) - Q(g, -1, 0) - Q(g1, -1, 0)) +
                                          a2 * (Q(g, 0, 0) - Q(g, -1, 0) - Q(g2, -1, 0)));
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y1, -1, 1) - Q(y1, -1, 0)) : R(0);
      const R uij_2 = (Q(y1, 0, 0) - Q(y1, -1, 0));
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_TIJ = huberW(hub_weight_y, d1);
      df_dy1_t -= betaTX * oneL * W_TIJ * (df_dy1 - Q(g1, -1, 0));
      if (hub_weight_y > d1) {
        const R dW_TIJ = W_TIJ / (hub_weight_y * hub_weight_y);
        df_dy1_t += betaTX * oneL * (dW_TIJ * betaTX * uij_2) * (uij_1 * (Q(g1, -1, 1) - Q(g1, -1, 0)) +
                                                                uij_2 * (Q(g1, 0, 0) - Q(g1, -1, 0)));
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y2, -1, 1) - Q(y2, -1, 0)) : R(0);
      const R uij_2 = (Q(y2, 0, 0) - Q(y2, -1, 0));
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_TIJ = huberW(hub_weight_y, d2);
      df_dy2_t -= betaTY * oneL * W_TIJ * (df_dy2 - Q(g2, -1, 0));
      if (hub_weight_y > d2) {
        const R dW_TIJ = W_TIJ / (hub_weight_y * hub_weight_y);
        df_dy2_t += betaTY * oneL * (dW_TIJ * betaTY * uij_2) * (uij_1 * (Q(g2, -1, 1) - Q(g2, -1, 0)) +
                                                                uij_2 * (Q(g2, 0, 0) - Q(g2, -1, 0)));
      }
    }
  }
  if (w > 0) {  // TGV.cu:1172-1227
    const R betaTX = bx[p - 1], betaTY = by[p - 1];
    const R wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : R(0);
    {
      const R zij_1 = (yk - Q(y, 0, -1) - Q(y1, 0, -1));
      const R zij_2 = (h < H - 1) ? (Q(y, 1, -1) - Q(y, 0, -1) - Q(y2, 0, -1)) : R(0);
      const R hub_weight_x = std::sqrt(zij_2 * zij_2 * wy_2 + zij_1 * zij_1 * wx_0);
      const R W_TIJ = huberW(hub_weight_x, d0);
      df_dy_t -= oneL * W_TIJ * ((df_dy - Q(g, 0, -1)) - Q(g1, 0, -1)) * wx_0;
      if (hub_weight_x > d0) {
        const R dW_TIJ = W_TIJ / (hub_weight_x * hub_weight_x);
        const R a1 = zij_1 * wx_0;
        const R a2 = zij_2 * wy_2;
        df_dy_t += oneL * (dW_TIJ * a1) * (a1 * (Q(g, 0, 0) - Q(g, 0, -1) - Q(g1, 0, -1)) +
                                          a2 * (Q(g, 1, -1) - Q(g, 0, -1) - Q(g2, 0, -1)));
      }
    }
    {
      const R uij_1 = (Q(y1, 0, 0) - Q(y1, 0, -1));
      const R uij_2 = (h < H - 1) ? (Q(y1, 1, -1) - Q(y1, 0, -1)) : R(0);
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_TIJ = huberW(hub_weight_y, d1);
      df_dy1_t -= betaTX * oneL * W_TIJ * (df_dy1 - Q(g1, 0, -1));
      if (hub_weight_y > d1) {
        const R dW_TIJ = W_TIJ / (hub_weight_y * hub_weight_y);
        df_dy1_t += betaTX * oneL * (dW_TIJ * betaTX * uij_1) * (uij_2 * (Q(g1, 1, -1) - Q(g1, 0, -1)) +
                                                                uij_1 * (Q(g1, 0, 0) - Q(g1, 0, -1)));
      }
    }
    {
      const R uij_1 = (Q(y2, 0, 0) - Q(y2, 0, -1));
      const R uij_2 = (h < H - 1) ? (Q(y2, 1, -1) - Q(y2, 0, -1)) : R(0);
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_TIJ = huberW(hub_weight_y, d2);
      df_dy2_t -= betaTY * oneL * W_TIJ * (df_dy2 - Q(g2, 0, -1));
      if (hub_weight_y > d2) {
        const R dW_TIJ = W_TIJ / (hub_weight_y * hub_weight_y);
        df_dy2_t += betaTY * oneL * (dW_TIJ * betaTY * uij_1) * (uij_2 * (Q(g2, 1, -1) - Q(g2, 0, -1)) +
                                                                uij_1 * (Q(g2, 0, 0) - Q(g2, 0, -1)));
      }
    }
  }
  {  // TGV.cu:1228-1333
    const R betaTX = bx[p], betaTY = by[p];
    {
      const R aij_1 = (w < W - 1) ? ((Q(y, 0, 1) - Q(y, 0, 0)) - Q(y1, 0, 0)) : R(0);
      const R aij_2 = (h < H - 1) ? ((Q(y, 1, 0) - Q(y, 0, 0)) - Q(y2, 0, 0)) : R(0);
      const R hub_weight_x = std::sqrt(aij_2 * aij_2 * wy_1 + aij_1 * aij_1 * wx_1);
      const R W_TIJ = huberW(hub_weight_x, d0);
      df_dy_t -= oneL * ((df_dy - Q(g, 1, 0)) + Q(g2, 0, 0)) * wy_1 * W_TIJ;
      df_dy_t -= oneL * ((df_dy - Q(g, 0, 1)) + Q(g1, 0, 0)) * wx_1 * W_TIJ;
      df_dy1_t -= oneL * W_TIJ * (df_dy1 - Q(g, 0, 1) + df_dy) * wx_1;
      df_dy2_t -= oneL * W_TIJ * (df_dy2 - Q(g, 1, 0) + df_dy) * wy_1;
      gwx0 = gwx0 + oneL * gxm * (df_dy - Q(g, 0, 1) + df_dy1) * aij_1 * W_TIJ;
      gwy0 = gwy0 + oneL * gxm * (df_dy - Q(g, 1, 0) + df_dy2) * aij_2 * W_TIJ;
      if (hub_weight_x > d0) {
        const R dW_TIJ = W_TIJ / (hub_weight_x * hub_weight_x);
        const R a2 = aij_2 * wy_1;
        const R a1 = aij_1 * wx_1;
        const R deriv_Tij = ((df_dy - Q(g, 0, 1) + df_dy1) * a1 + (df_dy - Q(g, 1, 0) + df_dy2) * a2) * oneL;
        df_dy_t += deriv_Tij * ((a1 + a2) * dW_TIJ);
        df_dy2_t += deriv_Tij * (a2 * dW_TIJ);
        df_dy1_t += deriv_Tij * (a1 * dW_TIJ);
        gwy0 = (R)((double)gwy0 - (double)(gxm * (aij_2 * dW_TIJ * aij_2)) * 0.5 * (double)deriv_Tij);
        gwx0 = (R)((double)gwx0 - (double)(gxm * (aij_1 * dW_TIJ * aij_1)) * 0.5 * (double)deriv_Tij);
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y1, 0, 1) - Q(y1, 0, 0)) : R(0);
      const R uij_2 = (h < H - 1) ? (Q(y1, 1, 0) - Q(y1, 0, 0)) : R(0);
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTX);
      const R W_YIJ = huberW(hub_weight_y, d1);
      if (h < H - 1) df_dy1_t -= betaTX * oneL * W_YIJ * (df_dy1 - Q(g1, 1, 0));  // y first here
      if (w < W - 1) df_dy1_t -= betaTX * oneL * W_YIJ * (df_dy1 - Q(g1, 0, 1));
      gwx1 = gwx1 + oneL * gxm * ((df_dy1 - Q(g1, 0, 1)) * uij_1 + (df_dy1 - Q(g1, 1, 0)) * uij_2) * W_YIJ;
      if (hub_weight_y > d1) {
        const R dW_YIJ = W_YIJ / (hub_weight_y * hub_weight_y);
        const R deriv_Yij = ((df_dy1 - Q(g1, 0, 1)) * uij_1 * betaTX + (df_dy1 - Q(g1, 1, 0)) * uij_2 * betaTX) * oneL;
        df_dy1_t += betaTX * dW_YIJ * (uij_1 + uij_2) * deriv_Yij;
        gwx1 = (R)((double)gwx1 - (double)(gxm * (uij_2 * dW_YIJ * uij_2 + uij_1 * dW_YIJ * uij_1)) * 0.5 * (double)deriv_Yij);
      }
    }
    {
      const R uij_1 = (w < W - 1) ? (Q(y2, 0, 1) - Q(y2, 0, 0)) : R(0);
      const R uij_2 = (h < H - 1) ? (Q(y2, 1, 0) - Q(y2, 0, 0)) : R(0);
      const R hub_weight_y = std::sqrt((uij_1 * uij_1 + uij_2 * uij_2) * betaTY);
      const R W_YIJ = huberW(hub_weight_y, d2);
      if (w < W - 1) df_dy2_t -= betaTY * oneL * W_YIJ * (df_dy2 - Q(g2, 0, 1));
      if (h < H - 1) df_dy2_t -= betaTY * oneL * W_YIJ * (df_dy2 - Q(g2, 1, 0));
      gwy1 = gwy1 + oneL * gxm * ((df_dy2 - Q(g2, 0, 1)) * uij_1 + (df_dy2 - Q(g2, 1, 0)) * uij_2) * W_YIJ;
      if (hub_weight_y > d2) {
        const R dW_YIJ = W_YIJ / (hub_weight_y * hub_weight_y);
        const R deriv_Yij = ((df_dy2 - Q(g2, 0, 1)) * uij_1 * betaTY + (df_dy2 - Q(g2, 1, 0)) * uij_2 * betaTY) * oneL;
        df_dy2_t += betaTY * dW_YIJ * (uij_1 + uij_2) * deriv_Yij;
        gwy1 = (R)((double)gwy1 - (double)(gxm * (uij_2 * dW_YIJ * uij_2 + uij_1 * dW_YIJ * uij_1)) * 0.5 * (double)deriv_Yij);
      }
    }
  }
#undef Q
  o0 = df_dy_t;
  o1 = df_dy1_t;
  o2 = df_dy2_t;
}

// One reverse step on one sample: TGV.cu:224-644 (bw_yk) / 1061-1472 (end).  All state tensors
// are (3,C,H,W); gwx, gwy are (2,H,W) accumulators; y is y_{k+1} (or the checkpoint y).
template <class R>
void adjoint_iter(const Weights<R>& wt, const R* cf, const R* b, const R* x05_it, R* gc, R* gb,
                  R* gwx, R* gwy, const R* g05_in, R* g05_out, R* gxk, R* gxk_m1, const R* y, int C,
                  int H, int W, R t, R oneL, const Mults& m, bool end_form, bool clamp, bool q7) {
  const size_t HW = (size_t)H * W, CHW = HW * C;
  auto clip = [&](R v) { return clamp ? std::fmax(-R(kClipLocalGrad), std::fmin(v, R(kClipLocalGrad))) : v; };
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      for (int ch = 0; ch < C; ch++) {
        const size_t q = ch * HW + p;
        const size_t o = ch * HW;
        R df_dy_t, df_dy1_t, df_dy2_t;
        if (end_form)
          jt_end_px<R>(y + o, y + CHW + o, y + 2 * CHW + o, g05_in + o, g05_in + CHW + o, g05_in + 2 * CHW + o,
                       wt, h, w, H, W, gwx[p], gwx[HW + p], gwy[p], gwy[HW + p], R(m.gx), oneL,
                       df_dy_t, df_dy1_t, df_dy2_t);
        else
          jt_main_px<R>(y + o, y + CHW + o, y + 2 * CHW + o, g05_in + o, g05_in + CHW + o, g05_in + 2 * CHW + o,
                        wt, h, w, H, W, gwx[p], gwx[HW + p], gwy[p], gwy[HW + p], R(m.gx), oneL, q7,
                        df_dy_t, df_dy1_t, df_dy2_t);
        // aux variables: momentum adjoint only, TGV.cu:560-577 / 1383-1399
        gxk_m1[CHW + q] = -t * df_dy1_t;
        df_dy1_t = clip((R)((double)gxk[CHW + q] + (1. + (double)t) * (double)df_dy1_t));
        g05_out[CHW + q] = df_dy1_t;
        gxk[CHW + q] = df_dy1_t;
        gxk_m1[2 * CHW + q] = -t * df_dy2_t;
        df_dy2_t = clip((R)((double)gxk[2 * CHW + q] + (1. + (double)t) * (double)df_dy2_t));
        g05_out[2 * CHW + q] = df_dy2_t;
        gxk[2 * CHW + q] = df_dy2_t;
        // u: TGV.cu:579-612 / 1403-1442
        R df_dxk = clip((R)((double)gxk[q] + (1. + (double)t) * (double)df_dy_t));
        gxk[q] = df_dxk;
        gxk_m1[q] = -t * df_dy_t;
        prox_adjoint<R>(df_dxk, b[q], x05_it[q], conf, g05_out[q], gc[p], gb[q], m, false);
      }
    }
}

// TGV.cu:2475-2618 with a batch loop around it.  d_x, d_y: (n,2,H,W); d_i, d_out: (n,3*C,H,W).
template <class R>
int forward(const R* d_x, const R* d_y, const R* d_c, const R* d_b, const R* d_i, R* d_out, int in,
            int ic, int ih, int iw, int its, int id) {
  if (static_cast<size_t>(id) >= (size_t)kUniqueIds) return 1;  // TGV.cu:2479-2483
  if (in < 1 || ic < 1 || ih < 1 || iw < 1 || its < 0) return 2;
  if ((int)std::floor(std::sqrt((double)its)) > kMaxCheckpoints) return 3;
  IdState<R>& st = states<R>()[id];
  const size_t HW = (size_t)ih * iw, CHW = HW * ic, S = 3 * CHW;
  const R oneL = R(1.0);  // TGV.cu:2527
  std::vector<Weights<R>> wts(in);
  for (int s = 0; s < in; s++) wts[s].build(d_x + s * 2 * HW, d_y + s * 2 * HW, ih, iw);

  std::vector<R> y0(d_i, d_i + in * S), y1(d_i, d_i + in * S);  // TGV.cu:2537-2541
  std::memcpy(d_out, d_i, in * S * sizeof(R));

  make_schedule(its, st.iterations, st.maxInterIts);
  st.intermediate_x.assign(st.iterations.size(), std::vector<R>());
  st.intermediate_y.assign(st.iterations.size(), std::vector<R>());
  make_step_sizes(its, st.stepSizes);
  st.n = in; st.ic = ic; st.ih = ih; st.iw = iw; st.its = its;

  size_t start_it = 0;
  for (int it = 0; it < its / 2; it++) {  // TGV.cu:2585-2614
    if (start_it < st.iterations.size() && st.iterations[start_it] == 2 * it) {
      st.intermediate_y[start_it].assign(y0.begin(), y0.end());
      st.intermediate_x[start_it].assign(d_out, d_out + in * S);
      start_it++;
    }
    for (int s = 0; s < in; s++) {
      R step = st.stepSizes[2 * it];
      forward_iter<R>(wts[s], d_c + s * HW, d_b + s * CHW, d_out + s * S, &y0[s * S], &y1[s * S],
                      nullptr, ic, ih, iw, step, oneL);
      step = st.stepSizes[2 * it + 1];
      forward_iter<R>(wts[s], d_c + s * HW, d_b + s * CHW, d_out + s * S, &y1[s * S], &y0[s * S],
                      nullptr, ic, ih, iw, step, oneL);
    }
  }
  for (size_t i = 0; i < st.iterations.size(); i++)
    if (st.intermediate_y[i].empty()) {
      st.intermediate_y[i].assign(in * S, R(0));
      st.intermediate_x[i].assign(in * S, R(0));
    }
  return 0;
}

// TGV.cu:2621-3063 with a batch loop around the kernel sequence.
// d_inGrad, d_outGradI: (n,3*C,H,W); d_outGradX/Y: (n,2,H,W); d_outGradC: (n,1,H,W); d_outGradB: (n,C,H,W).
template <class R>
int backward(const R* d_x, const R* d_y, const R* d_c, const R* d_b, R* d_inGrad, R* d_outGradX,
             R* d_outGradY, R* d_outGradC, R* d_outGradB, R* d_outGradI, int in, int ic, int ih,
             int iw, int its, int id) {
  if (static_cast<size_t>(id) >= (size_t)kUniqueIds) return 1;  // TGV.cu:2625-2629
  IdState<R>& st = states<R>()[id];
  if (st.its != its || st.n != in || st.ic != ic || st.ih != ih || st.iw != iw) return 4;
  const Quirks q = g_quirks;
  const size_t HW = (size_t)ih * iw, CHW = HW * ic, S = 3 * CHW;
  const R oneL = R(1.0);
  Mults m{kLocalGCMult, kLocalGXMult, kLocalGBMult};
  double globalMult = kGlobalGMult;
  if (!q.scale_factors) { m = Mults{1.f, 1.f, 1.f}; globalMult = 1.; }

  std::vector<Weights<R>> wts(in);
  for (int s = 0; s < in; s++) wts[s].build(d_x + s * 2 * HW, d_y + s * 2 * HW, ih, iw);

  // TGV.cu:2680-2684
  std::fill(d_outGradI, d_outGradI + in * S, R(0));
  std::fill(d_outGradX, d_outGradX + in * 2 * HW, R(0));
  std::fill(d_outGradY, d_outGradY + in * 2 * HW, R(0));
  std::fill(d_outGradC, d_outGradC + in * HW, R(0));
  std::fill(d_outGradB, d_outGradB + in * CHW, R(0));

  if (q.guard) {  // TGV.cu:2686-2703: any non-finite entry or an all-zero upstream => zeros, run unchanged
    int is_nan = 0, nnz = 0;
    std::vector<R> tempv(d_inGrad, d_inGrad + in * S);
    for (size_t i = 0; i < tempv.size(); i++) {
      if (!is_valid(tempv[i])) { is_nan++; tempv[i] = 0; }
      if (tempv[i] != 0) nnz++;
    }
    if (is_nan != 0 || nnz == 0) {
      std::copy(tempv.begin(), tempv.end(), d_inGrad);
      return 0;
    }
  }

  std::vector<R> gc(in * HW, 0), gx(in * 2 * HW, 0), gy(in * 2 * HW, 0), gb(in * CHW, 0);
  std::vector<R> y0(in * S), y1(in * S), dout(in * S);
  std::vector<R> g05_0(in * S, 0), g05_1(in * S, 0), gxk1(in * S, 0);
  std::vector<R> gxk0(d_inGrad, d_inGrad + in * S);  // TGV.cu:2726-2729
  std::vector<R> yk(in * S, 0);
  std::vector<R> xk05((size_t)std::max(st.maxInterIts, 1) * in * S);  // TGV.cu:2742
  std::vector<R> yhist;
  const bool keep_y = !q.getyk_rebuild || !q.end_uses_ckpt_y;
  if (keep_y) yhist.resize((size_t)std::max(st.maxInterIts, 1) * in * S);
  auto slot = [&](std::vector<R>& v, int j, int s) { return &v[((size_t)j * in + s) * S]; };

  std::vector<double> gc_storage(in * HW, 0), gx_storage(in * 2 * HW, 0), gy_storage(in * 2 * HW, 0),
      gb_storage(in * CHW, 0);  // TGV.cu:2744-2747

  int lastIt = its;
  const int nseg = (int)st.iterations.size();
  for (int outer = nseg - 1; outer >= 0; outer--) {  // TGV.cu:2751-2948
    const int nextLastIt = st.iterations[outer];
    y0 = st.intermediate_y[outer];
    y1 = st.intermediate_y[outer];
    dout = st.intermediate_x[outer];
    const int npairs = (lastIt - nextLastIt) / 2;
    for (int s = 0; s < in; s++) {
      const Weights<R>& wt = wts[s];
      const R *cs = d_c + s * HW, *bs = d_b + s * CHW;
      for (int it = 0; it < npairs; it++) {  // recompute, TGV.cu:2775-2814
        R step = st.stepSizes[nextLastIt + 2 * it];
        forward_iter<R>(wt, cs, bs, &dout[s * S], &y0[s * S], &y1[s * S], slot(xk05, 2 * it, s), ic, ih, iw, step, oneL);
        if (keep_y) std::memcpy(slot(yhist, 2 * it, s), &y1[s * S], S * sizeof(R));
        step = st.stepSizes[nextLastIt + 2 * it + 1];
        forward_iter<R>(wt, cs, bs, &dout[s * S], &y1[s * S], &y0[s * S], slot(xk05, 2 * it + 1, s), ic, ih, iw, step, oneL);
        if (keep_y) std::memcpy(slot(yhist, 2 * it + 1, s), &y0[s * S], S * sizeof(R));
      }
      for (int it = npairs - 1; it >= 0; it--) {  // reverse sweep, TGV.cu:2851-2933
        R step = st.stepSizes[nextLastIt + 2 * it + 1];
        if (outer == nseg - 1 && it == npairs - 1) {
          // the upstream gradient is read from the caller's tensor (d_gin), TGV.cu:2863-2864
          init_adjoint<R>(cs, bs, slot(xk05, 2 * it + 1, s), &gc[s * HW], &gb[s * CHW], &g05_1[s * S],
                          d_inGrad + s * S, ic, ih, iw, m);
        } else {
          const R* ysrc;
          if (q.getyk_rebuild) {
            get_yk<R>(cs, bs, slot(xk05, 2 * it + 1, s), slot(xk05, 2 * it, s), &yk[s * S], ic, ih, iw, step);
            ysrc = &yk[s * S];
          } else {
            ysrc = slot(yhist, 2 * it + 1, s);
          }
          adjoint_iter<R>(wt, cs, bs, slot(xk05, 2 * it + 1, s), &gc[s * HW], &gb[s * CHW], &gx[s * 2 * HW],
                          &gy[s * 2 * HW], &g05_0[s * S], &g05_1[s * S], &gxk0[s * S], &gxk1[s * S], ysrc,
                          ic, ih, iw, step, oneL, m, false, q.clamp != 0, q.dw_div != 0);
        }
        step = st.stepSizes[nextLastIt + 2 * it];
        if (it > 0) {
          const R* ysrc;
          if (q.getyk_rebuild) {
            get_yk<R>(cs, bs, slot(xk05, 2 * it, s), slot(xk05, 2 * it - 1, s), &yk[s * S], ic, ih, iw, step);
            ysrc = &yk[s * S];
          } else {
            ysrc = slot(yhist, 2 * it, s);
          }
          adjoint_iter<R>(wt, cs, bs, slot(xk05, 2 * it, s), &gc[s * HW], &gb[s * CHW], &gx[s * 2 * HW],
                          &gy[s * 2 * HW], &g05_1[s * S], &g05_0[s * S], &gxk1[s * S], &gxk0[s * S], ysrc,
                          ic, ih, iw, step, oneL, m, false, q.clamp != 0, q.dw_div != 0);
        } else {
          // TGV.cu:2914-2917: the checkpoint y stands in for y_{k0+1}
          const R* ysrc = q.end_uses_ckpt_y ? &st.intermediate_y[outer][s * S] : slot(yhist, 0, s);
          adjoint_iter<R>(wt, cs, bs, slot(xk05, 0, s), &gc[s * HW], &gb[s * CHW], &gx[s * 2 * HW],
                          &gy[s * 2 * HW], &g05_1[s * S], &g05_0[s * S], &gxk1[s * S], &gxk0[s * S], ysrc,
                          ic, ih, iw, step, oneL, m, q.end_uses_ckpt_y != 0, q.clamp != 0, q.dw_div != 0);
        }
      }
    }
    // copy_and_set_to_0, TGVH.cu:178-216, TGV.cu:2944
    for (size_t i = 0; i < gc.size(); i++) { gc_storage[i] = (double)gc[i] + gc_storage[i] / 1.; gc[i] = 0; }
    for (size_t i = 0; i < gx.size(); i++) { gx_storage[i] = (double)gx[i] + gx_storage[i] / 1.; gx[i] = 0; }
    for (size_t i = 0; i < gy.size(); i++) { gy_storage[i] = (double)gy[i] + gy_storage[i] / 1.; gy[i] = 0; }
    for (size_t i = 0; i < gb.size(); i++) { gb_storage[i] = (double)gb[i] + gb_storage[i] / 1.; gb[i] = 0; }
    lastIt = nextLastIt;
  }

  std::vector<R> gi(gxk1);  // g_x[1], all three variables
  if (!q.skip_iter0_adjoint && its / 2 > 0) {
    // true gradient wrt init: J^T(y_0) g05[0] + g_x[0]; weight gradients get iteration 0's term
    std::fill(gx.begin(), gx.end(), R(0));
    std::fill(gy.begin(), gy.end(), R(0));
    for (int s = 0; s < in; s++) {
      const R* yv = &st.intermediate_y[0][s * S];
      const R* gv = &g05_0[s * S];
      for (int h = 0; h < ih; h++)
        for (int w = 0; w < iw; w++)
          for (int ch = 0; ch < ic; ch++) {
            const size_t p = (size_t)h * iw + w, o = ch * HW;
            R a, b1, b2;
            jt_main_px<R>(yv + o, yv + CHW + o, yv + 2 * CHW + o, gv + o, gv + CHW + o, gv + 2 * CHW + o,
                          wts[s], h, w, ih, iw, gx[s * 2 * HW + p], gx[s * 2 * HW + HW + p],
                          gy[s * 2 * HW + p], gy[s * 2 * HW + HW + p], R(m.gx), oneL, q.dw_div != 0, a, b1, b2);
            gi[s * S + o + p] = a + gxk0[s * S + o + p];
            gi[s * S + CHW + o + p] = b1 + gxk0[s * S + CHW + o + p];
            gi[s * S + 2 * CHW + o + p] = b2 + gxk0[s * S + 2 * CHW + o + p];
          }
    }
    for (size_t i = 0; i < gx.size(); i++) { gx_storage[i] += (double)gx[i]; gy_storage[i] += (double)gy[i]; }
  }

  if (q.guard) {  // TGV.cu:2990-3021
    double run_step = double(st.run) / double(st.run + 1);
    double is_largest = 0, av_gc = 0;
    int num_above = 0, invalid = 0;
    check_gradUpdate(gc_storage.data(), gc_storage.size(), av_gc, is_largest, num_above, st.av_GC, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GC, gc_storage.data(), gc_storage.size(), run_step);
    check_gradUpdate(gx_storage.data(), gx_storage.size(), av_gc, is_largest, num_above, st.av_GX, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GX, gx_storage.data(), gx_storage.size(), run_step);
    check_gradUpdate(gy_storage.data(), gy_storage.size(), av_gc, is_largest, num_above, st.av_GY, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GY, gy_storage.data(), gy_storage.size(), run_step);
    check_gradUpdate(gb_storage.data(), gb_storage.size(), av_gc, is_largest, num_above, st.av_GB, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GB, gb_storage.data(), gb_storage.size(), run_step);
    // TGV.cu:3014-3021: only the first C*H*W floats (the u gradient) are inspected and rewritten.
    // With a batch that is the u block of every sample.
    std::vector<R> vf(in * CHW);
    for (int s = 0; s < in; s++) std::copy(&gi[s * S], &gi[s * S] + CHW, &vf[s * CHW]);
    check_gradUpdate(vf.data(), vf.size(), av_gc, is_largest, num_above, st.av_GI, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GI, vf.data(), vf.size(), run_step);
    for (int s = 0; s < in; s++) std::copy(&vf[s * CHW], &vf[s * CHW] + CHW, &gi[s * S]);
  }

  // TGV.cu:3024-3050
  for (size_t i = 0; i < in * HW; i++) d_outGradC[i] = (R)(gc_storage[i] * globalMult);
  for (int s = 0; s < in; s++) {
    const double L = wts[s].L;
    for (size_t i = 0; i < 2 * HW; i++) {
      d_outGradX[s * 2 * HW + i] = (R)(L * (double)(R)(gx_storage[s * 2 * HW + i] * globalMult));
      d_outGradY[s * 2 * HW + i] = (R)(L * (double)(R)(gy_storage[s * 2 * HW + i] * globalMult));
    }
  }
  for (size_t i = 0; i < in * CHW; i++) d_outGradB[i] = (R)(gb_storage[i] * globalMult);
  for (size_t i = 0; i < in * S; i++) d_outGradI[i] = gi[i];
  st.run++;  // TGV.cu:3061
  return 0;
}

}  // namespace

extern "C" {

int tgv_oracle_forward(const float* dx, const float* dy, const float* c, const float* b,
                       const float* init, float* out, int n, int ic, int ih, int iw, int its, int id) {
  return forward<float>(dx, dy, c, b, init, out, n, ic, ih, iw, its, id);
}
int tgv_oracle_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin,
                        float* gx, float* gy, float* gc, float* gb, float* gi, int n, int ic, int ih,
                        int iw, int its, int id) {
  return backward<float>(dx, dy, c, b, gin, gx, gy, gc, gb, gi, n, ic, ih, iw, its, id);
}
int tgv_oracle_forward_f64(const double* dx, const double* dy, const double* c, const double* b,
                           const double* init, double* out, int n, int ic, int ih, int iw, int its, int id) {
  return forward<double>(dx, dy, c, b, init, out, n, ic, ih, iw, its, id);
}
int tgv_oracle_backward_f64(const double* dx, const double* dy, const double* c, const double* b,
                            double* gin, double* gx, double* gy, double* gc, double* gb, double* gi,
                            int n, int ic, int ih, int iw, int its, int id) {
  return backward<double>(dx, dy, c, b, gin, gx, gy, gc, gb, gi, n, ic, ih, iw, its, id);
}

// quirk toggles, in the order of struct Quirks; all 1 = literal reference behaviour
void tgv_oracle_set_quirks(int end_uses_ckpt_y, int skip_iter0_adjoint, int getyk_rebuild,
                           int scale_factors, int clamp, int guard, int dw_div) {
  g_quirks.end_uses_ckpt_y = end_uses_ckpt_y;
  g_quirks.skip_iter0_adjoint = skip_iter0_adjoint;
  g_quirks.getyk_rebuild = getyk_rebuild;
  g_quirks.scale_factors = scale_factors;
  g_quirks.clamp = clamp;
  g_quirks.guard = guard;
  g_quirks.dw_div = dw_div;
}

void tgv_oracle_reset_id(int id) {
  if (id < 0 || id >= kUniqueIds) return;
  states<float>()[id] = IdState<float>();
  states<double>()[id] = IdState<double>();
}

// state6 = {run, av_GC, av_GX, av_GY, av_GB, av_GI}
int tgv_oracle_get_state(int id, double* state6, int f64) {
  if (id < 0 || id >= kUniqueIds) return 1;
  if (f64) {
    auto& s = states<double>()[id];
    state6[0] = s.run; state6[1] = s.av_GC; state6[2] = s.av_GX; state6[3] = s.av_GY; state6[4] = s.av_GB; state6[5] = s.av_GI;
  } else {
    auto& s = states<float>()[id];
    state6[0] = s.run; state6[1] = s.av_GC; state6[2] = s.av_GX; state6[3] = s.av_GY; state6[4] = s.av_GB; state6[5] = s.av_GI;
  }
  return 0;
}
int tgv_oracle_set_state(int id, const double* state6) {
  if (id < 0 || id >= kUniqueIds) return 1;
  auto& s = states<float>()[id];
  s.run = (int)state6[0]; s.av_GC = state6[1]; s.av_GX = state6[2]; s.av_GY = state6[3]; s.av_GB = state6[4]; s.av_GI = state6[5];
  auto& d = states<double>()[id];
  d.run = (int)state6[0]; d.av_GC = state6[1]; d.av_GX = state6[2]; d.av_GY = state6[3]; d.av_GB = state6[4]; d.av_GI = state6[5];
  return 0;
}

// Lipschitz bound of one sample from the unscaled fields dx, dy: (2,H,W).  Returns L; the
// per-pixel bound goes to storage (H*W floats) when non-null.
double tgv_oracle_lipschitz(const float* dx, const float* dy, int ih, int iw, float* storage) {
  const size_t HW = (size_t)ih * iw;
  return lipschitz<float>(dx, dy, dx + HW, dy + HW, ih, iw, storage);
}
double tgv_oracle_lipschitz_f64(const double* dx, const double* dy, int ih, int iw, double* storage) {
  const size_t HW = (size_t)ih * iw;
  return lipschitz<double>(dx, dy, dx + HW, dy + HW, ih, iw, storage);
}

// one forward iteration on one sample; dx, dy are the unscaled (2,H,W) fields, x/y/yout/x05 (3,C,H,W)
void tgv_oracle_forward_iter(const float* dx, const float* dy, const float* c, const float* b, float* x,
                             const float* y, float* yout, float* x05, int ic, int ih, int iw, float t) {
  Weights<float> wt;
  wt.build(dx, dy, ih, iw);
  forward_iter<float>(wt, c, b, x, y, yout, x05, ic, ih, iw, t, 1.0f);
}
void tgv_oracle_forward_iter_f64(const double* dx, const double* dy, const double* c, const double* b,
                                 double* x, const double* y, double* yout, double* x05, int ic, int ih,
                                 int iw, double t) {
  Weights<double> wt;
  wt.build(dx, dy, ih, iw);
  forward_iter<double>(wt, c, b, x, y, yout, x05, ic, ih, iw, t, 1.0);
}

// Transposed Jacobian of the gradient step alone (no momentum, no prox) on one single-channel
// sample in double precision: out (3,H,W) = J(y)^T g, gw (4,H,W) = the weight-gradient
// increments (gwx ch0, gwx ch1, gwy ch0, gwy ch1) with multiplier 1.  end_form selects the
// segment-start kernel's arithmetic, q7 the division quirk of the main form.
void tgv_oracle_jt_f64(const double* dx, const double* dy, const double* y, const double* g, int ih,
                       int iw, int end_form, int q7, double* out, double* gw) {
  Weights<double> wt;
  wt.build(dx, dy, ih, iw);
  const size_t HW = (size_t)ih * iw;
  std::fill(gw, gw + 4 * HW, 0.0);
  for (int h = 0; h < ih; h++)
    for (int w = 0; w < iw; w++) {
      const size_t p = (size_t)h * iw + w;
      if (end_form)
        jt_end_px<double>(y, y + HW, y + 2 * HW, g, g + HW, g + 2 * HW, wt, h, w, ih, iw, gw[p], gw[HW + p],
                          gw[2 * HW + p], gw[3 * HW + p], 1.0, 1.0, out[p], out[HW + p], out[2 * HW + p]);
      else
        jt_main_px<double>(y, y + HW, y + 2 * HW, g, g + HW, g + 2 * HW, wt, h, w, ih, iw, gw[p], gw[HW + p],
                           gw[2 * HW + p], gw[3 * HW + p], 1.0, 1.0, q7 != 0, out[p], out[HW + p], out[2 * HW + p]);
    }
}

// guard on a double vector (tensors C, X, Y, B) or a float vector (tensor I).
// stats4 = {av_gc, is_largest, num_above, invalid}.  Returns 0 plain / 1 rescaled / 2 killed.
int tgv_oracle_guard_f64(double* g, long n, int run, double* av, double* stats4) {
  double run_step = double(run) / double(run + 1);
  double av_gc = 0, is_largest = 0;
  int num_above = 0, invalid = 0;
  check_gradUpdate(g, (size_t)n, av_gc, is_largest, num_above, *av, invalid);
  int r = update_correct_av_step_host(run, av_gc, *av, g, (size_t)n, run_step);
  stats4[0] = av_gc; stats4[1] = is_largest; stats4[2] = num_above; stats4[3] = invalid;
  return r;
}
int tgv_oracle_guard_f32(float* g, long n, int run, double* av, double* stats4) {
  double run_step = double(run) / double(run + 1);
  double av_gc = 0, is_largest = 0;
  int num_above = 0, invalid = 0;
  check_gradUpdate(g, (size_t)n, av_gc, is_largest, num_above, *av, invalid);
  int r = update_correct_av_step_host(run, av_gc, *av, g, (size_t)n, run_step);
  stats4[0] = av_gc; stats4[1] = is_largest; stats4[2] = num_above; stats4[3] = invalid;
  return r;
}

void tgv_oracle_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n > 0 ? n : 1);
#else
  (void)n;
#endif
}

}  // extern "C"
