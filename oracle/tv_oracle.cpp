// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's Huber-TV FISTA inpainting layer.
//
// Nothing in the shipped package may import, link or call this file.  It exists so that the
// parity tests, the smoke check and the bench's cpu_baseline leg have something to compare the
// HIP path against.  Every function cites the reference lines it restates
// (paths relative to the reference root; TV.cu = cudaTV/cudaCode/TVInpaintFista.cu,
// TV.h = cudaTV/cudaCode/TVInpaintFista.h).
//
// Arithmetic conventions (chosen once, used by both this file and the HIP kernels):
//   * every floating-point expression is evaluated left to right exactly as written in the
//     reference source, in the type C++ promotion rules give it (a literal such as `1.` makes
//     the surrounding sub-expression double, as it does under nvcc);
//   * no fused multiply-add contraction (build with -ffp-contract=off); division and sqrt are
//     the correctly rounded IEEE ones.
// The reference's own build lets nvcc contract a*b+c into FMAs; that choice is not recoverable
// from the sources, so results agree with a CUDA run only to rounding (see the headers of
// tests/test_tv_oracle_pins.py and tests/test_tv_quirk_pins.py for what is pinned and how).
//
// Pin status of the functions below:
//   forward iteration / schedule / step sizes / prox ......... pinned (closed forms, sparse
//       Laplacian, convex fixed point, invariants)
//   adjoint chain with all quirk toggles OFF .................. pinned (autograd of an
//       independently written forward, finite differences)
//   what the backward pass does differently from the chain rule -- y rebuilt by the get_yk rule,
//   the checkpointed y at segment starts, the skipped Jacobian of iteration 0, the clamp
//       ............................................................ pinned one at a time
//       (tests/test_tv_quirk_pins.py: the exact adjoint recursion with autograd Jacobian products
//       and that one deviation; c = 0, regimes that never change, a fixed point and a sub-run
//       started at x_1 as model-free special cases); multipliers and the guard: ratio / table
//       tests in tests/test_tv_oracle_pins.py.
//   The numeric constants themselves (0.1, 1e4, 0.1 / 0.1 / 1.0 / 0.1, 50, 10, 0.975, 1e7) are
//   values read off the reference source; nothing else can fix them.
//
// The batch dimension n is an extension (the reference accepts n == 1 only, TV.cpp:61-65):
// samples are independent problems; guard statistics run over the whole batch tensor.

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

constexpr int kUniqueIds = 10;          // TV.h:5
constexpr int kMaxCheckpoints = 100;    // TV.h:9-15 (vectors of 100 entries)

// TV.cu:44,52,63-69,84-90
constexpr float kHDelta = 0.1f;
constexpr float kClipLocalGrad = 10000.0f;
constexpr float kLocalGCMult = 0.1f;
constexpr float kLocalGXMult = 0.1f;
constexpr float kLocalGBMult = 1.0f;
constexpr float kGlobalGMult = 0.1f;
constexpr double kKillT = 50.;
constexpr double kScaleT = 10.;
constexpr double kMemoryT = 0.975;

struct Quirks {
  int end_uses_ckpt_y = 1;     // adjoint of a segment's first iteration linearises at the checkpoint y (TV.cu:1724-1727)
  int skip_iter0_adjoint = 1;  // the gradient step of iteration 0 is never back-propagated (TV.cu:1696-1729,1816)
  int getyk_rebuild = 1;       // y is rebuilt from x05 by the get_yk rule (TV.cu:1130-1189); 0: use the y the recompute produced
  int scale_factors = 1;       // local/global gradient multipliers (TV.cu:63-69); 0: all 1
  int clamp = 1;               // clipLocalGrad (TV.cu:797-799)
  int guard = 1;               // upstream scrub + output guard (TV.cu:1609-1623,1760-1792)
};
Quirks g_quirks;

template <class R>
struct IdState {  // TV.h:7-50
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

// TV.cu:94-113
template <typename T>
bool is_valid(const T& value) {
  T max_value = std::numeric_limits<T>::max();
  T min_value = -max_value;
  bool is_inf = !(min_value <= value && value <= max_value);
  bool is_nan = value != value;
  return !is_inf && !is_nan;
}

// TV.cu:158-175
template <typename S>
void check_gradUpdate(std::vector<S>& tempc, double& av_gc, double& is_largest, int& num_above,
                      double av_gc_current, int& invalid) {
  const double maxTolerance = 10000000.;
  is_largest = 0;
  num_above = 0;
  av_gc = 0;
  invalid = 0;
  for (size_t i = 0; i < tempc.size(); i++)
    if (is_valid(tempc[i])) {
      double tca = std::abs(tempc[i]);
      double step = double(i) / double(i + 1);
      av_gc = (1. - step) * tca + step * av_gc;
      is_largest = std::max(tca, is_largest);
      if (tca > maxTolerance) {
        tempc[i] = 0;
        num_above++;
      }
    } else {
      tempc[i] = 0;
      av_gc = av_gc_current * 1000.;
      invalid++;
    }
}

// TV.cu:128-155.  Returns 0 = plain running-mean update, 1 = rescaled, 2 = killed.
template <typename S>
int update_correct_av_step_host(int run, double av_gc, double& av_GC, std::vector<S>& tempc,
                                double run_step) {
  if (run >= 10 && av_GC * kKillT < av_gc) {
    for (size_t i = 0; i < tempc.size(); i++) tempc[i] = 0.0;
    av_GC = av_GC * run_step + (1. - run_step) * kScaleT * av_GC;
    return 2;
  }
  const double scale = kScaleT;
  if (run >= 10 && av_GC * scale < av_gc) {
    double mult = scale * av_GC / av_gc;
    for (size_t i = 0; i < tempc.size(); i++) tempc[i] *= mult;
    av_GC = av_GC * run_step + (1. - run_step) * av_gc * mult;
    return 1;
  } else {
    av_GC = av_GC * run_step + (1. - run_step) * av_gc;
  }
  return 0;
}

// Checkpoint schedule, TV.cu:1499-1508,1523.
void make_schedule(int its, std::vector<int>& iterations, int& maxInterIts) {
  iterations.assign((size_t)std::floor(std::sqrt((double)its)), 0);
  maxInterIts = 0;
  for (size_t i = 0; i < iterations.size(); i++) {
    iterations[i] = (int)(std::floor(i * std::sqrt((double)its) * 0.5) * 2);
    if (i > 0) maxInterIts = std::max(maxInterIts, iterations[i] - iterations[i - 1]);
  }
  if (!iterations.empty()) maxInterIts = std::max(maxInterIts, its - iterations.back());
}

// FISTA extrapolation factors, TV.cu:1525-1532 (computed in double, stored as float).
void make_step_sizes(int its, std::vector<float>& stepSizes) {
  stepSizes.assign((size_t)std::max(its, 0), 0.f);
  double t(1), t_(1);
  for (size_t i = 0; i < stepSizes.size(); i++) {
    t_ = t;
    t = (1. + std::sqrt(1. + 4. * t * t)) / 2.;
    stepSizes[i] = (float)std::max(0.0, (t_ - 1.) / t);
  }
}

// Shared-memory tile read with zero padding outside the image (TV.cu:1229,1237).
template <class R>
inline R padded(const R* f, int h, int w, int H, int W) {
  return (h >= 0 && h < H && w >= 0 && w < W) ? f[(size_t)h * W + w] : R(0);
}

// One forward iteration on one sample: TV.cu:1194-1319 (x05 == nullptr) and 1321-1455 (x05 given).
// wx, wy are the L-scaled private copies (TV.cu:1483-1489); y and yout must not alias.
template <class R>
void forward_iter(const R* wx, const R* wy, const R* cf, const R* b, R* x, const R* y, R* yout,
                  R* x05, int C, int H, int W, R t) {
  const size_t HW = (size_t)H * W;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      const R wx_0 = (w > 0) ? wx[p - 1] : R(0);
      const R wx_1 = (w < W - 1) ? wx[p] : R(0);
      const R wy_0 = (h > 0) ? wy[p - W] : R(0);
      const R wy_1 = (h < H - 1) ? wy[p] : R(0);
      const R wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : R(0);
      const R wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : R(0);
      const R delta = R(kHDelta);
      for (int ch = 0; ch < C; ch++) {
        const R* yc_ = y + ch * HW;
        const R x_ = x[ch * HW + p];
        const R bb = b[ch * HW + p];
        R x_loc = bb;
        R yc = yc_[p];
        R yt = yc;
        if (h > 0) {  // TV.cu:1250-1259
          const R yu = padded(yc_, h - 1, w, H, W), yur = padded(yc_, h - 1, w + 1, H, W);
          R hub_weight = std::sqrt((yc - yu) * (yc - yu) * wy_0 + (yu - yur) * (yu - yur) * wx_2);
          yt -= (yc - yu) * (wy_0 / std::fmax(R(1), hub_weight / delta));
        }
        if (w > 0) {  // TV.cu:1260-1266
          const R yl = padded(yc_, h, w - 1, H, W), yld = padded(yc_, h + 1, w - 1, H, W);
          R hub_weight = std::sqrt((yc - yl) * (yc - yl) * wx_0 + (yl - yld) * (yl - yld) * wy_2);
          yt -= (yc - yl) * (wx_0 / std::fmax(R(1), hub_weight / delta));
        }
        {  // TV.cu:1268-1274
          const R yd = padded(yc_, h + 1, w, H, W), yr = padded(yc_, h, w + 1, H, W);
          R hub_weight = std::sqrt((yc - yd) * (yc - yd) * wy_1 + (yc - yr) * (yc - yr) * wx_1);
          yt -= (yc - yd) * (wy_1 / std::fmax(R(1), hub_weight / delta));
          yt -= (yc - yr) * (wx_1 / std::fmax(R(1), hub_weight / delta));
        }
        if (x05) x05[ch * HW + p] = yt;  // TV.cu:1414
        // Huber-1 data prox, TV.cu:1286-1292
        x_loc = (conf * bb + yt) / (R(1) + conf);
        yc = yt - conf;
        yt = yt + conf;
        if (yc > R(1) + bb) x_loc = yc;
        if (yt < bb - R(1)) x_loc = yt;
        // momentum, TV.cu:1315-1316
        yout[ch * HW + p] = x_loc + t * (x_loc - x_);
        x[ch * HW + p] = x_loc;
      }
    }
}

// TV.cu:1130-1189 (Huber-1 branch): rebuild y_{k+1} from x05[it], x05[it-1].
template <class R>
void get_yk(const R* cf, const R* b, const R* x05_it, const R* x05_itm1, R* yk_out, int C, int H,
            int W, R t) {
  const size_t HW = (size_t)H * W;
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
      }
    }
}

struct Mults {
  float gc, gx, gb;
};

// Prox adjoint + confidence / rhs gradient of one channel value, shared tail of
// TV.cu:240-255 (init), 806-828 (bw_yk) and the same lines of the end kernel.
// `init_kernel` selects the init kernel's `d_gb = 0` assignment (TV.cu:254).
template <class R>
inline void prox_adjoint(R df_dxk, R bb, R x05v, R conf, R& g05_out, R& gc_acc, R& gb_acc,
                         const Mults& m, bool init_kernel) {
  const R diff = bb - x05v;
  const R sign = (diff < 0) ? R(-1.) : R(1.);
  if (1. + (double)conf >= (double)(sign * diff)) {
    if (init_kernel) {  // statement order of TV.cu:246-248
      g05_out = df_dxk / (R(1) + conf);
      gc_acc += df_dxk * (bb / (R(1) + conf) - (conf * bb + x05v) / ((R(1) + conf) * (R(1) + conf))) * R(m.gc);
      gb_acc += df_dxk * conf / (R(1) + conf) * R(m.gb);
    } else {  // TV.cu:812-814
      gc_acc += df_dxk * (bb / (R(1) + conf) - (conf * bb + x05v) / ((R(1) + conf) * (R(1) + conf))) * R(m.gc);
      g05_out = df_dxk / (R(1) + conf);
      gb_acc += df_dxk * conf / (R(1) + conf) * R(m.gb);
    }
  } else {
    if (init_kernel) {  // TV.cu:252-254
      g05_out = df_dxk;
      gc_acc += sign * df_dxk * R(m.gc);
      gb_acc = 0;
    } else if (conf >= sign * diff) {  // TV.cu:818-822 (unreachable for conf >= 0, restated)
      g05_out = 0;
      gb_acc += df_dxk * R(m.gb);
    } else {  // TV.cu:825-826
      g05_out = df_dxk;
      gc_acc += sign * df_dxk * R(m.gc);
    }
  }
}

// TV.cu:222-287 on one sample.
template <class R>
void init_adjoint(const R* cf, const R* b, const R* x05_it, R* gc, R* gb, R* g05, const R* gin,
                  int C, int H, int W, const Mults& m) {
  const size_t HW = (size_t)H * W;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      for (int ch = 0; ch < C; ch++) {
        const size_t q = ch * HW + p;
        prox_adjoint<R>(gin[q], b[q], x05_it[q], conf, g05[q], gc[p], gb[q], m, true);
      }
    }
}

// Transposed Jacobian of the Huber-TV gradient step at one pixel of one channel plus the
// pixel's own-triangle weight gradients: TV.cu:651-771 (`end_form` == false) and the same
// block of the end kernel TV.cu:922-1040 (`end_form` == true; identical algebra, different
// operand order in the active-triangle weight gradient).
template <class R>
inline R jt_gradstep_px(const R* y, const R* g, const R* wx, const R* wy, int h, int w, int H,
                        int W, R& gwx_p, R& gwy_p, R gxmult, bool end_form) {
  const size_t p = (size_t)h * W + w;
  const R delta = R(kHDelta);
  const R wx_0 = (w > 0) ? wx[p - 1] : R(0);
  const R wx_1 = (w < W - 1) ? wx[p] : R(0);
  const R wy_0 = (h > 0) ? wy[p - W] : R(0);
  const R wy_1 = (h < H - 1) ? wy[p] : R(0);
  const R yk = y[p];
  const R df_dy = g[p];
  R df_dy_t = df_dy;
  if (h > 0) {  // triangle owned by the pixel above, TV.cu:655-686
    const R wx_2 = (h > 0 && w < W - 1) ? wx[p - W] : R(0);
    const R yu = padded(y, h - 1, w, H, W), yur = padded(y, h - 1, w + 1, H, W);
    const R gu = padded(g, h - 1, w, H, W), gur = padded(g, h - 1, w + 1, H, W);
    const R wy_nyy2_T2 = (yk - yu) * (yk - yu) * wy_0;
    const R wx_nyx2_T2 = (yu - yur) * (yu - yur) * wx_2;
    const R hub_weight = std::sqrt(wx_nyx2_T2 + wy_nyy2_T2);
    if (hub_weight > delta) {
      const R nom = delta / hub_weight;
      const R denom = nom / (R(2) * hub_weight * hub_weight);
      df_dy_t -= (df_dy - gu) * (wy_0 * nom);
      const R temp = -denom * R(2) * (yk - yu) * wy_0;
      df_dy_t -= (df_dy - gu) * wy_0 * (yk - yu) * temp;
      df_dy_t -= (gur - gu) * wx_2 * (yur - yu) * temp;
    } else {
      df_dy_t -= (df_dy - gu) * wy_0;
    }
  }
  if (w > 0) {  // triangle owned by the pixel to the left, TV.cu:687-720
    const R wy_2 = (w > 0 && h < H - 1) ? wy[p - 1] : R(0);
    const R yl = padded(y, h, w - 1, H, W), yld = padded(y, h + 1, w - 1, H, W);
    const R gl = padded(g, h, w - 1, H, W), gld = padded(g, h + 1, w - 1, H, W);
    const R wx_nyx2_T1 = (yk - yl) * (yk - yl) * wx_0;
    const R wy_nyy2_T1 = (yl - yld) * (yl - yld) * wy_2;
    const R hub_weight = std::sqrt(wx_nyx2_T1 + wy_nyy2_T1);
    if (hub_weight > delta) {
      const R nom = delta / hub_weight;
      const R denom = nom / (R(2) * hub_weight * hub_weight);
      df_dy_t -= (df_dy - gl) * (wx_0 * nom);
      const R temp = -denom * R(2) * (yk - yl) * wx_0;
      df_dy_t -= (df_dy - gl) * wx_0 * (yk - yl) * temp;
      df_dy_t -= (gld - gl) * wy_2 * (yld - yl) * temp;
    } else {
      df_dy_t -= (df_dy - gl) * wx_0;
    }
  }
  {  // the pixel's own triangle, TV.cu:722-771
    const R yr = padded(y, h, w + 1, H, W), yd = padded(y, h + 1, w, H, W);
    const R gr = padded(g, h, w + 1, H, W), gd = padded(g, h + 1, w, H, W);
    const R wx_nyx2_T0 = (yk - yr) * (yk - yr) * wx_1;
    const R wy_nyy2_T0 = (yk - yd) * (yk - yd) * wy_1;
    const R hub_weight = std::sqrt(wx_nyx2_T0 + wy_nyy2_T0);
    if (hub_weight > delta) {
      const R nom = delta / hub_weight;
      const R denom = nom / (R(2) * hub_weight * hub_weight);
      df_dy_t -= (df_dy - gd) * (wy_1 * nom);
      df_dy_t -= (df_dy - gr) * (wx_1 * nom);
      const R temp = denom * R(2) * ((yd - yk) * wy_1 + (yr - yk) * wx_1);
      df_dy_t -= (df_dy - gd) * wy_1 * (yk - yd) * temp;
      df_dy_t -= (df_dy - gr) * wx_1 * (yk - yr) * temp;
      if (!end_form) {  // TV.cu:749-759
        if (w < W - 1)
          gwx_p = gwx_p - gxmult * (yk - yr) *
                              ((df_dy - gr) * (nom - wx_nyx2_T0 * denom) -
                               (df_dy - gd) * (yk - yr) * (yk - yd) * denom * wy_1);
        if (h < H - 1)
          gwy_p = gwy_p - gxmult * (yk - yd) *
                              ((df_dy - gd) * (nom - wy_nyy2_T0 * denom) -
                               (df_dy - gr) * (yk - yd) * (yk - yr) * denom * wx_1);
      } else {  // TV.cu:1019-1027
        if (w < W - 1)
          gwx_p = gwx_p - gxmult * ((df_dy - gr) * (yk - yr) * (nom - wx_nyx2_T0 * denom) -
                                    (df_dy - gd) * (yk - yr) * (yk - yr) * (yk - yd) * denom * wy_1);
        if (h < H - 1)
          gwy_p = gwy_p - gxmult * ((df_dy - gd) * (yk - yd) * (nom - wy_nyy2_T0 * denom) -
                                    (df_dy - gr) * (yk - yd) * (yk - yd) * (yk - yr) * denom * wx_1);
      }
    } else {  // TV.cu:763-769
      df_dy_t -= (df_dy - gd) * wy_1;
      df_dy_t -= (df_dy - gr) * wx_1;
      if (w < W - 1) gwx_p = gwx_p - gxmult * (yk - yr) * (df_dy - gr);
      if (h < H - 1) gwy_p = gwy_p - gxmult * (yk - yd) * (df_dy - gd);
    }
  }
  return df_dy_t;
}

// One reverse step on one sample: TV.cu:586-859 (bw_yk) / 862-1126 (end).  g05_in/g05_out and
// gxk/gxk_m1 are the ping-pong pairs of TV.cu:1638-1641; y is y_{k+1} (or the checkpoint y for
// the end kernel).
template <class R>
void adjoint_iter(const R* wx, const R* wy, const R* cf, const R* b, const R* x05_it, R* gc,
                  R* gb, R* gwx, R* gwy, const R* g05_in, R* g05_out, R* gxk, R* gxk_m1,
                  const R* y, int C, int H, int W, R t, const Mults& m, bool end_form,
                  bool clamp) {
  const size_t HW = (size_t)H * W;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      const R conf = cf[p];
      for (int ch = 0; ch < C; ch++) {
        const size_t q = ch * HW + p;
        const R df_dy_t = jt_gradstep_px<R>(y + ch * HW, g05_in + ch * HW, wx, wy, h, w, H, W,
                                            gwx[p], gwy[p], R(m.gx), end_form);
        // momentum adjoint, TV.cu:796-801 (the literal `1.` makes the product double)
        R df_dxk = (R)((double)gxk[q] + (1. + (double)t) * (double)df_dy_t);
        if (clamp) df_dxk = std::fmax(-R(kClipLocalGrad), std::fmin(df_dxk, R(kClipLocalGrad)));  // CUDA max/min semantics
        gxk[q] = df_dxk;
        gxk_m1[q] = -t * df_dy_t;
        prox_adjoint<R>(df_dxk, b[q], x05_it[q], conf, g05_out[q], gc[p], gb[q], m, false);
      }
    }
}

// J^T only (no momentum / prox); used when the iteration-0 quirk is switched off.
template <class R>
void jt_only(const R* wx, const R* wy, const R* g05_in, const R* y, R* gy_out, R* gwx, R* gwy,
             int C, int H, int W, const Mults& m) {
  const size_t HW = (size_t)H * W;
  for (int h = 0; h < H; h++)
    for (int w = 0; w < W; w++) {
      const size_t p = (size_t)h * W + w;
      for (int ch = 0; ch < C; ch++)
        gy_out[ch * HW + p] = jt_gradstep_px<R>(y + ch * HW, g05_in + ch * HW, wx, wy, h, w, H, W,
                                                gwx[p], gwy[p], R(m.gx), false);
    }
}

// TV.cu:1463-1559 with a batch loop around it.
template <class R>
int forward(const R* d_x, const R* d_y, const R* d_c, const R* d_b, const R* d_i, R* d_out, int in,
            int ic, int ih, int iw, int its, int id) {
  if (static_cast<size_t>(id) >= (size_t)kUniqueIds) return 1;  // TV.cu:1468-1472
  if (in < 1 || ic < 1 || ih < 1 || iw < 1 || its < 0) return 2;
  if ((int)std::floor(std::sqrt((double)its)) > kMaxCheckpoints) return 3;  // TV.h:9-15
  IdState<R>& st = states<R>()[id];
  const size_t HW = (size_t)ih * iw, CHW = HW * ic;
  const double L = 1. / 8.;  // TV.cu:1478
  std::vector<R> wx(in * HW), wy(in * HW);
  for (size_t i = 0; i < in * HW; i++) {  // TV.cu:1488-1489
    wx[i] = (R)(L * (double)d_x[i]);
    wy[i] = (R)(L * (double)d_y[i]);
  }
  std::vector<R> y0(d_i, d_i + in * CHW), y1(d_i, d_i + in * CHW);  // TV.cu:1495-1497
  std::memcpy(d_out, d_i, in * CHW * sizeof(R));

  make_schedule(its, st.iterations, st.maxInterIts);
  st.intermediate_x.assign(st.iterations.size(), std::vector<R>());
  st.intermediate_y.assign(st.iterations.size(), std::vector<R>());
  make_step_sizes(its, st.stepSizes);
  st.n = in; st.ic = ic; st.ih = ih; st.iw = iw; st.its = its;

  size_t start_it = 0;
  for (int it = 0; it < its / 2; it++) {  // TV.cu:1539-1556
    if (start_it < st.iterations.size() && st.iterations[start_it] == 2 * it) {
      st.intermediate_y[start_it].assign(y0.begin(), y0.end());
      st.intermediate_x[start_it].assign(d_out, d_out + in * CHW);
      start_it++;
    }
    for (int s = 0; s < in; s++) {
      R step = st.stepSizes[2 * it];
      forward_iter<R>(&wx[s * HW], &wy[s * HW], d_c + s * HW, d_b + s * CHW, d_out + s * CHW,
                      &y0[s * CHW], &y1[s * CHW], nullptr, ic, ih, iw, step);
      step = st.stepSizes[2 * it + 1];
      forward_iter<R>(&wx[s * HW], &wy[s * HW], d_c + s * HW, d_b + s * CHW, d_out + s * CHW,
                      &y1[s * CHW], &y0[s * CHW], nullptr, ic, ih, iw, step);
    }
  }
  // Checkpoints the loop never reached (its < 2) stay unset; mirror calloc'ed zeros (TV.cu:1515).
  for (size_t i = 0; i < st.iterations.size(); i++)
    if (st.intermediate_y[i].empty()) {
      st.intermediate_y[i].assign(in * CHW, R(0));
      st.intermediate_x[i].assign(in * CHW, R(0));
    }
  return 0;
}

// TV.cu:1570-1831 with a batch loop around the kernel sequence.
template <class R>
int backward(const R* d_x, const R* d_y, const R* d_c, const R* d_b, R* d_inGrad, R* d_outGradX,
             R* d_outGradY, R* d_outGradC, R* d_outGradB, R* d_outGradI, int in, int ic, int ih,
             int iw, int its, int id) {
  if (static_cast<size_t>(id) >= (size_t)kUniqueIds) return 1;  // TV.cu:1580-1584
  IdState<R>& st = states<R>()[id];
  if (st.its != its || st.n != in || st.ic != ic || st.ih != ih || st.iw != iw) return 4;
  const Quirks q = g_quirks;
  const size_t HW = (size_t)ih * iw, CHW = HW * ic;
  const double L = 1. / 8.;
  Mults m{kLocalGCMult, kLocalGXMult, kLocalGBMult};
  double globalMult = kGlobalGMult;
  if (!q.scale_factors) { m = Mults{1.f, 1.f, 1.f}; globalMult = 1.; }

  std::vector<R> wx(in * HW), wy(in * HW);
  for (size_t i = 0; i < in * HW; i++) {  // TV.cu:1592-1593
    wx[i] = (R)(L * (double)d_x[i]);
    wy[i] = (R)(L * (double)d_y[i]);
  }
  // fp32 per-segment accumulators live in the output tensors, TV.cu:1603-1607
  std::vector<R> gc(in * HW, 0), gx(in * HW, 0), gy(in * HW, 0), gb(in * CHW, 0);

  if (q.guard) {  // TV.cu:1609-1623: scrub non-finite upstream entries in the caller's buffer
    for (size_t i = 0; i < in * CHW; i++)
      if (!is_valid(d_inGrad[i])) d_inGrad[i] = 0;
  }

  std::vector<R> y0(in * CHW), y1(in * CHW), dout(in * CHW);
  std::vector<R> g05_0(in * CHW, 0), g05_1(in * CHW, 0), gxk1(in * CHW, 0), gxk0(in * CHW, 0);  // TV.cu:1638-1648
  std::vector<R> yk(in * CHW, 0);
  std::vector<R> xk05((size_t)std::max(st.maxInterIts, 1) * in * CHW);  // TV.cu:1660, slot-major
  std::vector<R> yhist;  // only for the quirk-free modes
  const bool keep_y = !q.getyk_rebuild || !q.end_uses_ckpt_y;
  if (keep_y) yhist.resize((size_t)std::max(st.maxInterIts, 1) * in * CHW);
  auto slot = [&](std::vector<R>& v, int j, int s) { return &v[((size_t)j * in + s) * CHW]; };

  std::vector<double> gc_storage(in * HW, 0), gx_storage(in * HW, 0), gy_storage(in * HW, 0),
      gb_storage(in * CHW, 0);  // TV.cu:1663-1666

  int lastIt = its;
  const int nseg = (int)st.iterations.size();
  for (int outer = nseg - 1; outer >= 0; outer--) {  // TV.cu:1669-1733
    const int nextLastIt = st.iterations[outer];
    y0 = st.intermediate_y[outer];
    y1 = st.intermediate_y[outer];
    dout = st.intermediate_x[outer];
    const int npairs = (lastIt - nextLastIt) / 2;
    for (int s = 0; s < in; s++) {
      const R *wxs = &wx[s * HW], *wys = &wy[s * HW], *cs = d_c + s * HW, *bs = d_b + s * CHW;
      for (int it = 0; it < npairs; it++) {  // recompute, TV.cu:1678-1687
        R step = st.stepSizes[nextLastIt + 2 * it];
        forward_iter<R>(wxs, wys, cs, bs, &dout[s * CHW], &y0[s * CHW], &y1[s * CHW],
                        slot(xk05, 2 * it, s), ic, ih, iw, step);
        if (keep_y) std::memcpy(slot(yhist, 2 * it, s), &y1[s * CHW], CHW * sizeof(R));
        step = st.stepSizes[nextLastIt + 2 * it + 1];
        forward_iter<R>(wxs, wys, cs, bs, &dout[s * CHW], &y1[s * CHW], &y0[s * CHW],
                        slot(xk05, 2 * it + 1, s), ic, ih, iw, step);
        if (keep_y) std::memcpy(slot(yhist, 2 * it + 1, s), &y0[s * CHW], CHW * sizeof(R));
      }
      for (int it = npairs - 1; it >= 0; it--) {  // reverse sweep, TV.cu:1696-1729
        R step = st.stepSizes[nextLastIt + 2 * it + 1];
        if (outer == nseg - 1 && it == npairs - 1) {
          init_adjoint<R>(cs, bs, slot(xk05, 2 * it + 1, s), &gc[s * HW], &gb[s * CHW],
                          &g05_1[s * CHW], d_inGrad + s * CHW, ic, ih, iw, m);
        } else {
          const R* ysrc;
          if (q.getyk_rebuild) {
            get_yk<R>(cs, bs, slot(xk05, 2 * it + 1, s), slot(xk05, 2 * it, s), &yk[s * CHW], ic,
                      ih, iw, step);
            ysrc = &yk[s * CHW];
          } else {
            ysrc = slot(yhist, 2 * it + 1, s);
          }
          adjoint_iter<R>(wxs, wys, cs, bs, slot(xk05, 2 * it + 1, s), &gc[s * HW], &gb[s * CHW],
                          &gx[s * HW], &gy[s * HW], &g05_0[s * CHW], &g05_1[s * CHW],
                          &gxk0[s * CHW], &gxk1[s * CHW], ysrc, ic, ih, iw, step, m, false,
                          q.clamp != 0);
        }
        step = st.stepSizes[nextLastIt + 2 * it];
        if (it > 0) {
          const R* ysrc;
          if (q.getyk_rebuild) {
            get_yk<R>(cs, bs, slot(xk05, 2 * it, s), slot(xk05, 2 * it - 1, s), &yk[s * CHW], ic,
                      ih, iw, step);
            ysrc = &yk[s * CHW];
          } else {
            ysrc = slot(yhist, 2 * it, s);
          }
          adjoint_iter<R>(wxs, wys, cs, bs, slot(xk05, 2 * it, s), &gc[s * HW], &gb[s * CHW],
                          &gx[s * HW], &gy[s * HW], &g05_1[s * CHW], &g05_0[s * CHW],
                          &gxk1[s * CHW], &gxk0[s * CHW], ysrc, ic, ih, iw, step, m, false,
                          q.clamp != 0);
        } else {
          // TV.cu:1724-1727: the checkpoint y stands in for y_{k0+1}
          const R* ysrc = q.end_uses_ckpt_y ? &st.intermediate_y[outer][s * CHW] : slot(yhist, 0, s);
          adjoint_iter<R>(wxs, wys, cs, bs, slot(xk05, 0, s), &gc[s * HW], &gb[s * CHW],
                          &gx[s * HW], &gy[s * HW], &g05_1[s * CHW], &g05_0[s * CHW],
                          &gxk1[s * CHW], &gxk0[s * CHW], ysrc, ic, ih, iw, step, m,
                          q.end_uses_ckpt_y != 0, q.clamp != 0);
        }
      }
    }
    // copy_and_set_to_0, TV.cu:178-218,1730
    for (size_t i = 0; i < in * HW; i++) { gc_storage[i] = (double)gc[i] + gc_storage[i] / 1.; gc[i] = 0; }
    for (size_t i = 0; i < in * HW; i++) { gx_storage[i] = (double)gx[i] + gx_storage[i] / 1.; gx[i] = 0; }
    for (size_t i = 0; i < in * HW; i++) { gy_storage[i] = (double)gy[i] + gy_storage[i] / 1.; gy[i] = 0; }
    for (size_t i = 0; i < in * CHW; i++) { gb_storage[i] = (double)gb[i] + gb_storage[i] / 1.; gb[i] = 0; }
    lastIt = nextLastIt;
  }

  std::vector<R> vf(gxk1);  // TV.cu:1784-1785: g_x[1]
  if (!q.skip_iter0_adjoint && its / 2 > 0) {
    // true gradient wrt init: J^T(y_0) g05[0] + g_x[0]; weight gradients get iteration 0's term
    std::vector<R> gy0(in * CHW);
    std::fill(gx.begin(), gx.end(), R(0));
    std::fill(gy.begin(), gy.end(), R(0));
    for (int s = 0; s < in; s++)
      jt_only<R>(&wx[s * HW], &wy[s * HW], &g05_0[s * CHW], &st.intermediate_y[0][s * CHW],
                 &gy0[s * CHW], &gx[s * HW], &gy[s * HW], ic, ih, iw, m);
    for (size_t i = 0; i < in * CHW; i++) vf[i] = gy0[i] + gxk0[i];
    for (size_t i = 0; i < in * HW; i++) { gx_storage[i] += (double)gx[i]; gy_storage[i] += (double)gy[i]; }
  }

  if (q.guard) {  // TV.cu:1760-1791
    double run_step = std::min(kMemoryT, double(st.run) / double(st.run + 1));
    double is_largest = 0, av_gc = 0;
    int num_above = 0, invalid = 0;
    check_gradUpdate(gc_storage, av_gc, is_largest, num_above, st.av_GC, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GC, gc_storage, run_step);
    check_gradUpdate(gx_storage, av_gc, is_largest, num_above, st.av_GX, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GX, gx_storage, run_step);
    check_gradUpdate(gy_storage, av_gc, is_largest, num_above, st.av_GY, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GY, gy_storage, run_step);
    check_gradUpdate(gb_storage, av_gc, is_largest, num_above, st.av_GB, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GB, gb_storage, run_step);
    check_gradUpdate(vf, av_gc, is_largest, num_above, st.av_GI, invalid);
    update_correct_av_step_host(st.run, av_gc, st.av_GI, vf, run_step);
  }

  // TV.cu:1795-1818
  for (size_t i = 0; i < in * HW; i++) d_outGradC[i] = (R)(gc_storage[i] * globalMult);
  for (size_t i = 0; i < in * HW; i++) d_outGradX[i] = (R)(L * (double)(R)(gx_storage[i] * globalMult));
  for (size_t i = 0; i < in * HW; i++) d_outGradY[i] = (R)(L * (double)(R)(gy_storage[i] * globalMult));
  for (size_t i = 0; i < in * CHW; i++) d_outGradB[i] = (R)(gb_storage[i] * globalMult);
  for (size_t i = 0; i < in * CHW; i++) d_outGradI[i] = R(0) + vf[i];
  st.run++;  // TV.cu:1829
  return 0;
}

}  // namespace

extern "C" {

int tv_oracle_forward(const float* dx, const float* dy, const float* c, const float* b,
                      const float* init, float* out, int n, int ic, int ih, int iw, int its, int id) {
  return forward<float>(dx, dy, c, b, init, out, n, ic, ih, iw, its, id);
}
int tv_oracle_backward(const float* dx, const float* dy, const float* c, const float* b, float* gin,
                       float* gx, float* gy, float* gc, float* gb, float* gi, int n, int ic, int ih,
                       int iw, int its, int id) {
  return backward<float>(dx, dy, c, b, gin, gx, gy, gc, gb, gi, n, ic, ih, iw, its, id);
}
int tv_oracle_forward_f64(const double* dx, const double* dy, const double* c, const double* b,
                          const double* init, double* out, int n, int ic, int ih, int iw, int its, int id) {
  return forward<double>(dx, dy, c, b, init, out, n, ic, ih, iw, its, id);
}
int tv_oracle_backward_f64(const double* dx, const double* dy, const double* c, const double* b,
                           double* gin, double* gx, double* gy, double* gc, double* gb, double* gi,
                           int n, int ic, int ih, int iw, int its, int id) {
  return backward<double>(dx, dy, c, b, gin, gx, gy, gc, gb, gi, n, ic, ih, iw, its, id);
}

// quirk toggles, in the order of struct Quirks; all 1 = literal reference behaviour
void tv_oracle_set_quirks(int end_uses_ckpt_y, int skip_iter0_adjoint, int getyk_rebuild,
                          int scale_factors, int clamp, int guard) {
  g_quirks.end_uses_ckpt_y = end_uses_ckpt_y;
  g_quirks.skip_iter0_adjoint = skip_iter0_adjoint;
  g_quirks.getyk_rebuild = getyk_rebuild;
  g_quirks.scale_factors = scale_factors;
  g_quirks.clamp = clamp;
  g_quirks.guard = guard;
}

void tv_oracle_reset_id(int id) {
  if (id < 0 || id >= kUniqueIds) return;
  states<float>()[id] = IdState<float>();
  states<double>()[id] = IdState<double>();
}

// state6 = {run, av_GC, av_GX, av_GY, av_GB, av_GI}
int tv_oracle_get_state(int id, double* state6, int f64) {
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
int tv_oracle_set_state(int id, const double* state6) {
  if (id < 0 || id >= kUniqueIds) return 1;
  auto& s = states<float>()[id];
  s.run = (int)state6[0]; s.av_GC = state6[1]; s.av_GX = state6[2]; s.av_GY = state6[3]; s.av_GB = state6[4]; s.av_GI = state6[5];
  auto& d = states<double>()[id];
  d.run = (int)state6[0]; d.av_GC = state6[1]; d.av_GX = state6[2]; d.av_GY = state6[3]; d.av_GB = state6[4]; d.av_GI = state6[5];
  return 0;
}

// returns the number of checkpoints; iterations_out must hold floor(sqrt(its)) ints
int tv_oracle_schedule(int its, int* iterations_out, int* max_inter_its) {
  std::vector<int> it;
  int m = 0;
  make_schedule(its, it, m);
  for (size_t i = 0; i < it.size(); i++) iterations_out[i] = it[i];
  *max_inter_its = m;
  return (int)it.size();
}
void tv_oracle_step_sizes(int its, float* out) {
  std::vector<float> s;
  make_step_sizes(its, s);
  for (size_t i = 0; i < s.size(); i++) out[i] = s[i];
}

// one forward iteration on one sample with already L-scaled weights (x updated in place)
void tv_oracle_forward_iter(const float* wx, const float* wy, const float* c, const float* b, float* x,
                            const float* y, float* yout, float* x05, int ic, int ih, int iw, float t) {
  forward_iter<float>(wx, wy, c, b, x, y, yout, x05, ic, ih, iw, t);
}
void tv_oracle_forward_iter_f64(const double* wx, const double* wy, const double* c, const double* b,
                                double* x, const double* y, double* yout, double* x05, int ic, int ih,
                                int iw, double t) {
  forward_iter<double>(wx, wy, c, b, x, y, yout, x05, ic, ih, iw, t);
}

// the y rebuild of the backward pass on one sample: y_{k+1} from x05[k] (x05_it) and x05[k-1] (x05_itm1)
void tv_oracle_get_yk_f64(const double* c, const double* b, const double* x05_it, const double* x05_itm1,
                          double* yk_out, int ic, int ih, int iw, double t) {
  get_yk<double>(c, b, x05_it, x05_itm1, yk_out, ic, ih, iw, t);
}
void tv_oracle_get_yk(const float* c, const float* b, const float* x05_it, const float* x05_itm1, float* yk_out,
                      int ic, int ih, int iw, float t) {
  get_yk<float>(c, b, x05_it, x05_itm1, yk_out, ic, ih, iw, t);
}

// guard on a double vector (tensors C, X, Y, B) or a float vector (tensor I); `av` is the
// running mean, updated in place.  stats4 = {av_gc, is_largest, num_above, invalid}.
// Returns 0 plain / 1 rescaled / 2 killed.
int tv_oracle_guard_f64(double* g, long n, int run, double* av, double* stats4) {
  std::vector<double> v(g, g + n);
  double run_step = std::min(kMemoryT, double(run) / double(run + 1));
  double av_gc = 0, is_largest = 0;
  int num_above = 0, invalid = 0;
  check_gradUpdate(v, av_gc, is_largest, num_above, *av, invalid);
  int r = update_correct_av_step_host(run, av_gc, *av, v, run_step);
  std::copy(v.begin(), v.end(), g);
  stats4[0] = av_gc; stats4[1] = is_largest; stats4[2] = num_above; stats4[3] = invalid;
  return r;
}
int tv_oracle_guard_f32(float* g, long n, int run, double* av, double* stats4) {
  std::vector<float> v(g, g + n);
  double run_step = std::min(kMemoryT, double(run) / double(run + 1));
  double av_gc = 0, is_largest = 0;
  int num_above = 0, invalid = 0;
  check_gradUpdate(v, av_gc, is_largest, num_above, *av, invalid);
  int r = update_correct_av_step_host(run, av_gc, *av, v, run_step);
  std::copy(v.begin(), v.end(), g);
  stats4[0] = av_gc; stats4[1] = is_largest; stats4[2] = num_above; stats4[3] = invalid;
  return r;
}

void tv_oracle_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n > 0 ? n : 1);
#else
  (void)n;
#endif
}
int tv_oracle_max_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
