// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's two small flow layers that sit
// upstream of the inpainting layer: the quadratic sub-pixel fit of a matching cost (cudaQuadFit)
// and the median of a per-pixel displacement histogram (cudaMedian).
//
// Nothing in the shipped package may import, link or call this file.  It exists so that the
// parity tests, the smoke check and the bench's cpu_baseline leg have something to compare the
// HIP path against.  Every function cites the reference lines it restates (paths relative to the
// reference root; QF.cu = cudaQuadFit/cudaCode/quadFit.cu, QF.cpp = cudaQuadFit/QuadFit_cuda.cpp,
// MM.cu = cudaMedian/cudaCode/medimax.cu, MM.cpp = cudaMedian/median_cuda.cpp).
//
// Arithmetic conventions: every floating-point expression is evaluated left to right exactly as
// written in the reference source, in the type C++ promotion rules give it (a literal such as
// `2.` or `0.5` makes the surrounding sub-expression double, as it does under nvcc); no fused
// multiply-add contraction (build with -ffp-contract=off); IEEE division.  The templates are
// instantiated for float (the layer) and double (for the pins).
//
// Pin status:
//   quadfit forward ...... pinned (numpy.polyfit parabola through the three costs of each axis,
//                          costs from an independent gather; validity rules by construction)
//   quadfit backward ..... pinned (torch.autograd through an independently written forward,
//                          central finite differences)
//   median forward ....... pinned (inverse of the piecewise-linear CDF of the histogram density)
//   median backward ...... pinned (autograd of the median of the sum-normalised histogram); the
//                          gradient is the one of the NORMALISED histogram evaluated as if the
//                          input summed to one (MM.cu:62-64,78-81) -- that reading is by source.
//   The order in which the reference's atomicAdd calls land (QF.cu:279-283,296) is not defined;
//   this restatement adds in pixel order.  Agreement with a CUDA run is to rounding only.
//
// Extensions over the reference: the flow tensor may carry more than two channels (the Python
// module passes three, QuadFitting.py:53, while the kernel indexes a two-channel tensor,
// QF.cu:314): `fc` is its channel count and channels 0 and 1 are read.  The output of the fit
// has three channels (QF.cu:315; the binding allocates two, QF.cpp:60).

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

int g_threads = 0;

int threads_for(int work) {
#ifdef _OPENMP
  const int t = g_threads > 0 ? g_threads : omp_get_max_threads();
  return std::max(1, std::min(t, work));
#else
  return 1;
#endif
}

// ---------------------------------------------------------------------------------------------
// Quadratic fit.  Shared head of both kernels: QF.cu:22-80 == QF.cu:149-190.
// ---------------------------------------------------------------------------------------------
template <typename R>
struct Fit {
  bool inside;
  int ix, iy, ixm, iym, ixp, iyp;
  R c00, c0p, cp0, c0m, cm0;
  R ax, ay, bx, by, fx, fy;
  int validX, validY;
};

template <typename R>
Fit<R> fit_pixel(const R* im0, const R* im1, const R* flow, int n, int d, int H, int W, int fc, int h, int w) {
  Fit<R> f{};
  const size_t HW = (size_t)H * W;
  const R* fl = flow + (size_t)n * fc * HW;
  // QF.cu:31-38
  const R idx = w + fl[(size_t)h * W + w];
  const R idy = h + fl[HW + (size_t)h * W + w];
  // (written so that a NaN displacement counts as leaving the image; the reference's form of the test lets it
  // through and then indexes with an undefined integer)
  if (!(idx <= W - 1 && idx >= 0 && idy <= H - 1 && idy >= 0)) {
    f.inside = false;
    return f;
  }
  f.inside = true;
  // QF.cu:47-53
  f.ix = (int)std::floor(idx + 0.5);
  f.iy = (int)std::floor(idy + 0.5);
  f.ixm = std::max(f.ix - 1, 0);
  f.iym = std::max(f.iy - 1, 0);
  f.ixp = std::min(f.ix + 1, W - 1);
  f.iyp = std::min(f.iy + 1, H - 1);
  // QF.cu:56-71
  R c00(0), c0p(0), cp0(0), c0m(0), cm0(0);
  const R* a = im0 + (size_t)n * d * HW;
  const R* b = im1 + (size_t)n * d * HW;
  for (int cc = 0; cc < d; cc++) {
    const R I1 = a[(size_t)cc * HW + (size_t)h * W + w];
    const R* q = b + (size_t)cc * HW;
    c00 += I1 * q[(size_t)f.iy * W + f.ix];
    c0p += I1 * q[(size_t)f.iy * W + f.ixp];
    cp0 += I1 * q[(size_t)f.iyp * W + f.ix];
    c0m += I1 * q[(size_t)f.iy * W + f.ixm];
    cm0 += I1 * q[(size_t)f.iym * W + f.ix];
  }
  f.c00 = c00; f.c0p = c0p; f.cp0 = cp0; f.c0m = c0m; f.cm0 = cm0;
  // QF.cu:75-80
  f.ax = (R)(0.5 * (c0p + c0m - 2. * c00));
  f.ay = (R)(0.5 * (cp0 + cm0 - 2. * c00));
  f.bx = (R)(0.5 * (c0p - c0m));
  f.by = (R)(0.5 * (cp0 - cm0));
  // QF.cu:83-89
  f.validX = (f.ax < 0 && f.ax * f.ax >= 0.25 * f.bx * f.bx);
  f.validY = (f.ay < 0 && f.ay * f.ay >= 0.25 * f.by * f.by);
  if (!(f.ix < W - 1 && f.ix > 0)) f.validX = 0;
  if (!(f.iy < H - 1 && f.iy > 0)) f.validY = 0;
  // QF.cu:92-104
  f.fx = 0;
  f.fy = 0;
  if (f.validX) f.fx = (R)(-0.5 * f.bx / f.ax);
  if (f.validY) f.fy = (R)(-0.5 * f.by / f.ay);
  return f;
}

// QF.cu:14-139 and the driver QF.cu:308-331: out (n, 3, h, w) = (fx, fy, score), zero where the
// displaced pixel leaves the image.
template <typename R>
void quadfit_forward(const R* im0, const R* im1, const R* flow, R* out, int N, int d, int H, int W, int fc) {
  const size_t HW = (size_t)H * W;
  std::fill(out, out + (size_t)N * 3 * HW, R(0));  // QF.cu:318
#pragma omp parallel for collapse(2) num_threads(threads_for(N * H))
  for (int n = 0; n < N; n++)
    for (int h = 0; h < H; h++)
      for (int w = 0; w < W; w++) {
        Fit<R> f = fit_pixel(im0, im1, flow, n, d, H, W, fc, h, w);
        if (!f.inside) continue;
        R* o = out + (size_t)n * 3 * HW + (size_t)h * W + w;
        // QF.cu:125-133 (the stores happen only at interior columns / rows, where fx / fy may be
        // non-zero; elsewhere the fit is zero and so is the untouched output)
        if (f.ix < W - 1 && f.ix > 0) o[0] = f.fx; else f.fx = 0;
        if (f.iy < H - 1 && f.iy > 0) o[HW] = f.fy; else f.fy = 0;
        // QF.cu:136-137
        const R score = f.ax * f.fx * f.fx + f.bx * f.fx + f.c00 + f.ay * f.fy * f.fy + f.by * f.fy;
        o[2 * HW] = score;
      }
}

// QF.cu:145-300 and the driver QF.cu:338-369.  gin (n, 3, h, w); g0, g1 like the features.
template <typename R>
void quadfit_backward(const R* im0, const R* im1, const R* flow, const R* gin, R* g0, R* g1, int N, int d, int H,
                      int W, int fc) {
  const size_t HW = (size_t)H * W;
  std::fill(g0, g0 + (size_t)N * d * HW, R(0));  // QF.cu:353-354
  std::fill(g1, g1 + (size_t)N * d * HW, R(0));
#pragma omp parallel for num_threads(threads_for(N))
  for (int n = 0; n < N; n++)
    for (int h = 0; h < H; h++)
      for (int w = 0; w < W; w++) {
        const Fit<R> f = fit_pixel(im0, im1, flow, n, d, H, W, fc, h, w);
        if (!f.inside) continue;
        const int validX = f.validX, validY = f.validY;
        const R ax = f.ax, ay = f.ay, fx = f.fx, fy = f.fy;
        // QF.cu:244-253
        const R dfx_dbx = validX ? (R)(-1. / (2. * ax)) : (R)0.;
        const R dfx_dax = validX ? -fx / ax : (R)0.;
        const R dfy_dby = validY ? (R)(-1. / (2. * ay)) : (R)0.;
        const R dfy_day = validY ? -fy / ay : (R)0.;
        const R ds_dax = validX ? fx * fx : (R)0.;
        const R ds_dbx = validX ? fx : (R)0.;
        const R ds_dc = (validX || validY) ? (R)1. : (R)0.;
        const R ds_day = validY ? fy * fy : (R)0.;
        const R ds_dby = validY ? fy : (R)0.;
        // QF.cu:261-263
        const size_t p = (size_t)h * W + w;
        const R dFdfx = gin[(size_t)n * 3 * HW + p];
        const R dFdfy = gin[(size_t)n * 3 * HW + HW + p];
        const R dFds = gin[(size_t)n * 3 * HW + 2 * HW + p];
        for (int cc = 0; cc < d; cc++) {  // QF.cu:265-298
          const size_t base = ((size_t)n * d + cc) * HW;
          const R* q = im1 + base;
          R* G1 = g1 + base;
          const R I1 = im0[base + p];
          const R I2 = q[(size_t)f.iy * W + f.ix];
          const R I2_0p = q[(size_t)f.iy * W + f.ixp];
          const R I2_0m = q[(size_t)f.iy * W + f.ixm];
          const R I2_p0 = q[(size_t)f.iyp * W + f.ix];
          const R I2_m0 = q[(size_t)f.iym * W + f.ix];
          if (validX || validY) {
            G1[(size_t)f.iy * W + f.ix] += (R)(0.5 * I1 * (-2. * dFdfx * dfx_dax - 2. * dFdfy * dfy_day - 2. * dFds * ds_dax - 2. * dFds * ds_day + 2. * dFds * ds_dc));
            G1[(size_t)f.iy * W + f.ixp] += (R)(0.5 * I1 * (dFdfx * dfx_dax + dFdfx * dfx_dbx + dFds * ds_dax + dFds * ds_dbx));
            G1[(size_t)f.iy * W + f.ixm] += (R)(0.5 * I1 * (dFdfx * dfx_dax - dFdfx * dfx_dbx + dFds * ds_dax - dFds * ds_dbx));
            G1[(size_t)f.iyp * W + f.ix] += (R)(0.5 * I1 * (dFdfy * dfy_day + dFdfy * dfy_dby + dFds * ds_day + dFds * ds_dby));
            G1[(size_t)f.iym * W + f.ix] += (R)(0.5 * I1 * (dFdfy * dfy_day - dFdfy * dfy_dby + dFds * ds_day - dFds * ds_dby));
            g0[base + p] = (R)(0.5 * (I2 * (-2. * dFdfx * dfx_dax - 2. * dFdfy * dfy_day - 2. * dFds * ds_dax - 2. * dFds * ds_day + 2. * dFds * ds_dc) +
                                      I2_0p * (dFdfx * dfx_dax + dFdfx * dfx_dbx + dFds * ds_dax + dFds * ds_dbx) +
                                      I2_0m * (dFdfx * dfx_dax - dFdfx * dfx_dbx + dFds * ds_dax - dFds * ds_dbx) +
                                      I2_p0 * (dFdfy * dfy_day + dFdfy * dfy_dby + dFds * ds_day + dFds * ds_dby) +
                                      I2_m0 * (dFdfy * dfy_day - dFdfy * dfy_dby + dFds * ds_day - dFds * ds_dby)));
          } else {  // only the centre cost carries a gradient
            g0[base + p] = I2 * dFds;
            G1[(size_t)f.iy * W + f.ix] += I1 * dFds;
          }
        }
      }
}

// ---------------------------------------------------------------------------------------------
// Median.  vol (n, h, w, D) with the D histogram bins innermost (MM.cu:134; MM.cpp:43-46);
// out (n, 2, h, w) = (position of the median, mass of the bin that holds it).
// ---------------------------------------------------------------------------------------------
// MM.cu:17-44, driver 131-168
template <typename R>
void median_forward(const R* vol, R* out, int N, int H, int W, int D) {
  const size_t HW = (size_t)H * W;
  std::fill(out, out + (size_t)N * 2 * HW, R(0));  // MM.cu:155
#pragma omp parallel for collapse(2) num_threads(threads_for(N * H))
  for (int n = 0; n < N; n++)
    for (int h = 0; h < H; h++)
      for (int w = 0; w < W; w++) {
        const R* p = vol + ((size_t)n * HW + (size_t)h * W + w) * D;
        R score = 0;
        const R w2 = 0;
        for (int c = 0; c < D; ++c) {
          const R cScore = p[c];
          if (score < 0.5 && score + cScore >= 0.5) {
            const R alpha = (R)((1. - 2. * score - cScore) / (2. * cScore));  // MM.cu:34
            out[(size_t)n * 2 * HW + (size_t)h * W + w] = (R)(R(c) - w2 + alpha);
            out[(size_t)n * 2 * HW + HW + (size_t)h * W + w] = cScore;
            break;
          }
          score = score + cScore;
        }
      }
}

// MM.cu:46-93 (the variant the driver launches, MM.cu:186), driver 170-190
template <typename R>
void median_backward(const R* vol, const R* gin, R* gvol, int N, int H, int W, int D) {
  const size_t HW = (size_t)H * W;
  std::fill(gvol, gvol + (size_t)N * HW * D, R(0));  // MM.cu:176
#pragma omp parallel for collapse(2) num_threads(threads_for(N * H))
  for (int n = 0; n < N; n++)
    for (int h = 0; h < H; h++)
      for (int w = 0; w < W; w++) {
        const R* p = vol + ((size_t)n * HW + (size_t)h * W + w) * D;
        R* g = gvol + ((size_t)n * HW + (size_t)h * W + w) * D;
        const R g0 = gin[(size_t)n * 2 * HW + (size_t)h * W + w];
        const R g1 = gin[(size_t)n * 2 * HW + HW + (size_t)h * W + w];
        R score = 0, alpha = 0, pmid = 1.;
        for (int c = 0; c < D; ++c) {  // MM.cu:59-75
          const R cScore = p[c];
          if (score < 0.5 && score + cScore >= 0.5) {
            pmid = cScore;
            alpha = (R)((1. - 2. * score - cScore) / (2. * cScore));
            g[c] = g0 * alpha / (-pmid) + g1;
            break;
          }
          score = score + cScore;
        }
        score = 0;
        for (int c = 0; c < D; ++c) {  // MM.cu:77-92
          const R cScore = p[c];
          if (score + cScore < 0.5)
            g[c] = (R)(-g0 / (2. * pmid));
          else if (score >= 0.5)
            g[c] = (R)(+g0 / (2. * pmid));
          score = score + cScore;
        }
      }
}

// ---------------------------------------------------------------------------------------------
// Glue between two levels of a coarse-to-fine hierarchy of inpainting layers (the reference's README.md:64-71
// describes the hierarchy; it ships no code for the glue, so this is the build's own definition):
//   up   = scale * bilinear x2 upsampling of the coarse solution -- the definition of bilinear resampling with
//          half-pixel centres: source coordinate (dst + 0.5) / 2 - 0.5 clamped at 0, neighbours clamped at the border;
//          flow vectors are measured in pixels, hence scale = 2;
//   wx,wy = exp(-alpha |I(h, w+1) - I(h, w)|), exp(-alpha |I(h+1, w) - I(h, w)|), 1 in the last column / row --
//          the edge weights of the fine level from its guidance image (single precision: exp_nonpos below).
// Pins: torch.nn.functional.interpolate(mode="bilinear", align_corners=False) and its autograd adjoint.
// ---------------------------------------------------------------------------------------------
template <typename R>
void axis_taps(int dst, int size, int& i0, int& i1, R& l0, R& l1) {
  R src = (R)((dst + 0.5) * 0.5 - 0.5);
  if (src < 0) src = 0;
  i0 = (int)src;
  i1 = std::min(i0 + 1, size - 1);
  l1 = src - (R)i0;
  l0 = (R)1 - l1;
}

template <typename R>
void upsample2x(const R* in, R* out, int planes, int H, int W, R scale) {
  const int H2 = 2 * H, W2 = 2 * W;
#pragma omp parallel for num_threads(threads_for(planes))
  for (int q = 0; q < planes; q++) {
    const R* a = in + (size_t)q * H * W;
    R* o = out + (size_t)q * H2 * W2;
    for (int y = 0; y < H2; y++) {
      int y0, y1;
      R h0, h1;
      axis_taps<R>(y, H, y0, y1, h0, h1);
      for (int x = 0; x < W2; x++) {
        int x0, x1;
        R w0, w1;
        axis_taps<R>(x, W, x0, x1, w0, w1);
        const R v = h0 * (w0 * a[(size_t)y0 * W + x0] + w1 * a[(size_t)y0 * W + x1]) +
                    h1 * (w0 * a[(size_t)y1 * W + x0] + w1 * a[(size_t)y1 * W + x1]);
        o[(size_t)y * W2 + x] = scale * v;
      }
    }
  }
}

// adjoint of upsample2x applied to ga (+ gb when given): every coarse pixel collects, in a fixed order (fine rows
// ascending, then fine columns ascending), the fine pixels it was a tap of
template <typename R>
void upsample2x_adjoint(const R* ga, const R* gb, R* out, int planes, int H, int W, R scale) {
  const int H2 = 2 * H, W2 = 2 * W;
#pragma omp parallel for num_threads(threads_for(planes))
  for (int q = 0; q < planes; q++) {
    const R* g0 = ga + (size_t)q * H2 * W2;
    const R* g1 = gb ? gb + (size_t)q * H2 * W2 : nullptr;
    R* o = out + (size_t)q * H * W;
    for (int cy = 0; cy < H; cy++)
      for (int cx = 0; cx < W; cx++) {
        R acc = 0;
        for (int y = std::max(2 * cy - 1, 0); y <= std::min(2 * cy + 2, H2 - 1); y++) {
          int y0, y1;
          R h0, h1;
          axis_taps<R>(y, H, y0, y1, h0, h1);
          R wy = 0;  // weight of coarse row cy in fine row y (both taps can fall on the same clamped row)
          if (y0 == cy) wy += h0;
          if (y1 == cy) wy += h1;
          if (wy == 0) continue;
          for (int x = std::max(2 * cx - 1, 0); x <= std::min(2 * cx + 2, W2 - 1); x++) {
            int x0, x1;
            R w0, w1;
            axis_taps<R>(x, W, x0, x1, w0, w1);
            R wx = 0;
            if (x0 == cx) wx += w0;
            if (x1 == cx) wx += w1;
            if (wx == 0) continue;
            R g = g0[(size_t)y * W2 + x];
            if (g1) g = g + g1[(size_t)y * W2 + x];
            acc += (wy * wx) * g;
          }
        }
        o[(size_t)cy * W + cx] = scale * acc;
      }
  }
}

// exp(x) for x <= 0 in single precision with a FIXED sequence of IEEE operations (Cody-Waite reduction by
// ln 2, degree-7 Taylor polynomial in Horner form, exact scaling), so that a device and a host evaluation agree
// bit for bit; about 1 ulp from the true value.  The double instantiation uses the library's exp.
inline float exp_nonpos(float x) {
  if (!(x > -87.0f)) return 0.0f;
  const float n = std::rint(x * 1.44269504f);
  float r = x - n * 0.693359375f;
  r = r - n * -2.12194440e-4f;
  float p = 1.98412698e-4f;
  p = p * r + 1.38888889e-3f;
  p = p * r + 8.33333333e-3f;
  p = p * r + 4.16666667e-2f;
  p = p * r + 1.66666667e-1f;
  p = p * r + 0.5f;
  p = p * r + 1.0f;
  p = p * r + 1.0f;
  return std::ldexp(p, (int)n);
}
inline double exp_nonpos(double x) { return std::exp(x); }

template <typename R>
void edge_weights(const R* img, R* wx, R* wy, int planes, int H, int W, R alpha) {
  for (int q = 0; q < planes; q++) {
    const R* a = img + (size_t)q * H * W;
    for (int y = 0; y < H; y++)
      for (int x = 0; x < W; x++) {
        const size_t p = (size_t)q * H * W + (size_t)y * W + x;
        wx[p] = x + 1 < W ? exp_nonpos(-alpha * std::fabs(a[(size_t)y * W + x + 1] - a[(size_t)y * W + x])) : (R)1;
        wy[p] = y + 1 < H ? exp_nonpos(-alpha * std::fabs(a[(size_t)(y + 1) * W + x] - a[(size_t)y * W + x])) : (R)1;
      }
  }
}

}  // namespace

extern "C" {

int hierarchy_oracle_upsample2x(const float* in, float* out, int planes, int h, int w, float scale) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  upsample2x<float>(in, out, planes, h, w, scale);
  return 0;
}
int hierarchy_oracle_upsample2x_f64(const double* in, double* out, int planes, int h, int w, double scale) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  upsample2x<double>(in, out, planes, h, w, scale);
  return 0;
}
int hierarchy_oracle_upsample2x_adjoint(const float* ga, const float* gb, float* out, int planes, int h, int w, float scale) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  upsample2x_adjoint<float>(ga, gb, out, planes, h, w, scale);
  return 0;
}
int hierarchy_oracle_upsample2x_adjoint_f64(const double* ga, const double* gb, double* out, int planes, int h, int w,
                                            double scale) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  upsample2x_adjoint<double>(ga, gb, out, planes, h, w, scale);
  return 0;
}
int hierarchy_oracle_edge_weights(const float* img, float* wx, float* wy, int planes, int h, int w, float alpha) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  edge_weights<float>(img, wx, wy, planes, h, w, alpha);
  return 0;
}
int hierarchy_oracle_edge_weights_f64(const double* img, double* wx, double* wy, int planes, int h, int w, double alpha) {
  if (planes < 1 || h < 1 || w < 1) return 1;
  edge_weights<double>(img, wx, wy, planes, h, w, alpha);
  return 0;
}


void flowaux_oracle_set_threads(int t) { g_threads = t; }

int quadfit_oracle_forward(const float* im0, const float* im1, const float* flow, float* out, int n, int c, int h,
                           int w, int fc) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || fc < 2) return 1;
  quadfit_forward<float>(im0, im1, flow, out, n, c, h, w, fc);
  return 0;
}
int quadfit_oracle_forward_f64(const double* im0, const double* im1, const double* flow, double* out, int n, int c,
                               int h, int w, int fc) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || fc < 2) return 1;
  quadfit_forward<double>(im0, im1, flow, out, n, c, h, w, fc);
  return 0;
}
int quadfit_oracle_backward(const float* im0, const float* im1, const float* flow, const float* gin, float* g0,
                            float* g1, int n, int c, int h, int w, int fc) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || fc < 2) return 1;
  quadfit_backward<float>(im0, im1, flow, gin, g0, g1, n, c, h, w, fc);
  return 0;
}
int quadfit_oracle_backward_f64(const double* im0, const double* im1, const double* flow, const double* gin,
                                double* g0, double* g1, int n, int c, int h, int w, int fc) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || fc < 2) return 1;
  quadfit_backward<double>(im0, im1, flow, gin, g0, g1, n, c, h, w, fc);
  return 0;
}

int median_oracle_forward(const float* vol, float* out, int n, int h, int w, int d) {
  if (n < 1 || h < 1 || w < 1 || d < 1) return 1;
  median_forward<float>(vol, out, n, h, w, d);
  return 0;
}
int median_oracle_forward_f64(const double* vol, double* out, int n, int h, int w, int d) {
  if (n < 1 || h < 1 || w < 1 || d < 1) return 1;
  median_forward<double>(vol, out, n, h, w, d);
  return 0;
}
int median_oracle_backward(const float* vol, const float* gin, float* gvol, int n, int h, int w, int d) {
  if (n < 1 || h < 1 || w < 1 || d < 1) return 1;
  median_backward<float>(vol, gin, gvol, n, h, w, d);
  return 0;
}
int median_oracle_backward_f64(const double* vol, const double* gin, double* gvol, int n, int h, int w, int d) {
  if (n < 1 || h < 1 || w < 1 || d < 1) return 1;
  median_backward<double>(vol, gin, gvol, n, h, w, d);
  return 0;
}

}  // extern "C"
