// Wave-strip kernels of the TGV layer (the default path; adjoint pairs hold up to 4 flow channels, more run in groups).
//
// Same execution scheme as the TV layer's strip kernels: one wavefront owns 62 adjacent columns (one
// pixel per lane, lanes 0 and 63 are aprons) by R rows of one sample and walks them top to bottom
// without LDS and without barriers; rows stream through rotating register buffers; neighbouring
// lanes exchange values with wave-wide DPP shifts.
//
// Triangle sharing: the pixel q = (h, w) owns the triangle (q, right of q, below q) and with it three
// Huber terms: the coupling term on z = grad u - v and the two smoothness terms on grad v1, grad v2.
// The reference evaluates each of them three times (at q, at the pixel below, at the pixel to the
// right) with operands that are bit-identical or exact negations of each other, so the owner forms
// every product once and hands the neighbours' shares on: down the column in registers, to the
// right through a DPP shift.  Results are bit-identical to the per-pixel evaluation.
//
// rsqrt: the layer defines CUDA's rsqrtf as 1.0f / sqrtf(x) (both correctly rounded);
// rsq_exact() below returns those bits (checked exhaustively by inpaint_selftest_rsqrt).
#pragma once

#include <type_traits>

#include "exact_math.h"
#include "tv_strip_kernels.h"

namespace tgvstrip {

using inpaint::div_by;
using inpaint::exact_div;
using inpaint::exact_rcp;
using inpaint::div_by_fifth;
using inpaint::exact_sqrt;
using inpaint::rcp_refined;
using tvstrip::from_left_lane;
using tvstrip::from_right_lane;
using tvstrip::ldg;
using tvstrip::stg;
using tvstrip::stg_nt;
using tvstrip::lds_barrier;

// A copy of a store offset made INSIDE the block that stores.  Instruction selection folds "scalar base + 32-bit vector
// offset" into a store only if the offset's widening to 64 bits sits in the store's own basic block; the offset of a row is
// computed before the `if (store_lane)` blocks, its widening lands there too, and every store of a block then computes a
// 64-bit vector address of its own (19 per row in step B of the pair kernel).  The empty asm pins the copy in the block.
__device__ __forceinline__ unsigned offset_here(unsigned off) {
  asm volatile("" : "+v"(off));
  return off;
}
using tvstrip::strip_geometry;
using tvstrip::strip_geometry_block;
using tvstrip::StripGeom;

constexpr int kCols = 62;  // output columns per wavefront (lanes 0 and 63 are aprons)
constexpr int kCols2 = 60;  // two fused forward iterations (lanes 0, 1, 62, 63 are aprons)
constexpr float kD0 = 0.2f, kD1 = 0.2f, kD2 = 0.2f;  // TGV.cu:58-60
static_assert(kD0 == 0.2f && kD1 == 0.2f && kD2 == 0.2f, "the segment-start form divides by the threshold with div_by_fifth");
constexpr float kClipLocalGrad = 2000.0f;            // TGV.cu:78
constexpr float kLocalGCMult = 0.1f;                 // TGV.cu:87
constexpr float kLocalGXMult = 0.1f;                 // TGV.cu:89

// 1.0f / sqrtf(x) with both operations correctly rounded; +inf at 0.  Inputs below 2^-96 may be
// one ulp off, which no caller can see: their Huber weight is 1 either way.
__device__ __forceinline__ float rsq_exact(float x) {
  const float r = exact_rcp(exact_sqrt(x));
  return (x == 0.0f) ? __builtin_inff() : r;
}

// A wavefront whose 64 lanes all hold a Huber argument A <= kHuberQuiet skips the square root and the reciprocal of that
// term: the weight is exactly 1 there.  min(1, fl(fl(1 / fl(sqrt(A))) * 0.2f)) is 1 at A = 0.0399f (the product is
// 1.0012...) and every operation in it is monotone in A, so it is 1 for every A below as well (0 gives +inf * 0.2f);
// the segment-start form 1 / max(1, sqrt(A) / 0.2f) is 1 there too (sqrt(0.0399f) / 0.2f = 0.9987).  A NaN fails the
// comparison and takes the full path.  The test is per wavefront, so no lane diverges and the bits cannot change; what
// changes is the time, which now depends on the data: the smoothness terms of v1, v2 are quiet in whole rows of smooth
// flow, the coupling term in most of them.  inpaint_selftest_rsqrt checks the claim at the threshold on the device.
constexpr float kHuberQuiet = 0.0399f;
__device__ __forceinline__ bool wave_any(bool p) { return __builtin_amdgcn_ballot_w64(p) != 0ull; }

// Huber weight of the main kernels: min(1, rsqrt(A) * delta)  (TGV.cu:1624 and siblings)
__device__ __forceinline__ float huber_w_full(float A, float delta) { return fminf(1.f, rsq_exact(A) * delta); }
__device__ __forceinline__ float huber_w(float A, float delta) {
  static_assert(kD0 == 0.2f, "kHuberQuiet is the bound for a threshold of 0.2f");
  if (!wave_any(A > kHuberQuiet)) return 1.f;
  return huber_w_full(A, delta);
}

// -------------------------------------------------------------------------------------------------
// Forward iteration, TGV.cu:1546-1776 (and 2005-2235 when x05 is given).
//
// Per triangle (owner q) six products are formed once:
//     Fa = wy (z2 hwx)    Fb = wx (z1 hwx)         z = (y_q - y_right + y1_q, y_q - y_down + y2_q)
//     G1y = bx (u12 hwy1) G1x = bx (u11 hwy1)      u1 = (y1_q - y1_right, y1_q - y1_down)
//     G2y = by (u22 hwy2) G2x = by (u21 hwy2)      u2 likewise on y2
// q subtracts all of them (TGV.cu:1678-1684), the pixel below subtracts -Fa, -G1y, -G2y
// (TGV.cu:1637-1639) and the pixel to the right -Fb, -G1x, -G2x (TGV.cu:1665-1667).
// -------------------------------------------------------------------------------------------------
template <int C>
struct FwdRow {
  float y[3][C], x[3][C], bb[C], c, rc1, wxs, wys, bxs, bys;
};

template <int C, bool X05>
__global__ __launch_bounds__(256) void tgv_forward_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ xin, float* __restrict__ xout, const float* __restrict__ yin,
    float* __restrict__ yout, float* __restrict__ x05, int N, int H, int W, float t, int R, int strips_x,
    int strips_y, int Ct) {
  StripGeom g;
  if (!strip_geometry(g, kCols, R, W, strips_x, strips_y, N)) return;
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 0 && g.lane < 63 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;  // the pixel has a right neighbour
  const int Reff = min(R, H - g.hs);
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                     *const cf_p = cf + poff;
  const float *y_p[3][C], *x_p[3][C], *b_p[C];
  float *yo_p[3][C], *xo_p[3][C], *xh_p[3][C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    b_p[ch] = b + ((size_t)g.n * Ct + ch) * HW;
#pragma unroll
    for (int v = 0; v < 3; v++) {
      const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)ch * HW;
      y_p[v][ch] = yin + q; x_p[v][ch] = xin + q;
      yo_p[v][ch] = yout + q; xo_p[v][ch] = xout + q; xh_p[v][ch] = X05 ? x05 + q : nullptr;
    }
  }

  auto load_row = [&](int k, FwdRow<C>& in) {  // row k of the strip = image row hs - 1 + k
    const int kk = min(k, Reff + 1);
    const int h = g.hs - 1 + kk;
    const unsigned row = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4;
    // the rows above and below the strip contribute y (and, above, the weights) only; their other
    // fields are read from the strip's own first / last row, which is in L1 anyway
    const int hw = g.hs - 1 + min(kk, Reff);
    const unsigned row_w = (unsigned)(hw < 0 ? 0 : hw) * W4;
    const unsigned row_p = (unsigned)(g.hs - 1 + max(1, min(kk, Reff))) * W4;
    in.c = ldg(cf_p, row_p + wc);
    in.wxs = ldg(wx_p, row_w + wc);
    in.wys = ldg(wy_p, row_w + wc);
    in.bxs = ldg(bx_p, row_w + wc);
    in.bys = ldg(by_p, row_w + wc);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.bb[ch] = ldg(b_p[ch], row_p + wc);
#pragma unroll
      for (int v = 0; v < 3; v++) {
        in.y[v][ch] = ldg(y_p[v][ch], row + wc);
        in.x[v][ch] = ldg(x_p[v][ch], row_p + wc);
      }
    }
  };
  auto absorb = [&](int k, FwdRow<C>& o) {
    const int h = g.hs - 1 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const inpaint::LaneMask inside(ok);
    o.rc1 = rcp_refined(1.f + o.c);
    o.wxs = (ok && rmask) ? o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? o.wys : 0.f;
    o.bxs = inside(o.bxs);
    o.bys = inside(o.bys);
#pragma unroll
    for (int ch = 0; ch < C; ch++)
#pragma unroll
      for (int v = 0; v < 3; v++) o.y[v][ch] = inside(o.y[v][ch]);
  };

  float upFa[C], upG1y[C], upG2y[C];  // terms handed down to the row below
#pragma unroll
  for (int ch = 0; ch < C; ch++) upFa[ch] = upG1y[ch] = upG2y[ch] = 0.f;

  auto compute = [&](int r, const FwdRow<C>& cur, const FwdRow<C>& nxt, auto first) {
    const int h = g.hs - 1 + r;
    const bool dmask = h >= 0 && h < H - 1;  // the pixel has a lower neighbour
    const unsigned roff = (unsigned)(h >= 0 ? h : 0) * W4 + wc;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float yc = cur.y[0][ch], y1c = cur.y[1][ch], y2c = cur.y[2][ch];
      const float yr = from_right_lane(yc), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
      const float yd = nxt.y[0][ch], y1d = nxt.y[1][ch], y2d = nxt.y[2][ch];
      // own triangle, TGV.cu:1669-1684
      const float zij_1 = rmask ? ((yc - yr) + y1c) : 0.f;
      const float zij_2 = dmask ? ((yc - yd) + y2c) : 0.f;
      const float hwx = huber_w(zij_2 * zij_2 * cur.wys + zij_1 * zij_1 * cur.wxs, kD0);
      const float u11 = rmask ? (y1c - y1r) : 0.f;
      const float u12 = dmask ? (y1c - y1d) : 0.f;
      const float hwy1 = huber_w(cur.bxs * (u12 * u12 + u11 * u11), kD1);
      const float u21 = rmask ? (y2c - y2r) : 0.f;
      const float u22 = dmask ? (y2c - y2d) : 0.f;
      const float hwy2 = huber_w(cur.bys * (u22 * u22 + u21 * u21), kD2);
      const float Fa = cur.wys * (zij_2 * hwx), Fb = cur.wxs * (zij_1 * hwx);
      const float G1y = cur.bxs * (u12 * hwy1), G1x = cur.bxs * (u11 * hwy1);
      const float G2y = cur.bys * (u22 * hwy2), G2x = cur.bys * (u21 * hwy2);
      const float aFa = upFa[ch], aG1y = upG1y[ch], aG2y = upG2y[ch];
      upFa[ch] = Fa; upG1y[ch] = G1y; upG2y[ch] = G2y;
      if (first.value) continue;
      const float lFb = from_left_lane(Fb), lG1x = from_left_lane(G1x), lG2x = from_left_lane(G2x);
      float yt = yc, y1n = y1c, y2n = y2c;
      yt -= -aFa;    // TGV.cu:1637
      y1n -= -aG1y;  // TGV.cu:1638
      y2n -= -aG2y;  // TGV.cu:1639
      yt -= -lFb;    // TGV.cu:1665
      y1n -= -lG1x;  // TGV.cu:1666
      y2n -= -lG2x;  // TGV.cu:1667
      yt -= Fa;          // TGV.cu:1678
      y1n -= G1y;        // TGV.cu:1679
      y2n -= G2y + Fa;   // TGV.cu:1680
      yt -= Fb;          // TGV.cu:1682
      y1n -= G1x + Fb;   // TGV.cu:1683
      y2n -= G2x;        // TGV.cu:1684
      const float y1o = y1n + t * (y1n - cur.x[1][ch]);  // TGV.cu:1686-1687
      const float y2o = y2n + t * (y2n - cur.x[2][ch]);
      const float xh = yt;
      const float c = cur.c, bv = cur.bb[ch];
      float x_loc = div_by(c * bv + yt, 1.f + c, cur.rc1);  // TGV.cu:1740
      const float lo = yt - c, hi = yt + c;
      if (lo > 1.f + bv) x_loc = lo;
      if (hi < bv - 1.f) x_loc = hi;
      const float yn = x_loc + t * (x_loc - cur.x[0][ch]);  // TGV.cu:1772
      if (store_lane) {
        stg(yo_p[0][ch], roff, yn);
        stg(yo_p[1][ch], roff, y1o);
        stg(yo_p[2][ch], roff, y2o);
        stg(xo_p[0][ch], roff, x_loc);
        stg(xo_p[1][ch], roff, y1n);
        stg(xo_p[2][ch], roff, y2n);
        if (X05) {
          stg(xh_p[0][ch], roff, xh);
          stg(xh_p[1][ch], roff, y1n);
          stg(xh_p[2][ch], roff, y2n);
        }
      }
    }
  };
  const std::true_type kFirst{};
  const std::false_type kRow{};

  FwdRow<C> b0, b1, b2, b3;
  load_row(0, b0);
  load_row(1, b1);
  load_row(2, b2);
  load_row(3, b3);
  absorb(0, b0);
  absorb(1, b1);
  compute(0, b0, b1, kFirst);
  load_row(4, b0);
  for (int r = 1; r <= Reff; r += 4) {  // cur / next rotate through (b1,b2) (b2,b3) (b3,b0) (b0,b1)
    absorb(r + 1, b2);
    compute(r, b1, b2, kRow);
    load_row(r + 4, b1);
    if (r + 1 > Reff) break;
    absorb(r + 2, b3);
    compute(r + 1, b2, b3, kRow);
    load_row(r + 5, b2);
    if (r + 2 > Reff) break;
    absorb(r + 3, b0);
    compute(r + 2, b3, b0, kRow);
    load_row(r + 6, b3);
    if (r + 3 > Reff) break;
    absorb(r + 4, b1);
    compute(r + 3, b0, b1, kRow);
    load_row(r + 7, b0);
  }
}

// -------------------------------------------------------------------------------------------------
// Two forward iterations per launch (A = iteration k, B = k+1), the arithmetic of tgv_forward_strip
// applied twice.  B runs one row behind A in the same wavefront and takes A's new y and x from
// registers (the scheme of tvstrip::tv_forward_strip2).  Lanes cover columns w0-2 .. w0+61; A's
// update is valid on lanes 1..62, B's on lanes 2..61, the 60 output columns.  A's result outside
// the image is masked to the zero padding B must see.
// -------------------------------------------------------------------------------------------------
template <int C>
struct Fwd2Row {
  float y[3][C], x[3][C], bb[C], c, wxs, wys, bxs, bys;
};

// RING (recompute launches after a segment's first): the input iterate is not read but rebuilt from the x05 rows of
// the two iterations before it, which the ring holds anyway -- u: x = prox(x05[j-1]), y = x + tP (x - prox(x05[j-2]));
// v1, v2: x = x05[j-1], y = x + tP (x - x05[j-2]), the forward pass's own expressions -- and no iterate is written.
// yin / xin then point at those two rows.
// STORE = false: the launch stores no iterate at all (xout, yout ignored), and its row loop carries no code for it.
template <int C, bool X05, bool RING = false, bool STORE = true>
__global__ __launch_bounds__(256) void tgv_forward_strip2(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ xin, const float* __restrict__ xin_aux, float* __restrict__ xout,
    const float* __restrict__ yin, float* __restrict__ yout, float* __restrict__ x05a, float* __restrict__ x05b,
    int store_x_aux, int N, int H, int W, float tA, float tB, float tP, int R, int strips_x, int strips_y, int Ct,
    int groups, float* __restrict__ keep_x = nullptr, float* __restrict__ keep_y = nullptr) {
  // keep_x / keep_y (optional, not with RING): the input iterate is copied there on the strip's own rows as it passes
  // through -- how the starting point reaches checkpoint 0 without a copy launch
  // groups > 1: the launch covers `groups` consecutive channel groups of C channels each, every strip once per group
  // (forward channels never couple)
  StripGeom g;
  if (!strip_geometry(g, kCols2, R, W, strips_x, strips_y, N * groups, 2)) return;
  const int ch_first = (g.n % groups) * C;
  g.n /= groups;
  // the output iterate is stored where the caller wants it: x and y separately, or neither (a launch whose successor
  // rebuilds its input from the x05 rows)
  const bool store_x = STORE && xout != nullptr, store_y = STORE && yout != nullptr;
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                     *const cf_p = cf + poff;
  const float *y_p[3][C], *x_p[3][C], *b_p[C];
  float *yo_p[3][C], *xo_p[3][C], *xa_p[3][C], *xb_p[3][C], *kx_p[3][C], *ky_p[3][C];
  const bool keep_xin = !RING && keep_x != nullptr, keep_yin = !RING && keep_y != nullptr;
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    b_p[ch] = b + ((size_t)g.n * Ct + ch_first + ch) * HW;
#pragma unroll
    for (int v = 0; v < 3; v++) {
      const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)(ch_first + ch) * HW;
      // v1, v2 of an iterate equal the x05 rows of the iteration that made it (no prox on them): a recompute launch
      // reads them from the ring (xin_aux) instead of a second copy, and does not write that copy (store_x_aux == 0)
      y_p[v][ch] = yin + q; x_p[v][ch] = ((v > 0 && xin_aux) ? xin_aux : xin) + q;
      yo_p[v][ch] = yout + q; xo_p[v][ch] = xout + q;
      xa_p[v][ch] = X05 ? x05a + q : nullptr; xb_p[v][ch] = X05 ? x05b + q : nullptr;
      kx_p[v][ch] = keep_xin ? keep_x + q : nullptr; ky_p[v][ch] = keep_yin ? keep_y + q : nullptr;
    }
  }
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates

  auto load_row = [&](int k, Fwd2Row<C>& in) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    const unsigned row = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4;
    const unsigned row_w = (unsigned)min(max(h, 0), h_hi) * W4;
    const unsigned row_p = (unsigned)min(max(h, h_lo), h_hi) * W4;
    const unsigned row_c = RING ? row : row_p;  // rebuilding y needs c and b wherever y is read
    in.c = ldg(cf_p, row_c + wc);
    in.wxs = ldg(wx_p, row_w + wc);
    in.wys = ldg(wy_p, row_w + wc);
    in.bxs = ldg(bx_p, row_w + wc);
    in.bys = ldg(by_p, row_w + wc);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.bb[ch] = ldg(b_p[ch], row_c + wc);
#pragma unroll
      for (int v = 0; v < 3; v++) {
        in.y[v][ch] = ldg(y_p[v][ch], row + wc);
        in.x[v][ch] = ldg(x_p[v][ch], row_c + wc);
      }
    }
  };
  // Huber-1 prox of the data term (TGV.cu:1740-1744)
  auto prox = [&](float yt, float c, float rc1, float bv) {
    float x_loc = div_by(c * bv + yt, 1.f + c, rc1);
    const float lo = yt - c, hi = yt + c;
    if (lo > 1.f + bv) x_loc = lo;
    if (hi < bv - 1.f) x_loc = hi;
    return x_loc;
  };
  auto absorb = [&](int k, Fwd2Row<C>& o) {
    const int h = g.hs - 2 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const inpaint::LaneMask inside(ok);
    if (RING) {  // o.y holds x05[j-1], o.x holds x05[j-2]
      const float rc1 = rcp_refined(1.f + o.c);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xj = prox(o.y[0][ch], o.c, rc1, o.bb[ch]);
        const float xm = prox(o.x[0][ch], o.c, rc1, o.bb[ch]);
        o.x[0][ch] = xj;
        o.y[0][ch] = xj + tP * (xj - xm);  // TGV.cu:1773
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = o.y[v][ch], xmv = o.x[v][ch];
          o.x[v][ch] = xv;
          o.y[v][ch] = xv + tP * (xv - xmv);  // TGV.cu:1686-1690
        }
      }
    }
    o.wxs = (ok && rmask) ? o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? o.wys : 0.f;
    o.bxs = inside(o.bxs);
    o.bys = inside(o.bys);
#pragma unroll
    for (int ch = 0; ch < C; ch++)
#pragma unroll
      for (int v = 0; v < 3; v++) o.y[v][ch] = inside(o.y[v][ch]);
  };

  struct Tri {  // the six products of one triangle (TGV.cu:1669-1684)
    float Fa, Fb, G1y, G1x, G2y, G2x;
  };
  auto triangle = [&](float yc, float y1c, float y2c, float yd, float y1d, float y2d, float wxs, float wys, float bxs,
                      float bys, bool dmask) {
    Tri r;
    const float yr = from_right_lane(yc), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
    const float zij_1 = rmask ? ((yc - yr) + y1c) : 0.f;
    const float zij_2 = dmask ? ((yc - yd) + y2c) : 0.f;
    const float hwx = huber_w(zij_2 * zij_2 * wys + zij_1 * zij_1 * wxs, kD0);
    const float u11 = rmask ? (y1c - y1r) : 0.f;
    const float u12 = dmask ? (y1c - y1d) : 0.f;
    const float hwy1 = huber_w(bxs * (u12 * u12 + u11 * u11), kD1);
    const float u21 = rmask ? (y2c - y2r) : 0.f;
    const float u22 = dmask ? (y2c - y2d) : 0.f;
    const float hwy2 = huber_w(bys * (u22 * u22 + u21 * u21), kD2);
    r.Fa = wys * (zij_2 * hwx);
    r.Fb = wxs * (zij_1 * hwx);
    r.G1y = bxs * (u12 * hwy1);
    r.G1x = bxs * (u11 * hwy1);
    r.G2y = bys * (u22 * hwy2);
    r.G2x = bys * (u21 * hwy2);
    return r;
  };
  // gradient step on (u, v1, v2), prox on u, extrapolation (TGV.cu:1637-1690, 1740-1773)
  struct Upd {
    float xh, y1n, y2n, x_loc, yn, y1o, y2o;
  };
  auto update = [&](float yc, float y1c, float y2c, const Tri& t, float aFa, float aG1y, float aG2y, float c, float rc1,
                    float bv, float x0, float x1, float x2, float tm) {
    Upd u;
    const float lFb = from_left_lane(t.Fb), lG1x = from_left_lane(t.G1x), lG2x = from_left_lane(t.G2x);
    float yt = yc, y1n = y1c, y2n = y2c;
    yt -= -aFa;
    y1n -= -aG1y;
    y2n -= -aG2y;
    yt -= -lFb;
    y1n -= -lG1x;
    y2n -= -lG2x;
    yt -= t.Fa;
    y1n -= t.G1y;
    y2n -= t.G2y + t.Fa;
    yt -= t.Fb;
    y1n -= t.G1x + t.Fb;
    y2n -= t.G2x;
    u.y1o = y1n + tm * (y1n - x1);
    u.y2o = y2n + tm * (y2n - x2);
    u.xh = yt;
    u.y1n = y1n;
    u.y2n = y2n;
    const float x_loc = prox(yt, c, rc1, bv);
    u.x_loc = x_loc;
    u.yn = x_loc + tm * (x_loc - x0);
    return u;
  };

  float upA[3][C], upB[3][C];  // terms handed down to the next row (Fa, G1y, G2y), per iteration
  float pyB[3][C], pxB[3][C], pbb[C], pc = 0.f, prc1 = 1.f, pwxs = 0.f, pwys = 0.f, pbxs = 0.f, pbys = 0.f;
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    pbb[ch] = 0.f;
#pragma unroll
    for (int v = 0; v < 3; v++) upA[v][ch] = upB[v][ch] = pyB[v][ch] = pxB[v][ch] = 0.f;
  }

  auto step = [&](int k, const Fwd2Row<C>& cur, const Fwd2Row<C>& nxt, auto do_a, auto tri_b, auto do_b) {
    const int h = g.hs - 2 + k;  // A's row; B's row is h - 1
    const bool in_img = g.col_ok && h >= 0 && h < H;
    const bool dmaskA = h >= 0 && h < H - 1, dmaskB = h - 1 >= 0 && h - 1 < H - 1;
    const unsigned roffA = (unsigned)min(max(h, 0), H - 1) * W4 + wc;
    const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
    const bool storeA = store_lane && k >= 2 && k <= Reff + 1;
    const float rc1A = rcp_refined(1.f + cur.c);
    const float rc1B = prc1;  // iteration A formed it for this row one step ago
    float nyB[3][C], nxB[3][C];
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const Tri t = triangle(cur.y[0][ch], cur.y[1][ch], cur.y[2][ch], nxt.y[0][ch], nxt.y[1][ch], nxt.y[2][ch], cur.wxs,
                             cur.wys, cur.bxs, cur.bys, dmaskA);
      const float aFa = upA[0][ch], aG1y = upA[1][ch], aG2y = upA[2][ch];
      upA[0][ch] = t.Fa; upA[1][ch] = t.G1y; upA[2][ch] = t.G2y;
#pragma unroll
      for (int v = 0; v < 3; v++) nyB[v][ch] = nxB[v][ch] = 0.f;
      if (do_a.value) {
        const Upd u = update(cur.y[0][ch], cur.y[1][ch], cur.y[2][ch], t, aFa, aG1y, aG2y, cur.c, rc1A, cur.bb[ch],
                             cur.x[0][ch], cur.x[1][ch], cur.x[2][ch], tA);
        nyB[0][ch] = in_img ? u.yn : 0.f;  // B reads zero padding outside the image
        nyB[1][ch] = in_img ? u.y1o : 0.f;
        nyB[2][ch] = in_img ? u.y2o : 0.f;
        nxB[0][ch] = u.x_loc; nxB[1][ch] = u.y1n; nxB[2][ch] = u.y2n;
        if (X05 && storeA) {
          stg(xa_p[0][ch], roffA, u.xh);
          stg(xa_p[1][ch], roffA, u.y1n);
          stg(xa_p[2][ch], roffA, u.y2n);
        }
        if (!RING && storeA) {  // (own rows are inside the image: cur.y is the loaded value there)
#pragma unroll
          for (int v = 0; v < 3; v++) {
            if (keep_xin) stg(kx_p[v][ch], roffA, cur.x[v][ch]);
            if (keep_yin) stg(ky_p[v][ch], roffA, cur.y[v][ch]);
          }
        }
      }
    }
    if (tri_b.value) {
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const Tri t = triangle(pyB[0][ch], pyB[1][ch], pyB[2][ch], nyB[0][ch], nyB[1][ch], nyB[2][ch], pwxs, pwys, pbxs,
                               pbys, dmaskB);
        const float aFa = upB[0][ch], aG1y = upB[1][ch], aG2y = upB[2][ch];
        upB[0][ch] = t.Fa; upB[1][ch] = t.G1y; upB[2][ch] = t.G2y;
        if (do_b.value) {
          const Upd u = update(pyB[0][ch], pyB[1][ch], pyB[2][ch], t, aFa, aG1y, aG2y, pc, rc1B, pbb[ch], pxB[0][ch],
                               pxB[1][ch], pxB[2][ch], tB);
          if (store_lane) {
            if (store_y) {  // (half of a checkpoint: read once, by the backward pass -- it need not stay in the caches)
              stg_nt(yo_p[0][ch], roffB, u.yn);
              stg_nt(yo_p[1][ch], roffB, u.y1o);
              stg_nt(yo_p[2][ch], roffB, u.y2o);
            }
            if (store_x) {
              stg(xo_p[0][ch], roffB, u.x_loc);
              if (store_x_aux) {
                stg(xo_p[1][ch], roffB, u.y1n);
                stg(xo_p[2][ch], roffB, u.y2n);
              }
            }
            if (X05) {
              stg(xb_p[0][ch], roffB, u.xh);
              stg(xb_p[1][ch], roffB, u.y1n);
              stg(xb_p[2][ch], roffB, u.y2n);
            }
          }
        }
      }
    }
    pc = cur.c; prc1 = rc1A; pwxs = cur.wxs; pwys = cur.wys; pbxs = cur.bxs; pbys = cur.bys;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      pbb[ch] = cur.bb[ch];
#pragma unroll
      for (int v = 0; v < 3; v++) { pyB[v][ch] = nyB[v][ch]; pxB[v][ch] = nxB[v][ch]; }
    }
  };
  const std::true_type kYes{};
  const std::false_type kNo{};

  Fwd2Row<C> b0, b1, b2, b3;
  load_row(0, b0);
  load_row(1, b1);
  load_row(2, b2);
  load_row(3, b3);
  absorb(0, b0);
  absorb(1, b1);
  step(0, b0, b1, kNo, kNo, kNo);
  load_row(4, b0);
  absorb(2, b2);
  step(1, b1, b2, kYes, kNo, kNo);
  load_row(5, b1);
  absorb(3, b3);
  step(2, b2, b3, kYes, kYes, kNo);
  load_row(6, b2);
  for (int k = 3; k <= klast; k += 4) {  // cur / next rotate through (b3,b0) (b0,b1) (b1,b2) (b2,b3)
    absorb(k + 1, b0);
    step(k, b3, b0, kYes, kYes, kYes);
    load_row(k + 4, b3);
    if (k + 1 > klast) break;
    absorb(k + 2, b1);
    step(k + 1, b0, b1, kYes, kYes, kYes);
    load_row(k + 5, b0);
    if (k + 2 > klast) break;
    absorb(k + 3, b2);
    step(k + 2, b1, b2, kYes, kYes, kYes);
    load_row(k + 6, b1);
    if (k + 3 > klast) break;
    absorb(k + 4, b3);
    step(k + 3, b2, b3, kYes, kYes, kYes);
    load_row(k + 7, b2);
  }
}

// -------------------------------------------------------------------------------------------------
// Adjoint iteration with the y rebuild fused in: TGV.cu:224-644 (+1478-1541); END = the
// segment-start variant TGV.cu:1061-1472 that reads y from the checkpoint and writes the Huber
// weights with sqrt and divisions.
//
// Per triangle (owner q), with dy = (g_q - g_right + g1_q, g_q - g_down + g2_q), a = (z1 wx, z2 wy),
// deriv = dy1 a1 + dy2 a2, and for each smoothness term dg = (g1_q - g1_right, g1_q - g1_down),
// S = dg1 u1 + dg2 u2:
//     coupling term     Da = (W dy2) wy, Ea = deriv (a2 dW)  -> q's v2 row, negated: u row of the pixel below
//                       Db = (W dy1) wx, Eb = deriv (a1 dW)  -> q's v1 row, negated: u row of the pixel to the right
//     smoothness terms  Hy = (b Wy) dg2, Ny = (b ((dWy b) u2)) S -> q (Hy), negated: the pixel below
//                       Hx = (b Wy) dg1, Nx = (b ((dWy b) u1)) S -> q (Hx), negated: the pixel to the right
// Every product keeps the reference's operand order; an inactive triangle contributes E = N = 0.
// -------------------------------------------------------------------------------------------------
template <int C>
struct AdjRow {
  float c, rc1, wxs, wys, bxs, bys;
  float y[3][C];   // y[0]: loaded as x05[k-1] (or the checkpoint y) and rebuilt in place; y[1], y[2]: x05[k] aux (or checkpoint)
  float xa[C];     // x05[k] of u, for the prox regime
  float xl[C];     // FIRST only: u of the last x05 row, which the sweep's first step linearises at
  float yp[2][C];  // corrected gradient only: aux of x05[k-1] (or of the checkpointed x), for the momentum of aux y
  float bb[C], g[3][C];
  float gx_i[3][C], gb_i[C], gc_i, gwx0_i, gwx1_i, gwy0_i, gwy1_i;
  double opc_d;
};

// ADJ > 0 selects the corrected gradient (not the reference's): y is the forward pass's own y -- u: x+ + t (x+ - x-)
// with x+ = prox(x05[k]) and x- = prox(x05[k-1]) (ADJ == 1) or the checkpointed x of a segment start passed as
// x05b (ADJ == 2); aux: x05[k] + t (x05[k] - x05[k-1]), momentum included (TGV.cu:1686-1690) --, the upper-triangle
// v2 block multiplies by hub^2 like its siblings, and the per-step multipliers are 1.  END must be false then.
// FIRST: this step is the second of the reverse sweep, and the launch performs the sweep's first step (TGV.cu:151-218,
// a pointwise map: the prox adjoint on u, the auxiliary variables pass through) on the way in: g05_in is the caller's
// upstream gradient and x05l the last x05 row; every row that is loaded gets its incoming adjoint from them, and the
// strip's own rows add the first step's share to the accumulators, channel by channel, before the step's own (the
// order of two launches).  The accumulators and the partial g_x start at zero here, so the launch does not read them
// (gc_in, gb_in, gwx_in, gwy_in, gxk are not used) and the caller need not clear anything: every later launch reads
// only what the launch before it wrote in full.
template <int C, bool END, bool FINAL, int ADJ = 0, bool FIRST = false>
__global__ __launch_bounds__(256) void tgv_adjoint_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ x05a, const float* __restrict__ x05b, const float* __restrict__ yck,
    const float* __restrict__ gc_in, float* __restrict__ gc, const float* __restrict__ gb_in, float* __restrict__ gb,
    const float* __restrict__ gwx_in, float* __restrict__ gwx, const float* __restrict__ gwy_in,
    float* __restrict__ gwy, const float* __restrict__ g05_in, float* __restrict__ g05_out,
    const float* __restrict__ gxk, float* __restrict__ gxk_m1, float* __restrict__ gx_final, int N, int H, int W,
    float t, int R, int strips_x, int strips_y, int Ct, const float* __restrict__ x05l = nullptr) {
  static_assert(!(FIRST && END), "the first step is fused into a segment's inner steps only");
  StripGeom g;
  if (!strip_geometry(g, kCols, R, W, strips_x, strips_y, N)) return;
  const int Reff = min(R, H - g.hs);
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 0 && g.lane < 63 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;
  const double opt = 1. + (double)t;
  static_assert(!(END && ADJ), "the corrected gradient has no segment-start form");
  const float gxm = ADJ ? 1.f : kLocalGXMult;
  constexpr float kGC = ADJ ? 1.f : kLocalGCMult;
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                     *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwx0i_p = gwx_in + 2 * poff, *const gwx1i_p = gwx_in + 2 * poff + HW,
                     *const gwy0i_p = gwy_in + 2 * poff, *const gwy1i_p = gwy_in + 2 * poff + HW;
  float *const gco_p = gc + poff, *const gwx0o_p = gwx + 2 * poff, *const gwx1o_p = gwx + 2 * poff + HW,
               *const gwy0o_p = gwy + 2 * poff, *const gwy1o_p = gwy + 2 * poff + HW;
  const float *ys_p[3][C], *yp_p[2][C], *xa_p[C], *xl_p[C], *b_p[C], *g_p[3][C], *gxi_p[3][C], *gbi_p[C];
  float *g05o_p[3][C], *gxm_p[3][C], *gbo_p[C], *gxf_p[3][C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t qb = ((size_t)g.n * Ct + ch) * HW;
    b_p[ch] = b + qb; gbi_p[ch] = gb_in + qb; gbo_p[ch] = gb + qb;
#pragma unroll
    for (int v = 0; v < 3; v++) {
      const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)ch * HW;
      // y sources: u from x05[k-1] (rebuilt with x05[k]), aux straight from x05[k] (TGV.cu:1536-1537);
      // END: all three from the checkpoint y
      ys_p[v][ch] = (END ? yck : (v == 0 ? x05b : x05a)) + q;
      if (v > 0) yp_p[v - 1][ch] = x05b + q;
      g_p[v][ch] = g05_in + q; gxi_p[v][ch] = gxk + q;
      g05o_p[v][ch] = g05_out + q; gxm_p[v][ch] = gxk_m1 + q; gxf_p[v][ch] = FINAL ? gx_final + q : nullptr;
    }
    xa_p[ch] = x05a + (size_t)g.n * 3 * CHW + (size_t)ch * HW;
    xl_p[ch] = FIRST ? x05l + (size_t)g.n * 3 * CHW + (size_t)ch * HW : nullptr;
  }

  auto load_row = [&](int k, AdjRow<C>& in) {
    const int kk = min(k, Reff + 1);
    const int h = g.hs - 1 + kk;
    const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    const int hw = g.hs - 1 + min(kk, Reff);
    const unsigned off_w = (unsigned)(hw < 0 ? 0 : hw) * W4 + wc;
    const unsigned off_p = (unsigned)(g.hs - 1 + max(1, min(kk, Reff))) * W4 + wc;
    in.c = ldg(cf_p, off);
    in.wxs = ldg(wx_p, off_w);
    in.wys = ldg(wy_p, off_w);
    in.bxs = ldg(bx_p, off_w);
    in.bys = ldg(by_p, off_w);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.xa[ch] = ldg(xa_p[ch], off);
      if (FIRST) in.xl[ch] = ldg(xl_p[ch], off);
      in.bb[ch] = ldg(b_p[ch], off);
      in.gb_i[ch] = FIRST ? 0.f : ldg(gbi_p[ch], off_p);  // (FIRST: nothing accumulated yet, no partial g_x: zeros)
#pragma unroll
      for (int v = 0; v < 3; v++) {
        in.y[v][ch] = ldg(ys_p[v][ch], off);
        if (ADJ && v > 0) in.yp[v - 1][ch] = ldg(yp_p[v - 1][ch], off);
        in.g[v][ch] = ldg(g_p[v][ch], off);
        in.gx_i[v][ch] = FIRST ? 0.f : ldg(gxi_p[v][ch], off_p);
      }
    }
    in.gc_i = FIRST ? 0.f : ldg(gci_p, off_p);
    in.gwx0_i = FIRST ? 0.f : ldg(gwx0i_p, off_p);
    in.gwx1_i = FIRST ? 0.f : ldg(gwx1i_p, off_p);
    in.gwy0_i = FIRST ? 0.f : ldg(gwy0i_p, off_p);
    in.gwy1_i = FIRST ? 0.f : ldg(gwy1i_p, off_p);
  };
  auto absorb = [&](int k, AdjRow<C>& o) {
    const int h = g.hs - 1 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const inpaint::LaneMask inside(ok);
    o.c = inside(o.c);
    o.rc1 = rcp_refined(1.f + o.c);
    o.opc_d = 1. + (double)o.c;
    o.wxs = (ok && rmask) ? o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? o.wys : 0.f;
    o.bxs = inside(o.bxs);
    o.bys = inside(o.bys);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float xa = inside(o.xa[ch]), xb = inside(o.y[0][ch]), bv = inside(o.bb[ch]);
      if (ADJ) {
        const float xn = tvstrip::prox_huber1(xa, o.c, o.rc1, bv);
        const float xo = ADJ == 2 ? xb : tvstrip::prox_huber1(xb, o.c, o.rc1, bv);
        o.y[0][ch] = xn + t * (xn - xo);  // TGV.cu:1773
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = inside(o.y[v][ch]), xp = inside(o.yp[v - 1][ch]);
          o.y[v][ch] = xv + t * (xv - xp);  // TGV.cu:1686-1690
        }
      } else {
        o.y[0][ch] = END ? xb : tvstrip::rebuild_y_fast(bv, xa, xb, o.c, o.rc1, o.opc_d, t);
        o.y[1][ch] = inside(o.y[1][ch]);
        o.y[2][ch] = inside(o.y[2][ch]);
      }
      o.xa[ch] = xa;
      o.bb[ch] = bv;
#pragma unroll
      for (int v = 0; v < 3; v++) o.g[v][ch] = inside(o.g[v][ch]);
    }
    if (FIRST) {
      // the sweep's first step at this row (TGV.cu:166-182): the upstream gradient of u through the prox at the last
      // x05 row.  The accumulators belong to the strip's own rows; what rows above and below make of them is never used.
      const float opc = 1.f + o.c;
      const float rc2 = rcp_refined(opc * opc);
      float gcv = o.gc_i;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float df = o.g[0][ch], bv = o.bb[ch], xh = inside(o.xl[ch]);
        const float diff = bv - xh;
        const float sign = (diff < 0) ? -1.f : 1.f;
        const bool quad = (o.opc_d >= (double)(sign * diff));
        const float gc_q = df * (div_by(bv, opc, o.rc1) - div_by(o.c * bv + xh, opc * opc, rc2)) * kGC;
        const float gb_q = div_by(df * o.c, opc, o.rc1) * 1.0f;
        o.g[0][ch] = quad ? div_by(df, opc, o.rc1) : df;
        gcv += quad ? gc_q : sign * df * kGC;
        o.gb_i[ch] = quad ? o.gb_i[ch] + gb_q : 0.f;  // (TGV.cu:181 writes zero outside the quadratic regime)
      }
      o.gc_i = gcv;
    }
  };

  // terms handed down to the row below: coupling (Da, Ea) and the two smoothness terms (Hy, Ny)
  float dDa[C], dEa[C], dH1[C], dN1[C], dH2[C], dN2[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) dDa[ch] = dEa[ch] = dH1[ch] = dN1[ch] = dH2[ch] = dN2[ch] = 0.f;

  // Huber weight, activity and weight derivative of one term in the kernel's own form
  auto huber = [&](float A, float delta, float& Wt, bool& act, float& dW, float& hub2) {
    if (!wave_any(A > kHuberQuiet)) {  // no lane of the wavefront is near the threshold: weight 1, term inactive
      Wt = 1.f; act = false; dW = 0.f; hub2 = 1.f;
      return;
    }
    if (END) {  // TGV.cu:1132-1138
      const float hub = exact_sqrt(A);
      Wt = exact_rcp(fmaxf(1.f, div_by_fifth(hub)));  // delta is 0.2f for all three terms
      act = hub > delta;
      hub2 = hub * hub;
      dW = exact_div(Wt, hub2);
    } else {  // TGV.cu:313-319
      const float hub = rsq_exact(A);
      Wt = fminf(1.f, hub * delta);
      act = Wt < 1.0f;
      hub2 = hub * hub;
      dW = Wt * hub2;
    }
  };

  auto compute = [&](int r, const AdjRow<C>& cur, const AdjRow<C>& nxt, auto first) {
    const int h = g.hs - 1 + r;  // owner row of this step
    const bool dmask = h >= 0 && h < H - 1;
    const unsigned roff = (unsigned)(h >= 0 ? h : 0) * W4 + wc;
    float gcv = cur.gc_i, gwx0 = cur.gwx0_i, gwx1 = cur.gwx1_i, gwy0 = cur.gwy0_i, gwy1 = cur.gwy1_i, rc2 = 0.f;
    if (!first.value) rc2 = rcp_refined((1.f + cur.c) * (1.f + cur.c));
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float yk = cur.y[0][ch], y1c = cur.y[1][ch], y2c = cur.y[2][ch];
      const float gk = cur.g[0][ch], g1k = cur.g[1][ch], g2k = cur.g[2][ch];
      const float yr = from_right_lane(yk), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
      const float gr = from_right_lane(gk), g1r = from_right_lane(g1k), g2r = from_right_lane(g2k);
      const float yd = nxt.y[0][ch], y1d = nxt.y[1][ch], y2d = nxt.y[2][ch];
      const float gd = nxt.g[0][ch], g1d = nxt.g[1][ch], g2d = nxt.g[2][ch];
      const float wxv = cur.wxs, wyv = cur.wys, bX = cur.bxs, bY = cur.bys;

      // ---- coupling term, TGV.cu:421-455 / 1230-1260 ----
      const float aij_1 = rmask ? ((yr - yk) - y1c) : 0.f;
      const float aij_2 = dmask ? ((yd - yk) - y2c) : 0.f;
      float Wt, dW, hub2;
      bool act;
      huber(aij_2 * aij_2 * wyv + aij_1 * aij_1 * wxv, kD0, Wt, act, dW, hub2);
      const float dy1 = gk - gr + g1k;
      const float dy2 = gk - gd + g2k;
      const float a1 = aij_1 * wxv, a2 = aij_2 * wyv;
      const float deriv = dy1 * a1 + dy2 * a2;
      const float Da = Wt * dy2 * wyv, Db = Wt * dy1 * wxv;
      const float Ea = act ? deriv * (a2 * dW) : 0.f;
      const float Eb = act ? deriv * (a1 * dW) : 0.f;
      const float E0 = act ? deriv * ((a1 + a2) * dW) : 0.f;

      // ---- smoothness term of v1, TGV.cu:457-479 / 1262-1284 ----
      const float u11 = rmask ? (y1r - y1c) : 0.f;
      const float u12 = dmask ? (y1d - y1c) : 0.f;
      float W1, dW1, h1sq;
      bool act1;
      huber((u11 * u11 + u12 * u12) * bX, kD1, W1, act1, dW1, h1sq);
      const float dg1x = g1k - g1r, dg1y = g1k - g1d;
      const float H1x = rmask ? bX * W1 * dg1x : 0.f;
      const float H1y = dmask ? bX * W1 * dg1y : 0.f;
      const float S1 = dg1x * u11 + dg1y * u12;
      const float dv1 = dg1x * u11 * bX + dg1y * u12 * bX;
      const float R1 = act1 ? bX * dW1 * (u11 + u12) * dv1 : 0.f;
      const float N1y = act1 ? bX * (dW1 * bX * u12) * S1 : 0.f;
      const float N1x = act1 ? bX * (dW1 * bX * u11) * S1 : 0.f;

      // ---- smoothness term of v2, TGV.cu:481-505 / 1286-1310 ----
      const float u21 = rmask ? (y2r - y2c) : 0.f;
      const float u22 = dmask ? (y2d - y2c) : 0.f;
      float W2, dW2, h2sq;
      bool act2;
      huber((u21 * u21 + u22 * u22) * bY, kD2, W2, act2, dW2, h2sq);
      const float dg2x = g2k - g2r, dg2y = g2k - g2d;
      const float H2x = rmask ? bY * W2 * dg2x : 0.f;
      const float H2y = dmask ? bY * W2 * dg2y : 0.f;
      const float S2 = dg2x * u21 + dg2y * u22;
      const float dv2 = dg2x * u21 * bY + dg2y * u22 * bY;
      const float R2 = act2 ? bY * dW2 * (u21 + u22) * dv2 : 0.f;
      // the main kernel's upper-triangle v2 block divides by hub^2 where every sibling multiplies (TGV.cu:355)
      const float dW2_below = (END || ADJ) ? dW2 : exact_div(W2, h2sq);
      const float N2y = act2 ? bY * (dW2_below * bY * u22) * S2 : 0.f;
      const float N2x = act2 ? bY * (dW2 * bY * u21) * S2 : 0.f;

      // shares of the pixel to the right
      const float lDb = from_left_lane(Db), lEb = from_left_lane(Eb);
      const float lH1 = from_left_lane(H1x), lN1 = from_left_lane(N1x);
      const float lH2 = from_left_lane(H2x), lN2 = from_left_lane(N2x);
      // shares handed down from the row above
      const float aDa = dDa[ch], aEa = dEa[ch], aH1 = dH1[ch], aN1 = dN1[ch], aH2 = dH2[ch], aN2 = dN2[ch];
      dDa[ch] = Da; dEa[ch] = Ea; dH1[ch] = H1y; dN1[ch] = N1y; dH2[ch] = H2y; dN2[ch] = N2y;

      if (!first.value) {
        // weight gradients of the pixel's own triangle (edge weights: channel 0, beta: channel 1)
        if (END) {  // TGV.cu:1245-1246
          gwx0 = gwx0 + gxm * dy1 * aij_1 * Wt;
          gwy0 = gwy0 + gxm * dy2 * aij_2 * Wt;
        } else {  // TGV.cu:438-439
          gwx0 = gwx0 + gxm * dy1 * (aij_1 * Wt);
          gwy0 = gwy0 + gxm * dy2 * (aij_2 * Wt);
        }
        {  // the literal 0.5 makes these updates double (TGV.cu:452-453)
          const float ny = (float)((double)gwy0 - (double)(gxm * (aij_2 * dW * aij_2)) * 0.5 * (double)deriv);
          const float nx = (float)((double)gwx0 - (double)(gxm * (aij_1 * dW * aij_1)) * 0.5 * (double)deriv);
          gwy0 = act ? ny : gwy0;
          gwx0 = act ? nx : gwx0;
        }
        gwx1 = gwx1 + gxm * S1 * W1;  // TGV.cu:468-469
        {
          const float n1 = (float)((double)gwx1 - (double)(gxm * (u12 * dW1 * u12 + u11 * dW1 * u11)) * 0.5 * (double)dv1);
          gwx1 = act1 ? n1 : gwx1;  // TGV.cu:478
        }
        gwy1 = gwy1 + gxm * S2 * W2;  // TGV.cu:494-495
        {
          const float n2 = (float)((double)gwy1 - (double)(gxm * (u22 * dW2 * u22 + u21 * dW2 * u21)) * 0.5 * (double)dv2);
          gwy1 = act2 ? n2 : gwy1;  // TGV.cu:503
        }

        float t0 = gk, t1 = g1k, t2 = g2k;
        // triangles of the pixel above (TGV.cu:304-360)
        t0 -= -aDa;
        t0 += -aEa;
        t1 -= -aH1;
        t1 += -aN1;
        t2 -= -aH2;
        t2 += -aN2;
        // triangles of the pixel to the left (TGV.cu:361-418)
        t0 -= -lDb;
        t0 += -lEb;
        t1 -= -lH1;
        t1 += -lN1;
        t2 -= -lH2;
        t2 += -lN2;
        // own triangle
        if (END) {  // TGV.cu:1241-1244
          t0 -= dy2 * wyv * Wt;
          t0 -= dy1 * wxv * Wt;
          t1 -= Wt * (g1k - gr + gk) * wxv;
          t2 -= Wt * (g2k - gd + gk) * wyv;
        } else {  // TGV.cu:435-437
          t0 -= Wt * (dy2 * wyv + dy1 * wxv);
          t1 -= Db;
          t2 -= Da;
        }
        t0 += E0;  // TGV.cu:447-449
        t2 += Ea;
        t1 += Eb;
        if (END) {  // TGV.cu:1271-1274: the v1 block takes the lower neighbour first
          t1 -= H1y;
          t1 -= H1x;
        } else {  // TGV.cu:463-466
          t1 -= H1x;
          t1 -= H1y;
        }
        t1 += R1;
        t2 -= H2x;  // TGV.cu:489-492
        t2 -= H2y;
        t2 += R2;

        // aux variables: momentum adjoint only (TGV.cu:560-577)
        const float gxm1 = -t * t1;
        float d1 = (float)((double)cur.gx_i[1][ch] + opt * (double)t1);
        d1 = fmaxf(-kClipLocalGrad, fminf(d1, kClipLocalGrad));
        const float gxm2 = -t * t2;
        float d2 = (float)((double)cur.gx_i[2][ch] + opt * (double)t2);
        d2 = fmaxf(-kClipLocalGrad, fminf(d2, kClipLocalGrad));
        // u: momentum adjoint (TGV.cu:579-585), then prox adjoint (TGV.cu:592-612)
        float df = (float)((double)cur.gx_i[0][ch] + opt * (double)t0);
        df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
        const float gxm0 = -t * t0;
        const float conf = cur.c, bv = cur.bb[ch], xh = cur.xa[ch];
        const float diff = bv - xh;
        const float sign = (diff < 0) ? -1.f : 1.f;
        const bool quad = (cur.opc_d >= (double)(sign * diff));
        const float opc = 1.f + conf;
        const float gc_q = df * (div_by(bv, opc, cur.rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
        const float g05_q = div_by(df, opc, cur.rc1);
        const float gb_q = div_by(df * conf, opc, cur.rc1) * 1.0f;
        const bool mid = !quad && (conf >= sign * diff);
        const float g05v = quad ? g05_q : (mid ? 0.f : df);
        gcv += quad ? gc_q : (mid ? 0.f : sign * df * kGC);
        float gbv = cur.gb_i[ch];
        gbv += quad ? gb_q : (mid ? df * 1.0f : 0.f);
        if (store_lane) {
          if (FINAL) {  // only the last step's g_x is read again (TGV.cu:3047)
            stg(gxf_p[0][ch], roff, df);
            stg(gxf_p[1][ch], roff, d1);
            stg(gxf_p[2][ch], roff, d2);
          }
          stg(gxm_p[0][ch], roff, gxm0);
          stg(gxm_p[1][ch], roff, gxm1);
          stg(gxm_p[2][ch], roff, gxm2);
          stg(g05o_p[0][ch], roff, g05v);
          stg(g05o_p[1][ch], roff, d1);
          stg(g05o_p[2][ch], roff, d2);
          stg(gbo_p[ch], roff, gbv);
        }
      }
    }
    if (!first.value && store_lane) {
      stg(gco_p, roff, gcv);
      stg(gwx0o_p, roff, gwx0);
      stg(gwx1o_p, roff, gwx1);
      stg(gwy0o_p, roff, gwy0);
      stg(gwy1o_p, roff, gwy1);
    }
  };
  const std::true_type kFirst{};
  const std::false_type kRow{};

  AdjRow<C> b0, b1, b2;
  load_row(0, b0);
  load_row(1, b1);
  load_row(2, b2);
  absorb(0, b0);
  absorb(1, b1);
  compute(0, b0, b1, kFirst);
  load_row(3, b0);
  for (int r = 1; r <= Reff; r += 3) {  // cur / next rotate through (b1,b2) (b2,b0) (b0,b1)
    absorb(r + 1, b2);
    compute(r, b1, b2, kRow);
    load_row(r + 3, b1);
    if (r + 1 > Reff) break;
    absorb(r + 2, b0);
    compute(r + 1, b2, b0, kRow);
    load_row(r + 4, b2);
    if (r + 2 > Reff) break;
    absorb(r + 3, b1);
    compute(r + 2, b0, b1, kRow);
    load_row(r + 5, b0);
  }
}

// -------------------------------------------------------------------------------------------------
// Accumulators at a segment end, in all pair kernels below: a BEND launch stores the segment's sums as a record; the
// zeros the reference leaves in the accumulators (TGVH.cu:178-216) are written by the very last launch of the sweep only
// (FINAL).  After any other BEND launch the accumulator set it would have written holds stale values, and the caller
// hands the next launch a field of zeros as gc_in / gb_in / gwx_in / gwy_in instead.
// -------------------------------------------------------------------------------------------------
// Two adjoint steps per launch (A = local iteration j, B = j-1): the arithmetic of
// tgv_adjoint_strip applied twice, B one row behind A in the same wavefront (the scheme of
// tvstrip::tv_adjoint_strip2).  A's g05[j] and partial g_x[j] stay in registers; the seven
// accumulators are read and written once for both steps.  BEND: B is the segment's first iteration
// (checkpoint y, segment-start arithmetic) and the segment flush is fused: the fp32 segment sums go into the
// segment's record (added into the fp64 totals after the last segment).  FINAL: B's completed g_x is stored and the accumulators are left at zero.
// To fit two wavefronts per SIMD the row buffers hold only what a row's neighbours need; the fields
// that only the pixel's own update reads (partial g_x, accumulators) are loaded one step ahead into a
// single set of registers.
// -------------------------------------------------------------------------------------------------
template <int C>
struct Adj2Row {
  float c, wxs, wys, bxs, bys;
  float yA[3][C];  // yA[0] rebuilt from x05[j], x05[j-1]; yA[1], yA[2] = aux of x05[j]
  float yB[3][C];  // yB[0] rebuilt from x05[j-1], x05[j-2] (loaded there); yB[1], yB[2] = aux of x05[j-1]; BEND: checkpoint y
  float xa0[C], xb0[C], bb[C], g[3][C];
  float pv[2][C];  // corrected gradient only: aux of x05[j-1]
};
template <int C>
struct Adj2Late {
  float gx_i[3][C], gb_i[C], gc_i, gwx0_i, gwx1_i, gwy0_i, gwy1_i;
};

template <int C, bool BEND, bool FINAL>
__global__ __launch_bounds__(256) void tgv_adjoint_strip2(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ x05a, const float* __restrict__ x05b, const float* __restrict__ x05c,
    const float* __restrict__ gc_in, float* __restrict__ gc, const float* __restrict__ gb_in, float* __restrict__ gb,
    const float* __restrict__ gwx_in, float* __restrict__ gwx, const float* __restrict__ gwy_in,
    float* __restrict__ gwy, const float* __restrict__ g05_in, float* __restrict__ g05_out,
    const float* __restrict__ gxk, float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  StripGeom g;
  if (!strip_geometry(g, kCols2, R, W, strips_x, strips_y, N, 2)) return;
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const float gxm = kLocalGXMult;
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                     *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwx0i_p = gwx_in + 2 * poff, *const gwx1i_p = gwx_in + 2 * poff + HW,
                     *const gwy0i_p = gwy_in + 2 * poff, *const gwy1i_p = gwy_in + 2 * poff + HW;
  float *const gco_p = gc + poff, *const gwx0o_p = gwx + 2 * poff, *const gwx1o_p = gwx + 2 * poff + HW,
               *const gwy0o_p = gwy + 2 * poff, *const gwy1o_p = gwy + 2 * poff + HW;
  const float *xa_p[3][C], *xb_p[3][C], *xc_p[C], *b_p[C], *g_p[3][C], *gxi_p[3][C], *gbi_p[C];
  float *g05o_p[3][C], *gxm_p[3][C], *gbo_p[C], *gxf_p[3][C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t qb = ((size_t)g.n * Ct + ch) * HW;
    b_p[ch] = b + qb; gbi_p[ch] = gb_in + qb; gbo_p[ch] = gb + qb;
    xc_p[ch] = x05c + (size_t)g.n * 3 * CHW + (size_t)ch * HW;  // u of x05[j-2] (BEND: u of the checkpoint y)
#pragma unroll
    for (int v = 0; v < 3; v++) {
      const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)ch * HW;
      xa_p[v][ch] = x05a + q;
      xb_p[v][ch] = ((BEND && v > 0) ? x05c : x05b) + q;  // B's aux y: x05[j-1], or the checkpoint when BEND
      g_p[v][ch] = g05_in + q; gxi_p[v][ch] = gxk + q;
      g05o_p[v][ch] = g05_out + q; gxm_p[v][ch] = gxk_m1 + q; gxf_p[v][ch] = FINAL ? gx_final + q : nullptr;
    }
  }
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  auto load_row = [&](int k, Adj2Row<C>& in) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
    in.c = ldg(cf_p, off);
    in.wxs = ldg(wx_p, off_w);
    in.wys = ldg(wy_p, off_w);
    in.bxs = ldg(bx_p, off_w);
    in.bys = ldg(by_p, off_w);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.xa0[ch] = ldg(xa_p[0][ch], off);
      in.yA[1][ch] = ldg(xa_p[1][ch], off);
      in.yA[2][ch] = ldg(xa_p[2][ch], off);
      in.xb0[ch] = ldg(xb_p[0][ch], off);
      in.yB[1][ch] = ldg(xb_p[1][ch], off);
      in.yB[2][ch] = ldg(xb_p[2][ch], off);
      in.yB[0][ch] = ldg(xc_p[ch], off);
      in.bb[ch] = ldg(b_p[ch], off);
#pragma unroll
      for (int v = 0; v < 3; v++) in.g[v][ch] = ldg(g_p[v][ch], off);
    }
  };
  auto load_late = [&](int k, Adj2Late<C>& in) {  // what A's update of row k and the accumulators of that pixel need
    const int h = g.hs - 2 + min(k, klast);
    const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
    const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.gb_i[ch] = ldg(gbi_p[ch], off_o);
#pragma unroll
      for (int v = 0; v < 3; v++) in.gx_i[v][ch] = ldg(gxi_p[v][ch], off_a);
    }
    in.gc_i = ldg(gci_p, off_o);
    in.gwx0_i = ldg(gwx0i_p, off_o);
    in.gwx1_i = ldg(gwx1i_p, off_o);
    in.gwy0_i = ldg(gwy0i_p, off_o);
    in.gwy1_i = ldg(gwy1i_p, off_o);
  };
  auto absorb = [&](int k, Adj2Row<C>& o) {
    const int h = g.hs - 2 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const inpaint::LaneMask inside(ok);
    o.c = inside(o.c);
    const float rc1 = rcp_refined(1.f + o.c);
    const double opc_d = 1. + (double)o.c;
    o.wxs = (ok && rmask) ? o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? o.wys : 0.f;
    o.bxs = inside(o.bxs);
    o.bys = inside(o.bys);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float xa = inside(o.xa0[ch]), xb = inside(o.xb0[ch]), xc = inside(o.yB[0][ch]), bv = inside(o.bb[ch]);
      o.yA[0][ch] = tvstrip::rebuild_y_fast(bv, xa, xb, o.c, rc1, opc_d, tA);
      o.yB[0][ch] = BEND ? xc : tvstrip::rebuild_y_fast(bv, xb, xc, o.c, rc1, opc_d, tB);
      o.xa0[ch] = xa;
      o.xb0[ch] = xb;
      o.bb[ch] = bv;
#pragma unroll
      for (int v = 1; v < 3; v++) {
        o.yA[v][ch] = inside(o.yA[v][ch]);
        o.yB[v][ch] = inside(o.yB[v][ch]);
      }
#pragma unroll
      for (int v = 0; v < 3; v++) o.g[v][ch] = inside(o.g[v][ch]);
    }
  };

  // Huber weight, activity and weight derivative of one term, in the main or the segment-start form
  auto huber = [&](float A, float delta, float& Wt, bool& act, float& dW, float& hub2, auto end_form) {
    if (!wave_any(A > kHuberQuiet)) {  // no lane of the wavefront is near the threshold: weight 1, term inactive
      Wt = 1.f; act = false; dW = 0.f; hub2 = 1.f;
      return;
    }
    if (end_form.value) {  // TGV.cu:1132-1138
      const float hub = exact_sqrt(A);
      Wt = exact_rcp(fmaxf(1.f, div_by_fifth(hub)));  // delta is 0.2f for all three terms
      act = hub > delta;
      hub2 = hub * hub;
      dW = exact_div(Wt, hub2);
    } else {  // TGV.cu:313-319
      const float hub = rsq_exact(A);
      Wt = fminf(1.f, hub * delta);
      act = Wt < 1.0f;
      hub2 = hub * hub;
      dW = Wt * hub2;
    }
  };

  struct Acc {  // the weight-gradient accumulators of one pixel
    float gwx0, gwx1, gwy0, gwy1;
  };
  struct T3 {
    float t0, t1, t2;
  };
  // One pixel of one step: the triangle owned by the pixel (all shares), the terms handed down
  // (dn[6], read then replaced) and, when upd, the pixel's weight gradients and J^T g.
  auto pixel = [&](float yk, float y1c, float y2c, float yd, float y1d, float y2d, float gk, float g1k, float g2k,
                   float gd, float g1d, float g2d, float wxv, float wyv, float bX, float bY, bool dmask, float* dn,
                   Acc& acc, auto end_form, auto upd) {
    const float yr = from_right_lane(yk), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
    const float gr = from_right_lane(gk), g1r = from_right_lane(g1k), g2r = from_right_lane(g2k);
    // ---- coupling term ----
    const float aij_1 = rmask ? ((yr - yk) - y1c) : 0.f;
    const float aij_2 = dmask ? ((yd - yk) - y2c) : 0.f;
    float Wt, dW, hub2;
    bool act;
    huber(aij_2 * aij_2 * wyv + aij_1 * aij_1 * wxv, kD0, Wt, act, dW, hub2, end_form);
    const float dy1 = gk - gr + g1k;
    const float dy2 = gk - gd + g2k;
    const float a1 = aij_1 * wxv, a2 = aij_2 * wyv;
    const float deriv = dy1 * a1 + dy2 * a2;
    const float Da = Wt * dy2 * wyv, Db = Wt * dy1 * wxv;
    const float Ea = act ? deriv * (a2 * dW) : 0.f;
    const float Eb = act ? deriv * (a1 * dW) : 0.f;
    const float E0 = act ? deriv * ((a1 + a2) * dW) : 0.f;
    // ---- smoothness term of v1 ----
    const float u11 = rmask ? (y1r - y1c) : 0.f;
    const float u12 = dmask ? (y1d - y1c) : 0.f;
    float W1, dW1, h1sq;
    bool act1;
    huber((u11 * u11 + u12 * u12) * bX, kD1, W1, act1, dW1, h1sq, end_form);
    const float dg1x = g1k - g1r, dg1y = g1k - g1d;
    const float H1x = rmask ? bX * W1 * dg1x : 0.f;
    const float H1y = dmask ? bX * W1 * dg1y : 0.f;
    const float S1 = dg1x * u11 + dg1y * u12;
    const float dv1 = dg1x * u11 * bX + dg1y * u12 * bX;
    const float R1 = act1 ? bX * dW1 * (u11 + u12) * dv1 : 0.f;
    const float N1y = act1 ? bX * (dW1 * bX * u12) * S1 : 0.f;
    const float N1x = act1 ? bX * (dW1 * bX * u11) * S1 : 0.f;
    // ---- smoothness term of v2 ----
    const float u21 = rmask ? (y2r - y2c) : 0.f;
    const float u22 = dmask ? (y2d - y2c) : 0.f;
    float W2, dW2, h2sq;
    bool act2;
    huber((u21 * u21 + u22 * u22) * bY, kD2, W2, act2, dW2, h2sq, end_form);
    const float dg2x = g2k - g2r, dg2y = g2k - g2d;
    const float H2x = rmask ? bY * W2 * dg2x : 0.f;
    const float H2y = dmask ? bY * W2 * dg2y : 0.f;
    const float S2 = dg2x * u21 + dg2y * u22;
    const float dv2 = dg2x * u21 * bY + dg2y * u22 * bY;
    const float R2 = act2 ? bY * dW2 * (u21 + u22) * dv2 : 0.f;
    const float dW2_below = end_form.value ? dW2 : exact_div(W2, h2sq);  // TGV.cu:355
    const float N2y = act2 ? bY * (dW2_below * bY * u22) * S2 : 0.f;
    const float N2x = act2 ? bY * (dW2 * bY * u21) * S2 : 0.f;

    const float lDb = from_left_lane(Db), lEb = from_left_lane(Eb);
    const float lH1 = from_left_lane(H1x), lN1 = from_left_lane(N1x);
    const float lH2 = from_left_lane(H2x), lN2 = from_left_lane(N2x);
    const float aDa = dn[0], aEa = dn[1], aH1 = dn[2], aN1 = dn[3], aH2 = dn[4], aN2 = dn[5];
    dn[0] = Da; dn[1] = Ea; dn[2] = H1y; dn[3] = N1y; dn[4] = H2y; dn[5] = N2y;
    T3 r{0.f, 0.f, 0.f};
    if (upd.value) {
      if (end_form.value) {
        acc.gwx0 = acc.gwx0 + gxm * dy1 * aij_1 * Wt;
        acc.gwy0 = acc.gwy0 + gxm * dy2 * aij_2 * Wt;
      } else {
        acc.gwx0 = acc.gwx0 + gxm * dy1 * (aij_1 * Wt);
        acc.gwy0 = acc.gwy0 + gxm * dy2 * (aij_2 * Wt);
      }
      {
        const float ny = (float)((double)acc.gwy0 - (double)(gxm * (aij_2 * dW * aij_2)) * 0.5 * (double)deriv);
        const float nx = (float)((double)acc.gwx0 - (double)(gxm * (aij_1 * dW * aij_1)) * 0.5 * (double)deriv);
        acc.gwy0 = act ? ny : acc.gwy0;
        acc.gwx0 = act ? nx : acc.gwx0;
      }
      acc.gwx1 = acc.gwx1 + gxm * S1 * W1;
      {
        const float n1 = (float)((double)acc.gwx1 - (double)(gxm * (u12 * dW1 * u12 + u11 * dW1 * u11)) * 0.5 * (double)dv1);
        acc.gwx1 = act1 ? n1 : acc.gwx1;
      }
      acc.gwy1 = acc.gwy1 + gxm * S2 * W2;
      {
        const float n2 = (float)((double)acc.gwy1 - (double)(gxm * (u22 * dW2 * u22 + u21 * dW2 * u21)) * 0.5 * (double)dv2);
        acc.gwy1 = act2 ? n2 : acc.gwy1;
      }
      float t0 = gk, t1 = g1k, t2 = g2k;
      t0 -= -aDa;
      t0 += -aEa;
      t1 -= -aH1;
      t1 += -aN1;
      t2 -= -aH2;
      t2 += -aN2;
      t0 -= -lDb;
      t0 += -lEb;
      t1 -= -lH1;
      t1 += -lN1;
      t2 -= -lH2;
      t2 += -lN2;
      if (end_form.value) {
        t0 -= dy2 * wyv * Wt;
        t0 -= dy1 * wxv * Wt;
        t1 -= Wt * (g1k - gr + gk) * wxv;
        t2 -= Wt * (g2k - gd + gk) * wyv;
      } else {
        t0 -= Wt * (dy2 * wyv + dy1 * wxv);
        t1 -= Db;
        t2 -= Da;
      }
      t0 += E0;
      t2 += Ea;
      t1 += Eb;
      if (end_form.value) {
        t1 -= H1y;
        t1 -= H1x;
      } else {
        t1 -= H1x;
        t1 -= H1y;
      }
      t1 += R1;
      t2 -= H2x;
      t2 -= H2y;
      t2 += R2;
      r.t0 = t0; r.t1 = t1; r.t2 = t2;
    }
    return r;
  };
  // momentum adjoint of the three variables and prox adjoint of u (TGV.cu:560-612)
  struct Tail {
    float df, d1, d2, gxm0, gxm1, gxm2, g05v, gc_add, gb_add;
  };
  auto tail = [&](const T3& t, float gx0, float gx1, float gx2, double opt, float tm, float conf, float bv, float xh) {
    Tail o;
    o.gxm1 = -tm * t.t1;
    float d1 = (float)((double)gx1 + opt * (double)t.t1);
    o.d1 = fmaxf(-kClipLocalGrad, fminf(d1, kClipLocalGrad));
    o.gxm2 = -tm * t.t2;
    float d2 = (float)((double)gx2 + opt * (double)t.t2);
    o.d2 = fmaxf(-kClipLocalGrad, fminf(d2, kClipLocalGrad));
    float df = (float)((double)gx0 + opt * (double)t.t0);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    o.df = df;
    o.gxm0 = -tm * t.t0;
    const float rc1 = rcp_refined(1.f + conf);
    const float rc2 = rcp_refined((1.f + conf) * (1.f + conf));
    const double opc_d = 1. + (double)conf;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kLocalGCMult;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    o.g05v = quad ? g05_q : (mid ? 0.f : df);
    o.gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kLocalGCMult);
    o.gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
    return o;
  };

  float dnA[C][6], dnB[C][6];  // terms handed down to the next row, per step
  // row k-1 as step B sees it
  float pG[3][C], pgxm[3][C], pyB[3][C], pxb0[C], pbb[C], pgb[C], pgc = 0.f;
  Acc pacc{0.f, 0.f, 0.f, 0.f};
  float pc = 0.f, pwxs = 0.f, pwys = 0.f, pbxs = 0.f, pbys = 0.f;
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    pxb0[ch] = pbb[ch] = pgb[ch] = 0.f;
#pragma unroll
    for (int i = 0; i < 6; i++) dnA[ch][i] = dnB[ch][i] = 0.f;
#pragma unroll
    for (int v = 0; v < 3; v++) pG[v][ch] = pgxm[v][ch] = pyB[v][ch] = 0.f;
  }
  const std::true_type kYes{};
  const std::false_type kNo{};
  const std::integral_constant<bool, BEND> kBEnd{};

  auto step = [&](int k, const Adj2Row<C>& cur, const Adj2Row<C>& nxt, const Adj2Late<C>& late, auto do_a, auto tri_b,
                  auto do_b) {
    const int h = g.hs - 2 + k;  // A's row; B's row is h - 1
    const bool in_img = g.col_ok && h >= 0 && h < H;
    const bool dmaskA = h >= 0 && h < H - 1, dmaskB = h - 1 >= 0 && h - 1 < H - 1;
    const unsigned roffB_ = (unsigned)max(h - 1, 0) * W4 + wc;
    float nG[3][C], ngxm[3][C], ngb[C];
    float gcv = late.gc_i;
    Acc accA{late.gwx0_i, late.gwx1_i, late.gwy0_i, late.gwy1_i};
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const T3 t = pixel(cur.yA[0][ch], cur.yA[1][ch], cur.yA[2][ch], nxt.yA[0][ch], nxt.yA[1][ch], nxt.yA[2][ch],
                         cur.g[0][ch], cur.g[1][ch], cur.g[2][ch], nxt.g[0][ch], nxt.g[1][ch], nxt.g[2][ch], cur.wxs,
                         cur.wys, cur.bxs, cur.bys, dmaskA, dnA[ch], accA, kNo, do_a);
#pragma unroll
      for (int v = 0; v < 3; v++) nG[v][ch] = ngxm[v][ch] = 0.f;
      ngb[ch] = late.gb_i[ch];
      if (do_a.value) {
        const Tail o = tail(t, late.gx_i[0][ch], late.gx_i[1][ch], late.gx_i[2][ch], optA, tA, cur.c, cur.bb[ch], cur.xa0[ch]);
        gcv += o.gc_add;
        ngb[ch] += o.gb_add;
        nG[0][ch] = in_img ? o.g05v : 0.f;  // B reads zero padding outside the image
        nG[1][ch] = in_img ? o.d1 : 0.f;
        nG[2][ch] = in_img ? o.d2 : 0.f;
        ngxm[0][ch] = o.gxm0; ngxm[1][ch] = o.gxm1; ngxm[2][ch] = o.gxm2;
      }
    }
    if (tri_b.value) {
      float gcB = pgc;
      Acc accB = pacc;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const T3 t = pixel(pyB[0][ch], pyB[1][ch], pyB[2][ch], cur.yB[0][ch], cur.yB[1][ch], cur.yB[2][ch], pG[0][ch],
                           pG[1][ch], pG[2][ch], nG[0][ch], nG[1][ch], nG[2][ch], pwxs, pwys, pbxs, pbys, dmaskB,
                           dnB[ch], accB, kBEnd, do_b);
        if (do_b.value) {
          const Tail o = tail(t, pgxm[0][ch], pgxm[1][ch], pgxm[2][ch], optB, tB, pc, pbb[ch], pxb0[ch]);
          gcB += o.gc_add;
          const float gbv = pgb[ch] + o.gb_add;
          if (store_lane) {
            const unsigned roffB = offset_here(roffB_);
            if (FINAL) {
              stg(gxf_p[0][ch], roffB, o.df);
              stg(gxf_p[1][ch], roffB, o.d1);
              stg(gxf_p[2][ch], roffB, o.d2);
            }
            stg(gxm_p[0][ch], roffB, o.gxm0);
            stg(gxm_p[1][ch], roffB, o.gxm1);
            stg(gxm_p[2][ch], roffB, o.gxm2);
            stg(g05o_p[0][ch], roffB, o.g05v);
            stg(g05o_p[1][ch], roffB, o.d1);
            stg(g05o_p[2][ch], roffB, o.d2);
            if (BEND) {  // segment flush, fused: fp32 segment sum into the segment's record; zero at the sweep's end (TGVH.cu:178-216)
              seg_gb[((size_t)g.n * Ct + ch) * HW + (roffB >> 2)] = gbv;
              if (FINAL) stg(gbo_p[ch], roffB, 0.f);
            } else {
              stg(gbo_p[ch], roffB, gbv);
            }
          }
        }
      }
      if (do_b.value && store_lane) {
        const unsigned roffB = offset_here(roffB_);
        if (BEND) {
          const size_t e1 = poff + (roffB >> 2), e2 = 2 * poff + (roffB >> 2);
          seg_gc[e1] = gcB;
          seg_gwx[e2] = accB.gwx0;
          seg_gwx[e2 + HW] = accB.gwx1;
          seg_gwy[e2] = accB.gwy0;
          seg_gwy[e2 + HW] = accB.gwy1;
          if (FINAL) stg(gco_p, roffB, 0.f);
          if (FINAL) stg(gwx0o_p, roffB, 0.f);
          if (FINAL) stg(gwx1o_p, roffB, 0.f);
          if (FINAL) stg(gwy0o_p, roffB, 0.f);
          if (FINAL) stg(gwy1o_p, roffB, 0.f);
        } else {
          stg(gco_p, roffB, gcB);
          stg(gwx0o_p, roffB, accB.gwx0);
          stg(gwx1o_p, roffB, accB.gwx1);
          stg(gwy0o_p, roffB, accB.gwy0);
          stg(gwy1o_p, roffB, accB.gwy1);
        }
      }
    }
    pgc = gcv; pacc = accA;
    pc = cur.c; pwxs = cur.wxs; pwys = cur.wys; pbxs = cur.bxs; pbys = cur.bys;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      pgb[ch] = ngb[ch]; pxb0[ch] = cur.xb0[ch]; pbb[ch] = cur.bb[ch];
#pragma unroll
      for (int v = 0; v < 3; v++) { pG[v][ch] = nG[v][ch]; pgxm[v][ch] = ngxm[v][ch]; pyB[v][ch] = cur.yB[v][ch]; }
    }
  };

  Adj2Row<C> b0, b1, b2;
  Adj2Late<C> late;
  load_row(0, b0);
  load_row(1, b1);
  load_row(2, b2);
  load_late(1, late);
  absorb(0, b0);
  absorb(1, b1);
  step(0, b0, b1, late, kNo, kNo, kNo);
  load_row(3, b0);
  absorb(2, b2);
  step(1, b1, b2, late, kYes, kNo, kNo);
  load_row(4, b1);
  load_late(2, late);
  absorb(3, b0);
  step(2, b2, b0, late, kYes, kYes, kNo);
  load_row(5, b2);
  load_late(3, late);
  for (int k = 3; k <= klast; k += 3) {  // cur / next rotate through (b0,b1) (b1,b2) (b2,b0)
    absorb(k + 1, b1);
    step(k, b0, b1, late, kYes, kYes, kYes);
    load_row(k + 3, b0);
    load_late(k + 1, late);
    if (k + 1 > klast) break;
    absorb(k + 2, b2);
    step(k + 1, b1, b2, late, kYes, kYes, kYes);
    load_row(k + 4, b1);
    load_late(k + 2, late);
    if (k + 2 > klast) break;
    absorb(k + 3, b0);
    step(k + 2, b2, b0, late, kYes, kYes, kYes);
    load_row(k + 5, b2);
    load_late(k + 3, late);
  }
}

// -------------------------------------------------------------------------------------------------
// The same two adjoint steps per launch, split over the two wavefronts of a 128-thread workgroup:
// wavefront 0 runs step A (local iteration j) one row ahead and hands each row's results -- g05[j],
// the partial g_x[j] and the seven accumulators -- to wavefront 1 through LDS (7C+5 floats per lane,
// four slots, one LDS-only barrier per two rows); wavefront 1 runs step B (j-1) on them and stores.  Each
// wavefront holds one step's registers, so two workgroup pairs fit a SIMD where tgv_adjoint_strip2
// at two channels leaves room for one wavefront.  Arithmetic and memory traffic are those of
// tgv_adjoint_strip2 (wavefront 1 re-reads the weights, b and u of x05[j-1] from the cache).
// -------------------------------------------------------------------------------------------------
template <int C>
struct Adj2ARow {
  float c, wxs, wys, bxs, bys;
  float yA[3][C];  // yA[0] rebuilt from x05[j], x05[j-1]; yA[1], yA[2] = aux of x05[j]
  float xa0[C], xb0[C], bb[C], g[3][C];
  float pv[2][C];  // corrected gradient only: aux of x05[j-1]
};
template <int C>
struct Adj2BRow {
  float c, wxs, wys, bxs, bys;
  float yB[3][C];  // yB[0] rebuilt from x05[j-1], x05[j-2] (loaded there); yB[1], yB[2] = aux of x05[j-1]; BEND: checkpoint y
  float xb0[C], bb[C];
  float pv[2][C];  // corrected gradient only: aux of x05[j-2] (BEND: of the checkpointed x)
};

// TRUE_ADJ: the corrected gradient, as in tgv_adjoint_strip (with BEND, x05c is the checkpointed x of the segment start).
template <int C, bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(128) void tgv_adjoint_strip2w(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ x05a, const float* __restrict__ x05b, const float* __restrict__ x05c,
    const float* __restrict__ gc_in, float* __restrict__ gc, const float* __restrict__ gb_in, float* __restrict__ gb,
    const float* __restrict__ gwx_in, float* __restrict__ gwx, const float* __restrict__ gwy_in,
    float* __restrict__ gwy, const float* __restrict__ g05_in, float* __restrict__ g05_out,
    const float* __restrict__ gxk, float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  // floats step A hands to step B per row and lane: its results (7C + 5) and the row's inputs that both steps need
  // (c, four weights, b and the u of x05[j-1]: 2C + 5), which B would otherwise read from memory a second time
  constexpr int kHand = 9 * C + 10;
#ifndef TGV_ROWS_PER_BARRIER
#define TGV_ROWS_PER_BARRIER 2
#endif
  constexpr int kP = TGV_ROWS_PER_BARRIER;  // rows step A publishes per barrier
  __shared__ float hand[2 * kP][kHand][64];  // A fills kP slots while B works on the kP before them
  StripGeom g;
  if (!strip_geometry_block(g, kCols2, R, W, strips_x, strips_y, N, 2)) return;
  const int role = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wavefront 0: step A, wavefront 1: step B
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const float gxm = TRUE_ADJ ? 1.f : kLocalGXMult;
  constexpr float kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                     *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwx0i_p = gwx_in + 2 * poff, *const gwx1i_p = gwx_in + 2 * poff + HW,
                     *const gwy0i_p = gwy_in + 2 * poff, *const gwy1i_p = gwy_in + 2 * poff + HW;
  float *const gco_p = gc + poff, *const gwx0o_p = gwx + 2 * poff, *const gwx1o_p = gwx + 2 * poff + HW,
               *const gwy0o_p = gwy + 2 * poff, *const gwy1o_p = gwy + 2 * poff + HW;
  const float *xa_p[3][C], *xb_p[3][C], *xc_p[C], *pv_p[2][2][C], *b_p[C], *g_p[3][C], *gxi_p[3][C], *gbi_p[C];
  float *g05o_p[3][C], *gxm_p[3][C], *gbo_p[C], *gxf_p[3][C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t qb = ((size_t)g.n * Ct + ch) * HW;
    b_p[ch] = b + qb; gbi_p[ch] = gb_in + qb; gbo_p[ch] = gb + qb;
    xc_p[ch] = x05c + (size_t)g.n * 3 * CHW + (size_t)ch * HW;  // u of x05[j-2] (BEND: u of the checkpoint y)
#pragma unroll
    for (int v = 0; v < 3; v++) {
      const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)ch * HW;
      xa_p[v][ch] = x05a + q;
      xb_p[v][ch] = ((BEND && v > 0 && !TRUE_ADJ) ? x05c : x05b) + q;  // B's aux y: x05[j-1], or the checkpoint when BEND
      if (v > 0) {  // corrected gradient: the aux rows before A's and B's, for the momentum of aux y
        pv_p[0][v - 1][ch] = x05b + q;
        pv_p[1][v - 1][ch] = x05c + q;
      }
      g_p[v][ch] = g05_in + q; gxi_p[v][ch] = gxk + q;
      g05o_p[v][ch] = g05_out + q; gxm_p[v][ch] = gxk_m1 + q; gxf_p[v][ch] = FINAL ? gx_final + q : nullptr;
    }
  }
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  const auto row_offsets = [&](int k, unsigned& off, unsigned& off_w) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
  };

  // Huber weight, activity and weight derivative of one term, in the main or the segment-start form
  auto huber = [&](float A, float delta, float& Wt, bool& act, float& dW, float& hub2, auto end_form) {
    if (!wave_any(A > kHuberQuiet)) {  // no lane of the wavefront is near the threshold: weight 1, term inactive
      Wt = 1.f; act = false; dW = 0.f; hub2 = 1.f;
      return;
    }
    if (end_form.value) {  // TGV.cu:1132-1138
      const float hub = exact_sqrt(A);
      Wt = exact_rcp(fmaxf(1.f, div_by_fifth(hub)));  // delta is 0.2f for all three terms
      act = hub > delta;
      hub2 = hub * hub;
      dW = exact_div(Wt, hub2);
    } else {  // TGV.cu:313-319
      const float hub = rsq_exact(A);
      Wt = fminf(1.f, hub * delta);
      act = Wt < 1.0f;
      hub2 = hub * hub;
      dW = Wt * hub2;
    }
  };

  struct Acc {  // the weight-gradient accumulators of one pixel
    float gwx0, gwx1, gwy0, gwy1;
  };
  struct T3 {
    float t0, t1, t2;
  };
  // One pixel of one step: the triangle owned by the pixel (all shares), the terms handed down
  // (dn[6], read then replaced) and, when upd, the pixel's weight gradients and J^T g.
  auto pixel = [&](float yk, float y1c, float y2c, float yd, float y1d, float y2d, float gk, float g1k, float g2k,
                   float gd, float g1d, float g2d, float wxv, float wyv, float bX, float bY, bool dmask, float* dn,
                   Acc& acc, auto end_form, auto upd) {
    const float yr = from_right_lane(yk), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
    const float gr = from_right_lane(gk), g1r = from_right_lane(g1k), g2r = from_right_lane(g2k);
    // ---- coupling term ----
    const float aij_1 = rmask ? ((yr - yk) - y1c) : 0.f;
    const float aij_2 = dmask ? ((yd - yk) - y2c) : 0.f;
    float Wt, dW, hub2;
    bool act;
    huber(aij_2 * aij_2 * wyv + aij_1 * aij_1 * wxv, kD0, Wt, act, dW, hub2, end_form);
    const float dy1 = gk - gr + g1k;
    const float dy2 = gk - gd + g2k;
    const float a1 = aij_1 * wxv, a2 = aij_2 * wyv;
    const float deriv = dy1 * a1 + dy2 * a2;
    const float Da = Wt * dy2 * wyv, Db = Wt * dy1 * wxv;
    const float Ea = act ? deriv * (a2 * dW) : 0.f;
    const float Eb = act ? deriv * (a1 * dW) : 0.f;
    const float E0 = act ? deriv * ((a1 + a2) * dW) : 0.f;
    // ---- smoothness term of v1 ----
    const float u11 = rmask ? (y1r - y1c) : 0.f;
    const float u12 = dmask ? (y1d - y1c) : 0.f;
    float W1, dW1, h1sq;
    bool act1;
    huber((u11 * u11 + u12 * u12) * bX, kD1, W1, act1, dW1, h1sq, end_form);
    const float dg1x = g1k - g1r, dg1y = g1k - g1d;
    const float H1x = rmask ? bX * W1 * dg1x : 0.f;
    const float H1y = dmask ? bX * W1 * dg1y : 0.f;
    const float S1 = dg1x * u11 + dg1y * u12;
    const float dv1 = dg1x * u11 * bX + dg1y * u12 * bX;
    const float R1 = act1 ? bX * dW1 * (u11 + u12) * dv1 : 0.f;
    const float N1y = act1 ? bX * (dW1 * bX * u12) * S1 : 0.f;
    const float N1x = act1 ? bX * (dW1 * bX * u11) * S1 : 0.f;
    // ---- smoothness term of v2 ----
    const float u21 = rmask ? (y2r - y2c) : 0.f;
    const float u22 = dmask ? (y2d - y2c) : 0.f;
    float W2, dW2, h2sq;
    bool act2;
    huber((u21 * u21 + u22 * u22) * bY, kD2, W2, act2, dW2, h2sq, end_form);
    const float dg2x = g2k - g2r, dg2y = g2k - g2d;
    const float H2x = rmask ? bY * W2 * dg2x : 0.f;
    const float H2y = dmask ? bY * W2 * dg2y : 0.f;
    const float S2 = dg2x * u21 + dg2y * u22;
    const float dv2 = dg2x * u21 * bY + dg2y * u22 * bY;
    const float R2 = act2 ? bY * dW2 * (u21 + u22) * dv2 : 0.f;
    const float dW2_below = (end_form.value || TRUE_ADJ) ? dW2 : exact_div(W2, h2sq);  // TGV.cu:355
    const float N2y = act2 ? bY * (dW2_below * bY * u22) * S2 : 0.f;
    const float N2x = act2 ? bY * (dW2 * bY * u21) * S2 : 0.f;

    const float lDb = from_left_lane(Db), lEb = from_left_lane(Eb);
    const float lH1 = from_left_lane(H1x), lN1 = from_left_lane(N1x);
    const float lH2 = from_left_lane(H2x), lN2 = from_left_lane(N2x);
    const float aDa = dn[0], aEa = dn[1], aH1 = dn[2], aN1 = dn[3], aH2 = dn[4], aN2 = dn[5];
    dn[0] = Da; dn[1] = Ea; dn[2] = H1y; dn[3] = N1y; dn[4] = H2y; dn[5] = N2y;
    T3 r{0.f, 0.f, 0.f};
    if (upd.value) {
      if (end_form.value) {
        acc.gwx0 = acc.gwx0 + gxm * dy1 * aij_1 * Wt;
        acc.gwy0 = acc.gwy0 + gxm * dy2 * aij_2 * Wt;
      } else {
        acc.gwx0 = acc.gwx0 + gxm * dy1 * (aij_1 * Wt);
        acc.gwy0 = acc.gwy0 + gxm * dy2 * (aij_2 * Wt);
      }
      {
        const float ny = (float)((double)acc.gwy0 - (double)(gxm * (aij_2 * dW * aij_2)) * 0.5 * (double)deriv);
        const float nx = (float)((double)acc.gwx0 - (double)(gxm * (aij_1 * dW * aij_1)) * 0.5 * (double)deriv);
        acc.gwy0 = act ? ny : acc.gwy0;
        acc.gwx0 = act ? nx : acc.gwx0;
      }
      acc.gwx1 = acc.gwx1 + gxm * S1 * W1;
      {
        const float n1 = (float)((double)acc.gwx1 - (double)(gxm * (u12 * dW1 * u12 + u11 * dW1 * u11)) * 0.5 * (double)dv1);
        acc.gwx1 = act1 ? n1 : acc.gwx1;
      }
      acc.gwy1 = acc.gwy1 + gxm * S2 * W2;
      {
        const float n2 = (float)((double)acc.gwy1 - (double)(gxm * (u22 * dW2 * u22 + u21 * dW2 * u21)) * 0.5 * (double)dv2);
        acc.gwy1 = act2 ? n2 : acc.gwy1;
      }
      float t0 = gk, t1 = g1k, t2 = g2k;
      t0 -= -aDa;
      t0 += -aEa;
      t1 -= -aH1;
      t1 += -aN1;
      t2 -= -aH2;
      t2 += -aN2;
      t0 -= -lDb;
      t0 += -lEb;
      t1 -= -lH1;
      t1 += -lN1;
      t2 -= -lH2;
      t2 += -lN2;
      if (end_form.value) {
        t0 -= dy2 * wyv * Wt;
        t0 -= dy1 * wxv * Wt;
        t1 -= Wt * (g1k - gr + gk) * wxv;
        t2 -= Wt * (g2k - gd + gk) * wyv;
      } else {
        t0 -= Wt * (dy2 * wyv + dy1 * wxv);
        t1 -= Db;
        t2 -= Da;
      }
      t0 += E0;
      t2 += Ea;
      t1 += Eb;
      if (end_form.value) {
        t1 -= H1y;
        t1 -= H1x;
      } else {
        t1 -= H1x;
        t1 -= H1y;
      }
      t1 += R1;
      t2 -= H2x;
      t2 -= H2y;
      t2 += R2;
      r.t0 = t0; r.t1 = t1; r.t2 = t2;
    }
    return r;
  };
  // momentum adjoint of the three variables and prox adjoint of u (TGV.cu:560-612)
  struct Tail {
    float df, d1, d2, gxm0, gxm1, gxm2, g05v, gc_add, gb_add;
  };
  auto tail = [&](const T3& t, float gx0, float gx1, float gx2, double opt, float tm, float conf, float bv, float xh) {
    Tail o;
    o.gxm1 = -tm * t.t1;
    float d1 = (float)((double)gx1 + opt * (double)t.t1);
    o.d1 = fmaxf(-kClipLocalGrad, fminf(d1, kClipLocalGrad));
    o.gxm2 = -tm * t.t2;
    float d2 = (float)((double)gx2 + opt * (double)t.t2);
    o.d2 = fmaxf(-kClipLocalGrad, fminf(d2, kClipLocalGrad));
    float df = (float)((double)gx0 + opt * (double)t.t0);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    o.df = df;
    o.gxm0 = -tm * t.t0;
    const float rc1 = rcp_refined(1.f + conf);
    const float rc2 = rcp_refined((1.f + conf) * (1.f + conf));
    const double opc_d = 1. + (double)conf;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    o.g05v = quad ? g05_q : (mid ? 0.f : df);
    o.gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
    o.gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
    return o;
  };

  const std::true_type kYes{};
  const std::false_type kNo{};
  const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form

  if (role == 0) {
    // ---------------------------------- step A ----------------------------------
    auto load_row = [&](int k, Adj2ARow<C>& in) {
      unsigned off, off_w;
      row_offsets(k, off, off_w);
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
      in.bxs = ldg(bx_p, off_w);
      in.bys = ldg(by_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xa0[ch] = ldg(xa_p[0][ch], off);
        in.yA[1][ch] = ldg(xa_p[1][ch], off);
        in.yA[2][ch] = ldg(xa_p[2][ch], off);
        in.xb0[ch] = ldg(xb_p[0][ch], off);
        if (TRUE_ADJ) {
          in.pv[0][ch] = ldg(pv_p[0][0][ch], off);
          in.pv[1][ch] = ldg(pv_p[0][1][ch], off);
        }
        in.bb[ch] = ldg(b_p[ch], off);
#pragma unroll
        for (int v = 0; v < 3; v++) in.g[v][ch] = ldg(g_p[v][ch], off);
      }
    };
    auto load_late = [&](int k, Adj2Late<C>& in) {  // what A's update of row k and the accumulators of that pixel need
      const int h = g.hs - 2 + min(k, klast);
      const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
      const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.gb_i[ch] = ldg(gbi_p[ch], off_o);
#pragma unroll
        for (int v = 0; v < 3; v++) in.gx_i[v][ch] = ldg(gxi_p[v][ch], off_a);
      }
      in.gc_i = ldg(gci_p, off_o);
      in.gwx0_i = ldg(gwx0i_p, off_o);
      in.gwx1_i = ldg(gwx1i_p, off_o);
      in.gwy0_i = ldg(gwy0i_p, off_o);
      in.gwy1_i = ldg(gwy1i_p, off_o);
      // (the scheduler must not move the row loads that follow in front of these: see the order of the calls below)
      __builtin_amdgcn_sched_barrier(0);
    };
    auto absorb = [&](int k, Adj2ARow<C>& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      const float rc1 = rcp_refined(1.f + o.c);
      const double opc_d = 1. + (double)o.c;
      o.wxs = (ok && rmask) ? o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? o.wys : 0.f;
      o.bxs = inside(o.bxs);
      o.bys = inside(o.bys);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xa = inside(o.xa0[ch]), xb = inside(o.xb0[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pa = tvstrip::prox_huber1(xa, o.c, rc1, bv), pb = tvstrip::prox_huber1(xb, o.c, rc1, bv);
          o.yA[0][ch] = pa + tA * (pa - pb);  // TGV.cu:1773
        } else {
          o.yA[0][ch] = tvstrip::rebuild_y_fast(bv, xa, xb, o.c, rc1, opc_d, tA);
        }
        o.xa0[ch] = xa;
        o.xb0[ch] = xb;
        o.bb[ch] = bv;
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = inside(o.yA[v][ch]);
          o.yA[v][ch] = TRUE_ADJ ? xv + tA * (xv - inside(o.pv[v - 1][ch])) : xv;  // TGV.cu:1686-1690
        }
#pragma unroll
        for (int v = 0; v < 3; v++) o.g[v][ch] = inside(o.g[v][ch]);
      }
    };
    float dnA[C][6];
#pragma unroll
    for (int ch = 0; ch < C; ch++)
#pragma unroll
      for (int i = 0; i < 6; i++) dnA[ch][i] = 0.f;

    auto step = [&](int k, const Adj2ARow<C>& cur, const Adj2ARow<C>& nxt, const Adj2Late<C>& late, auto do_a) {
      const int h = g.hs - 2 + k;
      const bool in_img = g.col_ok && h >= 0 && h < H;
      const bool dmaskA = h >= 0 && h < H - 1;
      float (*slot)[64] = hand[k % (2 * kP)];
      float gcv = late.gc_i;
      Acc accA{late.gwx0_i, late.gwx1_i, late.gwy0_i, late.gwy1_i};
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const T3 t = pixel(cur.yA[0][ch], cur.yA[1][ch], cur.yA[2][ch], nxt.yA[0][ch], nxt.yA[1][ch], nxt.yA[2][ch],
                           cur.g[0][ch], cur.g[1][ch], cur.g[2][ch], nxt.g[0][ch], nxt.g[1][ch], nxt.g[2][ch], cur.wxs,
                           cur.wys, cur.bxs, cur.bys, dmaskA, dnA[ch], accA, kNo, do_a);
        float nG[3] = {0.f, 0.f, 0.f}, ngxm[3] = {0.f, 0.f, 0.f};
        float ngb = late.gb_i[ch];
        if (do_a.value) {
          const Tail o = tail(t, late.gx_i[0][ch], late.gx_i[1][ch], late.gx_i[2][ch], optA, tA, cur.c, cur.bb[ch], cur.xa0[ch]);
          gcv += o.gc_add;
          ngb += o.gb_add;
          nG[0] = in_img ? o.g05v : 0.f;  // B reads zero padding outside the image
          nG[1] = in_img ? o.d1 : 0.f;
          nG[2] = in_img ? o.d2 : 0.f;
          ngxm[0] = o.gxm0; ngxm[1] = o.gxm1; ngxm[2] = o.gxm2;
        }
#pragma unroll
        for (int v = 0; v < 3; v++) {
          slot[v * C + ch][g.lane] = nG[v];
          slot[3 * C + v * C + ch][g.lane] = ngxm[v];
        }
        slot[6 * C + ch][g.lane] = ngb;
      }
      slot[7 * C + 0][g.lane] = gcv;
      slot[7 * C + 1][g.lane] = accA.gwx0;
      slot[7 * C + 2][g.lane] = accA.gwx1;
      slot[7 * C + 3][g.lane] = accA.gwy0;
      slot[7 * C + 4][g.lane] = accA.gwy1;
      // row k's inputs as A absorbed them (zero outside the image): B takes them from here
      slot[7 * C + 5][g.lane] = cur.c;
      slot[7 * C + 6][g.lane] = cur.wxs;
      slot[7 * C + 7][g.lane] = cur.wys;
      slot[7 * C + 8][g.lane] = cur.bxs;
      slot[7 * C + 9][g.lane] = cur.bys;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        slot[7 * C + 10 + ch][g.lane] = cur.bb[ch];
        slot[8 * C + 10 + ch][g.lane] = cur.xb0[ch];
      }
    };

    // A publishes kP rows per barrier: the barrier after row k with k % kP == kP - 1 makes rows k-kP+1 .. k visible to
    // step B, which works on them while A fills the other kP slots (one barrier per row made each wavefront wait for
    // the other's slowest row)
    auto publish = [&](int k) {
      if (k % kP == kP - 1) lds_barrier();
    };
    // (The accumulators of row k+1 are asked for BEFORE the rows prefetched further ahead: loads return in order, so a
    // wait for the youngest load of the queue would drain every prefetched row with it.)
    Adj2ARow<C> b0, b1, b2;
    Adj2Late<C> late;
    load_row(0, b0);
    load_row(1, b1);
    load_late(1, late);
    load_row(2, b2);
    absorb(0, b0);
    absorb(1, b1);
    step(0, b0, b1, late, kNo);
    load_row(3, b0);
    publish(0);
    absorb(2, b2);
    step(1, b1, b2, late, kYes);
    load_late(2, late);
    load_row(4, b1);
    publish(1);
    absorb(3, b0);
    step(2, b2, b0, late, kYes);
    load_late(3, late);
    load_row(5, b2);
    publish(2);
    for (int k = 3; k <= klast; k += 3) {  // cur / next rotate through (b0,b1) (b1,b2) (b2,b0)
      absorb(k + 1, b1);
      step(k, b0, b1, late, kYes);
      load_late(k + 1, late);
      load_row(k + 3, b0);
      publish(k);
      if (k + 1 > klast) break;
      absorb(k + 2, b2);
      step(k + 1, b1, b2, late, kYes);
      load_late(k + 2, late);
      load_row(k + 4, b1);
      publish(k + 1);
      if (k + 2 > klast) break;
      absorb(k + 3, b0);
      step(k + 2, b2, b0, late, kYes);
      load_late(k + 3, late);
      load_row(k + 5, b2);
      publish(k + 2);
    }
    if (klast % kP != kP - 1) lds_barrier();  // the last rows have not been published yet
  } else {
    // ---------------------------------- step B ----------------------------------
    auto load_row = [&](int k, Adj2BRow<C>& in) {  // (c, the weights, b and x05[j-1]'s u come from step A, see absorb)
      unsigned off, off_w;
      row_offsets(k, off, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.yB[1][ch] = ldg(xb_p[1][ch], off);
        in.yB[2][ch] = ldg(xb_p[2][ch], off);
        in.yB[0][ch] = ldg(xc_p[ch], off);
        if (TRUE_ADJ) {
          in.pv[0][ch] = ldg(pv_p[1][0][ch], off);
          in.pv[1][ch] = ldg(pv_p[1][1][ch], off);
        }
      }
    };
    auto absorb = [&](int k, Adj2BRow<C>& o) {  // after await(k): row k's slot is visible
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      const float (*slot)[64] = hand[k % (2 * kP)];
      o.c = slot[7 * C + 5][g.lane];  // already zero outside the image
      o.wxs = slot[7 * C + 6][g.lane];
      o.wys = slot[7 * C + 7][g.lane];
      o.bxs = slot[7 * C + 8][g.lane];
      o.bys = slot[7 * C + 9][g.lane];
      const float rc1 = rcp_refined(1.f + o.c);
      const double opc_d = 1. + (double)o.c;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xb = slot[8 * C + 10 + ch][g.lane], xc = inside(o.yB[0][ch]), bv = slot[7 * C + 10 + ch][g.lane];
        if (TRUE_ADJ) {
          const float pb = tvstrip::prox_huber1(xb, o.c, rc1, bv);
          const float pc = BEND ? xc : tvstrip::prox_huber1(xc, o.c, rc1, bv);
          o.yB[0][ch] = pb + tB * (pb - pc);
        } else {
          o.yB[0][ch] = BEND ? xc : tvstrip::rebuild_y_fast(bv, xb, xc, o.c, rc1, opc_d, tB);
        }
        o.xb0[ch] = xb;
        o.bb[ch] = bv;
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = inside(o.yB[v][ch]);
          o.yB[v][ch] = TRUE_ADJ ? xv + tB * (xv - inside(o.pv[v - 1][ch])) : xv;
        }
      }
    };
    float dnB[C][6];
    // row k-1 as step B sees it
    float pG[3][C], pgxm[3][C], pyB[3][C], pxb0[C], pbb[C], pgb[C], pgc = 0.f;
    Acc pacc{0.f, 0.f, 0.f, 0.f};
    float pc = 0.f, pwxs = 0.f, pwys = 0.f, pbxs = 0.f, pbys = 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      pxb0[ch] = pbb[ch] = pgb[ch] = 0.f;
#pragma unroll
      for (int i = 0; i < 6; i++) dnB[ch][i] = 0.f;
#pragma unroll
      for (int v = 0; v < 3; v++) pG[v][ch] = pgxm[v][ch] = pyB[v][ch] = 0.f;
    }

    auto step = [&](int k, const Adj2BRow<C>& cur, auto tri_b, auto do_b) {
      const int h = g.hs - 2 + k;  // the row step A handed over; B's row is h - 1
      const bool dmaskB = h - 1 >= 0 && h - 1 < H - 1;
      const unsigned roffB_ = (unsigned)max(h - 1, 0) * W4 + wc;
      float (*slot)[64] = hand[k % (2 * kP)];
      float nG[3][C], ngxm[3][C], ngb[C];
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
#pragma unroll
        for (int v = 0; v < 3; v++) {
          nG[v][ch] = slot[v * C + ch][g.lane];
          ngxm[v][ch] = slot[3 * C + v * C + ch][g.lane];
        }
        ngb[ch] = slot[6 * C + ch][g.lane];
      }
      const float gcv = slot[7 * C + 0][g.lane];
      const Acc accA{slot[7 * C + 1][g.lane], slot[7 * C + 2][g.lane], slot[7 * C + 3][g.lane], slot[7 * C + 4][g.lane]};
      if (tri_b.value) {
        float gcB = pgc;
        Acc accB = pacc;
#pragma unroll
        for (int ch = 0; ch < C; ch++) {
          const T3 t = pixel(pyB[0][ch], pyB[1][ch], pyB[2][ch], cur.yB[0][ch], cur.yB[1][ch], cur.yB[2][ch], pG[0][ch],
                             pG[1][ch], pG[2][ch], nG[0][ch], nG[1][ch], nG[2][ch], pwxs, pwys, pbxs, pbys, dmaskB,
                             dnB[ch], accB, kBEnd, do_b);
          if (do_b.value) {
            const Tail o = tail(t, pgxm[0][ch], pgxm[1][ch], pgxm[2][ch], optB, tB, pc, pbb[ch], pxb0[ch]);
            gcB += o.gc_add;
            const float gbv = pgb[ch] + o.gb_add;
            if (store_lane) {
              const unsigned roffB = offset_here(roffB_);
              if (FINAL) {
                stg(gxf_p[0][ch], roffB, o.df);
                stg(gxf_p[1][ch], roffB, o.d1);
                stg(gxf_p[2][ch], roffB, o.d2);
              }
              stg(gxm_p[0][ch], roffB, o.gxm0);
              stg(gxm_p[1][ch], roffB, o.gxm1);
              stg(gxm_p[2][ch], roffB, o.gxm2);
              stg(g05o_p[0][ch], roffB, o.g05v);
              stg(g05o_p[1][ch], roffB, o.d1);
              stg(g05o_p[2][ch], roffB, o.d2);
              if (BEND) {  // segment flush, fused: fp32 segment sum into the segment's record; zero at the sweep's end (TGVH.cu:178-216)
                seg_gb[((size_t)g.n * Ct + ch) * HW + (roffB >> 2)] = gbv;
                if (FINAL) stg(gbo_p[ch], roffB, 0.f);
              } else {
                stg(gbo_p[ch], roffB, gbv);
              }
            }
          }
        }
        if (do_b.value && store_lane) {
          const unsigned roffB = offset_here(roffB_);
          if (BEND) {
            const size_t e1 = poff + (roffB >> 2), e2 = 2 * poff + (roffB >> 2);
            seg_gc[e1] = gcB;
            seg_gwx[e2] = accB.gwx0;
            seg_gwx[e2 + HW] = accB.gwx1;
            seg_gwy[e2] = accB.gwy0;
            seg_gwy[e2 + HW] = accB.gwy1;
            if (FINAL) stg(gco_p, roffB, 0.f);
            if (FINAL) stg(gwx0o_p, roffB, 0.f);
            if (FINAL) stg(gwx1o_p, roffB, 0.f);
            if (FINAL) stg(gwy0o_p, roffB, 0.f);
            if (FINAL) stg(gwy1o_p, roffB, 0.f);
          } else {
            stg(gco_p, roffB, gcB);
            stg(gwx0o_p, roffB, accB.gwx0);
            stg(gwx1o_p, roffB, accB.gwx1);
            stg(gwy0o_p, roffB, accB.gwy0);
            stg(gwy1o_p, roffB, accB.gwy1);
          }
        }
      }
      pgc = gcv; pacc = accA;
      pc = cur.c; pwxs = cur.wxs; pwys = cur.wys; pbxs = cur.bxs; pbys = cur.bys;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        pgb[ch] = ngb[ch]; pxb0[ch] = cur.xb0[ch]; pbb[ch] = cur.bb[ch];
#pragma unroll
        for (int v = 0; v < 3; v++) { pG[v][ch] = nG[v][ch]; pgxm[v][ch] = ngxm[v][ch]; pyB[v][ch] = cur.yB[v][ch]; }
      }
    };

    // B waits before every row k with k % kP == 0 for the barrier that published rows k .. k+kP-1
    auto await = [&](int k) {
      if (k % kP == 0) lds_barrier();
    };
    Adj2BRow<C> b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    await(0);
    absorb(0, b0);
    step(0, b0, kNo, kNo);
    load_row(3, b0);
    await(1);
    absorb(1, b1);
    step(1, b1, kNo, kNo);
    load_row(4, b1);
    await(2);
    absorb(2, b2);
    step(2, b2, kYes, kNo);
    load_row(5, b2);
    for (int k = 3; k <= klast; k += 3) {
      await(k);
      absorb(k, b0);
      step(k, b0, kYes, kYes);
      load_row(k + 3, b0);
      if (k + 1 > klast) break;
      await(k + 1);
      absorb(k + 1, b1);
      step(k + 1, b1, kYes, kYes);
      load_row(k + 4, b1);
      if (k + 2 > klast) break;
      await(k + 2);
      absorb(k + 2, b2);
      step(k + 2, b2, kYes, kYes);
      load_row(k + 5, b2);
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Two adjoint steps per launch for three and four flow channels: FOUR wavefronts per strip (256-thread
// workgroup).  The channels are split into two groups (the first CM, the second C1 <= CM of them);
// wavefronts 0 and 1 run step A on group 0 and group 1, wavefronts 2 and 3 step B on group 0 and
// group 1, each as the matching half of tgv_adjoint_strip2w.  The reference adds the terms of the five
// shared accumulators (gc, two channels of gwx, two of gwy) in the order A(ch 0 .. C-1), B(ch 0 .. C-1);
// here
//   A0 adds its terms to the accumulators read from memory and hands them on (LDS),
//   A1 adds its terms to what A0 handed on,
//   B0 does not touch the accumulators: it hands its terms on, one by one -- the gc term and, per weight
//      accumulator, the float that is added and the double that is subtracted after it (zero where the
//      Huber term is inactive: x - 0.0 is x),
//   B1 takes the accumulators after A1, applies B0's terms in channel order, then its own, and stores.
// Time runs in intervals of two rows with one LDS-only barrier between them: in interval t A0 works on
// rows 2t, 2t+1, A1 and B0 on the two rows before, B1 on the two before those; every record is written
// in one interval and read in the next, so two sets of two row slots per record type suffice.  Every
// wavefront passes the same number of barriers (intervals + 2).  Step B reads c, the weights, b and the
// u of x05[j-1] from memory itself (the records of two groups plus B0's terms fill the 64 KB of LDS a
// workgroup may hold).
// -------------------------------------------------------------------------------------------------
template <int CM, int C1, bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void tgv_adjoint_strip4w(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ bx,
    const float* __restrict__ by, const float* __restrict__ cf, const float* __restrict__ b,
    const float* __restrict__ x05a, const float* __restrict__ x05b, const float* __restrict__ x05c,
    const float* __restrict__ gc_in, float* __restrict__ gc, const float* __restrict__ gb_in, float* __restrict__ gb,
    const float* __restrict__ gwx_in, float* __restrict__ gwx, const float* __restrict__ gwy_in,
    float* __restrict__ gwy, const float* __restrict__ g05_in, float* __restrict__ g05_out,
    const float* __restrict__ gxk, float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  static_assert(C1 >= 1 && C1 <= CM, "the second group is the smaller one");
  constexpr int kP = 2;                // rows per interval
  constexpr int kSlots = 2 * kP;       // two sets of kP row slots
  constexpr int kRec = 7 * CM + 5;     // step A's results per row and lane: g05[j] (3), partial g_x[j] (3), gb per channel; the accumulators
  __shared__ float handA[2][kSlots][kRec][64];
  __shared__ float termF[kSlots][5 * CM][64];   // B0's terms: per channel the gc term and the four floats that are added
  __shared__ double termD[kSlots][4 * CM][64];  // ... and the four doubles that are subtracted after them
  StripGeom g;
  if (!strip_geometry_block(g, kCols2, R, W, strips_x, strips_y, N, 2)) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W, CHW = HW * Ct;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool rmask = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const float gxm = TRUE_ADJ ? 1.f : kLocalGXMult;
  constexpr float kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  const size_t poff = (size_t)g.n * HW;
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  const auto row_offsets = [&](int k, unsigned& off, unsigned& off_w) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
  };

  // Huber weight, activity and weight derivative of one term, in the main or the segment-start form
  auto huber = [&](float A, float delta, float& Wt, bool& act, float& dW, float& hub2, auto end_form) {
    if (!wave_any(A > kHuberQuiet)) {  // no lane of the wavefront is near the threshold: weight 1, term inactive
      Wt = 1.f; act = false; dW = 0.f; hub2 = 1.f;
      return;
    }
    if (end_form.value) {  // TGV.cu:1132-1138
      const float hub = exact_sqrt(A);
      Wt = exact_rcp(fmaxf(1.f, div_by_fifth(hub)));  // delta is 0.2f for all three terms
      act = hub > delta;
      hub2 = hub * hub;
      dW = exact_div(Wt, hub2);
    } else {  // TGV.cu:313-319
      const float hub = rsq_exact(A);
      Wt = fminf(1.f, hub * delta);
      act = Wt < 1.0f;
      hub2 = hub * hub;
      dW = Wt * hub2;
    }
  };

  struct Acc {  // the weight-gradient accumulators of one pixel
    float gwx0, gwx1, gwy0, gwy1;
  };
  // what one channel's triangle does to them: x = (float)((double)(x + add) - sub), sub = 0 where the term is inactive
  struct AccTerms {
    float add_wx0, add_wy0, add_wx1, add_wy1;
    double sub_wx0, sub_wy0, sub_wx1, sub_wy1;
  };
  auto apply_terms = [](Acc& acc, const AccTerms& t) {
    acc.gwx0 = (float)((double)(acc.gwx0 + t.add_wx0) - t.sub_wx0);
    acc.gwy0 = (float)((double)(acc.gwy0 + t.add_wy0) - t.sub_wy0);
    acc.gwx1 = (float)((double)(acc.gwx1 + t.add_wx1) - t.sub_wx1);
    acc.gwy1 = (float)((double)(acc.gwy1 + t.add_wy1) - t.sub_wy1);
  };
  struct T3 {
    float t0, t1, t2;
  };
  // One pixel of one step: the triangle owned by the pixel (all shares), the terms handed down
  // (dn[6], read then replaced) and, when upd, the pixel's weight-gradient terms and J^T g.
  auto pixel = [&](float yk, float y1c, float y2c, float yd, float y1d, float y2d, float gk, float g1k, float g2k,
                   float gd, float g1d, float g2d, float wxv, float wyv, float bX, float bY, bool dmask, float* dn,
                   AccTerms& at, auto end_form, auto upd) {
    const float yr = from_right_lane(yk), y1r = from_right_lane(y1c), y2r = from_right_lane(y2c);
    const float gr = from_right_lane(gk), g1r = from_right_lane(g1k), g2r = from_right_lane(g2k);
    // ---- coupling term ----
    const float aij_1 = rmask ? ((yr - yk) - y1c) : 0.f;
    const float aij_2 = dmask ? ((yd - yk) - y2c) : 0.f;
    float Wt, dW, hub2;
    bool act;
    huber(aij_2 * aij_2 * wyv + aij_1 * aij_1 * wxv, kD0, Wt, act, dW, hub2, end_form);
    const float dy1 = gk - gr + g1k;
    const float dy2 = gk - gd + g2k;
    const float a1 = aij_1 * wxv, a2 = aij_2 * wyv;
    const float deriv = dy1 * a1 + dy2 * a2;
    const float Da = Wt * dy2 * wyv, Db = Wt * dy1 * wxv;
    const float Ea = act ? deriv * (a2 * dW) : 0.f;
    const float Eb = act ? deriv * (a1 * dW) : 0.f;
    const float E0 = act ? deriv * ((a1 + a2) * dW) : 0.f;
    // ---- smoothness term of v1 ----
    const float u11 = rmask ? (y1r - y1c) : 0.f;
    const float u12 = dmask ? (y1d - y1c) : 0.f;
    float W1, dW1, h1sq;
    bool act1;
    huber((u11 * u11 + u12 * u12) * bX, kD1, W1, act1, dW1, h1sq, end_form);
    const float dg1x = g1k - g1r, dg1y = g1k - g1d;
    const float H1x = rmask ? bX * W1 * dg1x : 0.f;
    const float H1y = dmask ? bX * W1 * dg1y : 0.f;
    const float S1 = dg1x * u11 + dg1y * u12;
    const float dv1 = dg1x * u11 * bX + dg1y * u12 * bX;
    const float R1 = act1 ? bX * dW1 * (u11 + u12) * dv1 : 0.f;
    const float N1y = act1 ? bX * (dW1 * bX * u12) * S1 : 0.f;
    const float N1x = act1 ? bX * (dW1 * bX * u11) * S1 : 0.f;
    // ---- smoothness term of v2 ----
    const float u21 = rmask ? (y2r - y2c) : 0.f;
    const float u22 = dmask ? (y2d - y2c) : 0.f;
    float W2, dW2, h2sq;
    bool act2;
    huber((u21 * u21 + u22 * u22) * bY, kD2, W2, act2, dW2, h2sq, end_form);
    const float dg2x = g2k - g2r, dg2y = g2k - g2d;
    const float H2x = rmask ? bY * W2 * dg2x : 0.f;
    const float H2y = dmask ? bY * W2 * dg2y : 0.f;
    const float S2 = dg2x * u21 + dg2y * u22;
    const float dv2 = dg2x * u21 * bY + dg2y * u22 * bY;
    const float R2 = act2 ? bY * dW2 * (u21 + u22) * dv2 : 0.f;
    const float dW2_below = (end_form.value || TRUE_ADJ) ? dW2 : exact_div(W2, h2sq);  // TGV.cu:355
    const float N2y = act2 ? bY * (dW2_below * bY * u22) * S2 : 0.f;
    const float N2x = act2 ? bY * (dW2 * bY * u21) * S2 : 0.f;

    const float lDb = from_left_lane(Db), lEb = from_left_lane(Eb);
    const float lH1 = from_left_lane(H1x), lN1 = from_left_lane(N1x);
    const float lH2 = from_left_lane(H2x), lN2 = from_left_lane(N2x);
    const float aDa = dn[0], aEa = dn[1], aH1 = dn[2], aN1 = dn[3], aH2 = dn[4], aN2 = dn[5];
    dn[0] = Da; dn[1] = Ea; dn[2] = H1y; dn[3] = N1y; dn[4] = H2y; dn[5] = N2y;
    T3 r{0.f, 0.f, 0.f};
    if (upd.value) {
      if (end_form.value) {
        at.add_wx0 = gxm * dy1 * aij_1 * Wt;
        at.add_wy0 = gxm * dy2 * aij_2 * Wt;
      } else {
        at.add_wx0 = gxm * dy1 * (aij_1 * Wt);
        at.add_wy0 = gxm * dy2 * (aij_2 * Wt);
      }
      {
        const double sy = (double)(gxm * (aij_2 * dW * aij_2)) * 0.5 * (double)deriv;
        const double sx = (double)(gxm * (aij_1 * dW * aij_1)) * 0.5 * (double)deriv;
        at.sub_wy0 = act ? sy : 0.0;
        at.sub_wx0 = act ? sx : 0.0;
      }
      at.add_wx1 = gxm * S1 * W1;
      {
        const double s1 = (double)(gxm * (u12 * dW1 * u12 + u11 * dW1 * u11)) * 0.5 * (double)dv1;
        at.sub_wx1 = act1 ? s1 : 0.0;
      }
      at.add_wy1 = gxm * S2 * W2;
      {
        const double s2 = (double)(gxm * (u22 * dW2 * u22 + u21 * dW2 * u21)) * 0.5 * (double)dv2;
        at.sub_wy1 = act2 ? s2 : 0.0;
      }
      float t0 = gk, t1 = g1k, t2 = g2k;
      t0 -= -aDa;
      t0 += -aEa;
      t1 -= -aH1;
      t1 += -aN1;
      t2 -= -aH2;
      t2 += -aN2;
      t0 -= -lDb;
      t0 += -lEb;
      t1 -= -lH1;
      t1 += -lN1;
      t2 -= -lH2;
      t2 += -lN2;
      if (end_form.value) {
        t0 -= dy2 * wyv * Wt;
        t0 -= dy1 * wxv * Wt;
        t1 -= Wt * (g1k - gr + gk) * wxv;
        t2 -= Wt * (g2k - gd + gk) * wyv;
      } else {
        t0 -= Wt * (dy2 * wyv + dy1 * wxv);
        t1 -= Db;
        t2 -= Da;
      }
      t0 += E0;
      t2 += Ea;
      t1 += Eb;
      if (end_form.value) {
        t1 -= H1y;
        t1 -= H1x;
      } else {
        t1 -= H1x;
        t1 -= H1y;
      }
      t1 += R1;
      t2 -= H2x;
      t2 -= H2y;
      t2 += R2;
      r.t0 = t0; r.t1 = t1; r.t2 = t2;
    }
    return r;
  };
  // momentum adjoint of the three variables and prox adjoint of u (TGV.cu:560-612)
  struct Tail {
    float df, d1, d2, gxm0, gxm1, gxm2, g05v, gc_add, gb_add;
  };
  auto tail = [&](const T3& t, float gx0, float gx1, float gx2, double opt, float tm, float conf, float bv, float xh) {
    Tail o;
    o.gxm1 = -tm * t.t1;
    float d1 = (float)((double)gx1 + opt * (double)t.t1);
    o.d1 = fmaxf(-kClipLocalGrad, fminf(d1, kClipLocalGrad));
    o.gxm2 = -tm * t.t2;
    float d2 = (float)((double)gx2 + opt * (double)t.t2);
    o.d2 = fmaxf(-kClipLocalGrad, fminf(d2, kClipLocalGrad));
    float df = (float)((double)gx0 + opt * (double)t.t0);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    o.df = df;
    o.gxm0 = -tm * t.t0;
    const float rc1 = rcp_refined(1.f + conf);
    const float rc2 = rcp_refined((1.f + conf) * (1.f + conf));
    const double opc_d = 1. + (double)conf;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    o.g05v = quad ? g05_q : (mid ? 0.f : df);
    o.gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
    o.gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
    return o;
  };

  const std::true_type kYes{};
  const std::false_type kNo{};

  // ------------------------------------------ step A on one group ------------------------------------------
  auto role_a = [&](auto channels, auto group) {
    constexpr int C = decltype(channels)::value, G = decltype(group)::value;
    constexpr int chb = G ? CM : 0;  // the group's first channel
    const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                       *const cf_p = cf + poff;
    const float *const gci_p = gc_in + poff, *const gwx0i_p = gwx_in + 2 * poff, *const gwx1i_p = gwx_in + 2 * poff + HW,
                       *const gwy0i_p = gwy_in + 2 * poff, *const gwy1i_p = gwy_in + 2 * poff + HW;
    const float *xa_p[3][C], *xb0_p[C], *pv_p[2][C], *b_p[C], *g_p[3][C], *gxi_p[3][C], *gbi_p[C];
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const size_t qb = ((size_t)g.n * Ct + chb + ch) * HW;
      b_p[ch] = b + qb; gbi_p[ch] = gb_in + qb;
      xb0_p[ch] = x05b + (size_t)g.n * 3 * CHW + (size_t)(chb + ch) * HW;
#pragma unroll
      for (int v = 0; v < 3; v++) {
        const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)(chb + ch) * HW;
        xa_p[v][ch] = x05a + q;
        if (v > 0) pv_p[v - 1][ch] = x05b + q;  // corrected gradient: the aux rows before A's, for the momentum of aux y
        g_p[v][ch] = g05_in + q; gxi_p[v][ch] = gxk + q;
      }
    }
    auto load_row = [&](int k, Adj2ARow<C>& in) {
      unsigned off, off_w;
      row_offsets(k, off, off_w);
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
      in.bxs = ldg(bx_p, off_w);
      in.bys = ldg(by_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xa0[ch] = ldg(xa_p[0][ch], off);
        in.yA[1][ch] = ldg(xa_p[1][ch], off);
        in.yA[2][ch] = ldg(xa_p[2][ch], off);
        in.xb0[ch] = ldg(xb0_p[ch], off);
        if (TRUE_ADJ) {
          in.pv[0][ch] = ldg(pv_p[0][ch], off);
          in.pv[1][ch] = ldg(pv_p[1][ch], off);
        }
        in.bb[ch] = ldg(b_p[ch], off);
#pragma unroll
        for (int v = 0; v < 3; v++) in.g[v][ch] = ldg(g_p[v][ch], off);
      }
    };
    auto load_late = [&](int k, Adj2Late<C>& in) {  // what A's update of row k and the accumulators of that pixel need
      const int h = g.hs - 2 + min(k, klast);
      const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
      const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.gb_i[ch] = ldg(gbi_p[ch], off_o);
#pragma unroll
        for (int v = 0; v < 3; v++) in.gx_i[v][ch] = ldg(gxi_p[v][ch], off_a);
      }
      if (G == 0) {  // the second group continues the first group's sums
        in.gc_i = ldg(gci_p, off_o);
        in.gwx0_i = ldg(gwx0i_p, off_o);
        in.gwx1_i = ldg(gwx1i_p, off_o);
        in.gwy0_i = ldg(gwy0i_p, off_o);
        in.gwy1_i = ldg(gwy1i_p, off_o);
      } else {
        in.gc_i = in.gwx0_i = in.gwx1_i = in.gwy0_i = in.gwy1_i = 0.f;
      }
    };
    auto absorb = [&](int k, Adj2ARow<C>& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      const float rc1 = rcp_refined(1.f + o.c);
      const double opc_d = 1. + (double)o.c;
      o.wxs = (ok && rmask) ? o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? o.wys : 0.f;
      o.bxs = inside(o.bxs);
      o.bys = inside(o.bys);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xa = inside(o.xa0[ch]), xb = inside(o.xb0[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pa = tvstrip::prox_huber1(xa, o.c, rc1, bv), pb = tvstrip::prox_huber1(xb, o.c, rc1, bv);
          o.yA[0][ch] = pa + tA * (pa - pb);  // TGV.cu:1773
        } else {
          o.yA[0][ch] = tvstrip::rebuild_y_fast(bv, xa, xb, o.c, rc1, opc_d, tA);
        }
        o.xa0[ch] = xa;
        o.bb[ch] = bv;
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = inside(o.yA[v][ch]);
          o.yA[v][ch] = TRUE_ADJ ? xv + tA * (xv - inside(o.pv[v - 1][ch])) : xv;  // TGV.cu:1686-1690
        }
#pragma unroll
        for (int v = 0; v < 3; v++) o.g[v][ch] = inside(o.g[v][ch]);
      }
    };
    float dnA[C][6];
#pragma unroll
    for (int ch = 0; ch < C; ch++)
#pragma unroll
      for (int i = 0; i < 6; i++) dnA[ch][i] = 0.f;

    auto step = [&](int k, const Adj2ARow<C>& cur, const Adj2ARow<C>& nxt, const Adj2Late<C>& late, auto do_a) {
      const int h = g.hs - 2 + k;
      const bool in_img = g.col_ok && h >= 0 && h < H;
      const bool dmaskA = h >= 0 && h < H - 1;
      float (*slot)[64] = handA[G][k % kSlots];
      float gcv;
      Acc accA;
      if (G == 0) {
        gcv = late.gc_i;
        accA = Acc{late.gwx0_i, late.gwx1_i, late.gwy0_i, late.gwy1_i};
      } else {  // what the first group made of the row's accumulators, one interval ago
        const float (*prev)[64] = handA[0][k % kSlots];
        gcv = prev[7 * CM + 0][g.lane];
        accA = Acc{prev[7 * CM + 1][g.lane], prev[7 * CM + 2][g.lane], prev[7 * CM + 3][g.lane], prev[7 * CM + 4][g.lane]};
      }
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        AccTerms at;
        const T3 t = pixel(cur.yA[0][ch], cur.yA[1][ch], cur.yA[2][ch], nxt.yA[0][ch], nxt.yA[1][ch], nxt.yA[2][ch],
                           cur.g[0][ch], cur.g[1][ch], cur.g[2][ch], nxt.g[0][ch], nxt.g[1][ch], nxt.g[2][ch], cur.wxs,
                           cur.wys, cur.bxs, cur.bys, dmaskA, dnA[ch], at, kNo, do_a);
        float nG[3] = {0.f, 0.f, 0.f}, ngxm[3] = {0.f, 0.f, 0.f};
        float ngb = late.gb_i[ch];
        if (do_a.value) {
          apply_terms(accA, at);
          const Tail o = tail(t, late.gx_i[0][ch], late.gx_i[1][ch], late.gx_i[2][ch], optA, tA, cur.c, cur.bb[ch], cur.xa0[ch]);
          gcv += o.gc_add;
          ngb += o.gb_add;
          nG[0] = in_img ? o.g05v : 0.f;  // B reads zero padding outside the image
          nG[1] = in_img ? o.d1 : 0.f;
          nG[2] = in_img ? o.d2 : 0.f;
          ngxm[0] = o.gxm0; ngxm[1] = o.gxm1; ngxm[2] = o.gxm2;
        }
#pragma unroll
        for (int v = 0; v < 3; v++) {
          slot[v * CM + ch][g.lane] = nG[v];
          slot[3 * CM + v * CM + ch][g.lane] = ngxm[v];
        }
        slot[6 * CM + ch][g.lane] = ngb;
      }
      slot[7 * CM + 0][g.lane] = gcv;
      slot[7 * CM + 1][g.lane] = accA.gwx0;
      slot[7 * CM + 2][g.lane] = accA.gwx1;
      slot[7 * CM + 3][g.lane] = accA.gwy0;
      slot[7 * CM + 4][g.lane] = accA.gwy1;
    };
    // the barrier after row k with k % kP == kP - 1 ends the interval of rows k-kP+1 .. k
    auto publish = [&](int k) {
      if (k % kP == kP - 1) lds_barrier();
    };
    Adj2ARow<C> b0, b1, b2;
    Adj2Late<C> late;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    load_late(1, late);
    for (int t = 0; t < G; t++) lds_barrier();  // group 1 works one interval behind group 0
    absorb(0, b0);
    absorb(1, b1);
    step(0, b0, b1, late, kNo);
    load_row(3, b0);
    publish(0);
    absorb(2, b2);
    step(1, b1, b2, late, kYes);
    load_row(4, b1);
    load_late(2, late);
    publish(1);
    absorb(3, b0);
    step(2, b2, b0, late, kYes);
    load_row(5, b2);
    load_late(3, late);
    publish(2);
    for (int k = 3; k <= klast; k += 3) {  // cur / next rotate through (b0,b1) (b1,b2) (b2,b0)
      absorb(k + 1, b1);
      step(k, b0, b1, late, kYes);
      load_row(k + 3, b0);
      load_late(k + 1, late);
      publish(k);
      if (k + 1 > klast) break;
      absorb(k + 2, b2);
      step(k + 1, b1, b2, late, kYes);
      load_row(k + 4, b1);
      load_late(k + 2, late);
      publish(k + 1);
      if (k + 2 > klast) break;
      absorb(k + 3, b0);
      step(k + 2, b2, b0, late, kYes);
      load_row(k + 5, b2);
      load_late(k + 3, late);
      publish(k + 2);
    }
    if (klast % kP != kP - 1) lds_barrier();    // the last interval was a short one
    for (int t = G; t < 2; t++) lds_barrier();  // the intervals in which only the wavefronts behind still work
  };

  // ------------------------------------------ step B on one group ------------------------------------------
  auto role_b = [&](auto channels, auto group) {
    constexpr int C = decltype(channels)::value, G = decltype(group)::value;
    constexpr int chb = G ? CM : 0;
    const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const bx_p = bx + poff, *const by_p = by + poff,
                       *const cf_p = cf + poff;
    float *const gco_p = gc + poff, *const gwx0o_p = gwx + 2 * poff, *const gwx1o_p = gwx + 2 * poff + HW,
                 *const gwy0o_p = gwy + 2 * poff, *const gwy1o_p = gwy + 2 * poff + HW;
    const float *xb_p[3][C], *xc_p[C], *pv_p[2][C], *b_p[C];
    float *g05o_p[3][C], *gxm_p[3][C], *gbo_p[C], *gxf_p[3][C];
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const size_t qb = ((size_t)g.n * Ct + chb + ch) * HW;
      b_p[ch] = b + qb; gbo_p[ch] = gb + qb;
      xc_p[ch] = x05c + (size_t)g.n * 3 * CHW + (size_t)(chb + ch) * HW;  // u of x05[j-2] (BEND: u of the checkpoint y)
#pragma unroll
      for (int v = 0; v < 3; v++) {
        const size_t q = (size_t)g.n * 3 * CHW + (size_t)v * CHW + (size_t)(chb + ch) * HW;
        xb_p[v][ch] = ((BEND && v > 0 && !TRUE_ADJ) ? x05c : x05b) + q;  // B's aux y: x05[j-1], or the checkpoint when BEND
        if (v > 0) pv_p[v - 1][ch] = x05c + q;  // corrected gradient: the aux rows before B's
        g05o_p[v][ch] = g05_out + q; gxm_p[v][ch] = gxk_m1 + q; gxf_p[v][ch] = FINAL ? gx_final + q : nullptr;
      }
    }
    auto load_row = [&](int k, Adj2BRow<C>& in) {
      unsigned off, off_w;
      row_offsets(k, off, off_w);
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
      in.bxs = ldg(bx_p, off_w);
      in.bys = ldg(by_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xb0[ch] = ldg(x05b + (size_t)g.n * 3 * CHW + (size_t)(chb + ch) * HW, off);
        in.bb[ch] = ldg(b_p[ch], off);
        in.yB[1][ch] = ldg(xb_p[1][ch], off);
        in.yB[2][ch] = ldg(xb_p[2][ch], off);
        in.yB[0][ch] = ldg(xc_p[ch], off);
        if (TRUE_ADJ) {
          in.pv[0][ch] = ldg(pv_p[0][ch], off);
          in.pv[1][ch] = ldg(pv_p[1][ch], off);
        }
      }
    };
    auto absorb = [&](int k, Adj2BRow<C>& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      const float rc1 = rcp_refined(1.f + o.c);
      const double opc_d = 1. + (double)o.c;
      o.wxs = (ok && rmask) ? o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? o.wys : 0.f;
      o.bxs = inside(o.bxs);
      o.bys = inside(o.bys);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xb = inside(o.xb0[ch]), xc = inside(o.yB[0][ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pb = tvstrip::prox_huber1(xb, o.c, rc1, bv);
          const float pc = BEND ? xc : tvstrip::prox_huber1(xc, o.c, rc1, bv);
          o.yB[0][ch] = pb + tB * (pb - pc);
        } else {
          o.yB[0][ch] = BEND ? xc : tvstrip::rebuild_y_fast(bv, xb, xc, o.c, rc1, opc_d, tB);
        }
        o.xb0[ch] = xb;
        o.bb[ch] = bv;
#pragma unroll
        for (int v = 1; v < 3; v++) {
          const float xv = inside(o.yB[v][ch]);
          o.yB[v][ch] = TRUE_ADJ ? xv + tB * (xv - inside(o.pv[v - 1][ch])) : xv;
        }
      }
    };
    const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form
    float dnB[C][6];
    // row k-1 as step B sees it
    float pG[3][C], pgxm[3][C], pyB[3][C], pxb0[C], pbb[C], pgb[C], pgc = 0.f;
    Acc pacc{0.f, 0.f, 0.f, 0.f};
    float pc = 0.f, pwxs = 0.f, pwys = 0.f, pbxs = 0.f, pbys = 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      pxb0[ch] = pbb[ch] = pgb[ch] = 0.f;
#pragma unroll
      for (int i = 0; i < 6; i++) dnB[ch][i] = 0.f;
#pragma unroll
      for (int v = 0; v < 3; v++) pG[v][ch] = pgxm[v][ch] = pyB[v][ch] = 0.f;
    }

    auto step = [&](int k, const Adj2BRow<C>& cur, auto tri_b, auto do_b) {
      const int h = g.hs - 2 + k;  // the row step A handed over; B's row is h - 1
      const bool dmaskB = h - 1 >= 0 && h - 1 < H - 1;
      const unsigned roffB_ = (unsigned)max(h - 1, 0) * W4 + wc;
      const float (*slot)[64] = handA[G][k % kSlots];
      float (*tf)[64] = termF[k % kSlots];
      double (*td)[64] = termD[k % kSlots];
      float nG[3][C], ngxm[3][C], ngb[C];
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
#pragma unroll
        for (int v = 0; v < 3; v++) {
          nG[v][ch] = slot[v * CM + ch][g.lane];
          ngxm[v][ch] = slot[3 * CM + v * CM + ch][g.lane];
        }
        ngb[ch] = slot[6 * CM + ch][g.lane];
      }
      float gcv = 0.f;
      Acc accA{0.f, 0.f, 0.f, 0.f};
      if (G == 1) {  // the row's accumulators with every A term added
        gcv = slot[7 * CM + 0][g.lane];
        accA = Acc{slot[7 * CM + 1][g.lane], slot[7 * CM + 2][g.lane], slot[7 * CM + 3][g.lane], slot[7 * CM + 4][g.lane]};
      }
      if (tri_b.value) {
        float gcB = pgc;
        Acc accB = pacc;
        if (G == 1 && do_b.value) {  // the first group's B terms, in channel order, before this group's
#pragma unroll
          for (int ch = 0; ch < CM; ch++) {
            AccTerms at;
            at.add_wx0 = tf[5 * ch + 1][g.lane]; at.add_wy0 = tf[5 * ch + 2][g.lane];
            at.add_wx1 = tf[5 * ch + 3][g.lane]; at.add_wy1 = tf[5 * ch + 4][g.lane];
            at.sub_wx0 = td[4 * ch + 0][g.lane]; at.sub_wy0 = td[4 * ch + 1][g.lane];
            at.sub_wx1 = td[4 * ch + 2][g.lane]; at.sub_wy1 = td[4 * ch + 3][g.lane];
            apply_terms(accB, at);
            gcB += tf[5 * ch + 0][g.lane];
          }
        }
#pragma unroll
        for (int ch = 0; ch < C; ch++) {
          AccTerms at;
          const T3 t = pixel(pyB[0][ch], pyB[1][ch], pyB[2][ch], cur.yB[0][ch], cur.yB[1][ch], cur.yB[2][ch], pG[0][ch],
                             pG[1][ch], pG[2][ch], nG[0][ch], nG[1][ch], nG[2][ch], pwxs, pwys, pbxs, pbys, dmaskB,
                             dnB[ch], at, kBEnd, do_b);
          if (do_b.value) {
            const Tail o = tail(t, pgxm[0][ch], pgxm[1][ch], pgxm[2][ch], optB, tB, pc, pbb[ch], pxb0[ch]);
            if (G == 0) {
              tf[5 * ch + 0][g.lane] = o.gc_add;
              tf[5 * ch + 1][g.lane] = at.add_wx0; tf[5 * ch + 2][g.lane] = at.add_wy0;
              tf[5 * ch + 3][g.lane] = at.add_wx1; tf[5 * ch + 4][g.lane] = at.add_wy1;
              td[4 * ch + 0][g.lane] = at.sub_wx0; td[4 * ch + 1][g.lane] = at.sub_wy0;
              td[4 * ch + 2][g.lane] = at.sub_wx1; td[4 * ch + 3][g.lane] = at.sub_wy1;
            } else {
              apply_terms(accB, at);
              gcB += o.gc_add;
            }
            const float gbv = pgb[ch] + o.gb_add;
            if (store_lane) {
              const unsigned roffB = offset_here(roffB_);
              if (FINAL) {
                stg(gxf_p[0][ch], roffB, o.df);
                stg(gxf_p[1][ch], roffB, o.d1);
                stg(gxf_p[2][ch], roffB, o.d2);
              }
              stg(gxm_p[0][ch], roffB, o.gxm0);
              stg(gxm_p[1][ch], roffB, o.gxm1);
              stg(gxm_p[2][ch], roffB, o.gxm2);
              stg(g05o_p[0][ch], roffB, o.g05v);
              stg(g05o_p[1][ch], roffB, o.d1);
              stg(g05o_p[2][ch], roffB, o.d2);
              if (BEND) {  // segment flush, fused: fp32 segment sum into the segment's record; zero at the sweep's end (TGVH.cu:178-216)
                seg_gb[((size_t)g.n * Ct + chb + ch) * HW + (roffB >> 2)] = gbv;
                if (FINAL) stg(gbo_p[ch], roffB, 0.f);
              } else {
                stg(gbo_p[ch], roffB, gbv);
              }
            }
          }
        }
        if (G == 1 && do_b.value && store_lane) {
          const unsigned roffB = offset_here(roffB_);
          if (BEND) {
            const size_t e1 = poff + (roffB >> 2), e2 = 2 * poff + (roffB >> 2);
            seg_gc[e1] = gcB;
            seg_gwx[e2] = accB.gwx0;
            seg_gwx[e2 + HW] = accB.gwx1;
            seg_gwy[e2] = accB.gwy0;
            seg_gwy[e2 + HW] = accB.gwy1;
            if (FINAL) stg(gco_p, roffB, 0.f);
            if (FINAL) stg(gwx0o_p, roffB, 0.f);
            if (FINAL) stg(gwx1o_p, roffB, 0.f);
            if (FINAL) stg(gwy0o_p, roffB, 0.f);
            if (FINAL) stg(gwy1o_p, roffB, 0.f);
          } else {
            stg(gco_p, roffB, gcB);
            stg(gwx0o_p, roffB, accB.gwx0);
            stg(gwx1o_p, roffB, accB.gwx1);
            stg(gwy0o_p, roffB, accB.gwy0);
            stg(gwy1o_p, roffB, accB.gwy1);
          }
        }
      }
      pgc = gcv; pacc = accA;
      pc = cur.c; pwxs = cur.wxs; pwys = cur.wys; pbxs = cur.bxs; pbys = cur.bys;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        pgb[ch] = ngb[ch]; pxb0[ch] = cur.xb0[ch]; pbb[ch] = cur.bb[ch];
#pragma unroll
        for (int v = 0; v < 3; v++) { pG[v][ch] = nG[v][ch]; pgxm[v][ch] = ngxm[v][ch]; pyB[v][ch] = cur.yB[v][ch]; }
      }
    };

    // B waits before every row k with k % kP == 0 for the barrier that ended the interval in which rows k .. k+kP-1 were handed over
    auto await = [&](int k) {
      if (k % kP == 0) lds_barrier();
    };
    Adj2BRow<C> b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    for (int t = 0; t < G; t++) lds_barrier();  // group 1 works one interval behind group 0
    await(0);
    absorb(0, b0);
    step(0, b0, kNo, kNo);
    load_row(3, b0);
    await(1);
    absorb(1, b1);
    step(1, b1, kNo, kNo);
    load_row(4, b1);
    await(2);
    absorb(2, b2);
    step(2, b2, kYes, kNo);
    load_row(5, b2);
    for (int k = 3; k <= klast; k += 3) {
      await(k);
      absorb(k, b0);
      step(k, b0, kYes, kYes);
      load_row(k + 3, b0);
      if (k + 1 > klast) break;
      await(k + 1);
      absorb(k + 1, b1);
      step(k + 1, b1, kYes, kYes);
      load_row(k + 4, b1);
      if (k + 2 > klast) break;
      await(k + 2);
      absorb(k + 2, b2);
      step(k + 2, b2, kYes, kYes);
      load_row(k + 5, b2);
    }
    for (int t = G; t < 2; t++) lds_barrier();
  };

  const std::integral_constant<int, CM> kFirst{};
  const std::integral_constant<int, C1> kSecond{};
  const std::integral_constant<int, 0> kG0{};
  const std::integral_constant<int, 1> kG1{};
  if (wave == 0) role_a(kFirst, kG0);
  else if (wave == 1) role_a(kSecond, kG1);
  else if (wave == 2) role_b(kFirst, kG0);
  else role_b(kSecond, kG1);
}


}  // namespace tgvstrip
