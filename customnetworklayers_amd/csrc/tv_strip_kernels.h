// Wave-strip kernels of the TV layer: the fast path for image widths that are a multiple of 4.
//
// One wavefront owns a strip of kStripCols output columns x R rows of one sample and runs without
// LDS and without barriers.  Each lane holds 4 consecutive pixels of a row (float4 loads and
// stores); lane 0 is an apron lane that covers the 4 columns left of the strip and only supplies
// its triangle terms to lane 1.  Rows are walked top to bottom, starting one row above the strip.
//
// The reference evaluates, per pixel, the Huber weights of the three triangles the pixel belongs
// to.  The triangle owned by pixel q enters q, q's right neighbour and q's lower neighbour with
// bit-identical operands (the two squared differences are symmetric under negation and their sum
// commutes), so here the owner computes the weight once and passes it on: down the column in
// registers, to the right through one cross-lane move per row.  Results are bit-identical to the
// per-pixel evaluation; the work per pixel drops from 3 sqrt + 8 div to 1 sqrt + 3 div.
#pragma once

#include "exact_math.h"

namespace tvstrip {

using inpaint::div_by;
using inpaint::exact_sqrt;
using inpaint::rcp_refined;

constexpr int kLanePx = 4;
constexpr int kStripCols = 63 * kLanePx;  // 252 output columns per wavefront (lane 0 is the apron)
constexpr float kDelta = 0.1f;            // TV.cu:44
constexpr float kL = 0.125f;              // TV.cu:1478

struct F4 {
  float v[4];
};

__device__ __forceinline__ F4 load4(const float* __restrict__ p, bool ok) {
  F4 r;
  if (ok) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
  } else {
    r.v[0] = r.v[1] = r.v[2] = r.v[3] = 0.f;
  }
  return r;
}
__device__ __forceinline__ void store4(float* __restrict__ p, const F4& a) {
  *reinterpret_cast<float4*>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
}

// value held by the lane to the left (lane 0 gets its own back; it is the apron and never uses it)
__device__ __forceinline__ float from_left_lane(float v, int bperm_addr) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(bperm_addr, __float_as_int(v)));
}

struct StripGeom {
  int lane, w_first, hs, n;
  bool col_ok, store_lane;
  int bperm_left;
};

__device__ __forceinline__ bool strip_geometry(StripGeom& g, int R, int W, int strips_x, int strips_y, int N) {
  const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  g.lane = threadIdx.x & 63;
  const int sx = wave % strips_x;
  const int rest = wave / strips_x;
  const int sy = rest % strips_y;
  g.n = rest / strips_y;
  if (g.n >= N) return false;
  g.w_first = sx * kStripCols - kLanePx + kLanePx * g.lane;
  g.hs = sy * R;
  g.col_ok = g.w_first >= 0 && g.w_first < W;
  g.store_lane = g.lane > 0 && g.col_ok;
  g.bperm_left = ((g.lane + 63) & 63) << 2;
  return true;
}

// Forward iteration, TV.cu:1194-1319 (and 1321-1455 when x05 is given).
template <int R>
__global__ __launch_bounds__(256) void tv_forward_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* xin, float* xout, const float* __restrict__ yin,
    float* __restrict__ yout, float* __restrict__ x05, int N, int C, int H, int W, float t, int strips_x,
    int strips_y) {
  StripGeom g;
  if (!strip_geometry(g, R, W, strips_x, strips_y, N)) return;
  const size_t HW = (size_t)H * W;
  const float* wxp = wx + (size_t)g.n * HW;
  const float* wyp = wy + (size_t)g.n * HW;
  const float* cfp = cf + (size_t)g.n * HW;
  const int w0 = g.w_first;
  const bool left_ok = w0 - 1 >= 0 && w0 - 1 < W;
  const bool right_ok = w0 + kLanePx >= 0 && w0 + kLanePx < W;

  // masked, L-scaled weights of rows hs-1 .. hs+R-1, confidence of rows hs .. hs+R-1
  F4 wxs[R + 1], wys[R + 1], conf[R];
  float rc1[R][4];  // refined reciprocal of 1 + c
#pragma unroll
  for (int r = 0; r <= R; r++) {
    const int h = g.hs - 1 + r;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const size_t off = (size_t)(ok ? h : 0) * W + (ok ? w0 : 0);
    wxs[r] = load4(wxp + off, ok);
    wys[r] = load4(wyp + off, ok && h < H - 1);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      wxs[r].v[j] = (w0 + j < W - 1) ? kL * wxs[r].v[j] : 0.f;
      wys[r].v[j] = kL * wys[r].v[j];
    }
    if (r > 0) {
      conf[r - 1] = load4(cfp + off, ok);
#pragma unroll
      for (int j = 0; j < 4; j++) rc1[r - 1][j] = rcp_refined(1.f + conf[r - 1].v[j]);
    }
  }

  for (int ch = 0; ch < C; ch++) {
    const size_t coff = ((size_t)g.n * C + ch) * HW;
    const float* yp = yin + coff;
    // y rows hs-1 .. hs+R: own float4 plus the scalars left and right of it
    F4 y[R + 2];
    float yl[R + 2], yr[R + 2];
#pragma unroll
    for (int r = 0; r < R + 2; r++) {
      const int h = g.hs - 1 + r;
      const bool rok = h >= 0 && h < H;
      const size_t row = (size_t)(rok ? h : 0) * W;
      y[r] = load4(yp + row + (g.col_ok ? w0 : 0), rok && g.col_ok);
      yl[r] = (rok && left_ok) ? yp[row + w0 - 1] : 0.f;
      yr[r] = (rok && right_ok) ? yp[row + w0 + kLanePx] : 0.f;
    }
    F4 xo[R], bb[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const int h = g.hs + r;
      const bool ok = g.col_ok && h < H;
      const size_t off = coff + (size_t)(ok ? h : 0) * W + (ok ? w0 : 0);
      xo[r] = load4(xin + off, ok);
      bb[r] = load4(b + off, ok);
    }
    F4 qy_up;  // quotients wy/m of the row above
#pragma unroll
    for (int r = 0; r <= R; r++) {  // r indexes rows hs-1+r
      // own triangles of this row (TV.cu:1268-1274): norm, Huber divisor, the two quotients
      F4 qx, qy, d1, d2;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float yc = y[r].v[j];
        const float ydn = y[r + 1].v[j];
        const float yrt = (j < 3) ? y[r].v[j + 1] : yr[r];
        d1.v[j] = yc - ydn;
        d2.v[j] = yc - yrt;
        const float hub = exact_sqrt(d1.v[j] * d1.v[j] * wys[r].v[j] + d2.v[j] * d2.v[j] * wxs[r].v[j]);
        const float m = fmaxf(1.f, inpaint::exact_div(hub, kDelta));
        const float rm = rcp_refined(m);
        qy.v[j] = div_by(wys[r].v[j], m, rm);
        qx.v[j] = div_by(wxs[r].v[j], m, rm);
      }
      if (r > 0) {
        const int h = g.hs - 1 + r;
        const float qx_left = from_left_lane(qx.v[3], g.bperm_left);
        F4 xn, yn, xh;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float yc = y[r].v[j];
          const float yu = y[r - 1].v[j];
          const float ylf = (j > 0) ? y[r].v[j - 1] : yl[r];
          const float ql = (j > 0) ? qx.v[j - 1] : qx_left;
          float yt = yc;
          yt -= (yc - yu) * qy_up.v[j];   // TV.cu:1258
          yt -= (yc - ylf) * ql;          // TV.cu:1265
          yt -= d1.v[j] * qy.v[j];        // TV.cu:1272
          yt -= d2.v[j] * qx.v[j];        // TV.cu:1273
          xh.v[j] = yt;
          const float c = conf[r - 1].v[j], bv = bb[r - 1].v[j];
          float x_loc = div_by(c * bv + yt, 1.f + c, rc1[r - 1][j]);  // TV.cu:1288
          const float lo = yt - c, hi = yt + c;
          if (lo > 1.f + bv) x_loc = lo;
          if (hi < bv - 1.f) x_loc = hi;
          xn.v[j] = x_loc;
          yn.v[j] = x_loc + t * (x_loc - xo[r - 1].v[j]);  // TV.cu:1315
        }
        if (g.store_lane && h < H) {
          const size_t off = coff + (size_t)h * W + w0;
          store4(yout + off, yn);
          store4(xout + off, xn);
          if (x05) store4(x05 + off, xh);
        }
      }
      qy_up = qy;
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Adjoint iteration with the y rebuild fused in: TV.cu:586-859 (+1130-1189); END = the
// segment-start variant TV.cu:862-1126 that reads y from the checkpoint.
//
// Rows are streamed: the wavefront walks down its strip one row at a time, all channels per row,
// and prefetches the next row while it works on the current one.  Per triangle (owner q) the
// kernel forms, once, every term that the reference evaluates at q, at the pixel below q and at
// the pixel right of q:
//     O1..O4   the four own-triangle terms subtracted at q                     (TV.cu:732-743)
//     -O1, P1*tu, P2*tu   the three terms subtracted at the pixel below        (TV.cu:668-677)
//     -O2, P2*tl, P1*tl   the three terms subtracted at the pixel to the right (TV.cu:701-710)
// with P1 = (g_q-g_d) wy (y_q-y_d), P2 = (g_q-g_r) wx (y_q-y_r).  The operand order inside every
// product is the reference's (negating both factors of a product is exact), the order of the
// subtractions at each pixel is the reference's, and an inactive triangle is the active formula
// with nom = 1, denom = 0, which reproduces the inactive branch exactly.
// -------------------------------------------------------------------------------------------------
constexpr float kClipLocalGrad = 10000.0f;  // TV.cu:52
constexpr float kLocalGCMult = 0.1f;        // TV.cu:63
constexpr float kLocalGXMult = 0.1f;        // TV.cu:65

__device__ __forceinline__ float from_right_lane(float v, int bperm_addr) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(bperm_addr, __float_as_int(v)));
}

// y_{k+1} from x05[k] (xa) and x05[k-1] (xb), TV.cu:1149-1165; rc = rcp_refined(1 + conf)
__device__ __forceinline__ float rebuild_y_fast(float bb, float xa, float xb, float conf, float rc, float t) {
  float diff = bb - xa;
  float sign = (diff < 0) ? -1.f : 1.f;
  const bool quad = (1. + (double)conf >= (double)(sign * diff));
  const float cb = conf * bb;
  const float xk_q = div_by(cb + xa, 1.f + conf, rc);
  const float xkm_q = div_by(cb + xb, 1.f + conf, rc);
  const float y_q = xk_q + t * (xk_q - xkm_q);
  const float xk_l = (conf <= sign * diff) ? bb - diff + sign * conf : bb;
  diff = bb - xb;
  sign = (diff < 0) ? -1.f : 1.f;
  const float y_l = xk_l + t * (xk_l - ((conf <= sign * diff) ? bb - diff + sign * conf : bb));
  return quad ? y_q : y_l;
}

template <int C, bool END>
__global__ __launch_bounds__(256) void tv_adjoint_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ yck, float* __restrict__ gc, float* __restrict__ gb, float* __restrict__ gwx,
    float* __restrict__ gwy, const float* __restrict__ g05_in, float* __restrict__ g05_out,
    float* __restrict__ gxk, float* __restrict__ gxk_m1, int N, int H, int W, float t, int R, int strips_x,
    int strips_y) {
  StripGeom g;
  if (!strip_geometry(g, R, W, strips_x, strips_y, N)) return;
  const size_t HW = (size_t)H * W;
  const size_t poff = (size_t)g.n * HW;
  const int w0 = g.w_first;
  const bool last_lane = g.lane == 63;
  const bool right_ok = w0 + kLanePx < W;
  const int bperm_right = ((g.lane + 1) & 63) << 2;
  const double opt = 1. + (double)t;

  // raw loads of one row: everything the rebuild and the pixel update of that row need
  struct RowIn {
    F4 c, xa[C], xb[C], bb[C], gg[C];
  };
  auto load_row = [&](int h, RowIn& in) {
    const bool ok = g.col_ok && h >= 0 && h < H;
    const size_t off = (size_t)(ok ? h : 0) * W + (ok ? w0 : 0);
    in.c = load4(cf + poff + off, ok);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const size_t q = ((size_t)g.n * C + ch) * HW + off;
      if (END) {
        in.xa[ch] = load4(x05a + q, ok);
        in.xb[ch] = load4(yck + q, ok);  // the checkpoint y travels in the xb slot
      } else {
        in.xa[ch] = load4(x05a + q, ok);
        in.xb[ch] = load4(x05b + q, ok);
      }
      in.bb[ch] = load4(b + q, ok);
      in.gg[ch] = load4(g05_in + q, ok);
    }
  };
  // right neighbour of the last lane's fourth pixel: one scalar column, rebuilt the same way
  auto right_scalar = [&](int h, int ch, float& yv, float& gv) {
    yv = 0.f;
    gv = 0.f;
    if (h >= 0 && h < H && right_ok) {
      const size_t p = (size_t)h * W + w0 + kLanePx;
      const size_t q = ((size_t)g.n * C + ch) * HW + p;
      gv = g05_in[q];
      if (END) {
        yv = yck[q];
      } else {
        const float cv = cf[poff + p];
        yv = rebuild_y_fast(b[q], x05a[q], x05b[q], cv, rcp_refined(1.f + cv), t);
      }
    }
  };

  // state of the current row
  F4 c_cur, rc1_cur, y_cur[C], g_cur[C], xa_cur[C], b_cur[C];
  F4 dn1[C], dn3[C], dn4[C];  // terms handed down to the row below
  RowIn nxt;
  auto absorb = [&](const RowIn& in, F4& c_o, F4& rc1_o, F4* y_o, F4* g_o, F4* xa_o, F4* b_o) {
    c_o = in.c;
#pragma unroll
    for (int j = 0; j < 4; j++) rc1_o.v[j] = rcp_refined(1.f + in.c.v[j]);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
#pragma unroll
      for (int j = 0; j < 4; j++)
        y_o[ch].v[j] = END ? in.xb[ch].v[j]
                           : rebuild_y_fast(in.bb[ch].v[j], in.xa[ch].v[j], in.xb[ch].v[j], in.c.v[j], rc1_o.v[j], t);
      g_o[ch] = in.gg[ch];
      xa_o[ch] = in.xa[ch];
      b_o[ch] = in.bb[ch];
    }
  };

  {
    RowIn first;
    load_row(g.hs - 1, first);
    load_row(g.hs, nxt);
    absorb(first, c_cur, rc1_cur, y_cur, g_cur, xa_cur, b_cur);
  }
#pragma unroll
  for (int ch = 0; ch < C; ch++)
#pragma unroll
    for (int j = 0; j < 4; j++) dn1[ch].v[j] = dn3[ch].v[j] = dn4[ch].v[j] = 0.f;

  for (int r = 0; r <= R; r++) {
    const int h = g.hs - 1 + r;  // owner row of this step
    // next row: turn the prefetched loads into y / g, then prefetch the row after it
    F4 c_n, rc1_n, y_n[C], g_n[C], xa_n[C], b_n[C];
    absorb(nxt, c_n, rc1_n, y_n, g_n, xa_n, b_n);
    if (r < R) load_row(h + 2, nxt);

    // masked, L-scaled weights of the owner row
    const bool rok = g.col_ok && h >= 0 && h < H;
    const size_t roff = (size_t)(rok ? h : 0) * W + (rok ? w0 : 0);
    F4 wxs = load4(wx + poff + roff, rok);
    F4 wys = load4(wy + poff + roff, rok && h < H - 1);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      wxs.v[j] = (w0 + j < W - 1) ? kL * wxs.v[j] : 0.f;
      wys.v[j] = kL * wys.v[j];
    }
    const bool px_row = r > 0 && h < H;  // rows of this strip that produce output
    const bool do_store = px_row && g.store_lane;
    F4 gcv, gwxv, gwyv, rc2;
    if (r > 0) {
      gcv = load4(gc + poff + roff, do_store);
      gwxv = load4(gwx + poff + roff, do_store);
      gwyv = load4(gwy + poff + roff, do_store);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float d = (1.f + c_cur.v[j]) * (1.f + c_cur.v[j]);
        rc2.v[j] = rcp_refined(d);
      }
    }
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const size_t q = ((size_t)g.n * C + ch) * HW + roff;
      float yr = from_right_lane(y_cur[ch].v[0], bperm_right);
      float gr = from_right_lane(g_cur[ch].v[0], bperm_right);
      if (last_lane) right_scalar(h, ch, yr, gr);
      F4 gxv, gbv;
      if (r > 0) {
        gxv = load4(gxk + q, do_store);
        gbv = load4(gb + q, do_store);
      }
      F4 O1, O2, O3, O4, r3, r4, n3, n4;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float yk = y_cur[ch].v[j], yd = y_n[ch].v[j], yrt = (j < 3) ? y_cur[ch].v[j + 1] : yr;
        const float gk = g_cur[ch].v[j], gd = g_n[ch].v[j], grt = (j < 3) ? g_cur[ch].v[j + 1] : gr;
        const float wxv = wxs.v[j], wyv = wys.v[j];
        const float d1 = yk - yd, d2 = yk - yrt;
        const float a1 = d1 * d1 * wyv;  // wy_nyy2
        const float a2 = d2 * d2 * wxv;  // wx_nyx2
        const float hub = exact_sqrt(a2 + a1);
        const bool act = hub > kDelta;
        float nom = inpaint::exact_div(kDelta, hub);
        float denom = inpaint::exact_div(nom, 2.f * hub * hub);
        nom = act ? nom : 1.f;
        denom = act ? denom : 0.f;
        const float gpd = gk - gd, gpr = gk - grt;
        O1.v[j] = gpd * (wyv * nom);
        O2.v[j] = gpr * (wxv * nom);
        const float P1 = gpd * wyv * d1;
        const float P2 = gpr * wxv * d2;
        const float dd = denom * 2.0f;
        const float tp = dd * ((yd - yk) * wyv + (yrt - yk) * wxv);
        const float tu = dd * d1 * wyv;
        const float tl = dd * d2 * wxv;
        O3.v[j] = P1 * tp;
        O4.v[j] = P2 * tp;
        n3.v[j] = P1 * tu;
        n4.v[j] = P2 * tu;
        r3.v[j] = P2 * tl;
        r4.v[j] = P1 * tl;
        if (r > 0) {  // weight gradients of the pixel's own triangle, TV.cu:749-769 / 1019-1037
          float ux, uy;
          if (!END) {
            ux = kLocalGXMult * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
            uy = kLocalGXMult * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
          } else {
            const float ux_a = kLocalGXMult * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
            const float uy_a = kLocalGXMult * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
            ux = act ? ux_a : kLocalGXMult * d2 * gpr;
            uy = act ? uy_a : kLocalGXMult * d1 * gpd;
          }
          if (w0 + j < W - 1) gwxv.v[j] = gwxv.v[j] - ux;
          if (h < H - 1) gwyv.v[j] = gwyv.v[j] - uy;
        }
      }
      // terms arriving from the triangle of the pixel to the left
      const float l1 = from_left_lane(O2.v[3], g.bperm_left);
      const float l3 = from_left_lane(r3.v[3], g.bperm_left);
      const float l4 = from_left_lane(r4.v[3], g.bperm_left);
      if (r > 0) {
        F4 g05v, gxm;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float tt = g_cur[ch].v[j];
          tt -= -dn1[ch].v[j];                       // TV.cu:668 / 684
          tt -= dn3[ch].v[j];                        // TV.cu:675
          tt -= dn4[ch].v[j];                        // TV.cu:677
          tt -= -((j > 0) ? O2.v[j - 1] : l1);       // TV.cu:701 / 718
          tt -= (j > 0) ? r3.v[j - 1] : l3;          // TV.cu:707
          tt -= (j > 0) ? r4.v[j - 1] : l4;          // TV.cu:710
          tt -= O1.v[j];                             // TV.cu:732 / 763
          tt -= O2.v[j];                             // TV.cu:733 / 764
          tt -= O3.v[j];                             // TV.cu:741
          tt -= O4.v[j];                             // TV.cu:743
          // momentum adjoint, TV.cu:796-801
          float df = (float)((double)gxv.v[j] + opt * (double)tt);
          df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
          gxv.v[j] = df;
          gxm.v[j] = -t * tt;
          // prox adjoint, TV.cu:806-828
          const float conf = c_cur.v[j], bv = b_cur[ch].v[j], xh = xa_cur[ch].v[j];
          const float diff = bv - xh;
          const float sign = (diff < 0) ? -1.f : 1.f;
          const bool quad = (1. + (double)conf >= (double)(sign * diff));
          const float opc = 1.f + conf;
          const float gc_q = df * (div_by(bv, opc, rc1_cur.v[j]) - div_by(conf * bv + xh, opc * opc, rc2.v[j])) * kLocalGCMult;
          const float g05_q = div_by(df, opc, rc1_cur.v[j]);
          const float gb_q = div_by(df * conf, opc, rc1_cur.v[j]) * 1.0f;
          if (quad) {
            gcv.v[j] += gc_q;
            g05v.v[j] = g05_q;
            gbv.v[j] += gb_q;
          } else if (conf >= sign * diff) {  // TV.cu:818-822
            g05v.v[j] = 0.f;
            gbv.v[j] += df * 1.0f;
          } else {
            g05v.v[j] = df;
            gcv.v[j] += sign * df * kLocalGCMult;
          }
        }
        if (do_store) {
          store4(gxk + q, gxv);
          store4(gxk_m1 + q, gxm);
          store4(g05_out + q, g05v);
          store4(gb + q, gbv);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        dn1[ch].v[j] = O1.v[j];
        dn3[ch].v[j] = n3.v[j];
        dn4[ch].v[j] = n4.v[j];
      }
    }
    if (do_store) {
      store4(gc + poff + roff, gcv);
      store4(gwx + poff + roff, gwxv);
      store4(gwy + poff + roff, gwyv);
    }
    c_cur = c_n;
    rc1_cur = rc1_n;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      y_cur[ch] = y_n[ch];
      g_cur[ch] = g_n[ch];
      xa_cur[ch] = xa_n[ch];
      b_cur[ch] = b_n[ch];
    }
  }
}

}  // namespace tvstrip
