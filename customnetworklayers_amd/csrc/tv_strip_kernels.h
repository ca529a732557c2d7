// Wave-strip kernels of the TV layer (the default path for up to 4 channels).
//
// One wavefront owns a strip of one sample: 64 adjacent columns (one pixel per lane) by R rows, and
// walks it top to bottom without LDS and without barriers.  Lane 0 is an apron lane: it covers the
// column left of the strip and only feeds its triangle terms to lane 1 (the adjoint kernel also
// uses lane 63 as an apron on the right, because there a pixel's right neighbour is a rebuilt
// value and not a plain load).  Neighbouring lanes exchange values with wave-wide DPP shifts.
//
// Row streaming: row k (k = 0 is the row above the strip) is needed as the "next" row of step k-1
// and as the "current" row of step k.  Four row buffers rotate, so while step k computes, the loads
// of rows k+2 and k+3 are in flight; the loop body is four steps with the roles rotated, so no
// registers are copied.  A row buffer is 4C+4 registers, which keeps the kernels at several
// wavefronts per SIMD: the layer's images are small for this chip (about 7 rows of work per
// lane at 1 pixel per lane), so occupancy, not per-lane reuse, is what hides memory latency.
//
// Triangle sharing: the reference evaluates, per pixel, the Huber weights of the three triangles
// the pixel belongs to.  The triangle owned by pixel q enters q, q's right neighbour and q's lower
// neighbour with bit-identical operands (squared differences are symmetric under negation, their
// sum commutes), so the owner computes each term once and hands it on: down the column in
// registers, to the right through a DPP shift.  Results are bit-identical to the per-pixel
// evaluation; per pixel the work drops from 3 sqrt + 8 div to 1 sqrt + 3 div (forward).
#pragma once

#include <type_traits>

#include "exact_math.h"

namespace tvstrip {

using inpaint::div_by;
using inpaint::exact_sqrt;
using inpaint::rcp_refined;

constexpr int kFwdCols = 63;      // output columns per wavefront, forward (lane 0 is the apron)
constexpr int kAdjCols = 62;      // adjoint (lanes 0 and 63 are aprons)
constexpr int kFwd2Cols = 60;     // two fused forward iterations (lanes 0, 1, 62, 63 are aprons)
constexpr float kDelta = 0.1f;    // TV.cu:44
static_assert(kDelta == 0.1f, "the forward pass divides by the threshold with div_by_tenth");
constexpr float kL = 0.125f;      // TV.cu:1478
constexpr float kClipLocalGrad = 10000.0f;  // TV.cu:52
constexpr float kLocalGCMult = 0.1f;        // TV.cu:63
constexpr float kLocalGXMult = 0.1f;        // TV.cu:65

// value of the lane to the left / right; lanes without a source receive 0
__device__ __forceinline__ float from_left_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x138, 0xf, 0xf, false));  // wave_shr:1
}
__device__ __forceinline__ float from_right_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x130, 0xf, 0xf, false));  // wave_shl:1
}

// element `off_bytes / 4` of a wave-uniform plane: the byte offset is a 32-bit VGPR that is zero-extended
// and added to the SGPR base by the load / store itself
__device__ __forceinline__ float ldg(const float* base, unsigned off_bytes) {
  return *reinterpret_cast<const float*>(reinterpret_cast<const char*>(base) + off_bytes);
}
__device__ __forceinline__ void stg(float* base, unsigned off_bytes, float v) {
  *reinterpret_cast<float*>(reinterpret_cast<char*>(base) + off_bytes) = v;
}
// The same with the non-temporal hint, for data that is written once and not touched again for a long time (half of a
// checkpoint of the TGV layer, which only the backward pass reads): it leaves the caches to what the next launch reads
// again -- the iterate, the weights.  (Measured, config 2: forward pass 3.08 -> 3.00 ms.  The same hint on the TV layer's
// checkpoints costs 0.8%, and non-temporal LOADS of the rows a reverse sweep reads for the last time cost the TGV
// backward pass 2.7%: neighbouring strips share those lines.)
__device__ __forceinline__ void stg_nt(float* base, unsigned off_bytes, float v) {
  __builtin_nontemporal_store(v, reinterpret_cast<float*>(reinterpret_cast<char*>(base) + off_bytes));
}

struct StripGeom {
  int lane, w, hs, n;  // w: this lane's column, hs: first output row, n: sample (hs, n wave-uniform)
  bool col_ok;
};

// (The fp32 record of a segment's sums is written once and read once, after the last segment, by combine_segments_many:
// it is stored with the non-temporal hint, which keeps it out of the way of the fields the next launches reuse --
// -1.3% on the TV step; the same hint on the TGV layer's records measured +0.4% and is not used there.)
//
// The row loop is kept a straight line: loads are unconditional (clamped addresses) and stores sit in
// blocks small enough to be predicated rather than branched around.  A load or store behind a
// branch makes the compiler assume the path without it and drain the prefetched rows at every step.

__device__ __forceinline__ bool strip_geometry(StripGeom& g, int cols, int R, int W, int strips_x, int strips_y,
                                               int N, int left_apron = 1) {
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Neighbouring strips share
  // halo rows, the apron column and split cache lines, so strips are numbered such that every XCD
  // works through one contiguous band of the image: workgroup b serves logical block
  // (b % 8) * (gridDim.x / 8) + b / 8 (the grid is a multiple of 8 workgroups).
  const int per_xcd = gridDim.x >> 3;
  const int logical_block = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int wave = __builtin_amdgcn_readfirstlane(logical_block * (blockDim.x >> 6) + (threadIdx.x >> 6));
  g.lane = threadIdx.x & 63;
  const int sx = wave % strips_x;
  const int rest = wave / strips_x;
  const int sy = rest % strips_y;
  g.n = rest / strips_y;
  if (g.n >= N) return false;
  g.w = sx * cols - left_apron + g.lane;
  g.hs = sy * R;
  g.col_ok = g.w >= 0 && g.w < W;
  return true;
}

// The same numbering with ONE strip per workgroup (all wavefronts of the workgroup work on that strip).
__device__ __forceinline__ bool strip_geometry_block(StripGeom& g, int cols, int R, int W, int strips_x, int strips_y,
                                                     int N, int left_apron) {
  const int per_xcd = gridDim.x >> 3;
  const int strip = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  g.lane = threadIdx.x & 63;
  const int sx = strip % strips_x;
  const int rest = strip / strips_x;
  const int sy = rest % strips_y;
  g.n = rest / strips_y;
  if (g.n >= N) return false;
  g.w = sx * cols - left_apron + g.lane;
  g.hs = sy * R;
  g.col_ok = g.w >= 0 && g.w < W;
  return true;
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight (a full
// __syncthreads() drains the one counter this GPU keeps for loads and stores alike).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// -------------------------------------------------------------------------------------------------
// Forward iteration, TV.cu:1194-1319 (and 1321-1455 when x05 is given).
//
// Channel groups: a launch serves C consecutive channels of a tensor with Ct channels per sample; the caller passes
// the per-channel pointers already moved to the group's first channel.  (Forward channels never couple; the adjoint
// couples them through the per-pixel accumulators gc, gwx, gwy only, summed in channel order, so groups launched in
// channel order reproduce the sum of one launch over all channels.  flush_shared: only the last group of a
// segment-start step stores the segment record of those three and zeroes them.)
//
// Per triangle (owner q) the two products
//     E1 = (y_q - y_down) * (wy / m),   E2 = (y_q - y_right) * (wx / m),   m = max(1, |.|_q / delta)
// are formed once; q subtracts both, the pixel below q subtracts -E1 and the pixel right of q
// subtracts -E2, which are the reference's four updates with identical operands
// ((y_p - y_up) * q = -(y_up - y_p) * q exactly).
// -------------------------------------------------------------------------------------------------
template <int C>
struct FwdRow {
  float y[C], yr[C], x[C], bb[C], c, rc1, wxs, wys;
};

template <int C, bool X05>
__global__ __launch_bounds__(256) void tv_forward_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ xin, float* __restrict__ xout,
    const float* __restrict__ yin, float* __restrict__ yout, float* __restrict__ x05,
    int N, int H, int W, float t, int R, int strips_x, int strips_y, int Ct) {
  StripGeom g;
  if (!strip_geometry(g, kFwdCols, R, W, strips_x, strips_y, N)) return;
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;           // row pitch in bytes
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;   // clamped column (bytes): every address below is valid
  const bool right_ok = g.w + 1 < W;
  const unsigned wr = right_ok ? 4u * (g.w + 1) : 0u;
  const bool store_lane = g.lane > 0 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const int Reff = min(R, H - g.hs);  // output rows of this strip (the last strip may be ragged)
  // wave-uniform plane pointers + 32-bit element offsets: loads and stores take an SGPR base and a
  // VGPR offset, so no 64-bit address arithmetic is done per access
  const float* const wx_p = wx + (size_t)g.n * HW;
  const float* const wy_p = wy + (size_t)g.n * HW;
  const float* const cf_p = cf + (size_t)g.n * HW;
  const float *y_p[C], *x_p[C], *b_p[C];
  float *yo_p[C], *xo_p[C], *xh_p[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t q = ((size_t)g.n * Ct + ch) * HW;
    y_p[ch] = yin + q; x_p[ch] = xin + q; b_p[ch] = b + q;
    yo_p[ch] = yout + q; xo_p[ch] = xout + q; xh_p[ch] = X05 ? x05 + q : nullptr;
  }

  auto load_row = [&](int k, FwdRow<C>& in) {  // row k of the strip = image row hs - 1 + k
    const int kk = min(k, Reff + 1);  // rows past the last needed one re-read it
    const int h = g.hs - 1 + kk;
    const unsigned row = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4;
    // the rows above and below the strip only contribute y (and, above, the weights); their other
    // fields are read from the strip's own first / last row instead, which is in L1 anyway, so
    // that no cache line is fetched for a value that is never used
    const int hw = g.hs - 1 + min(kk, Reff);
    const unsigned row_w = (unsigned)(hw < 0 ? 0 : hw) * W4;
    const unsigned row_p = (unsigned)(g.hs - 1 + max(1, min(kk, Reff))) * W4;
    in.c = ldg(cf_p, row_p + wc);
    in.wxs = ldg(wx_p, row_w + wc);
    in.wys = ldg(wy_p, row_w + wc);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.y[ch] = ldg(y_p[ch], row + wc);
      in.yr[ch] = ldg(y_p[ch], row_w + wr);
      in.x[ch] = ldg(x_p[ch], row_p + wc);
      in.bb[ch] = ldg(b_p[ch], row_p + wc);
    }
  };
  // mask what lies outside the image, scale the weights, refine 1/(1+c): in place
  auto absorb = [&](int k, FwdRow<C>& o) {
    const int h = g.hs - 1 + k;
    const bool rok = h >= 0 && h < H;
    o.rc1 = rcp_refined(1.f + o.c);
    o.wxs = (rok && wx_ok) ? kL * o.wxs : 0.f;
    o.wys = (rok && g.col_ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      o.y[ch] = (rok && g.col_ok) ? o.y[ch] : 0.f;
      o.yr[ch] = (rok && right_ok) ? o.yr[ch] : 0.f;
    }
  };

  float e1_up[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) e1_up[ch] = 0.f;

  // one row step; `first` = the row above the strip, which only supplies its triangle terms
  auto compute = [&](int r, const FwdRow<C>& cur, const FwdRow<C>& nxt, auto first) {
    const int h = g.hs - 1 + r;
    const unsigned roff = (unsigned)(h >= 0 ? h : 0) * W4 + wc;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      // own triangle, TV.cu:1268-1274
      const float yc = cur.y[ch];
      const float d1 = yc - nxt.y[ch];
      const float d2 = yc - cur.yr[ch];
      const float hub = exact_sqrt(d1 * d1 * cur.wys + d2 * d2 * cur.wxs);
      const float m = fmaxf(1.f, inpaint::div_by_tenth(hub));
      const float rm = rcp_refined(m);
      const float e1 = d1 * div_by(cur.wys, m, rm);
      const float e2 = d2 * div_by(cur.wxs, m, rm);
      const float e1_above = e1_up[ch];
      e1_up[ch] = e1;
      if (first.value) continue;
      const float e2_left = from_left_lane(e2);
      float yt = yc;
      yt -= -e1_above;   // TV.cu:1258
      yt -= -e2_left;    // TV.cu:1265
      yt -= e1;          // TV.cu:1272
      yt -= e2;          // TV.cu:1273
      const float xh = yt;
      const float c = cur.c, bv = cur.bb[ch];
      float x_loc = div_by(c * bv + yt, 1.f + c, cur.rc1);  // TV.cu:1288
      const float lo = yt - c, hi = yt + c;
      if (lo > 1.f + bv) x_loc = lo;
      if (hi < bv - 1.f) x_loc = hi;
      const float yn = x_loc + t * (x_loc - cur.x[ch]);  // TV.cu:1315
      if (store_lane) {  // a block this small is predicated, not branched around
        stg(yo_p[ch], roff, yn);
        stg(xo_p[ch], roff, x_loc);
        if (X05) stg(xh_p[ch], roff, xh);
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
// Two forward iterations per launch (A = iteration k, B = iteration k+1), same arithmetic as
// tv_forward_strip applied twice.  B runs one row behind A inside the same wavefront: once A has
// updated row r+1, B owns everything its triangle of row r needs (A's new y of rows r and r+1, in
// registers) and, with the term handed down from row r-1, the update of row r.  A's new iterate
// never touches memory, so a pair moves the bytes of one iteration (plus the two x05 rows when the
// backward pass recomputes a segment).
//
// Lanes cover columns w0-2 .. w0+61.  A's update is valid on lanes 1..62 (it needs the left lane's
// triangle term and the right lane's y), B's on lanes 2..61, which are the 60 output columns.  Rows:
// the strip's R output rows need A on R+2 rows and the input y on R+4 rows.  Where A's result lies
// outside the image B must see the zero padding, so it is masked.
// -------------------------------------------------------------------------------------------------
template <int C>
struct Fwd2Row {
  float y[C], x[C], bb[C], c, wxs, wys;
};

// RING (recompute launches after a segment's first): the input iterate is not read but rebuilt from the x05 rows of
// the two iterations before it, which the ring holds anyway -- x = prox(x05[j-1]), y = x + tP (x - prox(x05[j-2])),
// the forward pass's own expressions -- and no iterate is written.  yin / xin then point at those two rows.
// STORE = false: the launch stores no iterate at all (xout, yout ignored), and its row loop carries no code for it.
template <int C, bool X05, bool RING = false, bool STORE = true>
__global__ __launch_bounds__(256) void tv_forward_strip2(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ xin, float* __restrict__ xout,
    const float* __restrict__ yin, float* __restrict__ yout, float* __restrict__ x05a, float* __restrict__ x05b,
    int N, int H, int W, float tA, float tB, float tP, int R, int strips_x, int strips_y, int Ct, int groups,
    float* __restrict__ keep_x = nullptr, float* __restrict__ keep_y = nullptr) {
  // keep_x / keep_y (optional, not with RING): the input iterate is copied there on the strip's own rows as it passes
  // through -- how the starting point reaches checkpoint 0 without a copy launch
  // groups > 1: the launch covers `groups` consecutive channel groups of C channels each, every strip once per group
  // (forward channels never couple): small images then spread over more wavefronts, each with a shorter row step
  StripGeom g;
  if (!strip_geometry(g, kFwd2Cols, R, W, strips_x, strips_y, N * groups, 2)) return;
  const int ch_first = (g.n % groups) * C;
  g.n /= groups;
  // the output iterate is stored where the caller wants it: x and y separately, or neither (a launch whose successor
  // rebuilds its input from the x05 rows)
  const bool store_x = STORE && xout != nullptr, store_y = STORE && yout != nullptr;
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // last step; strip row k is image row hs - 2 + k
  const float* const wx_p = wx + (size_t)g.n * HW;
  const float* const wy_p = wy + (size_t)g.n * HW;
  const float* const cf_p = cf + (size_t)g.n * HW;
  const float *y_p[C], *x_p[C], *b_p[C];
  float *yo_p[C], *xo_p[C], *xa_p[C], *xb_p[C], *kx_p[C], *ky_p[C];
  const bool keep_xin = !RING && keep_x != nullptr, keep_yin = !RING && keep_y != nullptr;
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t q = ((size_t)g.n * Ct + ch_first + ch) * HW;
    y_p[ch] = yin + q; x_p[ch] = xin + q; b_p[ch] = b + q;
    yo_p[ch] = yout + q; xo_p[ch] = xout + q;
    xa_p[ch] = X05 ? x05a + q : nullptr; xb_p[ch] = X05 ? x05b + q : nullptr;
    kx_p[ch] = keep_xin ? keep_x + q : nullptr; ky_p[ch] = keep_yin ? keep_y + q : nullptr;
  }
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates

  auto load_row = [&](int k, Fwd2Row<C>& in) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    const unsigned row = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4;
    // the outermost rows contribute y (and the upper one its weights) only: their other fields are
    // read from a row the strip needs anyway, so that no cache line is fetched for nothing
    const unsigned row_w = (unsigned)min(max(h, 0), h_hi) * W4;
    const unsigned row_p = (unsigned)min(max(h, h_lo), h_hi) * W4;
    const unsigned row_c = RING ? row : row_p;  // rebuilding y needs c and b wherever y is read
    in.c = ldg(cf_p, row_c + wc);
    in.wxs = ldg(wx_p, row_w + wc);
    in.wys = ldg(wy_p, row_w + wc);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.y[ch] = ldg(y_p[ch], row + wc);
      in.x[ch] = ldg(x_p[ch], row_c + wc);
      in.bb[ch] = ldg(b_p[ch], row_c + wc);
    }
  };
  // Huber-1 prox of the data term (TV.cu:1286-1292)
  auto prox = [&](float yt, float c, float rc1, float bv) {
    float x_loc = div_by(c * bv + yt, 1.f + c, rc1);
    const float lo = yt - c, hi = yt + c;
    if (lo > 1.f + bv) x_loc = lo;
    if (hi < bv - 1.f) x_loc = hi;
    return x_loc;
  };
  auto absorb = [&](int k, Fwd2Row<C>& o) {
    const int h = g.hs - 2 + k;
    const bool rok = h >= 0 && h < H;
    if (RING) {  // o.y holds x05[j-1], o.x holds x05[j-2]
      const float rc1 = rcp_refined(1.f + o.c);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xj = prox(o.y[ch], o.c, rc1, o.bb[ch]);
        const float xm = prox(o.x[ch], o.c, rc1, o.bb[ch]);
        o.x[ch] = xj;
        o.y[ch] = xj + tP * (xj - xm);  // TV.cu:1315
      }
    }
    o.wxs = (rok && wx_ok) ? kL * o.wxs : 0.f;
    o.wys = (rok && g.col_ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) o.y[ch] = (rok && g.col_ok) ? o.y[ch] : 0.f;
  };

  // one triangle (owner value yc, lower neighbour yd): the two products of TV.cu:1268-1274
  auto triangle = [&](float yc, float yd, float wxs, float wys, float& e1, float& e2) {
    const float d1 = yc - yd;
    const float d2 = yc - from_right_lane(yc);
    const float hub = exact_sqrt(d1 * d1 * wys + d2 * d2 * wxs);
    const float m = fmaxf(1.f, inpaint::div_by_tenth(hub));
    const float rm = rcp_refined(m);
    e1 = d1 * div_by(wys, m, rm);
    e2 = d2 * div_by(wxs, m, rm);
  };
  // gradient step + Huber-1 prox + extrapolation of one pixel (TV.cu:1258-1316)
  auto update = [&](float yc, float e1_above, float e2_left, float e1, float e2, float c, float rc1, float bv,
                    float xold, float t, float& xh, float& x_loc, float& yn) {
    float yt = yc;
    yt -= -e1_above;
    yt -= -e2_left;
    yt -= e1;
    yt -= e2;
    xh = yt;
    x_loc = prox(yt, c, rc1, bv);
    yn = x_loc + t * (x_loc - xold);
  };

  float upA[C], upB[C];        // triangle terms handed down to the next row, per iteration
  float pyB[C], pxB[C], pbb[C], pc = 0.f, prc1 = 1.f, pwxs = 0.f, pwys = 0.f;  // row k-1 as iteration B sees it
#pragma unroll
  for (int ch = 0; ch < C; ch++) upA[ch] = upB[ch] = pyB[ch] = pxB[ch] = pbb[ch] = 0.f;

  // step k: A's triangle of row k (+ A's update of row k when DO_A), then B's triangle of row k-1
  // (when TRI_B) and B's update of row k-1 (when DO_B)
  auto step = [&](int k, const Fwd2Row<C>& cur, const Fwd2Row<C>& nxt, auto do_a, auto tri_b, auto do_b) {
    const int h = g.hs - 2 + k;
    const bool in_img = g.col_ok && h >= 0 && h < H;
    const unsigned roffA = (unsigned)min(max(h, 0), H - 1) * W4 + wc;
    const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
    const bool storeA = store_lane && k >= 2 && k <= Reff + 1;  // A's pre-prox value, output rows only
    const float rc1A = rcp_refined(1.f + cur.c);
    const float rc1B = prc1;  // iteration A formed it for this row one step ago
    float nyB[C], nxB[C];
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      float e1, e2;
      triangle(cur.y[ch], nxt.y[ch], cur.wxs, cur.wys, e1, e2);
      const float e1_above = upA[ch];
      upA[ch] = e1;
      nyB[ch] = 0.f;
      nxB[ch] = 0.f;
      if (do_a.value) {
        float xh, x_loc, yn;
        update(cur.y[ch], e1_above, from_left_lane(e2), e1, e2, cur.c, rc1A, cur.bb[ch], cur.x[ch], tA, xh, x_loc, yn);
        nyB[ch] = in_img ? yn : 0.f;  // B reads zero padding outside the image (TV.cu:1229,1237)
        nxB[ch] = x_loc;
        if (X05 && storeA) stg(xa_p[ch], roffA, xh);
        if (!RING && storeA) {  // (own rows are inside the image: cur.y is the loaded value there)
          if (keep_xin) stg(kx_p[ch], roffA, cur.x[ch]);
          if (keep_yin) stg(ky_p[ch], roffA, cur.y[ch]);
        }
      }
    }
    if (tri_b.value) {
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        float e1, e2;
        triangle(pyB[ch], nyB[ch], pwxs, pwys, e1, e2);
        const float e1_above = upB[ch];
        upB[ch] = e1;
        if (do_b.value) {
          float xh, x_loc, yn;
          update(pyB[ch], e1_above, from_left_lane(e2), e1, e2, pc, rc1B, pbb[ch], pxB[ch], tB, xh, x_loc, yn);
          if (store_lane) {
            if (store_y) stg(yo_p[ch], roffB, yn);  // (half of a checkpoint; the non-temporal hint, which pays in the TGV layer, costs 0.8% here)
            if (store_x) stg(xo_p[ch], roffB, x_loc);
            if (X05) stg(xb_p[ch], roffB, xh);
          }
        }
      }
    }
    pc = cur.c; prc1 = rc1A; pwxs = cur.wxs; pwys = cur.wys;
#pragma unroll
    for (int ch = 0; ch < C; ch++) { pyB[ch] = nyB[ch]; pxB[ch] = nxB[ch]; pbb[ch] = cur.bb[ch]; }
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
// Adjoint iteration with the y rebuild fused in: TV.cu:586-859 (+1130-1189); END = the
// segment-start variant TV.cu:862-1126 that reads y from the checkpoint.  END is the last step of
// its segment, so it also performs the first half of the segment flush (copy_and_set_to_0, TV.cu:178-218): the
// fp32 segment sums are stored into the segment's own record (seg_*) and the accumulators are left at zero.  The
// records are added up into the fp64 totals in the reference's order after the last segment.
//
// Per triangle (owner q) the kernel forms, once, every term that the reference evaluates at q,
// at the pixel below q and at the pixel right of q:
//     O1..O4              the four own-triangle terms subtracted at q               (TV.cu:732-743)
//     -O1, P1*tu, P2*tu   the three terms subtracted at the pixel below             (TV.cu:668-677)
//     -O2, P2*tl, P1*tl   the three terms subtracted at the pixel to the right      (TV.cu:701-710)
// with P1 = (g_q-g_d) wy (y_q-y_d), P2 = (g_q-g_r) wx (y_q-y_r).  The operand order inside every
// product is the reference's (negating both factors of a product is exact), the order of the
// subtractions at each pixel is the reference's, and an inactive triangle is the active formula
// with nom = 1, denom = 0, which reproduces the inactive branch exactly.
// -------------------------------------------------------------------------------------------------

// y_{k+1} from x05[k] (xa) and x05[k-1] (xb), TV.cu:1149-1165; rc = rcp_refined(1 + conf)
__device__ __forceinline__ float rebuild_y_fast(float bb, float xa, float xb, float conf, float rc, double opc_d,
                                                float t) {
  float diff = bb - xa;
  float sign = (diff < 0) ? -1.f : 1.f;
  const bool quad = (opc_d >= (double)(sign * diff));  // opc_d = 1. + (double)conf
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

// The pieces of that rebuild for one half-step value v: q = the quadratic branch's iterate (TV.cu:1156-1157),
// l = the other branch's (TV.cu:1162-1164), quad = the regime test on v (TV.cu:1154).  rebuild_y_fast(bb, xa, xb, ...)
// is quad(xa) ? q(xa) + t (q(xa) - q(xb)) : l(xa) + t (l(xa) - l(xb)); a kernel that rebuilds two consecutive y
// evaluates the pieces of the shared middle value once.
struct RebuildPieces {
  float q, l;
  bool quad;
};
__device__ __forceinline__ RebuildPieces rebuild_pieces(float bb, float v, float conf, float rc, double opc_d) {
  RebuildPieces r;
  const float diff = bb - v;
  const float sign = (diff < 0) ? -1.f : 1.f;
  r.quad = (opc_d >= (double)(sign * diff));
  r.q = div_by(conf * bb + v, 1.f + conf, rc);
  r.l = (conf <= sign * diff) ? bb - diff + sign * conf : bb;
  return r;
}
__device__ __forceinline__ float rebuild_from(const RebuildPieces& a, const RebuildPieces& b, float t) {
  const float y_q = a.q + t * (a.q - b.q);
  const float y_l = a.l + t * (a.l - b.l);
  return a.quad ? y_q : y_l;
}

// y_{k+1} exactly as the forward pass made it: x_{k+1} = prox(x05[k]) (TV.cu:1286-1292), y_{k+1} = x_{k+1} +
// t (x_{k+1} - x_k) (TV.cu:1315); x_k is prox(x05[k-1]) or, at a segment start, the checkpointed iterate itself.
__device__ __forceinline__ float prox_huber1(float yt, float c, float rc1, float bv) {
  float x_loc = div_by(c * bv + yt, 1.f + c, rc1);
  const float lo = yt - c, hi = yt + c;
  if (lo > 1.f + bv) x_loc = lo;
  if (hi < bv - 1.f) x_loc = hi;
  return x_loc;
}

template <int C>
struct AdjRow {
  float c, rc1, wxs, wys, xa[C], y[C], bb[C], g[C];  // y is loaded as x05[k-1] (or the checkpoint y) and rebuilt in place
  float xl[C];                                       // FIRST only: the last x05 row, which the first step linearises at
  float gc_i, gwx_i, gwy_i, gx_i[C], gb_i[C];        // accumulators and partial g_x the row's pixel update continues
  double opc_d;                                      // 1. + (double)c, the left side of the prox regime test
};

// TRUE_ADJ selects the corrected gradient (not the reference's): y is the forward pass's own y (see prox_huber1;
// with END the y slot carries the checkpointed x of the segment start, not the checkpointed y), the segment-start
// step uses the main kernel's weight-gradient form, and the per-step multipliers are 1.
// FIRST: this step is the second of the reverse sweep, and the launch performs the sweep's first step (TV.cu:222-287,
// a pointwise map) on the way in: g05_in is the caller's upstream gradient and x05l the last x05 row; every row that is
// loaded gets its incoming adjoint from them, and the strip's own rows add the first step's share to the accumulators,
// channel by channel, before the step's own (the order of two launches).  The accumulators and the partial g_x start at
// zero here, so the launch does not read them (gc_in, gb_in, gwx_in, gwy_in, gxk are not used) and the caller need
// not clear anything: every later launch reads only what the launch before it wrote in full.
template <int C, bool END, bool FINAL, bool TRUE_ADJ = false, bool FIRST = false>
__global__ __launch_bounds__(256) void tv_adjoint_strip(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ yck, const float* __restrict__ gc_in, float* __restrict__ gc,
    const float* __restrict__ gb_in, float* __restrict__ gb, const float* __restrict__ gwx_in,
    float* __restrict__ gwx, const float* __restrict__ gwy_in, float* __restrict__ gwy,
    const float* __restrict__ g05_in, float* __restrict__ g05_out, const float* __restrict__ gxk,
    float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float t, int R, int strips_x, int strips_y, int Ct, int flush_shared, const float* __restrict__ x05l = nullptr) {
  static_assert(!(FIRST && END), "the first step is fused into a segment's inner steps only");
  StripGeom g;
  if (!strip_geometry(g, kAdjCols, R, W, strips_x, strips_y, N)) return;
  const int Reff = min(R, H - g.hs);
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;          // row pitch in bytes
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;  // clamped column (bytes)
  const bool store_lane = g.lane > 0 && g.lane < 63 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const double opt = 1. + (double)t;
  constexpr float kGX = TRUE_ADJ ? 1.f : kLocalGXMult, kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  // wave-uniform plane pointers + 32-bit element offsets (SGPR base, VGPR offset)
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwxi_p = gwx_in + poff, *const gwyi_p = gwy_in + poff;
  float *const gco_p = gc + poff, *const gwxo_p = gwx + poff, *const gwyo_p = gwy + poff;
  const float *xa_p[C], *xb_p[C], *b_p[C], *g_p[C], *gxi_p[C], *gbi_p[C], *xl_p[C];
  float *g05o_p[C], *gxm_p[C], *gbo_p[C], *gxf_p[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    const size_t q = ((size_t)g.n * Ct + ch) * HW;
    xa_p[ch] = x05a + q; xb_p[ch] = (END ? yck : x05b) + q;  // the checkpoint y travels in the y slot
    b_p[ch] = b + q; g_p[ch] = g05_in + q; gxi_p[ch] = gxk + q; gbi_p[ch] = gb_in + q;
    g05o_p[ch] = g05_out + q; gxm_p[ch] = gxk_m1 + q; gbo_p[ch] = gb + q;
    gxf_p[ch] = FINAL ? gx_final + q : nullptr;
    xl_p[ch] = FIRST ? x05l + q : nullptr;
  }

  auto load_row = [&](int k, AdjRow<C>& in) {
    const int kk = min(k, Reff + 1);
    const int h = g.hs - 1 + kk;
    const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    // the rows above and below the strip need y and g (and, above, the weights) only; what they do
    // not need is read from the strip's own first / last row, which is in L1 anyway
    const int hw = g.hs - 1 + min(kk, Reff);
    const unsigned off_w = (unsigned)(hw < 0 ? 0 : hw) * W4 + wc;
    const unsigned off_p = (unsigned)(g.hs - 1 + max(1, min(kk, Reff))) * W4 + wc;
    in.c = ldg(cf_p, off);
    in.wxs = ldg(wx_p, off_w);
    in.wys = ldg(wy_p, off_w);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.xa[ch] = ldg(xa_p[ch], off);
      in.y[ch] = ldg(xb_p[ch], off);
      in.bb[ch] = ldg(b_p[ch], off);
      in.g[ch] = ldg(g_p[ch], off);
      if (FIRST) in.xl[ch] = ldg(xl_p[ch], off);
      // (FIRST: nothing has been accumulated yet and there is no partial g_x: zeros, which nobody has to store first)
      in.gx_i[ch] = FIRST ? 0.f : ldg(gxi_p[ch], off_p);
      in.gb_i[ch] = FIRST ? 0.f : ldg(gbi_p[ch], off_p);
    }
    in.gc_i = FIRST ? 0.f : ldg(gci_p, off_p);
    in.gwx_i = FIRST ? 0.f : ldg(gwxi_p, off_p);
    in.gwy_i = FIRST ? 0.f : ldg(gwyi_p, off_p);
  };
  auto absorb = [&](int k, AdjRow<C>& o) {
    const int h = g.hs - 1 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const inpaint::LaneMask inside(ok);
    o.c = inside(o.c);
    o.rc1 = rcp_refined(1.f + o.c);
    o.opc_d = 1. + (double)o.c;
    o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float xa = inside(o.xa[ch]), xb = inside(o.y[ch]), bv = inside(o.bb[ch]);
      if (TRUE_ADJ) {
        const float xn = prox_huber1(xa, o.c, o.rc1, bv);
        const float xo = END ? xb : prox_huber1(xb, o.c, o.rc1, bv);
        o.y[ch] = xn + t * (xn - xo);
      } else {
        o.y[ch] = END ? xb : rebuild_y_fast(bv, xa, xb, o.c, o.rc1, o.opc_d, t);
      }
      o.g[ch] = inside(o.g[ch]);
      o.xa[ch] = xa;
      o.bb[ch] = bv;
    }
    if (FIRST) {
      // the sweep's first step at this row (TV.cu:240-255): the upstream gradient through the prox at the last x05 row.
      // The accumulators belong to the strip's own rows; what rows above and below make of them is never used.
      const float opc = 1.f + o.c;
      const float rc2 = rcp_refined(opc * opc);
      float gcv = o.gc_i;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float df = o.g[ch], bv = o.bb[ch], xh = inside(o.xl[ch]);
        const float diff = bv - xh;
        const float sign = (diff < 0) ? -1.f : 1.f;
        const bool quad = (o.opc_d >= (double)(sign * diff));
        const float gc_q = df * (div_by(bv, opc, o.rc1) - div_by(o.c * bv + xh, opc * opc, rc2)) * kGC;
        const float gb_q = div_by(df * o.c, opc, o.rc1) * 1.0f;
        o.g[ch] = quad ? div_by(df, opc, o.rc1) : df;
        gcv += quad ? gc_q : sign * df * kGC;
        o.gb_i[ch] = quad ? o.gb_i[ch] + gb_q : 0.f;  // (TV.cu:254 writes zero outside the quadratic regime)
      }
      o.gc_i = gcv;
    }
  };

  float dn1[C], dn3[C], dn4[C];  // terms handed down to the row below
#pragma unroll
  for (int ch = 0; ch < C; ch++) dn1[ch] = dn3[ch] = dn4[ch] = 0.f;

  auto compute = [&](int r, const AdjRow<C>& cur, const AdjRow<C>& nxt, auto first) {
    const int h = g.hs - 1 + r;  // owner row of this step
    const unsigned roff = (unsigned)(h >= 0 ? h : 0) * W4 + wc;
    float gcv = cur.gc_i, gwxv = cur.gwx_i, gwyv = cur.gwy_i, rc2 = 0.f;
    if (!first.value) rc2 = rcp_refined((1.f + cur.c) * (1.f + cur.c));
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float yrt = from_right_lane(cur.y[ch]);
      const float grt = from_right_lane(cur.g[ch]);
      const float gxv = cur.gx_i[ch];
      float gbv = cur.gb_i[ch];
      const float yk = cur.y[ch], yd = nxt.y[ch];
      const float gk = cur.g[ch], gd = nxt.g[ch];
      const float wxv = cur.wxs, wyv = cur.wys;
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
      const float O1 = gpd * (wyv * nom);
      const float O2 = gpr * (wxv * nom);
      const float P1 = gpd * wyv * d1;
      const float P2 = gpr * wxv * d2;
      const float dd = denom * 2.0f;
      const float tp = dd * ((yd - yk) * wyv + (yrt - yk) * wxv);
      const float tu = dd * d1 * wyv;
      const float tl = dd * d2 * wxv;
      const float O3 = P1 * tp, O4 = P2 * tp;
      const float n3 = P1 * tu, n4 = P2 * tu;
      // terms arriving from the triangle of the pixel to the left
      const float l1 = from_left_lane(O2);
      const float l3 = from_left_lane(P2 * tl);
      const float l4 = from_left_lane(P1 * tl);
      if (!first.value) {
        // weight gradients of the pixel's own triangle, TV.cu:749-769 / 1019-1037
        float ux, uy;
        if (!END || TRUE_ADJ) {
          ux = kGX * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
          uy = kGX * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
        } else {
          const float ux_a = kGX * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
          const float uy_a = kGX * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
          ux = act ? ux_a : kGX * d2 * gpr;
          uy = act ? uy_a : kGX * d1 * gpd;
        }
        if (g.w < W - 1) gwxv = gwxv - ux;
        if (h < H - 1) gwyv = gwyv - uy;

        float tt = gk;
        tt -= -dn1[ch];  // TV.cu:668 / 684
        tt -= dn3[ch];   // TV.cu:675
        tt -= dn4[ch];   // TV.cu:677
        tt -= -l1;       // TV.cu:701 / 718
        tt -= l3;        // TV.cu:707
        tt -= l4;        // TV.cu:710
        tt -= O1;        // TV.cu:732 / 763
        tt -= O2;        // TV.cu:733 / 764
        tt -= O3;        // TV.cu:741
        tt -= O4;        // TV.cu:743
        // momentum adjoint, TV.cu:796-801
        float df = (float)((double)gxv + opt * (double)tt);
        df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
        const float gxm = -t * tt;
        // prox adjoint, TV.cu:806-828
        const float conf = cur.c, bv = cur.bb[ch], xh = cur.xa[ch];
        const float diff = bv - xh;
        const float sign = (diff < 0) ? -1.f : 1.f;
        const bool quad = (cur.opc_d >= (double)(sign * diff));
        const float opc = 1.f + conf;
        const float gc_q = df * (div_by(bv, opc, cur.rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
        const float g05_q = div_by(df, opc, cur.rc1);
        const float gb_q = div_by(df * conf, opc, cur.rc1) * 1.0f;
        // three regimes (quadratic / TV.cu:818-822, unreachable for c >= 0 / linear) as selects;
        // adding +0 where the reference adds nothing leaves the accumulators unchanged
        const bool mid = !quad && (conf >= sign * diff);
        const float g05v = quad ? g05_q : (mid ? 0.f : df);
        gcv += quad ? gc_q : (mid ? 0.f : sign * df * kGC);
        gbv += quad ? gb_q : (mid ? df * 1.0f : 0.f);
        if (store_lane) {  // a block this small is predicated, not branched around
          if (FINAL) stg(gxf_p[ch], roff, df);  // only the last step's g_x is read again (TV.cu:800,1785)
          stg(gxm_p[ch], roff, gxm);
          stg(g05o_p[ch], roff, g05v);
          if (END) {  // segment flush, fused: fp32 segment sum into the segment's record, then zero (TV.cu:178-218)
            __builtin_nontemporal_store(gbv, &seg_gb[((size_t)g.n * Ct + ch) * HW + (roff >> 2)]);
            stg(gbo_p[ch], roff, 0.f);
          } else {
            stg(gbo_p[ch], roff, gbv);
          }
        }
      }
      dn1[ch] = O1;
      dn3[ch] = n3;
      dn4[ch] = n4;
    }
    if (!first.value && store_lane) {
      if (END && flush_shared) {
        const size_t e = poff + (roff >> 2);
        __builtin_nontemporal_store(gcv, &seg_gc[e]);
        __builtin_nontemporal_store(gwxv, &seg_gwx[e]);
        __builtin_nontemporal_store(gwyv, &seg_gwy[e]);
        stg(gco_p, roff, 0.f);
        stg(gwxo_p, roff, 0.f);
        stg(gwyo_p, roff, 0.f);
      } else {
        stg(gco_p, roff, gcv);
        stg(gwxo_p, roff, gwxv);
        stg(gwyo_p, roff, gwyv);
      }
    }
  };
  const std::true_type kFirst{};
  const std::false_type kRow{};

  AdjRow<C> b0, b1, b2, b3;
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
// Accumulators at a segment end, in all pair kernels below: a BEND launch stores the segment's sums as a record and
// does not write the zeros the reference leaves in the accumulators (TV.cu:178-218).  The accumulator set it would have
// written holds stale values afterwards: the caller hands the next segment's first launch a field of zeros as
// gc_in / gb_in / gwx_in / gwy_in instead, and a later backward pass starts by clearing the accumulators or from a
// launch that does not read them.
// -------------------------------------------------------------------------------------------------
// Two adjoint steps per launch (A = local iteration j, B = j-1), same arithmetic as tv_adjoint_strip
// applied twice.  B runs one row behind A in the same wavefront: A's outputs g05[j] (B's incoming
// adjoint) and the partial g_x[j] never touch memory, and the five accumulators are read and
// written once for both steps (each pixel adds A's contribution, then B's, as two launches would).
// BEND: B is the segment's first iteration (reads y from the checkpoint, end-form weight
// gradients, fused segment flush).  FINAL: B's completed g_x is stored (gradient wrt the start).
//
// Lanes cover columns w0-2 .. w0+61; A's update is valid on lanes 1..62, B's on 2..61 (the 60
// output columns).  The R output rows need A on R+2 rows; A's accumulator contributions on the two
// halo rows belong to the neighbouring strips and are dropped.
// -------------------------------------------------------------------------------------------------
template <int C>
struct Adj2Row {
  float c, rc1, wxs, wys;
  float xa[C], xb[C];  // x05[j], x05[j-1]: prox points of A and B
  float yA[C];         // loaded as nothing, rebuilt from xa, xb
  float yB[C];         // loaded as x05[j-2] (or the checkpoint y), rebuilt from xb and itself
  float bb[C], g[C], gx_i[C], gb_i[C], gc_i, gwx_i, gwy_i;
  double opc_d;
};

// TRUE_ADJ: the corrected gradient, as in tv_adjoint_strip (with BEND, x05c is the checkpointed x of the segment start).
template <int C, bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(256) void tv_adjoint_strip2(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ x05c, const float* __restrict__ gc_in, float* __restrict__ gc,
    const float* __restrict__ gb_in, float* __restrict__ gb, const float* __restrict__ gwx_in,
    float* __restrict__ gwx, const float* __restrict__ gwy_in, float* __restrict__ gwy,
    const float* __restrict__ g05_in, float* __restrict__ g05_out, const float* __restrict__ gxk,
    float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  StripGeom g;
  if (!strip_geometry(g, kFwd2Cols, R, W, strips_x, strips_y, N, 2)) return;
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwxi_p = gwx_in + poff, *const gwyi_p = gwy_in + poff;
  float *const gco_p = gc + poff, *const gwxo_p = gwx + poff, *const gwyo_p = gwy + poff;
  // One base pointer per tensor (the sample's first channel); channel ch sits chs[ch] bytes further (a 32-bit
  // offset: the host refuses planes of 2^29 pixels and more).  A pointer pair per tensor AND channel does not fit the
  // scalar registers: the compiler parks the surplus in lanes of a vector register and re-reads it at every row.
  const size_t q0 = (size_t)g.n * Ct * HW;
  const float *const xa_p = x05a + q0, *const xb_p = x05b + q0, *const xc_p = x05c + q0;  // x05c: x05[j-2], or the checkpoint y when BEND
  const float *const b_p = b + q0, *const g_p = g05_in + q0, *const gxi_p = gxk + q0, *const gbi_p = gb_in + q0;
  float *const g05o_p = g05_out + q0, *const gxm_p = gxk_m1 + q0, *const gbo_p = gb + q0;
  float *const gxf_p = FINAL ? gx_final + q0 : nullptr;
  unsigned chs[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) chs[ch] = (unsigned)ch * (4u * (unsigned)HW);
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  auto load_row = [&](int k, Adj2Row<C>& in) {
    const int kk = min(k, klast + 1);
    const int h = g.hs - 2 + kk;
    const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
    // what a row does not need is read from a row the strip needs anyway (no extra cache lines)
    const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
    const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
    const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
    in.c = ldg(cf_p, off);
    in.wxs = ldg(wx_p, off_w);
    in.wys = ldg(wy_p, off_w);
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      in.xa[ch] = ldg(xa_p, off + chs[ch]);
      in.xb[ch] = ldg(xb_p, off + chs[ch]);
      in.yB[ch] = ldg(xc_p, off + chs[ch]);
      in.bb[ch] = ldg(b_p, off + chs[ch]);
      in.g[ch] = ldg(g_p, off + chs[ch]);
      in.gx_i[ch] = ldg(gxi_p, off_a + chs[ch]);
      in.gb_i[ch] = ldg(gbi_p, off_o + chs[ch]);
    }
    in.gc_i = ldg(gci_p, off_o);
    in.gwx_i = ldg(gwxi_p, off_o);
    in.gwy_i = ldg(gwyi_p, off_o);
  };
  auto absorb = [&](int k, Adj2Row<C>& o) {
    const int h = g.hs - 2 + k;
    const bool ok = g.col_ok && h >= 0 && h < H;
    const std::conditional_t<BEND, inpaint::LaneSelect, inpaint::LaneMask> inside(ok);  // (the segment-end pair is short of registers)
    o.c = inside(o.c);
    o.rc1 = rcp_refined(1.f + o.c);
    o.opc_d = 1. + (double)o.c;
    o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
    o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const float xa = inside(o.xa[ch]), xb = inside(o.xb[ch]), xc = inside(o.yB[ch]), bv = inside(o.bb[ch]);
      if (TRUE_ADJ) {
        const float pa = prox_huber1(xa, o.c, o.rc1, bv), pb = prox_huber1(xb, o.c, o.rc1, bv);
        const float pc = BEND ? xc : prox_huber1(xc, o.c, o.rc1, bv);
        o.yA[ch] = pa + tA * (pa - pb);
        o.yB[ch] = pb + tB * (pb - pc);
      } else {
        // rebuild_y_fast(bv, xa, xb, ..., tA) and rebuild_y_fast(bv, xb, xc, ..., tB) with the pieces of xb formed once
        const RebuildPieces ra = rebuild_pieces(bv, xa, o.c, o.rc1, o.opc_d), rb = rebuild_pieces(bv, xb, o.c, o.rc1, o.opc_d);
        o.yA[ch] = rebuild_from(ra, rb, tA);
        o.yB[ch] = BEND ? xc : rebuild_from(rb, rebuild_pieces(bv, xc, o.c, o.rc1, o.opc_d), tB);
      }
      o.g[ch] = inside(o.g[ch]);
      o.xa[ch] = xa;
      o.xb[ch] = xb;
      o.bb[ch] = bv;
    }
  };

  constexpr float kGX = TRUE_ADJ ? 1.f : kLocalGXMult, kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  struct Tri {  // everything one triangle contributes (see tv_adjoint_strip)
    float O1, O2, O3, O4, n3, n4, l1, l3, l4, ux, uy;
  };
  auto triangle = [&](float yk, float yd, float gk, float gd, float wxv, float wyv, auto end_form) {
    Tri r;
    const float yrt = from_right_lane(yk);
    const float grt = from_right_lane(gk);
    const float d1 = yk - yd, d2 = yk - yrt;
    const float a1 = d1 * d1 * wyv;
    const float a2 = d2 * d2 * wxv;
    const float hub = exact_sqrt(a2 + a1);
    const bool act = hub > kDelta;
    float nom = inpaint::exact_div(kDelta, hub);
    float denom = inpaint::exact_div(nom, 2.f * hub * hub);
    nom = act ? nom : 1.f;
    denom = act ? denom : 0.f;
    const float gpd = gk - gd, gpr = gk - grt;
    r.O1 = gpd * (wyv * nom);
    r.O2 = gpr * (wxv * nom);
    const float P1 = gpd * wyv * d1;
    const float P2 = gpr * wxv * d2;
    const float dd = denom * 2.0f;
    // the reference's factor dd * ((yd - yk) * wyv + (yrt - yk) * wxv) is minus this one, exactly: a - b = -(b - a),
    // (-a) * w = -(a * w) and (-a) + (-b) = -(a + b) in IEEE arithmetic; O3, O4 carry the sign
    const float tp = dd * (d1 * wyv + d2 * wxv);
    const float tu = dd * d1 * wyv;
    const float tl = dd * d2 * wxv;
    r.O3 = -(P1 * tp);
    r.O4 = -(P2 * tp);
    r.n3 = P1 * tu;
    r.n4 = P2 * tu;
    r.l1 = from_left_lane(r.O2);
    r.l3 = from_left_lane(P2 * tl);
    r.l4 = from_left_lane(P1 * tl);
    if (!end_form.value) {  // TV.cu:749-769
      r.ux = kGX * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
      r.uy = kGX * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
    } else {  // TV.cu:1019-1037
      const float ux_a = kGX * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
      const float uy_a = kGX * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
      r.ux = act ? ux_a : kGX * d2 * gpr;
      r.uy = act ? uy_a : kGX * d1 * gpd;
    }
    return r;
  };
  // pixel update: J^T assembly, momentum adjoint, prox adjoint (TV.cu:668-743, 796-828)
  auto update = [&](float gk, const Tri& t, float a1_, float a3_, float a4_, float gxv, double opt, float tmom,
                    float conf, float rc1, float rc2, double opc_d, float bv, float xh, float& df, float& gxm,
                    float& g05v, float& gc_add, float& gb_add) {
    float tt = gk;
    tt -= -a1_;
    tt -= a3_;
    tt -= a4_;
    tt -= -t.l1;
    tt -= t.l3;
    tt -= t.l4;
    tt -= t.O1;
    tt -= t.O2;
    tt -= t.O3;
    tt -= t.O4;
    df = (float)((double)gxv + opt * (double)tt);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    gxm = -tmom * tt;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    g05v = quad ? g05_q : (mid ? 0.f : df);
    gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
    gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
  };

  float dA1[C], dA3[C], dA4[C], dB1[C], dB3[C], dB4[C];  // terms handed down, per step
  // row k-1 as step B sees it
  float pG[C], pgxm[C], pyB[C], pxb[C], pbb[C], pgb[C], pgc = 0.f, pgwx = 0.f, pgwy = 0.f;
  float pc = 0.f, prc1 = 1.f, prc2 = 1.f, pwxs = 0.f, pwys = 0.f;
  double popc_d = 1.;
#pragma unroll
  for (int ch = 0; ch < C; ch++) {
    dA1[ch] = dA3[ch] = dA4[ch] = dB1[ch] = dB3[ch] = dB4[ch] = 0.f;
    pG[ch] = pgxm[ch] = pyB[ch] = pxb[ch] = pbb[ch] = pgb[ch] = 0.f;
  }
  const std::true_type kYes{};
  const std::false_type kNo{};
  const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form

  auto step = [&](int k, const Adj2Row<C>& cur, const Adj2Row<C>& nxt, auto do_a, auto tri_b, auto do_b) {
    const int h = g.hs - 2 + k;  // A's row; B's row is h - 1
    const bool in_img = g.col_ok && h >= 0 && h < H;
    const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
    float nG[C], ngxm[C], ngb[C];
    float gcv = cur.gc_i, gwxv = cur.gwx_i, gwyv = cur.gwy_i;
    const float rc2A = rcp_refined((1.f + cur.c) * (1.f + cur.c));
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      const Tri t = triangle(cur.yA[ch], nxt.yA[ch], cur.g[ch], nxt.g[ch], cur.wxs, cur.wys, kNo);
      const float a1_ = dA1[ch], a3_ = dA3[ch], a4_ = dA4[ch];
      dA1[ch] = t.O1; dA3[ch] = t.n3; dA4[ch] = t.n4;
      nG[ch] = 0.f; ngxm[ch] = 0.f; ngb[ch] = cur.gb_i[ch];
      if (do_a.value) {
        if (g.w < W - 1) gwxv = gwxv - t.ux;
        if (h < H - 1) gwyv = gwyv - t.uy;
        float df, gxm, g05v, gc_add, gb_add;
        update(cur.g[ch], t, a1_, a3_, a4_, cur.gx_i[ch], optA, tA, cur.c, cur.rc1, rc2A, cur.opc_d, cur.bb[ch],
               cur.xa[ch], df, gxm, g05v, gc_add, gb_add);
        gcv += gc_add;
        ngb[ch] += gb_add;
        nG[ch] = in_img ? g05v : 0.f;  // B reads zero padding outside the image
        ngxm[ch] = gxm;
      }
    }
    if (tri_b.value) {
      float gcB = pgc, gwxB = pgwx, gwyB = pgwy;
      const float rc2B = prc2;  // step A formed it for this row one step ago
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const Tri t = triangle(pyB[ch], cur.yB[ch], pG[ch], nG[ch], pwxs, pwys, kBEnd);
        const float a1_ = dB1[ch], a3_ = dB3[ch], a4_ = dB4[ch];
        dB1[ch] = t.O1; dB3[ch] = t.n3; dB4[ch] = t.n4;
        if (do_b.value) {
          if (g.w < W - 1) gwxB = gwxB - t.ux;
          if (h - 1 < H - 1) gwyB = gwyB - t.uy;
          float df, gxm, g05v, gc_add, gb_add;
          update(pG[ch], t, a1_, a3_, a4_, pgxm[ch], optB, tB, pc, prc1, rc2B, popc_d, pbb[ch], pxb[ch], df, gxm, g05v,
                 gc_add, gb_add);
          gcB += gc_add;
          const float gbv = pgb[ch] + gb_add;
          if (store_lane) {
            if (FINAL) stg(gxf_p, roffB + chs[ch], df);
            stg(gxm_p, roffB + chs[ch], gxm);
            stg(g05o_p, roffB + chs[ch], g05v);
            if (BEND) {  // segment flush, fused (TV.cu:178-218)
              __builtin_nontemporal_store(gbv, &seg_gb[((size_t)g.n * Ct + ch) * HW + (roffB >> 2)]);
            } else {
              stg(gbo_p, roffB + chs[ch], gbv);
            }
          }
        }
      }
      if (do_b.value && store_lane) {
        if (BEND) {
          const size_t e = poff + (roffB >> 2);
          __builtin_nontemporal_store(gcB, &seg_gc[e]);
          __builtin_nontemporal_store(gwxB, &seg_gwx[e]);
          __builtin_nontemporal_store(gwyB, &seg_gwy[e]);
        } else {
          stg(gco_p, roffB, gcB);
          stg(gwxo_p, roffB, gwxB);
          stg(gwyo_p, roffB, gwyB);
        }
      }
    }
    pgc = gcv; pgwx = gwxv; pgwy = gwyv;
    pc = cur.c; prc1 = cur.rc1; prc2 = rc2A; popc_d = cur.opc_d; pwxs = cur.wxs; pwys = cur.wys;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      pG[ch] = nG[ch]; pgxm[ch] = ngxm[ch]; pgb[ch] = ngb[ch];
      pyB[ch] = cur.yB[ch]; pxb[ch] = cur.xb[ch]; pbb[ch] = cur.bb[ch];
    }
  };

  Adj2Row<C> b0, b1, b2, b3;
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
// The same two adjoint steps per launch for TWO channels with ONE CHANNEL PER WAVEFRONT (128-thread workgroup, one strip
// per workgroup), for launches that cannot fill the chip: such a launch lasts as long as one wavefront needs for its
// strip, and a wavefront with one channel needs half the time per row.  Both wavefronts run tv_adjoint_strip2's row loop
// on their own channel.  The channels meet in the three shared accumulators only, which the reference sums in the order
// A(ch 0), A(ch 1), B(ch 0), B(ch 1): wavefront 0 does not touch them but hands its terms (gc term, ux, uy of step A and
// of step B, six floats per row and lane) through LDS to wavefront 1, which works one row step behind, reads the
// accumulators, applies channel 0's terms before its own and stores.  One LDS-only barrier per row step; both wavefronts
// pass klast + 2 of them.
// -------------------------------------------------------------------------------------------------
template <bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(128) void tv_adjoint_strip2c(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ x05c, const float* __restrict__ gc_in, float* __restrict__ gc,
    const float* __restrict__ gb_in, float* __restrict__ gb, const float* __restrict__ gwx_in,
    float* __restrict__ gwx, const float* __restrict__ gwy_in, float* __restrict__ gwy,
    const float* __restrict__ g05_in, float* __restrict__ g05_out, const float* __restrict__ gxk,
    float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  constexpr int C = 1;  // channels per wavefront
  __shared__ float terms[2][6][64];  // wavefront 0's terms of a row step: gc term, ux, uy of step A and of step B
  StripGeom g;
  if (!strip_geometry_block(g, kFwd2Cols, R, W, strips_x, strips_y, N, 2)) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const size_t poff = (size_t)g.n * HW;
  const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
  const float *const gci_p = gc_in + poff, *const gwxi_p = gwx_in + poff, *const gwyi_p = gwy_in + poff;
  float *const gco_p = gc + poff, *const gwxo_p = gwx + poff, *const gwyo_p = gwy + poff;
  // One base pointer per tensor (the sample's first channel); channel ch sits chs[ch] bytes further (a 32-bit
  // offset: the host refuses planes of 2^29 pixels and more).  A pointer pair per tensor AND channel does not fit the
  // scalar registers: the compiler parks the surplus in lanes of a vector register and re-reads it at every row.
  const size_t q0 = ((size_t)g.n * Ct + wave) * HW;  // this wavefront's channel
  const float *const xa_p = x05a + q0, *const xb_p = x05b + q0, *const xc_p = x05c + q0;  // x05c: x05[j-2], or the checkpoint y when BEND
  const float *const b_p = b + q0, *const g_p = g05_in + q0, *const gxi_p = gxk + q0, *const gbi_p = gb_in + q0;
  float *const g05o_p = g05_out + q0, *const gxm_p = gxk_m1 + q0, *const gbo_p = gb + q0;
  float *const gxf_p = FINAL ? gx_final + q0 : nullptr;
  unsigned chs[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) chs[ch] = (unsigned)ch * (4u * (unsigned)HW);
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  auto run = [&](auto role) {
    constexpr int ROLE = decltype(role)::value;  // 0: channel 0, hands its accumulator terms on; 1: channel 1, owns the accumulators
    auto load_row = [&](int k, Adj2Row<C>& in) {
      const int kk = min(k, klast + 1);
      const int h = g.hs - 2 + kk;
      const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
      // what a row does not need is read from a row the strip needs anyway (no extra cache lines)
      const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
      const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
      const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
  #pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xa[ch] = ldg(xa_p, off + chs[ch]);
        in.xb[ch] = ldg(xb_p, off + chs[ch]);
        in.yB[ch] = ldg(xc_p, off + chs[ch]);
        in.bb[ch] = ldg(b_p, off + chs[ch]);
        in.g[ch] = ldg(g_p, off + chs[ch]);
        in.gx_i[ch] = ldg(gxi_p, off_a + chs[ch]);
        in.gb_i[ch] = ldg(gbi_p, off_o + chs[ch]);
      }
      in.gc_i = ldg(gci_p, off_o);
      in.gwx_i = ldg(gwxi_p, off_o);
      in.gwy_i = ldg(gwyi_p, off_o);
    };
    auto absorb = [&](int k, Adj2Row<C>& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const std::conditional_t<BEND, inpaint::LaneSelect, inpaint::LaneMask> inside(ok);  // (the segment-end pair is short of registers)
      o.c = inside(o.c);
      o.rc1 = rcp_refined(1.f + o.c);
      o.opc_d = 1. + (double)o.c;
      o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
  #pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xa = inside(o.xa[ch]), xb = inside(o.xb[ch]), xc = inside(o.yB[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pa = prox_huber1(xa, o.c, o.rc1, bv), pb = prox_huber1(xb, o.c, o.rc1, bv);
          const float pc = BEND ? xc : prox_huber1(xc, o.c, o.rc1, bv);
          o.yA[ch] = pa + tA * (pa - pb);
          o.yB[ch] = pb + tB * (pb - pc);
        } else {
          // rebuild_y_fast(bv, xa, xb, ..., tA) and rebuild_y_fast(bv, xb, xc, ..., tB) with the pieces of xb formed once
          const RebuildPieces ra = rebuild_pieces(bv, xa, o.c, o.rc1, o.opc_d), rb = rebuild_pieces(bv, xb, o.c, o.rc1, o.opc_d);
          o.yA[ch] = rebuild_from(ra, rb, tA);
          o.yB[ch] = BEND ? xc : rebuild_from(rb, rebuild_pieces(bv, xc, o.c, o.rc1, o.opc_d), tB);
        }
        o.g[ch] = inside(o.g[ch]);
        o.xa[ch] = xa;
        o.xb[ch] = xb;
        o.bb[ch] = bv;
      }
    };

    constexpr float kGX = TRUE_ADJ ? 1.f : kLocalGXMult, kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
    struct Tri {  // everything one triangle contributes (see tv_adjoint_strip)
      float O1, O2, O3, O4, n3, n4, l1, l3, l4, ux, uy;
    };
    auto triangle = [&](float yk, float yd, float gk, float gd, float wxv, float wyv, auto end_form) {
      Tri r;
      const float yrt = from_right_lane(yk);
      const float grt = from_right_lane(gk);
      const float d1 = yk - yd, d2 = yk - yrt;
      const float a1 = d1 * d1 * wyv;
      const float a2 = d2 * d2 * wxv;
      const float hub = exact_sqrt(a2 + a1);
      const bool act = hub > kDelta;
      float nom = inpaint::exact_div(kDelta, hub);
      float denom = inpaint::exact_div(nom, 2.f * hub * hub);
      nom = act ? nom : 1.f;
      denom = act ? denom : 0.f;
      const float gpd = gk - gd, gpr = gk - grt;
      r.O1 = gpd * (wyv * nom);
      r.O2 = gpr * (wxv * nom);
      const float P1 = gpd * wyv * d1;
      const float P2 = gpr * wxv * d2;
      const float dd = denom * 2.0f;
      // the reference's factor dd * ((yd - yk) * wyv + (yrt - yk) * wxv) is minus this one, exactly: a - b = -(b - a),
      // (-a) * w = -(a * w) and (-a) + (-b) = -(a + b) in IEEE arithmetic; O3, O4 carry the sign
      const float tp = dd * (d1 * wyv + d2 * wxv);
      const float tu = dd * d1 * wyv;
      const float tl = dd * d2 * wxv;
      r.O3 = -(P1 * tp);
      r.O4 = -(P2 * tp);
      r.n3 = P1 * tu;
      r.n4 = P2 * tu;
      r.l1 = from_left_lane(r.O2);
      r.l3 = from_left_lane(P2 * tl);
      r.l4 = from_left_lane(P1 * tl);
      if (!end_form.value) {  // TV.cu:749-769
        r.ux = kGX * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
        r.uy = kGX * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
      } else {  // TV.cu:1019-1037
        const float ux_a = kGX * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
        const float uy_a = kGX * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
        r.ux = act ? ux_a : kGX * d2 * gpr;
        r.uy = act ? uy_a : kGX * d1 * gpd;
      }
      return r;
    };
    // pixel update: J^T assembly, momentum adjoint, prox adjoint (TV.cu:668-743, 796-828)
    auto update = [&](float gk, const Tri& t, float a1_, float a3_, float a4_, float gxv, double opt, float tmom,
                      float conf, float rc1, float rc2, double opc_d, float bv, float xh, float& df, float& gxm,
                      float& g05v, float& gc_add, float& gb_add) {
      float tt = gk;
      tt -= -a1_;
      tt -= a3_;
      tt -= a4_;
      tt -= -t.l1;
      tt -= t.l3;
      tt -= t.l4;
      tt -= t.O1;
      tt -= t.O2;
      tt -= t.O3;
      tt -= t.O4;
      df = (float)((double)gxv + opt * (double)tt);
      df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
      gxm = -tmom * tt;
      const float diff = bv - xh;
      const float sign = (diff < 0) ? -1.f : 1.f;
      const bool quad = (opc_d >= (double)(sign * diff));
      const float opc = 1.f + conf;
      const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
      const float g05_q = div_by(df, opc, rc1);
      const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
      const bool mid = !quad && (conf >= sign * diff);
      g05v = quad ? g05_q : (mid ? 0.f : df);
      gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
      gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
    };

    float dA1[C], dA3[C], dA4[C], dB1[C], dB3[C], dB4[C];  // terms handed down, per step
    // row k-1 as step B sees it
    float pG[C], pgxm[C], pyB[C], pxb[C], pbb[C], pgb[C], pgc = 0.f, pgwx = 0.f, pgwy = 0.f;
    float pc = 0.f, prc1 = 1.f, prc2 = 1.f, pwxs = 0.f, pwys = 0.f;
    double popc_d = 1.;
  #pragma unroll
    for (int ch = 0; ch < C; ch++) {
      dA1[ch] = dA3[ch] = dA4[ch] = dB1[ch] = dB3[ch] = dB4[ch] = 0.f;
      pG[ch] = pgxm[ch] = pyB[ch] = pxb[ch] = pbb[ch] = pgb[ch] = 0.f;
    }
    const std::true_type kYes{};
    const std::false_type kNo{};
    const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form

    auto step = [&](int k, const Adj2Row<C>& cur, const Adj2Row<C>& nxt, auto do_a, auto tri_b, auto do_b) {
      const int h = g.hs - 2 + k;  // A's row; B's row is h - 1
      const bool in_img = g.col_ok && h >= 0 && h < H;
      const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
      float nG[C], ngxm[C], ngb[C];
      float (*slot)[64] = terms[k & 1];
      float gcv = cur.gc_i, gwxv = cur.gwx_i, gwyv = cur.gwy_i;
      if (ROLE == 1 && do_a.value) {  // channel 0's terms of this row first
        if (g.w < W - 1) gwxv = gwxv - slot[1][g.lane];
        if (h < H - 1) gwyv = gwyv - slot[2][g.lane];
        gcv += slot[0][g.lane];
      }
      const float rc2A = rcp_refined((1.f + cur.c) * (1.f + cur.c));
  #pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const Tri t = triangle(cur.yA[ch], nxt.yA[ch], cur.g[ch], nxt.g[ch], cur.wxs, cur.wys, kNo);
        const float a1_ = dA1[ch], a3_ = dA3[ch], a4_ = dA4[ch];
        dA1[ch] = t.O1; dA3[ch] = t.n3; dA4[ch] = t.n4;
        nG[ch] = 0.f; ngxm[ch] = 0.f; ngb[ch] = cur.gb_i[ch];
        if (do_a.value) {
          float df, gxm, g05v, gc_add, gb_add;
          update(cur.g[ch], t, a1_, a3_, a4_, cur.gx_i[ch], optA, tA, cur.c, cur.rc1, rc2A, cur.opc_d, cur.bb[ch],
                 cur.xa[ch], df, gxm, g05v, gc_add, gb_add);
          if (ROLE == 1) {
            if (g.w < W - 1) gwxv = gwxv - t.ux;
            if (h < H - 1) gwyv = gwyv - t.uy;
            gcv += gc_add;
          } else {
            slot[0][g.lane] = gc_add;
            slot[1][g.lane] = t.ux;
            slot[2][g.lane] = t.uy;
          }
          ngb[ch] += gb_add;
          nG[ch] = in_img ? g05v : 0.f;  // B reads zero padding outside the image
          ngxm[ch] = gxm;
        }
      }
      if (tri_b.value) {
        float gcB = pgc, gwxB = pgwx, gwyB = pgwy;
        if (ROLE == 1 && do_b.value) {  // channel 0's terms of B's row first
          if (g.w < W - 1) gwxB = gwxB - slot[4][g.lane];
          if (h - 1 < H - 1) gwyB = gwyB - slot[5][g.lane];
          gcB += slot[3][g.lane];
        }
        const float rc2B = prc2;  // step A formed it for this row one step ago
  #pragma unroll
        for (int ch = 0; ch < C; ch++) {
          const Tri t = triangle(pyB[ch], cur.yB[ch], pG[ch], nG[ch], pwxs, pwys, kBEnd);
          const float a1_ = dB1[ch], a3_ = dB3[ch], a4_ = dB4[ch];
          dB1[ch] = t.O1; dB3[ch] = t.n3; dB4[ch] = t.n4;
          if (do_b.value) {
            float df, gxm, g05v, gc_add, gb_add;
            update(pG[ch], t, a1_, a3_, a4_, pgxm[ch], optB, tB, pc, prc1, rc2B, popc_d, pbb[ch], pxb[ch], df, gxm, g05v,
                   gc_add, gb_add);
            if (ROLE == 1) {
              if (g.w < W - 1) gwxB = gwxB - t.ux;
              if (h - 1 < H - 1) gwyB = gwyB - t.uy;
              gcB += gc_add;
            } else {
              slot[3][g.lane] = gc_add;
              slot[4][g.lane] = t.ux;
              slot[5][g.lane] = t.uy;
            }
            const float gbv = pgb[ch] + gb_add;
            if (store_lane) {
              if (FINAL) stg(gxf_p, roffB + chs[ch], df);
              stg(gxm_p, roffB + chs[ch], gxm);
              stg(g05o_p, roffB + chs[ch], g05v);
              if (BEND) {  // segment flush, fused (TV.cu:178-218)
                __builtin_nontemporal_store(gbv, &seg_gb[((size_t)g.n * Ct + wave + ch) * HW + (roffB >> 2)]);
              } else {
                stg(gbo_p, roffB + chs[ch], gbv);
              }
            }
          }
        }
        if (ROLE == 1 && do_b.value && store_lane) {
          if (BEND) {
            const size_t e = poff + (roffB >> 2);
            __builtin_nontemporal_store(gcB, &seg_gc[e]);
            __builtin_nontemporal_store(gwxB, &seg_gwx[e]);
            __builtin_nontemporal_store(gwyB, &seg_gwy[e]);
          } else {
            stg(gco_p, roffB, gcB);
            stg(gwxo_p, roffB, gwxB);
            stg(gwyo_p, roffB, gwyB);
          }
        }
      }
      pgc = gcv; pgwx = gwxv; pgwy = gwyv;
      pc = cur.c; prc1 = cur.rc1; prc2 = rc2A; popc_d = cur.opc_d; pwxs = cur.wxs; pwys = cur.wys;
  #pragma unroll
      for (int ch = 0; ch < C; ch++) {
        pG[ch] = nG[ch]; pgxm[ch] = ngxm[ch]; pgb[ch] = ngb[ch];
        pyB[ch] = cur.yB[ch]; pxb[ch] = cur.xb[ch]; pbb[ch] = cur.bb[ch];
      }
    };

    Adj2Row<C> b0, b1, b2, b3;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    load_row(3, b3);
    if (ROLE == 1) lds_barrier();  // one row step behind wavefront 0
    absorb(0, b0);
    absorb(1, b1);
    step(0, b0, b1, kNo, kNo, kNo);
    lds_barrier();
    load_row(4, b0);
    absorb(2, b2);
    step(1, b1, b2, kYes, kNo, kNo);
    lds_barrier();
    load_row(5, b1);
    absorb(3, b3);
    step(2, b2, b3, kYes, kYes, kNo);
    lds_barrier();
    load_row(6, b2);
    for (int k = 3; k <= klast; k += 4) {  // cur / next rotate through (b3,b0) (b0,b1) (b1,b2) (b2,b3)
      absorb(k + 1, b0);
      step(k, b3, b0, kYes, kYes, kYes);
      lds_barrier();
      load_row(k + 4, b3);
      if (k + 1 > klast) break;
      absorb(k + 2, b1);
      step(k + 1, b0, b1, kYes, kYes, kYes);
      lds_barrier();
      load_row(k + 5, b0);
      if (k + 2 > klast) break;
      absorb(k + 3, b2);
      step(k + 2, b1, b2, kYes, kYes, kYes);
      lds_barrier();
      load_row(k + 6, b1);
      if (k + 3 > klast) break;
      absorb(k + 4, b3);
      step(k + 3, b2, b3, kYes, kYes, kYes);
      lds_barrier();
      load_row(k + 7, b2);
    }

    if (ROLE == 0) lds_barrier();  // wavefront 1's last row step
  };
  if (wave == 0) run(std::integral_constant<int, 0>{});
  else run(std::integral_constant<int, 1>{});
}

// -------------------------------------------------------------------------------------------------
// Two adjoint steps per launch in TWO wavefronts of a 128-thread workgroup (one strip per workgroup),
// for the channel counts whose two steps do not fit one wavefront's registers (3 and 4).  Same
// arithmetic, same rows and lanes as tv_adjoint_strip2: wavefront 0 runs step A (iteration j) on row
// k of the strip, wavefront 1 runs step B (iteration j-1) on row k-1.  What A computes for a row and
// B continues -- g05[j] and the partial g_x[j] per channel, the per-channel gb and the three shared
// accumulators with A's terms added (all channels of A first, then all channels of B: the reference's
// order) -- travels through LDS together with the row's inputs both steps need (c, 1/(1+c), the
// scaled weights, b and x05[j-1]), 5C + 7 floats per lane and row.  A publishes kP rows per barrier
// into 2 kP slots; B works on the kP rows before them.  Both wavefronts pass the same number of
// barriers, ceil((klast + 1) / kP).
// -------------------------------------------------------------------------------------------------
template <int C>
struct Adj2wRow {
  float c, rc1, wxs, wys;
  float xa[C], xb[C], yA[C], bb[C], g[C], gx_i[C], gb_i[C], gc_i, gwx_i, gwy_i;
  double opc_d;
};

template <int C, bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(128) void tv_adjoint_strip2w(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ x05c, const float* __restrict__ gc_in, float* __restrict__ gc,
    const float* __restrict__ gb_in, float* __restrict__ gb, const float* __restrict__ gwx_in,
    float* __restrict__ gwx, const float* __restrict__ gwy_in, float* __restrict__ gwy,
    const float* __restrict__ g05_in, float* __restrict__ g05_out, const float* __restrict__ gxk,
    float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  constexpr int kP = 2;                 // rows step A publishes per barrier
  constexpr int kHand = 5 * C + 7;      // floats per lane and row
  __shared__ float hand[2 * kP][kHand][64];
  StripGeom g;
  if (!strip_geometry_block(g, kFwd2Cols, R, W, strips_x, strips_y, N, 2)) return;
  const int role = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wavefront 0: step A, wavefront 1: step B
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const size_t poff = (size_t)g.n * HW;
  const size_t q0 = (size_t)g.n * Ct * HW;  // one base pointer per tensor, channel ch chs[ch] bytes further
  unsigned chs[C];
#pragma unroll
  for (int ch = 0; ch < C; ch++) chs[ch] = (unsigned)ch * (4u * (unsigned)HW);
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  constexpr float kGX = TRUE_ADJ ? 1.f : kLocalGXMult, kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  struct Tri {  // everything one triangle contributes (see tv_adjoint_strip)
    float O1, O2, O3, O4, n3, n4, l1, l3, l4, ux, uy;
  };
  auto triangle = [&](float yk, float yd, float gk, float gd, float wxv, float wyv, auto end_form) {
    Tri r;
    const float yrt = from_right_lane(yk);
    const float grt = from_right_lane(gk);
    const float d1 = yk - yd, d2 = yk - yrt;
    const float a1 = d1 * d1 * wyv;
    const float a2 = d2 * d2 * wxv;
    const float hub = exact_sqrt(a2 + a1);
    const bool act = hub > kDelta;
    float nom = inpaint::exact_div(kDelta, hub);
    float denom = inpaint::exact_div(nom, 2.f * hub * hub);
    nom = act ? nom : 1.f;
    denom = act ? denom : 0.f;
    const float gpd = gk - gd, gpr = gk - grt;
    r.O1 = gpd * (wyv * nom);
    r.O2 = gpr * (wxv * nom);
    const float P1 = gpd * wyv * d1;
    const float P2 = gpr * wxv * d2;
    const float dd = denom * 2.0f;
    const float tp = dd * (d1 * wyv + d2 * wxv);  // minus the reference's factor, exactly; O3, O4 carry the sign
    const float tu = dd * d1 * wyv;
    const float tl = dd * d2 * wxv;
    r.O3 = -(P1 * tp);
    r.O4 = -(P2 * tp);
    r.n3 = P1 * tu;
    r.n4 = P2 * tu;
    r.l1 = from_left_lane(r.O2);
    r.l3 = from_left_lane(P2 * tl);
    r.l4 = from_left_lane(P1 * tl);
    if (!end_form.value) {  // TV.cu:749-769
      r.ux = kGX * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
      r.uy = kGX * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
    } else {  // TV.cu:1019-1037
      const float ux_a = kGX * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
      const float uy_a = kGX * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
      r.ux = act ? ux_a : kGX * d2 * gpr;
      r.uy = act ? uy_a : kGX * d1 * gpd;
    }
    return r;
  };
  // pixel update: J^T assembly, momentum adjoint, prox adjoint (TV.cu:668-743, 796-828)
  auto update = [&](float gk, const Tri& t, float a1_, float a3_, float a4_, float gxv, double opt, float tmom,
                    float conf, float rc1, float rc2, double opc_d, float bv, float xh, float& df, float& gxm,
                    float& g05v, float& gc_add, float& gb_add) {
    float tt = gk;
    tt -= -a1_;
    tt -= a3_;
    tt -= a4_;
    tt -= -t.l1;
    tt -= t.l3;
    tt -= t.l4;
    tt -= t.O1;
    tt -= t.O2;
    tt -= t.O3;
    tt -= t.O4;
    df = (float)((double)gxv + opt * (double)tt);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    gxm = -tmom * tt;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    g05v = quad ? g05_q : (mid ? 0.f : df);
    gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
    gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
  };
  const std::true_type kYes{};
  const std::false_type kNo{};

  if (role == 0) {
    // ---------------------------------- step A ----------------------------------
    const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
    const float *const gci_p = gc_in + poff, *const gwxi_p = gwx_in + poff, *const gwyi_p = gwy_in + poff;
    const float *const xa_p = x05a + q0, *const xb_p = x05b + q0, *const b_p = b + q0, *const g_p = g05_in + q0;
    const float *const gxi_p = gxk + q0, *const gbi_p = gb_in + q0;
    auto load_row = [&](int k, Adj2wRow<C>& in) {
      const int kk = min(k, klast + 1);
      const int h = g.hs - 2 + kk;
      const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
      // what a row does not need is read from a row the strip needs anyway (no extra cache lines)
      const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
      const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
      const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xa[ch] = ldg(xa_p, off + chs[ch]);
        in.xb[ch] = ldg(xb_p, off + chs[ch]);
        in.bb[ch] = ldg(b_p, off + chs[ch]);
        in.g[ch] = ldg(g_p, off + chs[ch]);
        in.gx_i[ch] = ldg(gxi_p, off_a + chs[ch]);
        in.gb_i[ch] = ldg(gbi_p, off_o + chs[ch]);
      }
      in.gc_i = ldg(gci_p, off_o);
      in.gwx_i = ldg(gwxi_p, off_o);
      in.gwy_i = ldg(gwyi_p, off_o);
    };
    auto absorb = [&](int k, Adj2wRow<C>& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      o.rc1 = rcp_refined(1.f + o.c);
      o.opc_d = 1. + (double)o.c;
      o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xa = inside(o.xa[ch]), xb = inside(o.xb[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pa = prox_huber1(xa, o.c, o.rc1, bv), pb = prox_huber1(xb, o.c, o.rc1, bv);
          o.yA[ch] = pa + tA * (pa - pb);
        } else {
          o.yA[ch] = rebuild_y_fast(bv, xa, xb, o.c, o.rc1, o.opc_d, tA);
        }
        o.g[ch] = inside(o.g[ch]);
        o.xa[ch] = xa;
        o.xb[ch] = xb;
        o.bb[ch] = bv;
      }
    };
    float dA1[C], dA3[C], dA4[C];  // terms handed down to the row below
#pragma unroll
    for (int ch = 0; ch < C; ch++) dA1[ch] = dA3[ch] = dA4[ch] = 0.f;

    auto step = [&](int k, const Adj2wRow<C>& cur, const Adj2wRow<C>& nxt, auto do_a) {
      const int h = g.hs - 2 + k;
      const bool in_img = g.col_ok && h >= 0 && h < H;
      float (*slot)[64] = hand[k % (2 * kP)];
      float gcv = cur.gc_i, gwxv = cur.gwx_i, gwyv = cur.gwy_i;
      const float rc2A = rcp_refined((1.f + cur.c) * (1.f + cur.c));
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const Tri t = triangle(cur.yA[ch], nxt.yA[ch], cur.g[ch], nxt.g[ch], cur.wxs, cur.wys, kNo);
        const float a1_ = dA1[ch], a3_ = dA3[ch], a4_ = dA4[ch];
        dA1[ch] = t.O1; dA3[ch] = t.n3; dA4[ch] = t.n4;
        float nG = 0.f, ngxm = 0.f, ngb = cur.gb_i[ch];
        if (do_a.value) {
          if (g.w < W - 1) gwxv = gwxv - t.ux;
          if (h < H - 1) gwyv = gwyv - t.uy;
          float df, gxm, g05v, gc_add, gb_add;
          update(cur.g[ch], t, a1_, a3_, a4_, cur.gx_i[ch], optA, tA, cur.c, cur.rc1, rc2A, cur.opc_d, cur.bb[ch],
                 cur.xa[ch], df, gxm, g05v, gc_add, gb_add);
          gcv += gc_add;
          ngb += gb_add;
          nG = in_img ? g05v : 0.f;  // B reads zero padding outside the image
          ngxm = gxm;
        }
        slot[ch][g.lane] = nG;
        slot[C + ch][g.lane] = ngxm;
        slot[2 * C + ch][g.lane] = ngb;
        slot[3 * C + ch][g.lane] = cur.bb[ch];
        slot[4 * C + ch][g.lane] = cur.xb[ch];
      }
      slot[5 * C + 0][g.lane] = gcv;
      slot[5 * C + 1][g.lane] = gwxv;
      slot[5 * C + 2][g.lane] = gwyv;
      slot[5 * C + 3][g.lane] = cur.c;
      slot[5 * C + 4][g.lane] = cur.rc1;
      slot[5 * C + 5][g.lane] = cur.wxs;
      slot[5 * C + 6][g.lane] = cur.wys;
    };
    // the barrier after row k with k % kP == kP - 1 makes rows k-kP+1 .. k visible to step B
    auto publish = [&](int k) {
      if (k % kP == kP - 1) lds_barrier();
    };
    Adj2wRow<C> b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    absorb(0, b0);
    absorb(1, b1);
    step(0, b0, b1, kNo);
    load_row(3, b0);
    publish(0);
    for (int k = 1; k <= klast; k += 3) {  // cur / next rotate through (b1,b2) (b2,b0) (b0,b1)
      absorb(k + 1, b2);
      step(k, b1, b2, kYes);
      load_row(k + 3, b1);
      publish(k);
      if (k + 1 > klast) break;
      absorb(k + 2, b0);
      step(k + 1, b2, b0, kYes);
      load_row(k + 4, b2);
      publish(k + 1);
      if (k + 2 > klast) break;
      absorb(k + 3, b1);
      step(k + 2, b0, b1, kYes);
      load_row(k + 5, b0);
      publish(k + 2);
    }
    if (klast % kP != kP - 1) lds_barrier();  // the last rows have not been published yet
  } else {
    // ---------------------------------- step B ----------------------------------
    const float* const xc_p = x05c + q0;  // x05[j-2], or the checkpoint y when BEND
    float *const gco_p = gc + poff, *const gwxo_p = gwx + poff, *const gwyo_p = gwy + poff;
    float *const g05o_p = g05_out + q0, *const gxm_p = gxk_m1 + q0, *const gbo_p = gb + q0;
    float *const gxf_p = FINAL ? gx_final + q0 : nullptr;
    struct RowB {
      float xc[C];
    };
    auto load_row = [&](int k, RowB& in) {
      const int kk = min(k, klast + 1);
      const int h = g.hs - 2 + kk;
      const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
#pragma unroll
      for (int ch = 0; ch < C; ch++) in.xc[ch] = ldg(xc_p, off + chs[ch]);
    };
    const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form
    float dB1[C], dB3[C], dB4[C];
    // row k-1 as step B sees it
    float pG[C], pgxm[C], pyB[C], pxb[C], pbb[C], pgb[C], pgc = 0.f, pgwx = 0.f, pgwy = 0.f;
    float pc = 0.f, prc1 = 1.f, pwxs = 0.f, pwys = 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      dB1[ch] = dB3[ch] = dB4[ch] = 0.f;
      pG[ch] = pgxm[ch] = pyB[ch] = pxb[ch] = pbb[ch] = pgb[ch] = 0.f;
    }

    auto step = [&](int k, const RowB& in, auto tri_b, auto do_b) {
      const int h = g.hs - 2 + k;  // the row step A handed over; B's row is h - 1
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
      const float (*slot)[64] = hand[k % (2 * kP)];
      float nG[C], ngxm[C], ngb[C], bbv[C], xbv[C], yB[C];
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        nG[ch] = slot[ch][g.lane];
        ngxm[ch] = slot[C + ch][g.lane];
        ngb[ch] = slot[2 * C + ch][g.lane];
        bbv[ch] = slot[3 * C + ch][g.lane];
        xbv[ch] = slot[4 * C + ch][g.lane];
      }
      const float gcv = slot[5 * C + 0][g.lane], gwxv = slot[5 * C + 1][g.lane], gwyv = slot[5 * C + 2][g.lane];
      const float cc = slot[5 * C + 3][g.lane], rc1 = slot[5 * C + 4][g.lane];
      const float wxs = slot[5 * C + 5][g.lane], wys = slot[5 * C + 6][g.lane];
      const double opc_d = 1. + (double)cc;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {  // y of iteration j-1 on row k (the row below B's)
        const float xc = inside(in.xc[ch]);
        if (TRUE_ADJ) {
          const float pb = prox_huber1(xbv[ch], cc, rc1, bbv[ch]);
          const float pcv = BEND ? xc : prox_huber1(xc, cc, rc1, bbv[ch]);
          yB[ch] = pb + tB * (pb - pcv);
        } else {
          yB[ch] = BEND ? xc : rebuild_y_fast(bbv[ch], xbv[ch], xc, cc, rc1, opc_d, tB);
        }
      }
      if (tri_b.value) {
        float gcB = pgc, gwxB = pgwx, gwyB = pgwy;
        const float rc2B = rcp_refined((1.f + pc) * (1.f + pc));
        const double popc_d = 1. + (double)pc;
#pragma unroll
        for (int ch = 0; ch < C; ch++) {
          const Tri t = triangle(pyB[ch], yB[ch], pG[ch], nG[ch], pwxs, pwys, kBEnd);
          const float a1_ = dB1[ch], a3_ = dB3[ch], a4_ = dB4[ch];
          dB1[ch] = t.O1; dB3[ch] = t.n3; dB4[ch] = t.n4;
          if (do_b.value) {
            if (g.w < W - 1) gwxB = gwxB - t.ux;
            if (h - 1 < H - 1) gwyB = gwyB - t.uy;
            float df, gxm, g05v, gc_add, gb_add;
            update(pG[ch], t, a1_, a3_, a4_, pgxm[ch], optB, tB, pc, prc1, rc2B, popc_d, pbb[ch], pxb[ch], df, gxm, g05v,
                   gc_add, gb_add);
            gcB += gc_add;
            const float gbv = pgb[ch] + gb_add;
            if (store_lane) {
              if (FINAL) stg(gxf_p, roffB + chs[ch], df);
              stg(gxm_p, roffB + chs[ch], gxm);
              stg(g05o_p, roffB + chs[ch], g05v);
              if (BEND) {  // segment flush, fused (TV.cu:178-218)
                __builtin_nontemporal_store(gbv, &seg_gb[((size_t)g.n * Ct + ch) * HW + (roffB >> 2)]);
              } else {
                stg(gbo_p, roffB + chs[ch], gbv);
              }
            }
          }
        }
        if (do_b.value && store_lane) {
          if (BEND) {
            const size_t e = poff + (roffB >> 2);
            __builtin_nontemporal_store(gcB, &seg_gc[e]);
            __builtin_nontemporal_store(gwxB, &seg_gwx[e]);
            __builtin_nontemporal_store(gwyB, &seg_gwy[e]);
          } else {
            stg(gco_p, roffB, gcB);
            stg(gwxo_p, roffB, gwxB);
            stg(gwyo_p, roffB, gwyB);
          }
        }
      }
      pgc = gcv; pgwx = gwxv; pgwy = gwyv;
      pc = cc; prc1 = rc1; pwxs = wxs; pwys = wys;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        pG[ch] = nG[ch]; pgxm[ch] = ngxm[ch]; pgb[ch] = ngb[ch];
        pyB[ch] = yB[ch]; pxb[ch] = xbv[ch]; pbb[ch] = bbv[ch];
      }
    };
    // B waits before every row k with k % kP == 0 for the barrier that published rows k .. k+kP-1
    auto await = [&](int k) {
      if (k % kP == 0) lds_barrier();
    };
    RowB b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    await(0);
    step(0, b0, kNo, kNo);
    load_row(3, b0);
    await(1);
    step(1, b1, kNo, kNo);
    load_row(4, b1);
    await(2);
    step(2, b2, kYes, kNo);
    load_row(5, b2);
    for (int k = 3; k <= klast; k += 3) {
      await(k);
      step(k, b0, kYes, kYes);
      load_row(k + 3, b0);
      if (k + 1 > klast) break;
      await(k + 1);
      step(k + 1, b1, kYes, kYes);
      load_row(k + 4, b1);
      if (k + 2 > klast) break;
      await(k + 2);
      step(k + 2, b2, kYes, kYes);
      load_row(k + 5, b2);
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Two adjoint steps per launch for 5..8 channels: FOUR wavefronts per strip (256-thread workgroup).
// The channels are split into two groups (the first CM, the second C1 <= CM of them); wavefronts 0 and
// 1 run step A on group 0 and group 1, wavefronts 2 and 3 step B on group 0 and group 1, each as the
// matching half of tv_adjoint_strip2w.  The reference adds the terms of the three shared accumulators in
// the order A(ch 0 .. C-1), B(ch 0 .. C-1); here
//   A0 adds its terms to the accumulators read from memory and hands them on (LDS),
//   A1 adds its terms to what A0 handed on,
//   B0 does not touch the accumulators: it hands its terms on, one by one (gc term, ux, uy per channel),
//   B1 takes the accumulators after A1, adds B0's terms in channel order, then its own, and stores.
// Time runs in intervals of three rows with one LDS-only barrier between them: in interval t A0 works
// on rows 3t .. 3t+2, A1 and B0 on the three rows before, B1 on the three before those; every record
// is written in one interval and read in the next, so two sets of three row slots per record type
// suffice.  Every wavefront passes the same number of barriers (blocks + 2).
// -------------------------------------------------------------------------------------------------
template <int CM, int C1, bool BEND, bool FINAL, bool TRUE_ADJ = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void tv_adjoint_strip4w(
    const float* __restrict__ wx, const float* __restrict__ wy, const float* __restrict__ cf,
    const float* __restrict__ b, const float* __restrict__ x05a, const float* __restrict__ x05b,
    const float* __restrict__ x05c, const float* __restrict__ gc_in, float* __restrict__ gc,
    const float* __restrict__ gb_in, float* __restrict__ gb, const float* __restrict__ gwx_in,
    float* __restrict__ gwx, const float* __restrict__ gwy_in, float* __restrict__ gwy,
    const float* __restrict__ g05_in, float* __restrict__ g05_out, const float* __restrict__ gxk,
    float* __restrict__ gxk_m1, float* __restrict__ gx_final, float* __restrict__ seg_gc,
    float* __restrict__ seg_gb, float* __restrict__ seg_gwx, float* __restrict__ seg_gwy, int N, int H, int W,
    float tA, float tB, int R, int strips_x, int strips_y, int Ct) {
  static_assert(C1 >= 1 && C1 <= CM, "the second group is the smaller one");
  constexpr int kSlots = 6;                     // two sets of three rows
  __shared__ float handA[2][kSlots][3 * CM + 3][64];  // per group: g05[j], partial g_x[j], gb per channel; the accumulators
  __shared__ float handT[kSlots][3 * CM][64];         // B0's terms: gc term, ux, uy per channel
  StripGeom g;
  if (!strip_geometry_block(g, kFwd2Cols, R, W, strips_x, strips_y, N, 2)) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int Reff = min(R, H - g.hs);
  const int klast = Reff + 2;  // strip row k is image row hs - 2 + k
  const int nblocks = (klast + 3) / 3;
  const size_t HW = (size_t)H * W;
  const unsigned W4 = 4u * (unsigned)W;
  const unsigned wc = g.col_ok ? 4u * g.w : 0u;
  const bool store_lane = g.lane > 1 && g.lane < 62 && g.col_ok;
  const bool wx_ok = g.col_ok && g.w < W - 1;
  const double optA = 1. + (double)tA, optB = 1. + (double)tB;
  const size_t poff = (size_t)g.n * HW;
  const unsigned plane4 = 4u * (unsigned)HW;  // bytes from one channel to the next
  const int h_lo = max(g.hs - 1, 0), h_hi = min(g.hs + Reff, H - 1);  // rows A updates
  const int o_lo = g.hs, o_hi = g.hs + Reff - 1;                       // output rows

  constexpr float kGX = TRUE_ADJ ? 1.f : kLocalGXMult, kGC = TRUE_ADJ ? 1.f : kLocalGCMult;
  struct Tri {  // everything one triangle contributes (see tv_adjoint_strip)
    float O1, O2, O3, O4, n3, n4, l1, l3, l4, ux, uy;
  };
  auto triangle = [&](float yk, float yd, float gk, float gd, float wxv, float wyv, auto end_form) {
    Tri r;
    const float yrt = from_right_lane(yk);
    const float grt = from_right_lane(gk);
    const float d1 = yk - yd, d2 = yk - yrt;
    const float a1 = d1 * d1 * wyv;
    const float a2 = d2 * d2 * wxv;
    const float hub = exact_sqrt(a2 + a1);
    const bool act = hub > kDelta;
    float nom = inpaint::exact_div(kDelta, hub);
    float denom = inpaint::exact_div(nom, 2.f * hub * hub);
    nom = act ? nom : 1.f;
    denom = act ? denom : 0.f;
    const float gpd = gk - gd, gpr = gk - grt;
    r.O1 = gpd * (wyv * nom);
    r.O2 = gpr * (wxv * nom);
    const float P1 = gpd * wyv * d1;
    const float P2 = gpr * wxv * d2;
    const float dd = denom * 2.0f;
    const float tp = dd * (d1 * wyv + d2 * wxv);  // minus the reference's factor, exactly; O3, O4 carry the sign
    const float tu = dd * d1 * wyv;
    const float tl = dd * d2 * wxv;
    r.O3 = -(P1 * tp);
    r.O4 = -(P2 * tp);
    r.n3 = P1 * tu;
    r.n4 = P2 * tu;
    r.l1 = from_left_lane(r.O2);
    r.l3 = from_left_lane(P2 * tl);
    r.l4 = from_left_lane(P1 * tl);
    if (!end_form.value) {  // TV.cu:749-769
      r.ux = kGX * d2 * (gpr * (nom - a2 * denom) - gpd * d2 * d1 * denom * wyv);
      r.uy = kGX * d1 * (gpd * (nom - a1 * denom) - gpr * d1 * d2 * denom * wxv);
    } else {  // TV.cu:1019-1037
      const float ux_a = kGX * (gpr * d2 * (nom - a2 * denom) - gpd * d2 * d2 * d1 * denom * wyv);
      const float uy_a = kGX * (gpd * d1 * (nom - a1 * denom) - gpr * d1 * d1 * d2 * denom * wxv);
      r.ux = act ? ux_a : kGX * d2 * gpr;
      r.uy = act ? uy_a : kGX * d1 * gpd;
    }
    return r;
  };
  // pixel update: J^T assembly, momentum adjoint, prox adjoint (TV.cu:668-743, 796-828)
  auto update = [&](float gk, const Tri& t, float a1_, float a3_, float a4_, float gxv, double opt, float tmom,
                    float conf, float rc1, float rc2, double opc_d, float bv, float xh, float& df, float& gxm,
                    float& g05v, float& gc_add, float& gb_add) {
    float tt = gk;
    tt -= -a1_;
    tt -= a3_;
    tt -= a4_;
    tt -= -t.l1;
    tt -= t.l3;
    tt -= t.l4;
    tt -= t.O1;
    tt -= t.O2;
    tt -= t.O3;
    tt -= t.O4;
    df = (float)((double)gxv + opt * (double)tt);
    df = fmaxf(-kClipLocalGrad, fminf(df, kClipLocalGrad));
    gxm = -tmom * tt;
    const float diff = bv - xh;
    const float sign = (diff < 0) ? -1.f : 1.f;
    const bool quad = (opc_d >= (double)(sign * diff));
    const float opc = 1.f + conf;
    const float gc_q = df * (div_by(bv, opc, rc1) - div_by(conf * bv + xh, opc * opc, rc2)) * kGC;
    const float g05_q = div_by(df, opc, rc1);
    const float gb_q = div_by(df * conf, opc, rc1) * 1.0f;
    const bool mid = !quad && (conf >= sign * diff);
    g05v = quad ? g05_q : (mid ? 0.f : df);
    gc_add = quad ? gc_q : (mid ? 0.f : sign * df * kGC);
    gb_add = quad ? gb_q : (mid ? df * 1.0f : 0.f);
  };
  const std::true_type kYes{};
  const std::false_type kNo{};

  // ------------------------------------------ step A on one group ------------------------------------------
  auto role_a = [&](auto channels, auto group) {
    constexpr int C = decltype(channels)::value, G = decltype(group)::value;
    const size_t q0 = ((size_t)g.n * Ct + (G ? CM : 0)) * HW;  // the group's first channel; channel ch plane4 * ch bytes further
    const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
    const float *const gci_p = gc_in + poff, *const gwxi_p = gwx_in + poff, *const gwyi_p = gwy_in + poff;
    const float *const xa_p = x05a + q0, *const xb_p = x05b + q0, *const b_p = b + q0, *const g_p = g05_in + q0;
    const float *const gxi_p = gxk + q0, *const gbi_p = gb_in + q0;
    struct Row {
      float c, rc1, wxs, wys;
      float xa[C], xb[C], yA[C], bb[C], g[C], gx_i[C], gb_i[C], gc_i, gwx_i, gwy_i;
      double opc_d;
    };
    auto load_row = [&](int k, Row& in) {
      const int kk = min(k, klast + 1);
      const int h = g.hs - 2 + kk;
      const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
      const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
      const unsigned off_a = (unsigned)min(max(h, h_lo), h_hi) * W4 + wc;
      const unsigned off_o = (unsigned)min(max(h, o_lo), o_hi) * W4 + wc;
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xa[ch] = ldg(xa_p, off + plane4 * ch);
        in.xb[ch] = ldg(xb_p, off + plane4 * ch);
        in.bb[ch] = ldg(b_p, off + plane4 * ch);
        in.g[ch] = ldg(g_p, off + plane4 * ch);
        in.gx_i[ch] = ldg(gxi_p, off_a + plane4 * ch);
        in.gb_i[ch] = ldg(gbi_p, off_o + plane4 * ch);
      }
      if (G == 0) {  // the second group continues the first group's sums
        in.gc_i = ldg(gci_p, off_o);
        in.gwx_i = ldg(gwxi_p, off_o);
        in.gwy_i = ldg(gwyi_p, off_o);
      } else {
        in.gc_i = in.gwx_i = in.gwy_i = 0.f;
      }
    };
    auto absorb = [&](int k, Row& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      o.rc1 = rcp_refined(1.f + o.c);
      o.opc_d = 1. + (double)o.c;
      o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xa = inside(o.xa[ch]), xb = inside(o.xb[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pa = prox_huber1(xa, o.c, o.rc1, bv), pb = prox_huber1(xb, o.c, o.rc1, bv);
          o.yA[ch] = pa + tA * (pa - pb);
        } else {
          o.yA[ch] = rebuild_y_fast(bv, xa, xb, o.c, o.rc1, o.opc_d, tA);
        }
        o.g[ch] = inside(o.g[ch]);
        o.xa[ch] = xa;
        o.bb[ch] = bv;
      }
    };
    float dA1[C], dA3[C], dA4[C];  // terms handed down to the row below
#pragma unroll
    for (int ch = 0; ch < C; ch++) dA1[ch] = dA3[ch] = dA4[ch] = 0.f;

    auto step = [&](int k, const Row& cur, const Row& nxt, auto do_a) {
      const int h = g.hs - 2 + k;
      const bool in_img = g.col_ok && h >= 0 && h < H;
      float (*slot)[64] = handA[G][k % kSlots];
      float gcv, gwxv, gwyv;
      if (G == 0) {
        gcv = cur.gc_i; gwxv = cur.gwx_i; gwyv = cur.gwy_i;
      } else {  // what the first group made of the row's accumulators, one interval ago
        const float (*prev)[64] = handA[0][k % kSlots];
        gcv = prev[3 * CM + 0][g.lane]; gwxv = prev[3 * CM + 1][g.lane]; gwyv = prev[3 * CM + 2][g.lane];
      }
      const float rc2A = rcp_refined((1.f + cur.c) * (1.f + cur.c));
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const Tri t = triangle(cur.yA[ch], nxt.yA[ch], cur.g[ch], nxt.g[ch], cur.wxs, cur.wys, kNo);
        const float a1_ = dA1[ch], a3_ = dA3[ch], a4_ = dA4[ch];
        dA1[ch] = t.O1; dA3[ch] = t.n3; dA4[ch] = t.n4;
        float nG = 0.f, ngxm = 0.f, ngb = cur.gb_i[ch];
        if (do_a.value) {
          if (g.w < W - 1) gwxv = gwxv - t.ux;
          if (h < H - 1) gwyv = gwyv - t.uy;
          float df, gxm, g05v, gc_add, gb_add;
          update(cur.g[ch], t, a1_, a3_, a4_, cur.gx_i[ch], optA, tA, cur.c, cur.rc1, rc2A, cur.opc_d, cur.bb[ch],
                 cur.xa[ch], df, gxm, g05v, gc_add, gb_add);
          gcv += gc_add;
          ngb += gb_add;
          nG = in_img ? g05v : 0.f;  // B reads zero padding outside the image
          ngxm = gxm;
        }
        slot[ch][g.lane] = nG;
        slot[CM + ch][g.lane] = ngxm;
        slot[2 * CM + ch][g.lane] = ngb;
      }
      slot[3 * CM + 0][g.lane] = gcv;
      slot[3 * CM + 1][g.lane] = gwxv;
      slot[3 * CM + 2][g.lane] = gwyv;
    };
    Row b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    for (int t = 0; t < G; t++) lds_barrier();  // group 1 works one interval behind group 0
    absorb(0, b0);
    absorb(1, b1);
    step(0, b0, b1, kNo);
    load_row(3, b0);
    absorb(2, b2);
    step(1, b1, b2, kYes);
    load_row(4, b1);
    absorb(3, b0);
    step(2, b2, b0, kYes);
    load_row(5, b2);
    lds_barrier();
    for (int blk = 1; blk < nblocks; blk++) {  // b0 holds row k (absorbed), b1 and b2 rows k+1, k+2 (loaded)
      const int k = 3 * blk;
      absorb(k + 1, b1);
      step(k, b0, b1, kYes);
      load_row(k + 3, b0);
      if (k + 1 <= klast) {
        absorb(k + 2, b2);
        step(k + 1, b1, b2, kYes);
        load_row(k + 4, b1);
      }
      if (k + 2 <= klast) {
        absorb(k + 3, b0);
        step(k + 2, b2, b0, kYes);
        load_row(k + 5, b2);
      }
      lds_barrier();
    }
    for (int t = G; t < 2; t++) lds_barrier();  // the intervals in which only the wavefronts behind still work
  };

  // ------------------------------------------ step B on one group ------------------------------------------
  auto role_b = [&](auto channels, auto group) {
    constexpr int C = decltype(channels)::value, G = decltype(group)::value;
    const size_t q0 = ((size_t)g.n * Ct + (G ? CM : 0)) * HW;
    const int ch0 = G ? CM : 0;
    const float *const wx_p = wx + poff, *const wy_p = wy + poff, *const cf_p = cf + poff;
    const float *const xb_p = x05b + q0, *const xc_p = x05c + q0, *const b_p = b + q0;  // x05c: x05[j-2], or the checkpoint y when BEND
    float *const gco_p = gc + poff, *const gwxo_p = gwx + poff, *const gwyo_p = gwy + poff;
    float *const g05o_p = g05_out + q0, *const gxm_p = gxk_m1 + q0, *const gbo_p = gb + q0;
    float *const gxf_p = FINAL ? gx_final + q0 : nullptr;
    struct Row {
      float c, rc1, wxs, wys;
      float xb[C], yB[C], bb[C];  // yB is loaded as x05[j-2] (or the checkpoint y) and rebuilt in place
    };
    auto load_row = [&](int k, Row& in) {
      const int kk = min(k, klast + 1);
      const int h = g.hs - 2 + kk;
      const unsigned off = (unsigned)(h < 0 ? 0 : (h >= H ? H - 1 : h)) * W4 + wc;
      const unsigned off_w = (unsigned)min(max(h, 0), h_hi) * W4 + wc;
      in.c = ldg(cf_p, off);
      in.wxs = ldg(wx_p, off_w);
      in.wys = ldg(wy_p, off_w);
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        in.xb[ch] = ldg(xb_p, off + plane4 * ch);
        in.yB[ch] = ldg(xc_p, off + plane4 * ch);
        in.bb[ch] = ldg(b_p, off + plane4 * ch);
      }
    };
    auto absorb = [&](int k, Row& o) {
      const int h = g.hs - 2 + k;
      const bool ok = g.col_ok && h >= 0 && h < H;
      const inpaint::LaneMask inside(ok);
      o.c = inside(o.c);
      o.rc1 = rcp_refined(1.f + o.c);
      const double opc_d = 1. + (double)o.c;
      o.wxs = (ok && wx_ok) ? kL * o.wxs : 0.f;
      o.wys = (ok && h < H - 1) ? kL * o.wys : 0.f;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        const float xb = inside(o.xb[ch]), xc = inside(o.yB[ch]), bv = inside(o.bb[ch]);
        if (TRUE_ADJ) {
          const float pb = prox_huber1(xb, o.c, o.rc1, bv);
          const float pcv = BEND ? xc : prox_huber1(xc, o.c, o.rc1, bv);
          o.yB[ch] = pb + tB * (pb - pcv);
        } else {
          o.yB[ch] = BEND ? xc : rebuild_y_fast(bv, xb, xc, o.c, o.rc1, opc_d, tB);
        }
        o.xb[ch] = xb;
        o.bb[ch] = bv;
      }
    };
    const std::integral_constant<bool, BEND && !TRUE_ADJ> kBEnd{};  // the corrected gradient has one arithmetic form
    float dB1[C], dB3[C], dB4[C];
    // row k-1 as step B sees it
    float pG[C], pgxm[C], pyB[C], pxb[C], pbb[C], pgb[C], pgc = 0.f, pgwx = 0.f, pgwy = 0.f;
    float pc = 0.f, prc1 = 1.f, pwxs = 0.f, pwys = 0.f;
#pragma unroll
    for (int ch = 0; ch < C; ch++) {
      dB1[ch] = dB3[ch] = dB4[ch] = 0.f;
      pG[ch] = pgxm[ch] = pyB[ch] = pxb[ch] = pbb[ch] = pgb[ch] = 0.f;
    }

    auto step = [&](int k, const Row& cur, auto tri_b, auto do_b) {
      const int h = g.hs - 2 + k;  // the row step A handed over; B's row is h - 1
      const unsigned roffB = (unsigned)max(h - 1, 0) * W4 + wc;
      const float (*slot)[64] = handA[G][k % kSlots];
      float (*terms)[64] = handT[k % kSlots];
      float nG[C], ngxm[C], ngb[C];
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        nG[ch] = slot[ch][g.lane];
        ngxm[ch] = slot[CM + ch][g.lane];
        ngb[ch] = slot[2 * CM + ch][g.lane];
      }
      float gcv = 0.f, gwxv = 0.f, gwyv = 0.f;
      if (G == 1) {  // the row's accumulators with every A term added
        gcv = slot[3 * CM + 0][g.lane]; gwxv = slot[3 * CM + 1][g.lane]; gwyv = slot[3 * CM + 2][g.lane];
      }
      if (tri_b.value) {
        float gcB = pgc, gwxB = pgwx, gwyB = pgwy;
        if (G == 1 && do_b.value) {  // the first group's B terms, in channel order, before this group's
#pragma unroll
          for (int ch = 0; ch < CM; ch++) {
            if (g.w < W - 1) gwxB = gwxB - terms[CM + ch][g.lane];
            if (h - 1 < H - 1) gwyB = gwyB - terms[2 * CM + ch][g.lane];
            gcB += terms[ch][g.lane];
          }
        }
        const float rc2B = rcp_refined((1.f + pc) * (1.f + pc));
        const double popc_d = 1. + (double)pc;
#pragma unroll
        for (int ch = 0; ch < C; ch++) {
          const Tri t = triangle(pyB[ch], cur.yB[ch], pG[ch], nG[ch], pwxs, pwys, kBEnd);
          const float a1_ = dB1[ch], a3_ = dB3[ch], a4_ = dB4[ch];
          dB1[ch] = t.O1; dB3[ch] = t.n3; dB4[ch] = t.n4;
          if (do_b.value) {
            float df, gxm, g05v, gc_add, gb_add;
            update(pG[ch], t, a1_, a3_, a4_, pgxm[ch], optB, tB, pc, prc1, rc2B, popc_d, pbb[ch], pxb[ch], df, gxm, g05v,
                   gc_add, gb_add);
            if (G == 0) {
              terms[ch][g.lane] = gc_add;
              terms[CM + ch][g.lane] = t.ux;
              terms[2 * CM + ch][g.lane] = t.uy;
            } else {
              if (g.w < W - 1) gwxB = gwxB - t.ux;
              if (h - 1 < H - 1) gwyB = gwyB - t.uy;
              gcB += gc_add;
            }
            const float gbv = pgb[ch] + gb_add;
            if (store_lane) {
              if (FINAL) stg(gxf_p, roffB + plane4 * ch, df);
              stg(gxm_p, roffB + plane4 * ch, gxm);
              stg(g05o_p, roffB + plane4 * ch, g05v);
              if (BEND) {  // segment flush, fused (TV.cu:178-218)
                __builtin_nontemporal_store(gbv, &seg_gb[((size_t)g.n * Ct + ch0 + ch) * HW + (roffB >> 2)]);
              } else {
                stg(gbo_p, roffB + plane4 * ch, gbv);
              }
            }
          }
        }
        if (G == 1 && do_b.value && store_lane) {
          if (BEND) {
            const size_t e = poff + (roffB >> 2);
            __builtin_nontemporal_store(gcB, &seg_gc[e]);
            __builtin_nontemporal_store(gwxB, &seg_gwx[e]);
            __builtin_nontemporal_store(gwyB, &seg_gwy[e]);
          } else {
            stg(gco_p, roffB, gcB);
            stg(gwxo_p, roffB, gwxB);
            stg(gwyo_p, roffB, gwyB);
          }
        }
      }
      pgc = gcv; pgwx = gwxv; pgwy = gwyv;
      pc = cur.c; prc1 = cur.rc1; pwxs = cur.wxs; pwys = cur.wys;
#pragma unroll
      for (int ch = 0; ch < C; ch++) {
        pG[ch] = nG[ch]; pgxm[ch] = ngxm[ch]; pgb[ch] = ngb[ch];
        pyB[ch] = cur.yB[ch]; pxb[ch] = cur.xb[ch]; pbb[ch] = cur.bb[ch];
      }
    };
    Row b0, b1, b2;
    load_row(0, b0);
    load_row(1, b1);
    load_row(2, b2);
    for (int t = 0; t < 1 + G; t++) lds_barrier();  // one interval behind the group's step A
    absorb(0, b0);
    step(0, b0, kNo, kNo);
    load_row(3, b0);
    absorb(1, b1);
    step(1, b1, kNo, kNo);
    load_row(4, b1);
    absorb(2, b2);
    step(2, b2, kYes, kNo);
    load_row(5, b2);
    lds_barrier();
    for (int blk = 1; blk < nblocks; blk++) {  // b0, b1, b2 hold rows k, k+1, k+2 (loaded)
      const int k = 3 * blk;
      absorb(k, b0);
      step(k, b0, kYes, kYes);
      load_row(k + 3, b0);
      if (k + 1 <= klast) {
        absorb(k + 1, b1);
        step(k + 1, b1, kYes, kYes);
        load_row(k + 4, b1);
      }
      if (k + 2 <= klast) {
        absorb(k + 2, b2);
        step(k + 2, b2, kYes, kYes);
        load_row(k + 5, b2);
      }
      lds_barrier();
    }
    for (int t = 1 + G; t < 2; t++) lds_barrier();
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

}  // namespace tvstrip
