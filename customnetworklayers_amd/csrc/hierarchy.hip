// Glue between two levels of a coarse-to-fine hierarchy of inpainting layers for MI355X (gfx950):
// scaled bilinear x2 upsampling of the coarse solution (right-hand side and starting point of the
// fine level), the fine level's edge weights from its guidance image, and the adjoint of the
// upsampling.  C ABI in include/hierarchy.h.  Pointwise / small-stencil work, bound by HBM: every
// value is read once from memory (the overlapping stencil reads hit the vector L1) and written once.
//
// Arithmetic: the upsampling and its adjoint keep one fixed operation order (no contraction), so
// they are reproducible bit for bit by a plain C++ loop; so are the edge weights (own exp, see exp_nonpos).
#include <hip/hip_runtime.h>

#include "../../include/hierarchy.h"
#include "inpaint_common.h"

namespace {

using inpaint::fail;

// taps of fine index `dst` along one axis of coarse size `size`: source coordinate (dst + 0.5) / 2 - 0.5
// clamped at 0, right neighbour clamped at the border (all values are multiples of 1/4: exact)
__device__ __forceinline__ void axis_taps(int dst, int size, int& i0, int& i1, float& l0, float& l1) {
  float src = ((float)dst + 0.5f) * 0.5f - 0.5f;
  if (src < 0.f) src = 0.f;
  i0 = (int)src;
  i1 = min(i0 + 1, size - 1);
  l1 = src - (float)i0;
  l0 = 1.f - l1;
}

// exp(x) for x <= 0 with a fixed sequence of IEEE operations (Cody-Waite reduction by ln 2, degree-7 Taylor
// polynomial in Horner form, exact scaling): the same bits on the device and in a host evaluation of the same
// lines, about 1 ulp from the true value.  A one-ulp difference in an edge weight is enough to flip Huber
// switches in the layer that consumes it, so the library's expf (whose last bit is implementation defined) is
// not used.
__device__ __forceinline__ float exp_nonpos(float x) {
  if (!(x > -87.0f)) return 0.0f;
  const float n = rintf(x * 1.44269504f);
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
  return ldexpf(p, (int)n);
}

// one lane per pair of fine pixels (2 cx, 2 cx + 1) of one fine row: 8-byte stores, all channels
__global__ __launch_bounds__(256) void next_level_forward_kernel(const float* __restrict__ sol, const float* __restrict__ img,
                                                                 float* __restrict__ up, float* __restrict__ wx,
                                                                 float* __restrict__ wy, int N, int C, int H, int W,
                                                                 float scale, float alpha) {
  const int H2 = 2 * H, W2 = 2 * W;
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)N * H2 * W) return;
  const int cx = (int)(t % W);
  const int y = (int)((t / W) % H2);
  const int n = (int)(t / ((long long)W * H2));
  int y0, y1, xa0, xa1, xb0, xb1;
  float h0, h1, wa0, wa1, wb0, wb1;
  axis_taps(y, H, y0, y1, h0, h1);
  axis_taps(2 * cx, W, xa0, xa1, wa0, wa1);
  axis_taps(2 * cx + 1, W, xb0, xb1, wb0, wb1);
  for (int c = 0; c < C; c++) {
    const float* a = sol + ((size_t)n * C + c) * H * W;
    const float* r0 = a + (size_t)y0 * W;
    const float* r1 = a + (size_t)y1 * W;
    const float va = h0 * (wa0 * r0[xa0] + wa1 * r0[xa1]) + h1 * (wa0 * r1[xa0] + wa1 * r1[xa1]);
    const float vb = h0 * (wb0 * r0[xb0] + wb1 * r0[xb1]) + h1 * (wb0 * r1[xb0] + wb1 * r1[xb1]);
    float2 o;
    o.x = scale * va;
    o.y = scale * vb;
    *reinterpret_cast<float2*>(up + ((size_t)n * C + c) * H2 * W2 + (size_t)y * W2 + 2 * cx) = o;
  }
  if (img) {
    const float* I = img + (size_t)n * H2 * W2;
    const size_t p = (size_t)y * W2 + 2 * cx;
    const float i0 = I[p], i1 = I[p + 1];
    float2 ox, oy;
    ox.x = exp_nonpos(-alpha * fabsf(i1 - i0));
    ox.y = 2 * cx + 2 < W2 ? exp_nonpos(-alpha * fabsf(I[p + 2] - i1)) : 1.f;
    oy.x = y + 1 < H2 ? exp_nonpos(-alpha * fabsf(I[p + W2] - i0)) : 1.f;
    oy.y = y + 1 < H2 ? exp_nonpos(-alpha * fabsf(I[p + W2 + 1] - i1)) : 1.f;
    *reinterpret_cast<float2*>(wx + (size_t)n * H2 * W2 + p) = ox;
    *reinterpret_cast<float2*>(wy + (size_t)n * H2 * W2 + p) = oy;
  }
}

// one lane per coarse pixel: the fine pixels it was a tap of, rows then columns ascending
__global__ __launch_bounds__(256) void next_level_backward_kernel(const float* __restrict__ ga, const float* __restrict__ gb,
                                                                  float* __restrict__ out, int N, int C, int H, int W,
                                                                  float scale) {
  const int H2 = 2 * H, W2 = 2 * W;
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)N * H * W) return;
  const int cx = (int)(t % W);
  const int cy = (int)((t / W) % H);
  const int n = (int)(t / ((long long)W * H));
  const int ylo = max(2 * cy - 1, 0), xlo = max(2 * cx - 1, 0);
  float wyv[4], wxv[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    int i0, i1;
    float l0, l1;
    wyv[k] = 0.f;
    wxv[k] = 0.f;
    const int y = ylo + k, x = xlo + k;
    if (y <= min(2 * cy + 2, H2 - 1)) {
      axis_taps(y, H, i0, i1, l0, l1);
      if (i0 == cy) wyv[k] += l0;
      if (i1 == cy) wyv[k] += l1;
    }
    if (x <= min(2 * cx + 2, W2 - 1)) {
      axis_taps(x, W, i0, i1, l0, l1);
      if (i0 == cx) wxv[k] += l0;
      if (i1 == cx) wxv[k] += l1;
    }
  }
  for (int c = 0; c < C; c++) {
    const size_t plane = ((size_t)n * C + c) * H2 * W2;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (wyv[j] == 0.f) continue;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        if (wxv[k] == 0.f) continue;
        const size_t p = plane + (size_t)(ylo + j) * W2 + xlo + k;
        float g = ga[p];
        if (gb) g = g + gb[p];
        acc += (wyv[j] * wxv[k]) * g;
      }
    }
    out[((size_t)n * C + c) * H * W + (size_t)cy * W + cx] = scale * acc;
  }
}

}  // namespace

extern "C" {

const char* hierarchy_last_error(void) { return inpaint::error_buffer(); }

int hierarchy_next_level_forward(const float* sol, const float* img, float* up, float* wx, float* wy, int n, int c, int h,
                                 int w, float scale, float alpha, void* stream) {
  if (!sol || !up) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_forward: null pointer");
  if (img && (!wx || !wy)) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_forward: an image needs both weight outputs");
  if (n < 1 || c < 1 || h < 1 || w < 1) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_forward: bad shape %dx%dx%dx%d", n, c, h, w);
  if (h > 16383 || w > 16383) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_forward: level too large");
  if (((uintptr_t)up & 7) || (img && (((uintptr_t)wx & 7) || ((uintptr_t)wy & 7))))
    return fail(INPAINT_ERR_ARG, "hierarchy_next_level_forward: outputs must be 8-byte aligned");
  const long long total = (long long)n * 2 * h * w;
  hipLaunchKernelGGL(next_level_forward_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, sol, img,
                     up, wx, wy, n, c, h, w, scale, alpha);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

int hierarchy_next_level_backward(const float* g_b, const float* g_init, float* g_sol, int n, int c, int h, int w, float scale,
                                  void* stream) {
  if (!g_b || !g_sol) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_backward: null pointer");
  if (n < 1 || c < 1 || h < 1 || w < 1) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_backward: bad shape %dx%dx%dx%d", n, c, h, w);
  if (h > 16383 || w > 16383) return fail(INPAINT_ERR_ARG, "hierarchy_next_level_backward: level too large");
  const long long total = (long long)n * h * w;
  hipLaunchKernelGGL(next_level_backward_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, g_b,
                     g_init, g_sol, n, c, h, w, scale);
  INPAINT_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
