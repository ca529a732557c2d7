// On-device check of the cheap correctly-rounded division / square root against the compiler's
// IEEE expansions.  Diagnostic entry point of the library, used by the GPU test-suite.
#include "exact_math.h"
#include "inpaint_common.h"
#include "tgv_strip_kernels.h"

namespace {

using namespace inpaint;

__device__ inline bool same_bits(float a, float b) {
  return (__float_as_uint(a) == __float_as_uint(b)) || (a != a && b != b);
}

__device__ inline unsigned int mix(unsigned int x) {  // integer hash, good enough to spread operands
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// counts[0]: sqrt over 0 and every finite float in [2^-96, FLT_MAX]
// counts[1]: div_by_tenth(x) against x / 0.1f over 0 and every float in [2^-96, 2^96]
// counts[2]: n / d on hashed pairs, d in [2^-6, 2^40), |n| in [2^-60, 2^60) or 0, plus structured
//            denominators (all-ones and single-bit mantissas)
// counts[3]: shared-reciprocal form, two numerators per denominator in [1, 2^24)
__global__ __launch_bounds__(256) void selftest_kernel(unsigned long long* counts, unsigned int pair_rounds) {
  const unsigned int tid = blockIdx.x * blockDim.x + threadIdx.x;
  const unsigned int stride = gridDim.x * blockDim.x;
  unsigned int bad0 = 0, bad1 = 0, bad2 = 0, bad3 = 0;
  for (unsigned long long i = tid; i < 0x7f800000ULL; i += stride) {
    const float x = __uint_as_float((unsigned int)i);
    if (x == 0.f || x >= 1.2621774e-29f) bad0 += !same_bits(exact_sqrt(x), sqrtf(x));
    if (x == 0.f || (x >= 1.2621774e-29f && x <= 7.9228163e28f)) bad1 += !same_bits(div_by_tenth(x), x / 0.1f);
  }
  for (unsigned int k = 0; k < pair_rounds; k++) {
    const unsigned int h1 = mix(tid * 2654435761U + k * 40503U + 17U), h2 = mix(h1 ^ 0x9e3779b9U);
    // denominator: exponent in [-6, 40), mantissa hashed / structured
    unsigned int mant = h1 & 0x7fffffU;
    if ((k & 7) == 1) mant = 0x7fffffU;
    if ((k & 7) == 2) mant = 1U << (h1 % 23U);
    if ((k & 7) == 3) mant = 0x7fffffU ^ (1U << (h1 % 23U));
    const unsigned int dexp = 127U - 6U + ((h1 >> 23) % 46U);
    const float d = __uint_as_float((dexp << 23) | mant);
    const unsigned int nexp = 127U - 60U + ((h2 >> 23) % 120U);
    float n = __uint_as_float((h2 & 0x80000000U) | (nexp << 23) | (h2 & 0x7fffffU));
    if ((k & 63) == 5) n = 0.f;
    bad2 += !same_bits(exact_div(n, d), n / d);
    const float d1 = __uint_as_float(((127U + ((h1 >> 23) % 24U)) << 23) | mant);
    const float r = rcp_refined(d1);
    const float n2 = __uint_as_float(((127U - 20U + ((h2 >> 8) % 24U)) << 23) | (h1 & 0x7fffffU));
    bad3 += !same_bits(div_by(n, d1, r), n / d1);
    bad3 += !same_bits(div_by(n2, d1, r), n2 / d1);
  }
  if (bad0) atomicAdd(&counts[0], (unsigned long long)bad0);
  if (bad1) atomicAdd(&counts[1], (unsigned long long)bad1);
  if (bad2) atomicAdd(&counts[2], (unsigned long long)bad2);
  if (bad3) atomicAdd(&counts[3], (unsigned long long)bad3);
}

// counts[0]: rsq_exact(x) against 1.0f / sqrtf(x) over 0 and every float in [2^-96, 2^96]; and every float up to
//            kHuberQuiet has Huber weight 1 in both forms
// counts[1]: div_by_fifth(x) against x / 0.2f over the same set (the TGV layer's Huber threshold)
// counts[2]: exact_rcp(m) against 1 / m over every float m in [2^-40, 2^40): the reciprocal that every division starts
//            from, and the segment-start kernel's Huber weight
// counts[3]: w / h2 on hashed pairs, w in (2^-20, 1], h2 in [2^-14, 2^6): its weight derivative
__global__ __launch_bounds__(256) void selftest_rsqrt_kernel(unsigned long long* counts, unsigned int pair_rounds) {
  const unsigned int tid = blockIdx.x * blockDim.x + threadIdx.x;
  const unsigned int stride = gridDim.x * blockDim.x;
  unsigned int bad0 = 0, bad1 = 0, bad2 = 0, bad3 = 0;
  for (unsigned long long i = tid; i < 0x7f800000ULL; i += stride) {
    const float x = __uint_as_float((unsigned int)i);
    if (x == 0.f || (x >= 1.2621774e-29f && x <= 7.9228163e28f)) {
      bad0 += !same_bits(tgvstrip::rsq_exact(x), 1.0f / sqrtf(x));
      bad1 += !same_bits(div_by_fifth(x), x / 0.2f);
    }
    if (x >= 9.094947e-13f && x < 1.0995116e12f) bad2 += !same_bits(exact_rcp(x), 1.0f / x);
    // a Huber argument up to kHuberQuiet has weight exactly 1 and an inactive term, in both arithmetic forms: what the
    // strip kernels assume when a whole wavefront skips the square root
    if (x <= tgvstrip::kHuberQuiet) {
      const float root = exact_sqrt(x);
      bad0 += tgvstrip::huber_w_full(x, 0.2f) != 1.0f;
      bad0 += root > 0.2f || exact_rcp(fmaxf(1.f, div_by_fifth(root))) != 1.0f;
    }
  }
  for (unsigned int k = 0; k < pair_rounds; k++) {
    const unsigned int h1 = mix(tid * 2654435761U + k * 40503U + 29U), h2 = mix(h1 ^ 0x9e3779b9U);
    const float w = __uint_as_float(((127U - 20U + ((h1 >> 23) % 21U)) << 23) | (h1 & 0x7fffffU));
    const float h = __uint_as_float(((127U - 14U + ((h2 >> 23) % 20U)) << 23) | (h2 & 0x7fffffU));
    bad3 += !same_bits(exact_div(fminf(w, 1.0f), h), fminf(w, 1.0f) / h);
  }
  if (bad0) atomicAdd(&counts[0], (unsigned long long)bad0);
  if (bad1) atomicAdd(&counts[1], (unsigned long long)bad1);
  if (bad2) atomicAdd(&counts[2], (unsigned long long)bad2);
  if (bad3) atomicAdd(&counts[3], (unsigned long long)bad3);
}

// plain streaming copy, 16 bytes per lane.  One element per thread when the grid covers the buffer, with
// non-temporal loads and stores: the fastest of the shapes measured on this GPU for 1 GiB (6.6 TB/s read + written;
// the same loop on 8192 persistent workgroups reaches 4.6-4.9, a grid of half that many elements per thread 6.2).
typedef float copy_v4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void copy_kernel(const copy_v4* __restrict__ src, copy_v4* __restrict__ dst, long long n16) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (long long)gridDim.x * blockDim.x)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// NR planes read and summed, NW planes written: one 16-byte element per thread and plane (the streaming mix of a kernel
// that reads more than it writes; a plain copy is NR = NW = 1)
template <int NR, int NW>
__global__ __launch_bounds__(256) void stream_kernel(const copy_v4* __restrict__ src, copy_v4* __restrict__ dst, long long n16,
                                                     copy_v4* __restrict__ sink) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n16) return;
  copy_v4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < NR; r++) a += src[(long long)r * n16 + i];
#pragma unroll
  for (int w = 0; w < NW; w++) dst[(long long)w * n16 + i] = a;
  if (NW == 0 && a.x == 123.456f) *sink = a;  // (never true for the fill value: keeps the reads alive)
}
template <int NR, int NW>
static void launch_stream(int grid, hipStream_t stream, const copy_v4* src, copy_v4* dst, long long n16, copy_v4* sink) {
  hipLaunchKernelGGL((stream_kernel<NR, NW>), dim3(grid), dim3(256), 0, stream, src, dst, n16, sink);
}

// Every quotient of ordinary operands is, up to a power of two, n / d with n, d in [1, 2): all 2^23 x 2^23 pairs of
// mantissas, the library's division (reciprocal refined once, quotient corrected once) against the compiler's IEEE
// expansion.  One thread per denominator; blockIdx.y selects a sixteenth of the numerators.
// counts[0]: mismatches of div_by; counts[1]: mismatches of the uncorrected n * r (a check of the check: about a
// quarter of all pairs).
__global__ __launch_bounds__(256) void selftest_pairs_kernel(unsigned long long* counts, unsigned first_mantissa) {
  const unsigned dm = first_mantissa + blockIdx.x * blockDim.x + threadIdx.x;
  const float d = __uint_as_float(0x3f800000u | dm);
  const float r = rcp_refined(d);
  unsigned bad0 = 0, bad1 = 0;
  const unsigned n0 = blockIdx.y * (0x800000u / 16), n1 = n0 + 0x800000u / 16;
  for (unsigned nm = n0; nm < n1; nm++) {
    const float n = __uint_as_float(0x3f800000u | nm);
    const float ref = n / d;
    bad0 += !same_bits(div_by(n, d, r), ref);
    bad1 += !same_bits(n * r, ref);
  }
  if (bad0) atomicAdd(&counts[0], (unsigned long long)bad0);
  if (bad1) atomicAdd(&counts[1], (unsigned long long)bad1);
}

int run_selftest(void (*kernel)(unsigned long long*, unsigned int), unsigned long long* host4, unsigned int rounds) {
  unsigned long long* dev = nullptr;
  INPAINT_HIP(hipMalloc((void**)&dev, 4 * sizeof(unsigned long long)));
  INPAINT_HIP(hipMemset(dev, 0, 4 * sizeof(unsigned long long)));
  hipLaunchKernelGGL(kernel, dim3(4096), dim3(256), 0, 0, dev, rounds);
  INPAINT_HIP(hipGetLastError());
  INPAINT_HIP(hipMemcpy(host4, dev, 4 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  INPAINT_HIP(hipFree(dev));
  return 0;
}

}  // namespace

extern "C" int inpaint_selftest_rsqrt(unsigned long long* mismatches4_host, unsigned int pair_rounds) {
  return run_selftest(selftest_rsqrt_kernel, mismatches4_host, pair_rounds);
}

// Slices first_slice .. first_slice + slices - 1 of the 64 slices of 2^17 denominator mantissas each (all 2^23
// numerator mantissas per denominator: 1.1e12 pairs and about 0.6 s per slice on an MI355X).
extern "C" int inpaint_selftest_division_pairs(unsigned int first_slice, unsigned int slices, unsigned long long* mismatches2_host) {
  if (first_slice >= 64 || slices < 1 || first_slice + slices > 64 || !mismatches2_host)
    return inpaint::fail(INPAINT_ERR_ARG, "slices %u .. %u of 64", first_slice, first_slice + slices);
  unsigned long long* dev = nullptr;
  INPAINT_HIP(hipMalloc((void**)&dev, 2 * sizeof(unsigned long long)));
  INPAINT_HIP(hipMemset(dev, 0, 2 * sizeof(unsigned long long)));
  for (unsigned int s = first_slice; s < first_slice + slices; s++) {
    hipLaunchKernelGGL(selftest_pairs_kernel, dim3((1u << 17) / 256, 16), dim3(256), 0, 0, dev, s << 17);
    INPAINT_HIP(hipGetLastError());
    INPAINT_HIP(hipDeviceSynchronize());  // one launch at a time: each runs for about half a second
  }
  INPAINT_HIP(hipMemcpy(mismatches2_host, dev, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  INPAINT_HIP(hipFree(dev));
  return 0;
}

extern "C" int inpaint_selftest_math(unsigned long long* mismatches4_host, unsigned int pair_rounds) {
  unsigned long long* dev = nullptr;
  INPAINT_HIP(hipMalloc((void**)&dev, 4 * sizeof(unsigned long long)));
  INPAINT_HIP(hipMemset(dev, 0, 4 * sizeof(unsigned long long)));
  hipLaunchKernelGGL(selftest_kernel, dim3(4096), dim3(256), 0, 0, dev, pair_rounds);
  INPAINT_HIP(hipGetLastError());
  INPAINT_HIP(hipMemcpy(mismatches4_host, dev, 4 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  INPAINT_HIP(hipFree(dev));
  return 0;
}

// Diagnostic: what a plain device-to-device copy kernel reaches on this GPU, as a practical ceiling to quote beside
// the published HBM peak.  Copies `bytes` (rounded down to 16) from one fresh buffer to another `repeats` times after
// one warm-up launch and returns (bytes read + bytes written) / time in GB/s, timed with HIP events on `stream`.
extern "C" int inpaint_copy_bandwidth(long long bytes, int repeats, double* gbps_host, void* stream_) {
  if (bytes < 16 || repeats < 1 || !gbps_host) return inpaint::fail(INPAINT_ERR_ARG, "bad arguments");
  hipStream_t stream = (hipStream_t)stream_;
  const long long n16 = bytes / 16;
  copy_v4 *src = nullptr, *dst = nullptr;
  INPAINT_HIP(hipMalloc((void**)&src, (size_t)n16 * 16));
  if (hipMalloc((void**)&dst, (size_t)n16 * 16) != hipSuccess) {
    (void)hipFree(src);
    return inpaint::fail(INPAINT_ERR_HIP, "hipMalloc of the copy target failed");
  }
  INPAINT_HIP(hipMemsetAsync(src, 0x3c, (size_t)n16 * 16, stream));
  hipEvent_t e0, e1;
  INPAINT_HIP(hipEventCreate(&e0));
  INPAINT_HIP(hipEventCreate(&e1));
  const int grid = (int)std::min<long long>((n16 + 255) / 256, (1LL << 31) - 1);  // one element per thread
  hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, stream, src, dst, n16);
  INPAINT_HIP(hipEventRecord(e0, stream));
  for (int r = 0; r < repeats; r++) hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, stream, src, dst, n16);
  INPAINT_HIP(hipEventRecord(e1, stream));
  INPAINT_HIP(hipEventSynchronize(e1));
  float ms = 0;
  INPAINT_HIP(hipEventElapsedTime(&ms, e0, e1));
  INPAINT_HIP(hipGetLastError());
  *gbps_host = ms > 0 ? 2.0 * (double)n16 * 16 * repeats / (ms * 1e-3) / 1e9 : 0.0;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(src);
  (void)hipFree(dst);
  return 0;
}

// Diagnostic: the rate of a streaming kernel that reads `planes_read` planes and writes `planes_written` planes of
// `bytes_per_plane` each (16 bytes per thread and plane), bytes read + written per second in GB/s.  The memory system
// serves mixes of reads and writes more slowly than reads alone, so this, not the copy, is the practical ceiling of a
// kernel with that mix.  planes_read 1..4, planes_written 0..2.
extern "C" int inpaint_stream_bandwidth(long long bytes_per_plane, int planes_read, int planes_written, int repeats,
                                        double* gbps_host, void* stream_) {
  if (bytes_per_plane < 16 || repeats < 1 || !gbps_host || planes_read < 1 || planes_read > 4 || planes_written < 0 ||
      planes_written > 2)
    return inpaint::fail(INPAINT_ERR_ARG, "bad arguments (1..4 planes read, 0..2 written)");
  hipStream_t stream = (hipStream_t)stream_;
  const long long n16 = bytes_per_plane / 16;
  copy_v4 *src = nullptr, *dst = nullptr;
  INPAINT_HIP(hipMalloc((void**)&src, (size_t)n16 * 16 * planes_read));
  if (hipMalloc((void**)&dst, (size_t)n16 * 16 * std::max(planes_written, 1)) != hipSuccess) {
    (void)hipFree(src);
    return inpaint::fail(INPAINT_ERR_HIP, "hipMalloc of the stream target failed");
  }
  INPAINT_HIP(hipMemsetAsync(src, 0x3c, (size_t)n16 * 16 * planes_read, stream));
  hipEvent_t e0, e1;
  INPAINT_HIP(hipEventCreate(&e0));
  INPAINT_HIP(hipEventCreate(&e1));
  const int grid = (int)std::min<long long>((n16 + 255) / 256, (1LL << 31) - 1);
  typedef void (*Launch)(int, hipStream_t, const copy_v4*, copy_v4*, long long, copy_v4*);
  static const Launch table[4][3] = {{launch_stream<1, 0>, launch_stream<1, 1>, launch_stream<1, 2>},
                                     {launch_stream<2, 0>, launch_stream<2, 1>, launch_stream<2, 2>},
                                     {launch_stream<3, 0>, launch_stream<3, 1>, launch_stream<3, 2>},
                                     {launch_stream<4, 0>, launch_stream<4, 1>, launch_stream<4, 2>}};
  const Launch go = table[planes_read - 1][planes_written];
  go(grid, stream, src, dst, n16, dst);
  INPAINT_HIP(hipEventRecord(e0, stream));
  for (int r = 0; r < repeats; r++) go(grid, stream, src, dst, n16, dst);
  INPAINT_HIP(hipEventRecord(e1, stream));
  INPAINT_HIP(hipEventSynchronize(e1));
  float ms = 0;
  INPAINT_HIP(hipEventElapsedTime(&ms, e0, e1));
  INPAINT_HIP(hipGetLastError());
  *gbps_host = ms > 0 ? (double)(planes_read + planes_written) * (double)n16 * 16 * repeats / (ms * 1e-3) / 1e9 : 0.0;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(src);
  (void)hipFree(dst);
  return 0;
}
