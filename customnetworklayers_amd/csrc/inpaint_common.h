// Shared host/device plumbing of the TV and TGV inpainting layers: error reporting, the per-id
// device arena, the checkpoint schedule, and the on-device output guard.
#pragma once

#include <hip/hip_runtime.h>


#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/tvinpaint.h"
#include "../../include/inpaint_diagnostics.h"

namespace inpaint {

constexpr int kUniqueIds = 10;        // reference: __uniqueIds__, TVInpaintFista.h:5
constexpr int kMaxCheckpoints = 100;  // reference: idStruct vectors, TVInpaintFista.h:9-15

// ---------------------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------------------
inline char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}
#define INPAINT_HIP(call)                                                                      \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess)                                                                      \
      return inpaint::fail(INPAINT_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                           __FILE__, __LINE__);                                                \
  } while (0)

// ---------------------------------------------------------------------------------------------
// testing / tuning switches (INPAINT_* environment variables)
//
// Read once per process, on first use, and again only when somebody asks: *_reset_id() and inpaint_reload_env() do.
// A variable changed in the middle of a run therefore switches no kernel until one of those calls.
// ---------------------------------------------------------------------------------------------
struct Knobs {
  bool tv_tile_path = false;      // INPAINT_TV_PATH=tile: the LDS-tile kernels instead of the wave strips
  bool tv_fuse = true;            // INPAINT_TV_FUSE=0: one forward iteration per launch
  bool tv_fuse_adj = true;        // INPAINT_TV_FUSE_ADJ=0: one adjoint step per launch
  bool tv_fuse_first = true;      // INPAINT_TV_FUSE_FIRST=0: the reverse sweep's first step in a launch of its own
  bool tgv_fuse_first = true;     // INPAINT_TGV_FUSE_FIRST=0: the same for the TGV layer
  int tv_fwd_rows = 0;            // INPAINT_TV_FWD_ROWS / INPAINT_TV_ADJ_ROWS: strip height (0 = chosen per launch)
  int tv_adj_rows = 0;
  int tv_fwd_split = -1;          // INPAINT_TV_FWD_SPLIT=0|1: forward pairs with one channel per wavefront (-1 = by the size of the launch)
  int tv_adj_split = -1;          // INPAINT_TV_ADJ_SPLIT=0|1: the same for the adjoint pairs of two channels
  bool tgv_px_path = false;       // INPAINT_TGV_PATH=px: the per-pixel kernels
  bool tgv_fuse = true;           // INPAINT_TGV_FUSE=0
  bool tgv_fuse_adj = true;       // INPAINT_TGV_FUSE_ADJ=0
  int tgv_fwd_rows = 0;           // INPAINT_TGV_FWD_ROWS / INPAINT_TGV_ADJ_ROWS
  int tgv_adj_rows = 0;
  int tgv_fwd_split = -1;         // INPAINT_TGV_FWD_SPLIT=0|1: forward pairs with one channel per wavefront (-1 = by the size of the launch)
  int tgv_pair_waves = 0;         // INPAINT_TGV_PAIR_WAVES=1|2 (0 = by channel count)
  int keep = -1;                  // INPAINT_KEEP=0|1|2 (INPAINT_KEEP_LAST=0 is INPAINT_KEEP=0); -1 = the id's own mode
  double keep_gb = 32.0;          // INPAINT_KEEP_GB: budget of keep mode 2
  bool keep_gb_set = false;       // (the variable is set: the budget is the caller's, free device memory is not consulted)
  int stats_every = 0;            // INPAINT_STATS_EVERY=N: the guard's statistics on stderr every Nth backward pass of an id (a host wait; off by default)
  bool quadfit_px_path = false;   // INPAINT_QUADFIT_PATH=px: one pixel per lane, no LDS windows
  bool median_tile_per_wave = false;  // INPAINT_MEDIAN_PATH=tile: one tile of 64 pixels per wavefront for every bin count
  bool quadfit_reread = false;    // INPAINT_QUADFIT_PATH=reread: backward pass A reads the second map twice (any channel count)
  void load() {
    *this = Knobs();
    auto is = [](const char* name, const char* value) {
      const char* e = getenv(name);
      return e && strcmp(e, value) == 0;
    };
    auto rows = [](const char* name) {
      const char* e = getenv(name);
      const int v = e ? atoi(e) : 0;
      return (v >= 1 && v <= 4096) ? v : 0;
    };
    tv_tile_path = is("INPAINT_TV_PATH", "tile");
    tv_fuse = !is("INPAINT_TV_FUSE", "0");
    tv_fuse_adj = !is("INPAINT_TV_FUSE_ADJ", "0");
    tv_fuse_first = !is("INPAINT_TV_FUSE_FIRST", "0");
    tgv_fuse_first = !is("INPAINT_TGV_FUSE_FIRST", "0");
    tv_fwd_rows = rows("INPAINT_TV_FWD_ROWS");
    tv_adj_rows = rows("INPAINT_TV_ADJ_ROWS");
    tv_fwd_split = is("INPAINT_TV_FWD_SPLIT", "1") ? 1 : (is("INPAINT_TV_FWD_SPLIT", "0") ? 0 : -1);
    tv_adj_split = is("INPAINT_TV_ADJ_SPLIT", "1") ? 1 : (is("INPAINT_TV_ADJ_SPLIT", "0") ? 0 : -1);
    tgv_px_path = is("INPAINT_TGV_PATH", "px");
    tgv_fuse = !is("INPAINT_TGV_FUSE", "0");
    tgv_fuse_adj = !is("INPAINT_TGV_FUSE_ADJ", "0");
    tgv_fwd_rows = rows("INPAINT_TGV_FWD_ROWS");
    tgv_adj_rows = rows("INPAINT_TGV_ADJ_ROWS");
    tgv_fwd_split = is("INPAINT_TGV_FWD_SPLIT", "1") ? 1 : (is("INPAINT_TGV_FWD_SPLIT", "0") ? 0 : -1);
    tgv_pair_waves = is("INPAINT_TGV_PAIR_WAVES", "1") ? 1 : (is("INPAINT_TGV_PAIR_WAVES", "2") ? 2 : (getenv("INPAINT_TGV_PAIR_WAVES") ? 1 : 0));
    if (is("INPAINT_KEEP_LAST", "0")) keep = 0;
    if (const char* e = getenv("INPAINT_KEEP")) {
      const int v = atoi(e);
      if (v >= 0 && v <= 2) keep = v;
    }
    if (const char* e = getenv("INPAINT_KEEP_GB")) { keep_gb = atof(e); keep_gb_set = true; }
    if (const char* e = getenv("INPAINT_STATS_EVERY")) stats_every = std::max(0, atoi(e));
    quadfit_px_path = is("INPAINT_QUADFIT_PATH", "px");
    quadfit_reread = is("INPAINT_QUADFIT_PATH", "reread");
    median_tile_per_wave = is("INPAINT_MEDIAN_PATH", "tile");
  }
};
struct KnobsHolder {
  Knobs k;
  bool loaded = false;
};
inline KnobsHolder& knobs_holder() {
  static KnobsHolder h;
  return h;
}
inline const Knobs& knobs() {
  KnobsHolder& h = knobs_holder();
  if (!h.loaded) { h.k.load(); h.loaded = true; }
  return h.k;
}
inline void reload_knobs() {
  KnobsHolder& h = knobs_holder();
  h.k.load();
  h.loaded = true;
}

// ---------------------------------------------------------------------------------------------
// schedule (reference: TVInpaintFista.cu:1499-1508,1523 and 1525-1532; the TGV driver repeats both)
// ---------------------------------------------------------------------------------------------
inline void make_schedule(int its, std::vector<int>& iterations, int& max_inter_its) {
  const double root = std::sqrt((double)its);
  iterations.assign((size_t)std::floor(root), 0);
  max_inter_its = 0;
  for (size_t i = 0; i < iterations.size(); i++) {
    iterations[i] = (int)(std::floor(i * root * 0.5) * 2);
    if (i > 0) max_inter_its = std::max(max_inter_its, iterations[i] - iterations[i - 1]);
  }
  if (!iterations.empty()) max_inter_its = std::max(max_inter_its, its - iterations.back());
}

inline void make_step_sizes(int its, std::vector<float>& s) {
  s.assign((size_t)std::max(its, 0), 0.f);
  double t = 1, t_ = 1;
  for (size_t i = 0; i < s.size(); i++) {
    t_ = t;
    t = (1. + std::sqrt(1. + 4. * t * t)) / 2.;
    s[i] = (float)std::max(0.0, (t_ - 1.) / t);
  }
}

// ---------------------------------------------------------------------------------------------
// device arena: one hipMalloc per slot, re-made only when the shape changes
// ---------------------------------------------------------------------------------------------
// Where a slot's block comes from: hipMalloc / hipFree, or the caller's pool (t[g]vinpaint_set_allocator).
struct Allocator {
  inpaint_alloc_fn alloc = nullptr;
  inpaint_release_fn release = nullptr;
  void* user = nullptr;
};

struct Arena {
  char* base = nullptr;
  size_t bytes = 0, used = 0;
  int device = -1;
  Allocator owner;  // the pair that made `base` also takes it back
  int release() {
    if (base) {
      int cur = -1;
      (void)hipGetDevice(&cur);
      if (cur != device && device >= 0) (void)hipSetDevice(device);
      hipError_t e = hipSuccess;
      if (owner.release) owner.release(base, owner.user);
      else e = hipFree(base);
      if (cur != device && cur >= 0) (void)hipSetDevice(cur);
      base = nullptr;
      bytes = used = 0;
      if (e != hipSuccess) return fail(INPAINT_ERR_HIP, "hipFree failed: %s", hipGetErrorString(e));
    }
    return 0;
  }
  int reserve(size_t need, const Allocator& from, hipStream_t stream) {
    int rc = release();
    if (rc) return rc;
    INPAINT_HIP(hipGetDevice(&device));
    if (from.alloc && from.release) {
      base = static_cast<char*>(from.alloc((unsigned long long)need, device, (void*)stream, from.user));
      if (!base) return fail(INPAINT_ERR_HIP, "the caller's allocator returned no memory for %zu bytes", need);
      if (reinterpret_cast<uintptr_t>(base) & 255) {
        from.release(base, from.user);
        base = nullptr;
        return fail(INPAINT_ERR_HIP, "the caller's allocator returned a block that is not aligned to 256 bytes");
      }
      owner = from;
    } else {
      const hipError_t e = hipMalloc((void**)&base, need);
      if (e != hipSuccess) {
        base = nullptr;
        return fail(INPAINT_ERR_HIP, "hipMalloc of %zu bytes failed: %s", need, hipGetErrorString(e));
      }
      owner = Allocator();
    }
    bytes = need;
    used = 0;
    return 0;
  }
  template <class T>
  T* take(size_t count) {
    size_t off = (used + 255) & ~size_t(255);
    used = off + count * sizeof(T);
    return (used <= bytes) ? reinterpret_cast<T*>(base + off) : nullptr;
  }
  static size_t padded(size_t count, size_t elem) { return ((count * elem + 255) & ~size_t(255)) + 256; }
};

// Keep mode 2 asks for one x05 row per iteration.  When the slot has to grow for them and nobody stated a budget
// (INPAINT_KEEP_GB), rows that would take more than a quarter of what the device has free right now are not asked for:
// the forward pass keeps the last segment's rows instead (mode 1).  One hipMemGetInfo per (re)allocation, none per call.
inline bool rows_exceed_free_memory(double ring_bytes) {
  if (knobs().keep_gb_set) return false;
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return ring_bytes > 0.25 * (double)free_b;
}

// ---------------------------------------------------------------------------------------------
// strip height
// ---------------------------------------------------------------------------------------------
inline int compute_unit_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
              ? prop.multiProcessorCount
              : 256;
  }
  return cus;
}

// Rows per strip (one wavefront per strip, `waves_per_block` of them in a workgroup; `strips` = strips across the
// image width x samples).  Taller strips re-read fewer halo rows, but the launch should still put about two
// wavefronts on every SIMD (>= 1792 of them), and the workgroups are dealt to the CUs in whole numbers: the CU with
// one workgroup more than the others sets the time.  Among the heights that keep the device full, take the one that
// minimises (workgroups on the fullest CU) x (rows a wavefront walks: R + `lag` halo, pipeline and start-up rows).
// Measured: 4 x 2 x 384 x 1248, pair kernels: 16 rows (504 workgroups, two per CU) beat 8, 17, 18 and 24;
// 16 x 2 x 256 x 512: 19 rows (504 workgroups) 9.8 ms, 16 rows (576: three on some CUs) 12.0 ms.
inline int choose_strip_rows(long long strips, int ih, int waves_per_block, int lag) {
  const long long cus = compute_unit_count();
  int best = 0;
  long long best_cost = 0;
  for (int R = 3; R <= 32; R++) {
    const long long waves = strips * ((ih + R - 1) / R);
    if (waves < 1792) break;  // (waves fall as R grows)
    const long long blocks = (waves + waves_per_block - 1) / waves_per_block;
    const long long cost = ((blocks + cus - 1) / cus) * (R + lag);
    const bool even = ih % R == 0, best_even = best > 0 && ih % best == 0;
    if (best == 0 || cost < best_cost || (cost == best_cost && (even || !best_even))) {
      best = R;
      best_cost = cost;
    }
  }
  return best > 0 ? best : 2;
}

// ---------------------------------------------------------------------------------------------
// output guard (reference: check_gradUpdate + update_correct_av_step_host,
// TVInpaintFista.cu:128-175; TGV variant TGVInpaintFistaHelp.cu:119-216)
// ---------------------------------------------------------------------------------------------
struct GuardParams {
  double max_tolerance;  // entries above are zeroed (TV) or clamped to +-clamp_to (TGV)
  double clamp_to;       // 0: zero them
  double kill_t, scale_t, memory_t;
};

struct GuardStats {
  double sum;                        // sum of |g| over finite entries
  double tail_sum;                   // sum of |g| behind the last non-finite entry
  unsigned long long max_bits;       // bit pattern of max |g| (non-negative doubles order like integers)
  unsigned long long last_invalid1;  // 1 + index of the last non-finite entry, 0 if none
  unsigned int num_above, num_invalid;
};

constexpr int kGuardBlocks = 512;  // blocks per tensor in pass 1, each leaves one partial record

struct GuardState {  // lives in device memory, one per id
  double av[5];      // running means: C, X, Y, B, I
  double scale[5];   // multiplier chosen for the current backward (1, mult, or 0)
  double report[25]; // per tensor: mean |g|, max |g|, num_above, num_invalid, action
  GuardStats stats[5];
  unsigned int tickets[5];  // blocks of pass 2 that have added their share of a tail sum (zero between launches)
  // The TGV layer's verdict on the upstream gradient of the current backward pass (non-finite entries, or zero
  // everywhere: every output is zero, the running means and the run count stay as they are), and how many backward
  // passes so far had such an upstream.  The verdict stays on the device, so the host never waits for it: the host
  // counts every backward pass and the guard subtracts `skipped`.  Always zero in the TV layer.
  unsigned int upstream_bad, skipped;
  // pass 1 leaves per-block records here; they are combined in a fixed order (no atomics on one address, which
  // this GPU serialises at the memory side, and a mean that does not depend on the order of arrival)
  GuardStats partial[5][kGuardBlocks];
};
constexpr size_t kGuardHeaderBytes = offsetof(GuardState, partial);  // what the host reads back

// The decision rule, shared by the device kernel and the host-side test hook.
// Returns 0 plain / 1 rescaled / 2 killed.
__host__ __device__ inline int guard_decide_rule(int run, double av_gc, double& av_running, double& mult,
                                                 const GuardParams& p) {
  const double run_step = fmin(p.memory_t, double(run) / double(run + 1));
  if (run >= 10 && av_running * p.kill_t < av_gc) {
    mult = 0.0;
    av_running = av_running * run_step + (1. - run_step) * p.scale_t * av_running;
    return 2;
  }
  if (run >= 10 && av_running * p.scale_t < av_gc) {
    mult = p.scale_t * av_running / av_gc;
    av_running = av_running * run_step + (1. - run_step) * av_gc * mult;
    return 1;
  }
  mult = 1.0;
  av_running = av_running * run_step + (1. - run_step) * av_gc;
  return 0;
}

template <class T>
__device__ inline bool finite_value(T v) {
  return (v == v) && (fabs((double)v) <= (sizeof(T) == 4 ? 3.4028234663852886e38 : 1.7976931348623157e308));
}

__device__ inline double wave_sum(double v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}
__device__ inline unsigned long long wave_max(unsigned long long v) {
  for (int off = 32; off > 0; off >>= 1) {
    unsigned long long o = __shfl_down(v, off, 64);
    v = o > v ? o : v;
  }
  return v;
}
__device__ inline unsigned int wave_sum_u(unsigned int v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// pass 1: sum, max, counts, position of the last non-finite entry (one record per block); with clamp_mean
// (TGV) an entry above max_tol enters the mean as max_tol, the TV layer's mean takes it as it is.
// pass 2 (does nothing unless pass 1 saw a non-finite entry): sum of |g| behind the last one.
// pass 3: the decision.
// The five tensors of one backward in one launch for pass 1, one for passes 2 and 3 and one for the final scaling
// (blockIdx.y picks the tensor; blocks beyond a tensor's own grid find nothing to do).
struct GuardJobs {
  const void* ptr[5];
  long long n[5];
  int is_f32[5];
};

template <class T>
__device__ __forceinline__ void guard_reduce_body(const T* __restrict__ g, long long n, GuardStats* __restrict__ st,
                                                  double max_tol, bool clamp_mean) {
  __shared__ double s_sum[4];
  __shared__ unsigned long long s_mx[4], s_last[4];
  __shared__ unsigned int s_above[4], s_invalid[4];
  double s = 0;
  unsigned long long mx = 0, last = 0;
  unsigned int above = 0, invalid = 0;
#pragma unroll 4
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    T v = g[i];
    if (finite_value(v)) {
      double a = fabs((double)v);
      s += (clamp_mean && a > max_tol) ? max_tol : a;
      unsigned long long bits = (unsigned long long)__double_as_longlong(a);
      mx = bits > mx ? bits : mx;
      above += (a > max_tol);
    } else {
      invalid++;
      last = (unsigned long long)(i + 1);
    }
  }
  s = wave_sum(s);
  mx = wave_max(mx);
  last = wave_max(last);
  above = wave_sum_u(above);
  invalid = wave_sum_u(invalid);
  const int wv = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    s_sum[wv] = s; s_mx[wv] = mx; s_last[wv] = last; s_above[wv] = above; s_invalid[wv] = invalid;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < 4; k++) {
      s += s_sum[k];
      mx = s_mx[k] > mx ? s_mx[k] : mx;
      last = s_last[k] > last ? s_last[k] : last;
      above += s_above[k];
      invalid += s_invalid[k];
    }
    GuardStats r;
    r.sum = s; r.tail_sum = 0; r.max_bits = mx; r.last_invalid1 = last; r.num_above = above; r.num_invalid = invalid;
    *st = r;
  }
}

// launch with grid (kGuardBlocks, 5)
static __global__ __launch_bounds__(256) void guard_reduce_many(GuardJobs jobs, GuardState* __restrict__ gs, double max_tol,
                                                                bool clamp_mean) {
  const int k = blockIdx.y;
  GuardStats* st = &gs->partial[k][blockIdx.x];
  if (jobs.is_f32[k]) guard_reduce_body(static_cast<const float*>(jobs.ptr[k]), jobs.n[k], st, max_tol, clamp_mean);
  else guard_reduce_body(static_cast<const double*>(jobs.ptr[k]), jobs.n[k], st, max_tol, clamp_mean);
}

// the partial records of one tensor, combined by one wavefront in a fixed order (lane l takes records l, l+64, ...)
__device__ __forceinline__ GuardStats guard_combine(const GuardStats* __restrict__ part, int lane) {
  double s = 0;
  unsigned long long mx = 0, last = 0;
  unsigned int above = 0, invalid = 0;
  for (int i = lane; i < kGuardBlocks; i += 64) {
    s += part[i].sum;
    mx = part[i].max_bits > mx ? part[i].max_bits : mx;
    last = part[i].last_invalid1 > last ? part[i].last_invalid1 : last;
    above += part[i].num_above;
    invalid += part[i].num_invalid;
  }
  GuardStats r;
  r.sum = wave_sum(s);
  r.tail_sum = 0;
  r.max_bits = wave_max(mx);
  r.last_invalid1 = wave_max(last);
  r.num_above = wave_sum_u(above);
  r.num_invalid = wave_sum_u(invalid);
  r.sum = __shfl(r.sum, 0, 64);
  r.max_bits = __shfl(r.max_bits, 0, 64);
  r.last_invalid1 = __shfl(r.last_invalid1, 0, 64);
  r.num_above = __shfl(r.num_above, 0, 64);
  r.num_invalid = __shfl(r.num_invalid, 0, 64);
  return r;
}

// Passes 2 and 3 of one tensor.  Pass 2 does nothing unless pass 1 saw a non-finite entry: then every block adds its
// share of the sum of |g| behind the last one to stats->tail_sum and takes a ticket; the block with the last ticket has
// every share in front of it and goes on to pass 3.  Without non-finite entries block 0 does.  Pass 3, one wavefront:
// the partial records combined in a fixed order, then lane 0 turns the statistics into the tensor's multiplier and
// updates its running mean.  Sequential running mean of the reference, av_{i+1} = (|g_i| + i av_i)/(i+1) with a
// reset to 1000 * running mean at every non-finite entry, in closed form.
template <class T>
__device__ __forceinline__ void guard_tail_decide_body(const T* __restrict__ g, long long n, GuardState* __restrict__ gs, int k,
                                                       int run, const GuardParams& p, bool clamp_mean) {
  const GuardStats* __restrict__ part = gs->partial[k];
  GuardStats* __restrict__ st = &gs->stats[k];
  __shared__ unsigned long long s_last[4];
  __shared__ unsigned int s_invalid[4];
  __shared__ int s_decide;
  {
    unsigned long long last = 0;
    unsigned int invalid = 0;
    for (int i = threadIdx.x; i < kGuardBlocks; i += blockDim.x) {
      last = part[i].last_invalid1 > last ? part[i].last_invalid1 : last;
      invalid += part[i].num_invalid;
    }
    last = wave_max(last);
    invalid = wave_sum_u(invalid);
    if ((threadIdx.x & 63) == 0) { s_last[threadIdx.x >> 6] = last; s_invalid[threadIdx.x >> 6] = invalid; }
    __syncthreads();
  }
  const bool any_invalid = s_invalid[0] + s_invalid[1] + s_invalid[2] + s_invalid[3] != 0;
  if (!any_invalid) {
    if (blockIdx.x != 0) return;
  } else {
    unsigned long long last1 = s_last[0];
    for (int w = 1; w < 4; w++) last1 = s_last[w] > last1 ? s_last[w] : last1;
    double s = 0;
    for (long long i = (long long)last1 + (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (long long)gridDim.x * blockDim.x) {
      const double a = fabs((double)g[i]);
      s += (clamp_mean && a > p.max_tolerance) ? p.max_tolerance : a;
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0 && s != 0) atomicAdd(&st->tail_sum, s);
    __threadfence();  // the share is visible to the device before the ticket is taken
    __syncthreads();
    if (threadIdx.x == 0) s_decide = atomicAdd(&gs->tickets[k], 1u) == gridDim.x - 1;
    __syncthreads();
    if (!s_decide) return;
    __threadfence();
  }
  if (threadIdx.x >= 64) return;
  const int lane = threadIdx.x;
  GuardStats c = guard_combine(part, lane);
  if (lane != 0) return;
  // (cleared before pass 1; read where the other blocks' atomics have put it)
  c.tail_sum = any_invalid ? atomicAdd(&st->tail_sum, 0.0) : 0.0;
  if (any_invalid) gs->tickets[k] = 0;
  *st = c;
  if (gs->upstream_bad) return;  // (TGV) this backward pass returns zeros: no decision, running mean and report untouched
  run -= (int)gs->skipped;       // (TGV) backward passes that did not count
  double av_gc;
  if (n <= 0) {
    av_gc = 0;
  } else if (c.num_invalid == 0) {
    av_gc = c.sum / (double)n;
  } else {
    av_gc = ((double)c.last_invalid1 * (gs->av[k] * 1000.) + c.tail_sum) / (double)n;
  }
  double mult = 1.0;
  const int action = guard_decide_rule(run, av_gc, gs->av[k], mult, p);
  gs->scale[k] = mult;
  gs->report[5 * k + 0] = av_gc;
  gs->report[5 * k + 1] = __longlong_as_double((long long)c.max_bits);
  gs->report[5 * k + 2] = c.num_above;
  gs->report[5 * k + 3] = c.num_invalid;
  gs->report[5 * k + 4] = action;
}

// launch with grid (guard_grid(longest tensor), 5) and 256 threads
static __global__ __launch_bounds__(256) void guard_tail_decide_many(GuardJobs jobs, GuardState* __restrict__ gs, int run,
                                                                     GuardParams p, bool clamp_mean) {
  const int k = blockIdx.y;
  if (jobs.is_f32[k]) guard_tail_decide_body(static_cast<const float*>(jobs.ptr[k]), jobs.n[k], gs, k, run, p, clamp_mean);
  else guard_tail_decide_body(static_cast<const double*>(jobs.ptr[k]), jobs.n[k], gs, k, run, p, clamp_mean);
}

static __global__ void guard_clear_kernel(GuardState* gs) {
  int k = threadIdx.x;
  if (k < 5) {
    GuardStats z;
    z.sum = 0; z.tail_sum = 0; z.max_bits = 0; z.last_invalid1 = 0; z.num_above = 0; z.num_invalid = 0;
    gs->stats[k] = z;
    gs->tickets[k] = 0;
  }
}

inline int guard_grid(long long n) {
  long long blocks = (n + 256 * 16 - 1) / (256 * 16);
  return (int)std::max<long long>(1, std::min<long long>(blocks, 1024));
}

// ---------------------------------------------------------------------------------------------
// small generic kernels shared by both layers
// ---------------------------------------------------------------------------------------------
inline int grid1d(long long n) { return (int)std::max<long long>(1, std::min<long long>((n + 255) / 256, 1 << 20)); }
inline int grid_stride(long long n) { return (int)std::max<long long>(1, std::min<long long>((n + 1023) / 1024, 4096)); }

// Segment flush: fp32 accumulator into its fp64 total, then zero (copy_and_set_to_0,
// TVInpaintFista.cu:178-218; TGVInpaintFistaHelp.cu:178-216).
static __global__ __launch_bounds__(256) void flush_kernel(float* __restrict__ acc, double* __restrict__ total,
                                                           long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    total[i] = (double)acc[i] + total[i] / 1.;
    acc[i] = 0.f;
  }
}

// The same flush in two halves, for the paths that keep one fp32 record per segment: segment_store_many moves the
// accumulators of a finished segment into its record and zeroes them; combine_segments_many, after the last segment,
// adds the records into the fp64 totals in the order the reference flushes them (last segment first), with the
// reference's expression.  The totals then hold the bits they would after per-segment flushes, and nobody has read
// and rewritten them once per segment.
struct SegmentJobs {
  float* acc[4];     // accumulators (segment_store_many) -- unused by combine_segments_many
  float* seg[4];     // segment_store_many: this segment's record; combine_segments_many: record of segment 0
  double* total[4];  // combine_segments_many only
  long long n[4];    // elements per record
};
static __global__ __launch_bounds__(256) void segment_store_many(SegmentJobs jobs) {
  const int k = blockIdx.y;
  float* __restrict__ acc = jobs.acc[k];
  float* __restrict__ seg = jobs.seg[k];
  const long long n = jobs.n[k];
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    seg[i] = acc[i];
    acc[i] = 0.f;
  }
}
static __global__ __launch_bounds__(256) void combine_segments_many(SegmentJobs jobs, int nseg) {
  const int k = blockIdx.y;
  const float* __restrict__ seg = jobs.seg[k];
  double* __restrict__ total = jobs.total[k];
  const long long n = jobs.n[k];
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    double t = 0.;
    int o = nseg - 1;
    for (; o >= 3; o -= 4) {  // four records in flight at a time; the additions keep their order
      // (the records are read once, long after they were written: non-temporal loads)
      const float v0 = __builtin_nontemporal_load(seg + (long long)o * n + i), v1 = __builtin_nontemporal_load(seg + (long long)(o - 1) * n + i);
      const float v2 = __builtin_nontemporal_load(seg + (long long)(o - 2) * n + i), v3 = __builtin_nontemporal_load(seg + (long long)(o - 3) * n + i);
      t = (double)v0 + t / 1.;
      t = (double)v1 + t / 1.;
      t = (double)v2 + t / 1.;
      t = (double)v3 + t / 1.;
    }
    for (; o >= 0; o--) t = (double)__builtin_nontemporal_load(seg + (long long)o * n + i) + t / 1.;
    total[i] = t;
  }
}

static __global__ __launch_bounds__(256) void fill_zero_f32(float* __restrict__ p, long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x)
    p[i] = 0.f;
}

// One source copied into two destinations (the starting point into both halves of checkpoint 0).
static __global__ __launch_bounds__(256) void copy_twice_f32(const float* __restrict__ src, float* __restrict__ a, float* __restrict__ b,
                                                             long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    const float v = src[i];
    a[i] = v;
    b[i] = v;
  }
}

// Zero several buffers in one launch (blockIdx.y picks the buffer).
struct ZeroList {
  void* ptr[24];
  long long bytes[24];
};
static __global__ __launch_bounds__(256) void fill_zero_many(ZeroList z) {
  uint32_t* p = static_cast<uint32_t*>(z.ptr[blockIdx.y]);
  const long long n = z.bytes[blockIdx.y] / 4;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x)
    p[i] = 0u;
}

// Zero the non-finite entries of the caller's upstream gradient in place
// (TVInpaintFista.cu:1609-1623; TGVInpaintFistaBetas.cu:2690-2701).
static __global__ __launch_bounds__(256) void scrub_kernel(float* __restrict__ g, long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const float v = g[i];
    if (!finite_value(v)) g[i] = 0.f;
  }
}

// The start of a backward pass in one launch: the buffers of `z` zeroed (blockIdx.y < nz), the non-finite entries of the
// caller's upstream gradient zeroed in place (blockIdx.y == nz, as scrub_kernel) and the guard's statistics of the
// previous backward cleared (blockIdx.y == nz + 1, as guard_clear_kernel).  Launch with grid (blocks, nz + 2).
static __global__ __launch_bounds__(256) void backward_prologue_many(ZeroList z, int nz, float* __restrict__ upstream,
                                                                     long long upstream_n, GuardState* gs) {
  const int job = blockIdx.y;
  if (job < nz) {
    uint32_t* p = static_cast<uint32_t*>(z.ptr[job]);
    const long long n = z.bytes[job] / 4;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) p[i] = 0u;
  } else if (job == nz) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < upstream_n; i += (long long)gridDim.x * blockDim.x) {
      const float v = upstream[i];
      if (!finite_value(v)) upstream[i] = 0.f;
    }
  } else if (blockIdx.x == 0 && threadIdx.x < 5) {
    GuardStats zs;
    zs.sum = 0; zs.tail_sum = 0; zs.max_bits = 0; zs.last_invalid1 = 0; zs.num_above = 0; zs.num_invalid = 0;
    gs->stats[threadIdx.x] = zs;
    gs->tickets[threadIdx.x] = 0;
  }
}

// An entry beyond the guard's tolerance: zeroed (TV) or clamped to +-clamp_to (TGV).
template <class T>
__device__ inline T guard_limit(T v, const GuardParams& p) {
  if (!finite_value(v)) return T(0);
  if (fabs((double)v) > p.max_tolerance) return p.clamp_to > 0 ? (T)(v > 0 ? p.clamp_to : -p.clamp_to) : T(0);
  return v;
}

// Gradient wrt the starting point, guarded as a float tensor (TVInpaintFista.cu:1784-1791,1816).
static __global__ __launch_bounds__(256) void finalize_f32(const float* __restrict__ src, float* __restrict__ out,
                                                           long long n, const GuardState* __restrict__ gs, int k,
                                                           GuardParams p) {
  const double mult = gs->scale[k];
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    float v = guard_limit(src[i], p);
    if (mult != 1.0) v = (mult == 0.0) ? 0.f : (float)((double)v * mult);
    out[i] = 0.0f + v;
  }
}

// (TGV) every output of a backward pass whose upstream gradient was refused is zero
template <class T>
__device__ __forceinline__ void finalize_zero(T* __restrict__ out, long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) out[i] = T(0);
}

// Guarded fp64 totals -> fp32 outputs, the four tensors of one backward in one launch (blockIdx.y picks the tensor):
// limit, kill / rescale, global multiplier, then the chain factor of the weight scaling (TVInpaintFista.cu:1795-1818;
// TGVInpaintFistaBetas.cu:3024-3050).  The chain factor is chain_const, or chain_per_sample[i / per_sample] when that
// pointer is given.
struct FinalizeJobs {
  const double* total[4];
  float* out[4];
  long long n[4];
  double chain_const[4];
  const double* chain_per_sample[4];
  long long per_sample[4];
  // optional fifth job (grid.y == 5): a float tensor guarded as finalize_f32 does, with the guard's scale `f32_scale`
  const float* f32_src = nullptr;
  float* f32_out = nullptr;
  long long f32_n = 0;
  int f32_scale = 4;
};
static __global__ __launch_bounds__(256) void finalize_many(FinalizeJobs jobs, const GuardState* __restrict__ gs, GuardParams p,
                                                            float global_mult) {
  const int k = blockIdx.y;
  if (gs->upstream_bad) {
    if (k == 4) finalize_zero(jobs.f32_out, jobs.f32_n);
    else finalize_zero(jobs.out[k], jobs.n[k]);
    return;
  }
  if (k == 4) {  // (finalize_f32)
    const double mult = gs->scale[jobs.f32_scale];
    const float* __restrict__ src = jobs.f32_src;
    float* __restrict__ out = jobs.f32_out;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < jobs.f32_n; i += (long long)gridDim.x * blockDim.x) {
      float v = guard_limit(src[i], p);
      if (mult != 1.0) v = (mult == 0.0) ? 0.f : (float)((double)v * mult);
      out[i] = 0.0f + v;
    }
    return;
  }
  const double mult = gs->scale[k];
  const double* __restrict__ total = jobs.total[k];
  float* __restrict__ out = jobs.out[k];
  const double* __restrict__ chain_per_sample = jobs.chain_per_sample[k];
  const double chain_const = jobs.chain_const[k];
  const long long n = jobs.n[k], per_sample = jobs.per_sample[k];
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    double v = guard_limit(total[i], p);
    if (mult != 1.0) v = (mult == 0.0) ? 0.0 : v * mult;
    const float f = (float)(v * global_mult);
    const double chain = chain_per_sample ? chain_per_sample[i / per_sample] : chain_const;
    out[i] = (chain == 1.0) ? f : (float)(chain * (double)f);
  }
}

// Diagnostic: the device guard (the three kernels above, as a backward pass launches them) on one tensor handed over in
// host memory.  `values`: n doubles, or n floats with is_f32 (then the tensor takes the slot of the gradient wrt the
// starting point).  `out`: the n guarded values as floats (limit, kill / rescale; no global multiplier, no chain
// factor).  result7: mean |g|, max |g|, entries above the tolerance, non-finite entries, action (0 plain / 1 rescaled
// / 2 killed), the updated running mean, the multiplier.  Allocates and frees its own device memory.
inline int guard_selftest(const void* values, long long n, bool is_f32, int run, double running_mean, const GuardParams& p,
                          bool clamp_mean, float* out, double* result7) {
  if (!values || !out || !result7 || n < 1) return fail(INPAINT_ERR_ARG, "guard selftest: null pointer or n < 1");
  const int k = is_f32 ? 4 : 0;
  const size_t bytes = (size_t)n * (is_f32 ? sizeof(float) : sizeof(double));
  void* dv = nullptr;
  float* dout = nullptr;
  GuardState* gs = nullptr;
  auto release = [&]() {
    (void)hipFree(dv);
    (void)hipFree(dout);
    (void)hipFree(gs);
  };
  auto run_all = [&]() -> int {
    INPAINT_HIP(hipMalloc(&dv, bytes));
    INPAINT_HIP(hipMalloc((void**)&dout, (size_t)n * sizeof(float)));
    INPAINT_HIP(hipMalloc((void**)&gs, sizeof(GuardState)));
    INPAINT_HIP(hipMemcpy(dv, values, bytes, hipMemcpyHostToDevice));
    INPAINT_HIP(hipMemset(gs, 0, sizeof(GuardState)));
    INPAINT_HIP(hipMemcpy(&gs->av[k], &running_mean, sizeof(double), hipMemcpyHostToDevice));
    GuardJobs jobs;
    FinalizeJobs fin;
    for (int j = 0; j < 5; j++) {
      jobs.ptr[j] = nullptr; jobs.n[j] = 0; jobs.is_f32[j] = 0;
      if (j < 4) {
        fin.total[j] = nullptr; fin.out[j] = nullptr; fin.n[j] = 0;
        fin.chain_const[j] = 1.0; fin.chain_per_sample[j] = nullptr; fin.per_sample[j] = 1;
      }
    }
    jobs.ptr[k] = dv; jobs.n[k] = n; jobs.is_f32[k] = is_f32;
    if (is_f32) {
      fin.f32_src = static_cast<const float*>(dv); fin.f32_out = dout; fin.f32_n = n; fin.f32_scale = k;
    } else {
      fin.total[k] = static_cast<const double*>(dv); fin.out[k] = dout; fin.n[k] = n;
    }
    hipLaunchKernelGGL(guard_reduce_many, dim3(kGuardBlocks, 5), dim3(256), 0, 0, jobs, gs, p.max_tolerance, clamp_mean);
    hipLaunchKernelGGL(guard_tail_decide_many, dim3(guard_grid(n), 5), dim3(256), 0, 0, jobs, gs, run, p, clamp_mean);
    hipLaunchKernelGGL(finalize_many, dim3(grid_stride(n), 5), dim3(256), 0, 0, fin, gs, p, 1.f);
    INPAINT_HIP(hipGetLastError());
    INPAINT_HIP(hipDeviceSynchronize());
    INPAINT_HIP(hipMemcpy(out, dout, (size_t)n * sizeof(float), hipMemcpyDeviceToHost));
    INPAINT_HIP(hipMemcpy(result7, &gs->report[5 * k], 5 * sizeof(double), hipMemcpyDeviceToHost));
    INPAINT_HIP(hipMemcpy(result7 + 5, &gs->av[k], sizeof(double), hipMemcpyDeviceToHost));
    INPAINT_HIP(hipMemcpy(result7 + 6, &gs->scale[k], sizeof(double), hipMemcpyDeviceToHost));
    return 0;
  };
  const int rc = run_all();
  release();
  return rc;
}

// The guard's statistics of the backward pass just enqueued, on stderr in the reference's wording (TVInpaintFista.cu:1766-1790
// prints them on every 75th run of an id, TGVInpaintFistaBetas.cu:2996-3021 with the id in front).  Waits for the stream:
// only called when INPAINT_STATS_EVERY asks for it.  Nothing is printed for a backward pass whose upstream was refused.
inline int print_guard_report(const GuardState* dev, hipStream_t stream, int id, bool with_id) {
  GuardState host;
  INPAINT_HIP(hipStreamSynchronize(stream));
  INPAINT_HIP(hipMemcpy(&host, dev, kGuardHeaderBytes, hipMemcpyDeviceToHost));
  if (host.upstream_bad) return 0;
  static const char* const names[5] = {"conf ", "gradX ", "gradY ", "gradB ", "gradI "};
  for (int k = 0; k < 5; k++) {
    if (with_id) fprintf(stderr, "\nL %d Output gradient to %s %d %g  vs  %g vs %g ", id, names[k], (int)host.report[5 * k + 2],
                         host.report[5 * k + 0], host.av[k], host.report[5 * k + 1]);
    else fprintf(stderr, "\nOutput gradient to %s %d %g  vs  %g vs %g ", names[k], (int)host.report[5 * k + 2], host.report[5 * k + 0],
                 host.av[k], host.report[5 * k + 1]);
  }
  fprintf(stderr, "\n\n");
  return 0;
}

// Optional timing of a layer's dominant kernel with HIP events on the launch stream.  An event
// between two launches costs several microseconds of idle GPU, so a pair of events brackets a run
// of consecutive launches of that kernel (one reverse sweep), not every launch.
struct KernelTimer {
  bool enabled = false;
  std::vector<hipEvent_t> pool;  // start/stop pairs
  std::vector<int> counts;       // launches inside each pair
  size_t used = 0;
  void record(hipStream_t stream) {
    if (used == pool.size()) {
      hipEvent_t e;
      if (hipEventCreate(&e) != hipSuccess) { enabled = false; return; }
      pool.push_back(e);
    }
    (void)hipEventRecord(pool[used++], stream);
  }
  void begin(hipStream_t stream) {
    if (enabled) record(stream);
  }
  void end(hipStream_t stream, int launches) {
    if (!enabled) return;
    record(stream);
    counts.resize(used / 2, 0);
    if (used >= 2) counts[used / 2 - 1] = launches;
  }
  void reset() { used = 0; counts.clear(); }
  int read(double* total_ms, int* launches) {
    double total = 0;
    int count = 0;
    for (size_t i = 0; i + 1 < used; i += 2) {
      INPAINT_HIP(hipEventSynchronize(pool[i + 1]));
      float ms = 0;
      INPAINT_HIP(hipEventElapsedTime(&ms, pool[i], pool[i + 1]));
      total += ms;
      count += counts[i / 2];
    }
    reset();
    if (total_ms) *total_ms = total;
    if (launches) *launches = count;
    return 0;
  }
};

}  // namespace inpaint
