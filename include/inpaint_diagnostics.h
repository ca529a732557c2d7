/* Diagnostics and measurement hooks of libinpaint_hip.so.  None of these has a counterpart in the reference and none is
 * part of the operator boundary (include/tvinpaint.h, include/tgvinpaint.h): they are for the tests, the benchmark and
 * for whoever ports the kernels to another GPU.  Same conventions: plain pointers and sizes, 0 = ok, the text of an
 * error from tvinpaint_last_error().
 */
#ifndef INPAINT_DIAGNOSTICS_H_
#define INPAINT_DIAGNOSTICS_H_

#ifdef __cplusplus
extern "C" {
#endif

/* The output guard as the backward pass runs it on the device
 * (check_gradUpdate + update_correct_av_step_host, TVInpaintFista.cu:128-175, applied as
 * TVInpaintFista.cu:1760-1818) on ONE tensor handed over in host memory, so that tensors with non-finite and
 * out-of-tolerance entries can be checked.  values: n doubles, or n floats when is_f32 is set (the guard treats the
 * gradient wrt the starting point as a float tensor).  out: the n guarded values as floats (non-finite and
 * out-of-tolerance entries zeroed, then killed or rescaled; no further factor).  result7: mean |g| as the guard
 * counts it, max |g|, entries above the tolerance, non-finite entries, action (0 plain / 1 rescaled / 2 killed), the
 * updated running mean, the multiplier.  Allocates and frees its own device memory; synchronises the device. */
int tvinpaint_selftest_guard(const void* values, long long n, int is_f32, int run, double running_mean, float* out,
                             double* result7);

/* Timing of the main adjoint kernel (the dominant one) with HIP events recorded on the launch
 * stream around every launch.  profile(1) starts collecting, profile_read waits for the recorded
 * events, returns their summed duration and count and clears the collection. */
int tvinpaint_profile(int enable);
int tvinpaint_profile_read(double* total_ms, int* launches);

/* Compares the library's cheap correctly-rounded division / square root with the
 * compiler's IEEE expansions on the GPU (exhaustively over single floats, on `pair_rounds` hashed
 * pairs per thread otherwise) and returns the four mismatch counts (host array).  All must be 0. */
int inpaint_selftest_math(unsigned long long* mismatches4_host, unsigned int pair_rounds);

/* The library's division (reciprocal refined once, quotient corrected once) against the compiler's IEEE
 * expansion on ALL pairs of mantissas, n / d with n, d in [1, 2) -- every quotient of ordinary operands is one of
 * these up to a power of two.  The 2^23 denominator mantissas come in 64 slices of 2^17 (each with all 2^23
 * numerators: 1.1e12 pairs, about 0.6 s on an MI355X); the call checks slices first_slice .. first_slice + slices - 1
 * and returns two counts (host array): mismatches of the division, which must be 0, and mismatches of the
 * uncorrected product n * (1 / d), about a quarter of the pairs (shows that the comparison sees a wrong last bit). */
int inpaint_selftest_division_pairs(unsigned int first_slice, unsigned int slices, unsigned long long* mismatches2_host);

/* As tvinpaint_selftest_guard, with the TGV layer's guard (check_gradUpdate + update_correct_av_step_host,
 * TGVInpaintFistaHelp.cu:119-216: an entry above the tolerance enters the mean as the tolerance and is clamped to it,
 * not zeroed). */
int tgvinpaint_selftest_guard(const void* values, long long n, int is_f32, int run, double running_mean, float* out,
                              double* result7);

/* HIP-event timing of the main adjoint kernel, as tvinpaint_profile / tvinpaint_profile_read. */
int tgvinpaint_profile(int enable);
int tgvinpaint_profile_read(double* total_ms, int* launches);

/* Like inpaint_selftest_math: the TGV strip kernels' 1/sqrt(x), x/0.2f, the reciprocal 1/m over [2^-40, 2^40) and w/h^2
 * against the compiler's IEEE expansions on the GPU (host array of four mismatch counts, all 0). */
int inpaint_selftest_rsqrt(unsigned long long* mismatches4_host, unsigned int pair_rounds);

/* The rate a plain device-to-device copy kernel reaches on the current GPU (bytes read + bytes written per
 * second, in GB/s, host pointer), to quote beside the published HBM peak.  Allocates and frees two buffers of `bytes`,
 * copies `repeats` times after a warm-up launch, timed with HIP events on `stream`; waits for the result. */
int inpaint_copy_bandwidth(long long bytes, int repeats, double* gbps_host, void* stream);

/* The same for a streaming kernel that reads `planes_read` (1..4) planes and writes `planes_written` (0..2) planes of
 * `bytes_per_plane` each: the memory system serves a mix of reads and writes more slowly than either alone, so this is the
 * practical ceiling to hold a kernel with that mix against (the strip kernels read about two bytes for each one they
 * write).  Bytes read + written per second, GB/s. */
int inpaint_stream_bandwidth(long long bytes_per_plane, int planes_read, int planes_written, int repeats, double* gbps_host,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INPAINT_DIAGNOSTICS_H_ */
