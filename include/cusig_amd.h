/*
 * cusig_amd.h -- C ABI of the MI355X (gfx950) truncated-signature library.
 *
 * The shared object is named libcusig.so and exports, with identical names,
 * argument lists and status codes, the entry points that the reference binds
 * from its GPU plugin for the batched signature path, so the reference's
 * Python loader and wrappers work on it unchanged.
 *
 * Conventions (all entry points):
 *   - pointers are DEVICE pointers of the current HIP device; dense row-major
 *     buffers allocated by the caller; inputs are never modified;
 *   - `dimension` / `length` are the RAW path sizes (before lead-lag / time
 *     augmentation);
 *   - synchronous: device work has completed when the call returns;
 *   - never throws; returns 0 on success, 1 allocation failure, 2 invalid
 *     argument, 3 out of range, 10 runtime error (e.g. size overflow or a shape
 *     this build has no kernel for), 11 unknown, 100000 + hipError_t for device
 *     errors; a human-readable message for the calling thread is available from
 *     cusig_last_error_message().
 */
#ifndef CUSIG_AMD_H
#define CUSIG_AMD_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
#define CUSIG_AMD_NOEXCEPT noexcept
extern "C" {
#else
#define CUSIG_AMD_NOEXCEPT
#endif

#define CUSIG_AMD_API __attribute__((visibility("default")))

/* Truncated signature of a batch of paths.
 * path [batch, length, dimension]; out [batch, S] with S = sum_{k=1..degree} d^k
 * (+1 leading scalar when scalar_term), d = augmented dimension; level-major,
 * row-major words inside a level.
 * Replaces: siglib/cusig/cu_signature.cu:3497-3517 (signature_cuda_f / _d),
 * bound by pysiglib/load_siglib.py:484-488, called from pysiglib/sig.py:288-294. */
CUSIG_AMD_API int signature_cuda_f(const float* path, float* out, uint64_t batch_size, uint64_t dimension,
                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag, float end_time,
                                   bool horner, bool scalar_term, const float* correction,
                                   uint64_t correction_len, uint64_t correction_batch_stride,
                                   uint64_t correction_segment_stride) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int signature_cuda_d(const double* path, double* out, uint64_t batch_size, uint64_t dimension,
                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                   double end_time, bool horner, bool scalar_term, const double* correction,
                                   uint64_t correction_len, uint64_t correction_batch_stride,
                                   uint64_t correction_segment_stride) CUSIG_AMD_NOEXCEPT;

/* Gradient of a scalar loss w.r.t. the raw path, given the signature and the
 * loss gradient w.r.t. the signature (both [batch, S], same layout as above).
 * out [batch, length, dimension] is fully overwritten.
 * Replaces: siglib/cusig/cu_signature.cu:3524-3544 (sig_backprop_cuda_f / _d),
 * bound by pysiglib/load_siglib.py:490-494, called from pysiglib/sig_backprop.py:245-251. */
CUSIG_AMD_API int sig_backprop_cuda_f(const float* path, float* out, const float* sig_derivs, const float* sig,
                                      uint64_t batch_size, uint64_t dimension, uint64_t length, uint64_t degree,
                                      bool time_aug, bool lead_lag, float end_time, bool scalar_term,
                                      const float* correction, uint64_t correction_len,
                                      uint64_t correction_batch_stride,
                                      uint64_t correction_segment_stride) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_backprop_cuda_d(const double* path, double* out, const double* sig_derivs,
                                      const double* sig, uint64_t batch_size, uint64_t dimension,
                                      uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                      double end_time, bool scalar_term, const double* correction,
                                      uint64_t correction_len, uint64_t correction_batch_stride,
                                      uint64_t correction_segment_stride) CUSIG_AMD_NOEXCEPT;

/* sig_backprop_cuda_d for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * sig_backprop_cuda_d without the correction (none is applied), plus the stream (a hipStream_t; null = the null
 * stream) on which the kernels are enqueued.  The call does not wait: inputs must be ready on that stream, and the
 * result is ready when the stream reaches the end of the enqueued work.  Every buffer the kernels need beyond the
 * arguments (increments, increment gradient) lives in a fixed array of cusig_amd_noalloc_scratch_bytes() = 32 MiB
 * inside the library, one copy per GPU, held until the process ends; shapes that need more return status 2 before
 * anything is launched.  The call makes no hipMalloc / hipFree and uses no allocating library routine; paths are
 * always swept whole (no time split).  All calls on one GPU share that array: calls whose kernels may overlap on one
 * GPU (different streams, several threads) race. */
CUSIG_AMD_API int cusig_amd_sig_backprop_noalloc_d(const double* path, double* out, const double* sig_derivs,
                                                   const double* sig, uint64_t batch_size, uint64_t dimension,
                                                   uint64_t length, uint64_t degree, bool time_aug, bool lead_lag,
                                                   double end_time, bool scalar_term, void* stream) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API uint64_t cusig_amd_noalloc_scratch_bytes(void) CUSIG_AMD_NOEXCEPT;

/* Chen product of two signatures per batch item: out = sig1 (x) sig2, all [batch, S(+1)].
 * Replaces: siglib/cusig/cu_sig_combine.cu:157-169 (decl siglib/cusig/cusig.h:364-365),
 * bound by pysiglib/load_siglib.py:450-454, called from pysiglib/sig.py:113-121. */
CUSIG_AMD_API int sig_combine_cuda_f(const float* sig1, const float* sig2, float* out, uint64_t batch_size,
                                     uint64_t dimension, uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_combine_cuda_d(const double* sig1, const double* sig2, double* out, uint64_t batch_size,
                                     uint64_t dimension, uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Gradients of a loss w.r.t. sig1 and sig2 given its gradient w.r.t. sig1 (x) sig2 (scalar slots get 0).
 * Replaces: siglib/cusig/cu_sig_combine.cu:323-337 (decl siglib/cusig/cusig.h:387-388),
 * bound by pysiglib/load_siglib.py:466-471. */
CUSIG_AMD_API int sig_combine_backprop_cuda_f(const float* sig_combined_deriv, float* sig1_deriv, float* sig2_deriv,
                                              const float* sig1, const float* sig2, uint64_t batch_size,
                                              uint64_t dimension, uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_combine_backprop_cuda_d(const double* sig_combined_deriv, double* sig1_deriv, double* sig2_deriv,
                                              const double* sig1, const double* sig2, uint64_t batch_size,
                                              uint64_t dimension, uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Materialises the lead-lag / time augmentation: data_in [batch, length, dimension] ->
 * data_out [batch, len_eff, d_eff].
 * Replaces: siglib/cusig/cu_path_transforms.cu:48-127 (decl siglib/cusig/cusig.h:66-67),
 * bound by pysiglib/load_siglib.py:420-424, called from pysiglib/transform_path.py. */
CUSIG_AMD_API int transform_path_cuda_f(const float* data_in, float* data_out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t length, bool time_aug, bool lead_lag, float end_time) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int transform_path_cuda_d(const double* data_in, double* data_out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t length, bool time_aug, bool lead_lag, double end_time) CUSIG_AMD_NOEXCEPT;

/* Adjoint of the augmentation: derivs [batch, len_eff, d_eff] -> data_out [batch, length, dimension].
 * Replaces: siglib/cusig/cu_path_transforms.cu:129-205 (decl siglib/cusig/cusig.h:91-92),
 * bound by pysiglib/load_siglib.py:425-429. */
CUSIG_AMD_API int transform_path_backprop_cuda_f(const float* derivs, float* data_out, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t length, bool time_aug, bool lead_lag,
                                                 float end_time) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int transform_path_backprop_cuda_d(const double* derivs, double* data_out, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t length, bool time_aug, bool lead_lag,
                                                 double end_time) CUSIG_AMD_NOEXCEPT;

/* Signature of each straight-line displacement [batch, dimension] -> [batch, sig_length - !scalar_term].
 * Replaces: linear_sig_cuda_{f,d} (decl siglib/cusig/cusig.h:942-944; arithmetic siglib/cpsig/cp_sig_join.h:36-104),
 * bound by pysiglib/load_siglib.py (CUSIG_LINEAR_SIG), called from pysiglib/linear_sig.py. */
CUSIG_AMD_API int linear_sig_cuda_f(const float* displacement, float* out, uint64_t batch_size, uint64_t dimension,
                                    uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int linear_sig_cuda_d(const double* displacement, double* out, uint64_t batch_size, uint64_t dimension,
                                    uint64_t degree, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Appends (or prepends) one straight-line segment to each signature: out = sig (x) exp(z), resp. exp(z) (x) sig.
 * Replaces: sig_join_cuda_{f,d} (decl siglib/cusig/cusig.h:962-964; arithmetic siglib/cpsig/cp_sig_join.h:107-160),
 * bound by pysiglib/load_siglib.py:456-460, called from pysiglib/sig_join.py. */
CUSIG_AMD_API int sig_join_cuda_f(const float* sig, const float* displacement, float* out, uint64_t batch_size,
                                  uint64_t dimension, uint64_t degree, bool prepend, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_join_cuda_d(const double* sig, const double* displacement, double* out, uint64_t batch_size,
                                  uint64_t dimension, uint64_t degree, bool prepend, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Gradients of sig_join w.r.t. the signature (scalar slot zero) and the displacement.
 * Replaces: sig_join_backprop_cuda_{f,d} (decl siglib/cusig/cusig.h:984-986; arithmetic
 * siglib/cpsig/cp_sig_join.h:163-238), bound by pysiglib/load_siglib.py:461-465, called from
 * pysiglib/sig_join_backprop.py. */
CUSIG_AMD_API int sig_join_backprop_cuda_f(const float* d_out, float* d_sig, float* d_displacement, const float* sig,
                                           const float* displacement, uint64_t batch_size, uint64_t dimension,
                                           uint64_t degree, bool prepend, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_join_backprop_cuda_d(const double* d_out, double* d_sig, double* d_displacement, const double* sig,
                                           const double* displacement, uint64_t batch_size, uint64_t dimension,
                                           uint64_t degree, bool prepend, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Coefficients of selected words.  multi_idx: the words' letters end to end, degrees: their lengths (both uint64, on
 * the device); out [batch, num_multi_idx], or with `prefixes` per word the coefficients of all its non-empty
 * prefixes (one entry, 1, for the empty word).  Augmentations are applied beforehand (transform_path_cuda).
 * Replaces: sig_coef_cuda_{f,d} (decl siglib/cusig/cusig.h:468-470; arithmetic
 * siglib/cpsig/cp_sig_coef_impl.cpp:35-84,138-348), bound by pysiglib/load_siglib.py (CUSIG_SIG_COEF), called from
 * pysiglib/sig_coef.py. */
CUSIG_AMD_API int sig_coef_cuda_f(const float* path, float* out, const uint64_t* multi_idx, uint64_t num_multi_idx,
                                  const uint64_t* degrees, uint64_t batch_size, uint64_t dimension, uint64_t length,
                                  bool prefixes) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_coef_cuda_d(const double* path, double* out, const uint64_t* multi_idx, uint64_t num_multi_idx,
                                  const uint64_t* degrees, uint64_t batch_size, uint64_t dimension, uint64_t length,
                                  bool prefixes) CUSIG_AMD_NOEXCEPT;

/* Path gradient given dF/d(prefix coefficients); coefs and derivs have the `prefixes` layout of sig_coef_cuda.
 * Replaces: sig_coef_backprop_cuda_{f,d} (decl siglib/cusig/cusig.h:492-494; arithmetic
 * siglib/cpsig/cp_sig_coef_impl.cpp:360-485), bound by pysiglib/load_siglib.py (CUSIG_SIG_COEF_BACKPROP), called from
 * pysiglib/sig_coef_backprop.py. */
CUSIG_AMD_API int sig_coef_backprop_cuda_f(const float* path, float* out, const float* coefs, const float* derivs,
                                           const uint64_t* multi_idx, uint64_t num_multi_idx, const uint64_t* degrees,
                                           uint64_t batch_size, uint64_t dimension, uint64_t length) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_coef_backprop_cuda_d(const double* path, double* out, const double* coefs, const double* derivs,
                                           const uint64_t* multi_idx, uint64_t num_multi_idx, const uint64_t* degrees,
                                           uint64_t batch_size, uint64_t dimension, uint64_t length) CUSIG_AMD_NOEXCEPT;

/* Logarithm of each signature.  method 0: expanded (tensor) logarithm, same row layout in and out, scalar slot of
 * the result 0.  method 1: its coefficients at the Lyndon words, method 2: its coordinates in the Lyndon basis; both
 * write rows of log_sig_length(dimension, degree) values (no scalar slot) and need prepare_log_sig_cuda first
 * (status 5 otherwise).
 * Replaces: sig_to_log_sig_cuda_{f,d} (decl siglib/cusig/cusig.h:407-409; arithmetic siglib/cpsig/cp_tensor_log.h:40-170),
 * bound by pysiglib/load_siglib.py (CUSIG_SIG_TO_LOG_SIG), called from pysiglib/log_sig.py:223-311. */
CUSIG_AMD_API int sig_to_log_sig_cuda_f(const float* sig, float* out, uint64_t batch_size, uint64_t dimension, uint64_t degree,
                                        int method, bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_to_log_sig_cuda_d(const double* sig, double* out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t degree, int method, bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Prepares the tables of methods 1 and 2 for (dimension, degree) on the current device; preparing method 2 also
 * serves method 1; method 0 needs nothing; method 3 (BCH) returns status 10.  use_disk is accepted and ignored.
 * Replaces: prepare_log_sig_cuda (siglib/cusig/cusig.h:447; tables of siglib/shared/preparation/log_sig/lyndon_words.cpp),
 * bound by pysiglib/load_siglib.py:166-167, called from pysiglib/log_sig.py:93-187. */
CUSIG_AMD_API int prepare_log_sig_cuda(uint64_t dimension, uint64_t degree, int method, bool use_disk) CUSIG_AMD_NOEXCEPT;
/* Host-only view of the tables prepare_log_sig_cuda builds (needs no GPU; no counterpart in the reference's ABI): call
 * with null arrays for the sizes, then with `count` indices (positions of the Lyndon words in a scalar-free signature
 * row), `count + 1` row offsets and `nnz` columns / values of the strictly lower part of the inverse projection
 * (unit diagonal implicit; empty for method 1). */
CUSIG_AMD_API int cusig_amd_lyndon_tables(uint64_t dimension, uint64_t degree, int method, uint64_t* count, uint64_t* nnz,
                                          uint64_t* index, uint64_t* row_ptr, uint32_t* col, int32_t* val) CUSIG_AMD_NOEXCEPT;
/* Drops every prepared table.  Replaces: clear_cache_cuda (siglib/cusig/cusig.h:626), bound by
 * pysiglib/load_siglib.py:169-170, called from pysiglib/log_sig.py:190-240. */
CUSIG_AMD_API int clear_cache_cuda(bool use_disk) CUSIG_AMD_NOEXCEPT;

/* Gradient w.r.t. the signature given dF/d(log signature) (rows in the layout of `method`); scalar slot of the result 0.
 * Replaces: sig_to_log_sig_backprop_cuda_{f,d} (decl siglib/cusig/cusig.h:429-431; arithmetic
 * siglib/cpsig/cp_tensor_log.h:164-221), bound by pysiglib/load_siglib.py (CUSIG_SIG_TO_LOG_SIG_BACKPROP), called from
 * pysiglib/log_sig_backprop.py:30-137. */
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_f(const float* sig, float* out, const float* log_sig_derivs, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t degree, int method,
                                                 bool scalar_term) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_d(const double* sig, double* out, const double* log_sig_derivs,
                                                 uint64_t batch_size, uint64_t dimension, uint64_t degree, int method,
                                                 bool scalar_term) CUSIG_AMD_NOEXCEPT;

/* Message of the last failing call made by the calling thread ("" if none).
 * Replaces: cusig_last_error_message, probed by pysiglib/load_siglib.py:108-110
 * and read by pysiglib/error_codes.py:28-42. */
CUSIG_AMD_API const char* cusig_last_error_message(void) CUSIG_AMD_NOEXCEPT;

/* Releases the library's device workspaces; idempotent, never fails.
 * Replaces: siglib/cusig/cache_lifecycle/cusig_lifecycle.cu:31-50, registered at
 * interpreter exit by pysiglib/load_siglib.py:647-664. */
CUSIG_AMD_API void cusig_shutdown(void) CUSIG_AMD_NOEXCEPT;

/* (d^(degree+1) - 1)/(d - 1), 0 on 64-bit overflow.  Same contract as the CPU
 * library's sig_length (siglib/cpsig/cp_utils.cpp:91-105), which the reference's
 * Python wrapper calls to size its outputs (pysiglib/sig_length.py:91-94). */
CUSIG_AMD_API uint64_t cusig_amd_sig_length(uint64_t dimension, uint64_t degree) CUSIG_AMD_NOEXCEPT;

/* Measurement hooks used by the benchmark (no counterpart in the reference):
 * when enabled, the sweep kernel of every following call is bracketed with HIP
 * events on the stream it is launched on. */
CUSIG_AMD_API void cusig_amd_set_profiling(int enabled) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API float cusig_amd_last_kernel_ms(void) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API const char* cusig_amd_last_kernel_name(void) CUSIG_AMD_NOEXCEPT;
/* Measured ceiling of the vector multiply-add pipe: runs a kernel of independent FMAs (float64 or float32, unpacked) with
 * `waves_per_simd` (1..8) waves on every SIMD of the current device and stores the achieved TFLOP/s.  The benchmark
 * reports it beside the nominal peak.  Synchronous; returns a status like the operators.  No counterpart in the reference. */
CUSIG_AMD_API int cusig_amd_measure_fma_peak(int is_f64, int waves_per_simd, double* tflops) CUSIG_AMD_NOEXCEPT;
/* Whether the last signature_cuda_* call on this thread stored a NaN or an infinity: 1 yes, 0 no, -1 not
 * reported (the call failed, or ran in stream-ordered mode, where the answer is not known at return).  The
 * kernels that store the result set the flag, so a caller who must warn about overflow (pysiglib/sig.py:299-311
 * scans the result for NaN and Inf) needs no pass of its own over the output.  No counterpart in the reference. */
CUSIG_AMD_API int cusig_amd_last_sig_nonfinite(void) CUSIG_AMD_NOEXCEPT;
/* The tuning and test hooks declared from here on (cusig_amd_force_*, cusig_amd_set_point_fed, _set_lead_lag_sparse,
 * _set_chen_low_levels, _set_degree2_staged, _set_alloc_limit) are process-wide switches for offline sweeps and for the
 * test-suite.  They are ignored until cusig_amd_enable_test_hooks(1) has been called; cusig_amd_enable_test_hooks(0)
 * restores every default.  No counterpart in the reference. */
CUSIG_AMD_API void cusig_amd_enable_test_hooks(int enabled) CUSIG_AMD_NOEXCEPT;
/* Test hook: workspace requests of more than `bytes` bytes fail as if the device were out of memory (0: no limit), which
 * exercises the retry on halves of the batch (siglib/cusig/cu_runtime_utils.h:103-105,212-235) and the fall-back of the
 * degree-3 matrix form to the sweeps.  cusig_amd_alloc_retries counts the splits since the library was loaded. */
CUSIG_AMD_API void cusig_amd_set_alloc_limit(uint64_t bytes) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API int cusig_amd_alloc_retries(void) CUSIG_AMD_NOEXCEPT;
/* Bytes the library's grow-only workspace pool holds on the current device (released by cusig_shutdown).  A host-side
 * query; no counterpart in the reference. */
CUSIG_AMD_API uint64_t cusig_amd_workspace_bytes(void) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: number of time segments the forward sweep splits every path into (0 = automatic). */
CUSIG_AMD_API void cusig_amd_force_segments(int segments) CUSIG_AMD_NOEXCEPT;
/* Number of time segments per path in the last forward sweep on this thread (0 if no sweep kernel ran). */
CUSIG_AMD_API int cusig_amd_last_segments(void) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: 0 makes every forward sweep read increments computed by a kernel of their own; 1 (default) lets
 * the LDS-staged sweeps of plain paths (no time or lead-lag augmentation) of at most 16 channels take the
 * differences of consecutive points while they stage them. */
CUSIG_AMD_API void cusig_amd_set_point_fed(int on) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: 1 (default) lets the forward and backward sweeps of lead-lag paths that have such a form (up to 40
 * augmented channels; the LDS-staged kernels and the wider scalar-fed backward kernels) skip, in every step, the
 * multiply-adds by the channels that step cannot move (lead and lag halves move in turn; the increments there are
 * exactly zero and their gradients never reach the path gradient); 0 sweeps them like any other path. */
CUSIG_AMD_API void cusig_amd_set_lead_lag_sparse(int on) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: number of time segments the backward sweep splits every path into (0 = automatic, 1 = never). */
CUSIG_AMD_API void cusig_amd_force_bwd_segments(int segments) CUSIG_AMD_NOEXCEPT;
/* Test hook: 1 (default) lets single-precision backward sweeps of 33 and more augmented channels at degrees 3 .. 8 that
 * the compiled instance table does not cover run the by-row reverse sweep (a wave holds its tile of top-level adjoints
 * both by prefix and by letter, so no per-step reduction across lanes is left); 0 sends them to the general run-time
 * kernels. */
CUSIG_AMD_API void cusig_amd_set_rows_backward(int on) CUSIG_AMD_NOEXCEPT;
/* Test hook: the same switch for the forward sweep of such shapes (33 and more channels without a compiled instance,
 * degrees 3 .. 8): 1 (default) runs the by-row forward sweep (64 or 32 top-level letters per lane), 0 the general
 * run-time kernels. */
CUSIG_AMD_API void cusig_amd_set_rows_forward(int on) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: how increments reach the waves: -1 automatic, 0 scalar loads, 1 LDS-staged where compiled. */
CUSIG_AMD_API void cusig_amd_force_staged(int mode) CUSIG_AMD_NOEXCEPT;
/* Test hook: nonzero makes the coefficient-per-thread kernels use their 64-bit index arithmetic (otherwise only
 * taken for rows of 2^31 coefficients or more) whatever the size. */
CUSIG_AMD_API void cusig_amd_force_wide_index(int enabled) CUSIG_AMD_NOEXCEPT;
/* Test hook: kernels of the Chen product's adjoint (sig_combine_backprop, sig_join_backprop, the tensor logarithm's
 * backward, time-split sig_backprop): 0 = streaming kernels for rows of 4096 coefficients or more, 1 = streaming
 * kernels wherever they apply, 2 = item-per-word kernels only. */
CUSIG_AMD_API void cusig_amd_force_chen_adjoint(int mode) CUSIG_AMD_NOEXCEPT;
/* Test hook: the Chen product kernels of sig_combine and of the tensor logarithm can keep the factors' short levels in
 * LDS: 0 = never, 1 (default) = for float64 rows of large launches, 2 = always. */
CUSIG_AMD_API void cusig_amd_set_chen_low_levels(int enabled) CUSIG_AMD_NOEXCEPT;
/* Stream-ordered mode (no counterpart in the reference, off by default).  When enabled, signature_cuda_{f,d} and
 * sig_backprop_cuda_{f,d} enqueue their kernels on the null stream and return without waiting, and do not wait for
 * other streams on entry: inputs must be ordered before, and consumers after, the null stream (true for PyTorch's
 * default stream and for blocking streams).  Kernel faults then surface at the caller's next synchronisation.
 * Process-wide. */
CUSIG_AMD_API void cusig_amd_set_stream_ordered(int enabled) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: the closed-form degree-2 kernels (matrix cores): -1 automatic, 0 never, 1 whenever the degree is 2. */
CUSIG_AMD_API void cusig_amd_force_degree2(int mode) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: degree 3 as rocBLAS matrix products around a scan kernel (backward: two products, forward: one):
 * -1 automatic (backward from 48 channels in float32 and 36 in float64, forward from 112, given enough paths to fill
 * the chip, a librocblas that can be opened and a device that can hold the extra rows buffer of up to 1 GiB; otherwise
 * the sweeps serve the shape), 0 never, 1 whenever the degree is 3 and one path's rows fit the buffer. */
CUSIG_AMD_API void cusig_amd_force_degree3(int mode) CUSIG_AMD_NOEXCEPT;
/* Test hook: 1 routes every sweep of 2, 3 or 4 augmented channels that the run-time-degree kernels can serve
 * (degree >= 5, 4, 3 respectively) to them; by default they only serve degrees 17 .. 64. */
CUSIG_AMD_API void cusig_amd_force_deep(int enabled) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: 0 makes the degree-2 kernels build their operands straight from global memory instead of staging
 * them through LDS (the path taken anyway when a chunk of all channels does not fit). */
CUSIG_AMD_API void cusig_amd_set_degree2_staged(int enabled) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: with a forced partition, shapes served by a run-time-dimension kernel take its wide-layout variant. */
/* Tuning hook: nonzero makes every shape run the run-time-dimension kernels (and the by-row reverse sweep where it
 * applies), as if the shape had no compiled instance: the yardstick for deciding which instances earn their place. */
CUSIG_AMD_API void cusig_amd_ignore_instance_table(int on) CUSIG_AMD_NOEXCEPT;
CUSIG_AMD_API void cusig_amd_force_run_time_wide(int enabled) CUSIG_AMD_NOEXCEPT;
/* Tuning hook: prefer the compiled lane partition (tail, k) where a shape has several; tail = 0 restores
 * the defaults.  Not thread-safe; meant for offline sweeps. */
CUSIG_AMD_API void cusig_amd_force_partition(int tail, int k) CUSIG_AMD_NOEXCEPT;
/* Which kernel instance serves (dtype, augmented dimension, degree): returns 1 and
 * fills tail / k / specialised, or 0 if the shape has no kernel. */
CUSIG_AMD_API int cusig_amd_kernel_choice(int backward, int is_f64, uint64_t dimension, uint64_t degree,
                                          int* tail, int* k, int* specialised) CUSIG_AMD_NOEXCEPT;

#ifdef __cplusplus
}
#endif
#endif /* CUSIG_AMD_H */
