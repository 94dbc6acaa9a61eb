/*
 * sigref.h -- CPU oracle for the truncated path signature (TEST INFRASTRUCTURE ONLY).
 *
 * A dependency-free C restatement of the reference CPU library's forward and
 * backward signature algorithm.  It exists to check the GPU library and to be
 * timed as the CPU baseline; nothing in the shipped package may link or call it.
 */
#ifndef SIGREF_H
#define SIGREF_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* siglib/cpsig/cp_utils.cpp:91-105: (d^(N+1)-1)/(d-1); 0 on uint64 overflow. */
uint64_t sigref_sig_length(uint64_t dimension, uint64_t degree);
/* siglib/cpsig/cp_utils.cpp:40-50: level_index[k] = (d^k-1)/(d-1), n entries. */
int sigref_level_index(uint64_t *level_index, uint64_t dimension, uint64_t n);
/* number of hardware threads n_jobs = -1 resolves to */
int sigref_max_threads(void);
/* siglib/cpsig/multithreading.cpp:43-81: contiguous chunks over min(threads, batch) workers. */
void sigref_run_batch(uint64_t batch, int n_jobs, void *ctx, void (*worker)(void *, uint64_t, uint64_t));

/* Same argument meaning as the reference's signature_{f,d} / sig_backprop_{f,d}
 * (siglib/cpsig/cpsig.h:311-346) without the correction arguments.
 * Return 0 ok, 1 out of memory, 2 invalid argument, 10 overflow. */
int sigref_signature_f(const float *path, float *out, uint64_t batch, uint64_t dimension,
                       uint64_t length, uint64_t degree, int time_aug, int lead_lag,
                       float end_time, int horner, int scalar_term, int n_jobs);
int sigref_signature_d(const double *path, double *out, uint64_t batch, uint64_t dimension,
                       uint64_t length, uint64_t degree, int time_aug, int lead_lag,
                       double end_time, int horner, int scalar_term, int n_jobs);
int sigref_sig_backprop_f(const float *path, float *out, const float *sig_derivs, const float *sig,
                          uint64_t batch, uint64_t dimension, uint64_t length, uint64_t degree,
                          int time_aug, int lead_lag, float end_time, int scalar_term, int n_jobs);
int sigref_sig_backprop_d(const double *path, double *out, const double *sig_derivs, const double *sig,
                          uint64_t batch, uint64_t dimension, uint64_t length, uint64_t degree,
                          int time_aug, int lead_lag, double end_time, int scalar_term, int n_jobs);
/* Operators either side of the signature path, same argument meaning as the reference's
 * sig_combine_{f,d}, sig_combine_backprop_{f,d}, transform_path_{f,d}, transform_path_backprop_{f,d}
 * (siglib/cpsig/cpsig.h) without n_jobs. */
int sigref_sig_combine_f(const float *sig1, const float *sig2, float *out, uint64_t batch, uint64_t dimension,
                         uint64_t degree, int scalar_term);
int sigref_sig_combine_d(const double *sig1, const double *sig2, double *out, uint64_t batch, uint64_t dimension,
                         uint64_t degree, int scalar_term);
int sigref_sig_combine_backprop_f(const float *dout, float *d1, float *d2, const float *sig1, const float *sig2,
                                  uint64_t batch, uint64_t dimension, uint64_t degree, int scalar_term);
int sigref_sig_combine_backprop_d(const double *dout, double *d1, double *d2, const double *sig1, const double *sig2,
                                  uint64_t batch, uint64_t dimension, uint64_t degree, int scalar_term);
int sigref_transform_path_f(const float *in, float *out, uint64_t batch, uint64_t dimension, uint64_t length,
                            int time_aug, int lead_lag, float end_time);
int sigref_transform_path_d(const double *in, double *out, uint64_t batch, uint64_t dimension, uint64_t length,
                            int time_aug, int lead_lag, double end_time);
int sigref_transform_path_backprop_f(const float *derivs, float *out, uint64_t batch, uint64_t dimension,
                                     uint64_t length, int time_aug, int lead_lag);
int sigref_transform_path_backprop_d(const double *derivs, double *out, uint64_t batch, uint64_t dimension,
                                     uint64_t length, int time_aug, int lead_lag);
/* linear_sig_{f,d}, sig_join_{f,d}, sig_join_backprop_{f,d} of the reference (siglib/cpsig/cpsig.h) without n_jobs. */
int sigref_linear_sig_f(const float *displacement, float *out, uint64_t batch, uint64_t dimension, uint64_t degree,
                        int scalar_term);
int sigref_sig_join_f(const float *sig, const float *displacement, float *out, uint64_t batch, uint64_t dimension,
                      uint64_t degree, int prepend, int scalar_term);
int sigref_sig_join_backprop_f(const float *dout, float *dsig, float *ddisplacement, const float *sig,
                               const float *displacement, uint64_t batch, uint64_t dimension, uint64_t degree,
                               int prepend, int scalar_term);
int sigref_linear_sig_d(const double *displacement, double *out, uint64_t batch, uint64_t dimension, uint64_t degree,
                        int scalar_term);
int sigref_sig_join_d(const double *sig, const double *displacement, double *out, uint64_t batch, uint64_t dimension,
                      uint64_t degree, int prepend, int scalar_term);
int sigref_sig_join_backprop_d(const double *dout, double *dsig, double *ddisplacement, const double *sig,
                               const double *displacement, uint64_t batch, uint64_t dimension, uint64_t degree,
                               int prepend, int scalar_term);
/* sig_coef_{f,d}, sig_coef_backprop_{f,d} of the reference (siglib/cpsig/cpsig.h) without n_jobs. */
int sigref_sig_coef_f(const float *path, float *out, const uint64_t *multi_idx, uint64_t num_multi_idx,
                      const uint64_t *degrees, uint64_t batch, uint64_t dimension, uint64_t length, int time_aug,
                      int lead_lag, float end_time, int prefixes);
int sigref_sig_coef_backprop_f(const float *path, float *out, const float *coefs, const float *derivs,
                               const uint64_t *multi_idx, uint64_t num_multi_idx, const uint64_t *degrees, uint64_t batch,
                               uint64_t dimension, uint64_t length, int time_aug, int lead_lag, float end_time);
int sigref_sig_coef_d(const double *path, double *out, const uint64_t *multi_idx, uint64_t num_multi_idx,
                      const uint64_t *degrees, uint64_t batch, uint64_t dimension, uint64_t length, int time_aug,
                      int lead_lag, double end_time, int prefixes);
int sigref_sig_coef_backprop_d(const double *path, double *out, const double *coefs, const double *derivs,
                               const uint64_t *multi_idx, uint64_t num_multi_idx, const uint64_t *degrees, uint64_t batch,
                               uint64_t dimension, uint64_t length, int time_aug, int lead_lag, double end_time);
/* sig_to_log_sig_{f,d} and its backprop with method 0 (expanded tensor logarithm), dimension already augmented. */
int sigref_sig_to_log_sig_f(const float *sig, float *out, uint64_t batch, uint64_t dimension, uint64_t degree,
                            int scalar_term);
int sigref_sig_to_log_sig_backprop_f(const float *sig, float *out, const float *log_sig_derivs, uint64_t batch,
                                     uint64_t dimension, uint64_t degree, int scalar_term);
int sigref_sig_to_log_sig_d(const double *sig, double *out, uint64_t batch, uint64_t dimension, uint64_t degree,
                            int scalar_term);
int sigref_sig_to_log_sig_backprop_d(const double *sig, double *out, const double *log_sig_derivs, uint64_t batch,
                                     uint64_t dimension, uint64_t degree, int scalar_term);
#ifdef __cplusplus
}
#endif
#endif
