/*
 * xcorr_fft.h - C ABI of libxcorr_fft.so, the FFT-based comparison path of the cross-correlation
 * benchmark on MI355X (hipFFT + three small HIP kernels).
 *
 * The reference compares its definition-based kernels with cross-correlation through the
 * convolution theorem: zero-pad both inputs to twice their size, forward real-to-complex
 * FFT, multiply the left spectrum with the conjugate of the right one ("hadamard"),
 * inverse FFT; the un-normalised circular result is brought into the definition's layout
 * on the host (fft_helpers.hpp:193-262). This library provides the device side of that
 * path: plan objects in place of the cufftHandle calls of fft_helpers.hpp:113-192 and
 * the launchers run_hadamard_original, run_hadamard_n_to_m_over_right,
 * run_hadamard_n_to_m_over_output (kernels.cuh:7-39) and run_scatter (kernels.cuh:53-63).
 *
 * Conventions as in xcorr_hip.h: caller-owned device pointers, asynchronous on the given
 * stream (NULL = default stream), int status (XCORR_OK = 0), message from
 * xcorr_fft_last_error(). Complex data are interleaved (re, im) pairs of the element type;
 * a real-to-complex transform of a rows x cols matrix has rows x (cols/2 + 1) complex
 * elements.
 */
#ifndef XCORR_FFT_H
#define XCORR_FFT_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *xcorr_fft_last_error(void);

/* Batched 2-D transforms of `batch` contiguous rows x cols matrices; elem_bytes 4 (float)
 * or 8 (double). Forward: real -> complex (cufftPlanMany(..., R2C/D2Z, batch), e.g.
 * one_to_one.hpp:938-941); inverse: complex -> real, un-normalised (C2R/Z2D). */
int xcorr_fft_plan_forward(void **plan, unsigned rows, unsigned cols, unsigned batch, unsigned elem_bytes);
int xcorr_fft_plan_inverse(void **plan, unsigned rows, unsigned cols, unsigned batch, unsigned elem_bytes);
int xcorr_fft_plan_set_stream(void *plan, void *stream);
/* fft_real_to_complex / fft_complex_to_real (fft_helpers.hpp:113-192); the inverse transform may
 * overwrite its input */
int xcorr_fft_exec_forward(void *plan, const void *real_in, void *complex_out);
int xcorr_fft_exec_inverse(void *plan, void *complex_in, void *real_out);
int xcorr_fft_plan_destroy(void *plan);

/* deformed[b][i] = ref[i] * conj(deformed[b][i]) for the `batch` strips of
 * `subregions_per_pic` spectra (run_hadamard_original, kernels.cuh:7-15; hadamard.cu:34-55).
 * fft_cols x fft_rows is the size of one spectrum in complex elements. */
int xcorr_hadamard_original_f32(const void *ref, void *deformed, unsigned fft_cols, unsigned fft_rows, unsigned subregions_per_pic,
                                unsigned batch, unsigned threads_per_block, void *stream);
int xcorr_hadamard_original_f64(const void *ref, void *deformed, unsigned fft_cols, unsigned fft_rows, unsigned subregions_per_pic,
                                unsigned batch, unsigned threads_per_block, void *stream);

/* out[l * n_right + r] = left[l] * conj(right[r]) for all pairs. over_right: a thread keeps a
 * right value in a register and walks the left spectra (run_hadamard_n_to_m_over_right,
 * kernels.cuh:17-27); over_output: one output element per thread and step
 * (run_hadamard_n_to_m_over_output, kernels.cuh:29-39). */
int xcorr_hadamard_n_to_m_over_right_f32(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                         unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                         void *stream);
int xcorr_hadamard_n_to_m_over_right_f64(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                         unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                         void *stream);
int xcorr_hadamard_n_to_m_over_output_f32(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                          unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                          void *stream);
int xcorr_hadamard_n_to_m_over_output_f64(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                          unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                          void *stream);

/* Copies `n` dense src_rows x src_cols matrices into the top-left corner (offset dst_x, dst_y)
 * of `n` dst_rows x dst_cols matrices, i.e. zero padding on the device when `dst` was cleared
 * (run_scatter, kernels.cuh:53-63; the reference's kernel takes the column index modulo the row
 * count, scatter.cu:38, which is only right for square matrices - not reproduced). */
int xcorr_scatter_f32(const float *src, float *dst, unsigned src_cols, unsigned src_rows, unsigned n, unsigned dst_cols,
                      unsigned dst_rows, unsigned dst_x, unsigned dst_y, unsigned threads_per_block, unsigned items_per_thread,
                      void *stream);
int xcorr_scatter_f64(const double *src, double *dst, unsigned src_cols, unsigned src_rows, unsigned n, unsigned dst_cols,
                      unsigned dst_rows, unsigned dst_x, unsigned dst_y, unsigned threads_per_block, unsigned items_per_thread,
                      void *stream);

#ifdef __cplusplus
}
#endif

#endif
