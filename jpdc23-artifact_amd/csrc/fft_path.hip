// Device side of the FFT-based comparison path: hipFFT plans behind opaque handles and the
// element-wise kernels between the transforms (reference fft_helpers.hpp, hadamard.cu,
// scatter.cu). Built into its own library so that programs which only use the
// definition-based kernels do not load rocFFT.
#include <hip/hip_runtime.h>
#include <hipfft/hipfft.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/xcorr_fft.h"

namespace {

constexpr int OK = 0, ERR_INVALID_ARGUMENT = 1, ERR_RUNTIME = 2; // the codes of xcorr_hip.h

thread_local char error_text[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_text, sizeof(error_text), fmt, ap);
    va_end(ap);
    return code;
}

const char *fft_status_name(hipfftResult r) {
    switch (r) {
    case HIPFFT_SUCCESS: return "HIPFFT_SUCCESS";
    case HIPFFT_INVALID_PLAN: return "HIPFFT_INVALID_PLAN";
    case HIPFFT_ALLOC_FAILED: return "HIPFFT_ALLOC_FAILED";
    case HIPFFT_INVALID_TYPE: return "HIPFFT_INVALID_TYPE";
    case HIPFFT_INVALID_VALUE: return "HIPFFT_INVALID_VALUE";
    case HIPFFT_INTERNAL_ERROR: return "HIPFFT_INTERNAL_ERROR";
    case HIPFFT_EXEC_FAILED: return "HIPFFT_EXEC_FAILED";
    case HIPFFT_SETUP_FAILED: return "HIPFFT_SETUP_FAILED";
    case HIPFFT_INVALID_SIZE: return "HIPFFT_INVALID_SIZE";
    case HIPFFT_UNALIGNED_DATA: return "HIPFFT_UNALIGNED_DATA";
    case HIPFFT_NOT_SUPPORTED: return "HIPFFT_NOT_SUPPORTED";
    default: return "<unknown>";
    }
}

#define FFT_CALL(expr)                                                                                        \
    do {                                                                                                      \
        hipfftResult r_ = (expr);                                                                             \
        if (r_ != HIPFFT_SUCCESS) return fail(ERR_RUNTIME, "hipFFT error %d: %s in %s", (int)r_, fft_status_name(r_), #expr); \
    } while (0)

#define HIP_CALL(expr)                                                                                                 \
    do {                                                                                                               \
        hipError_t e_ = (expr);                                                                                        \
        if (e_ != hipSuccess) return fail(ERR_RUNTIME, "HIP error %d: %s in %s", (int)e_, hipGetErrorString(e_), #expr); \
    } while (0)

struct Plan {
    hipfftHandle handle;
    bool forward;
    unsigned elem_bytes;
};

int make_plan(void **out, unsigned rows, unsigned cols, unsigned batch, unsigned elem_bytes, bool forward) {
    if (!out) return fail(ERR_INVALID_ARGUMENT, "null plan pointer");
    if (rows == 0 || cols == 0 || batch == 0) return fail(ERR_INVALID_ARGUMENT, "empty transform: %u x %u, batch %u", rows, cols, batch);
    if (elem_bytes != 4 && elem_bytes != 8) return fail(ERR_INVALID_ARGUMENT, "element size %u is neither 4 nor 8", elem_bytes);
    int n[2] = {(int)rows, (int)cols};
    hipfftType type = forward ? (elem_bytes == 4 ? HIPFFT_R2C : HIPFFT_D2Z) : (elem_bytes == 4 ? HIPFFT_C2R : HIPFFT_Z2D);
    hipfftHandle h;
    // null embeds: dense matrices one after another (the strides and distances are then ignored)
    FFT_CALL(hipfftPlanMany(&h, 2, n, nullptr, 1, 0, nullptr, 1, 0, type, (int)batch));
    *out = new Plan{h, forward, elem_bytes};
    return OK;
}

// ---------------------------------------------------------------- kernels
template <typename C>
__device__ __forceinline__ C multiply_conjugate(C a, C b) { // a * conj(b)
    return C{a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y};
}

// One thread per element of the reference strip; it walks every gridDim.y-th of the `batch` strips of deformed spectra
// (the reference's kernel walks all of them, hadamard.cu:34-55: with one small left spectrum and thousands of right ones
// that is a few hundred threads in a loop of thousands of dependent memory round trips).
template <typename C>
__global__ void hadamard_original_kernel(const C *__restrict__ ref, C *__restrict__ deformed, size_t strip, unsigned batch) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= strip) return;
    const C r = ref[i];
    for (unsigned b = blockIdx.y; b < batch; b += gridDim.y) {
        C *p = deformed + (size_t)b * strip + i;
        *p = multiply_conjugate(r, *p);
    }
}

// Grid-stride over the right spectra; the right value stays in registers for all left spectra.
template <typename C>
__global__ void hadamard_over_right_kernel(const C *__restrict__ left, const C *__restrict__ right, C *__restrict__ out, size_t len,
                                           unsigned n_left, unsigned n_right) {
    const size_t total = len * n_right, stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const C r = right[i];
        const size_t e = i % len;
        for (unsigned l = 0; l < n_left; ++l) out[(size_t)l * total + i] = multiply_conjugate(left[(size_t)l * len + e], r);
    }
}

// Grid-stride over the output elements.
template <typename C>
__global__ void hadamard_over_output_kernel(const C *__restrict__ left, const C *__restrict__ right, C *__restrict__ out, size_t len,
                                            unsigned n_left, unsigned n_right) {
    const size_t per_left = len * n_right, total = per_left * n_left, stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const size_t l = i / per_left, ri = i % per_left;
        out[i] = multiply_conjugate(left[l * len + ri % len], right[ri]);
    }
}

template <typename T>
__global__ void scatter_kernel(const T *__restrict__ src, T *__restrict__ dst, unsigned src_cols, unsigned src_rows, size_t total,
                               unsigned dst_cols, unsigned dst_rows, unsigned dst_x, unsigned dst_y) {
    const size_t area = (size_t)src_cols * src_rows, stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const size_t m = i / area, o = i % area;
        const unsigned y = (unsigned)(o / src_cols), x = (unsigned)(o % src_cols);
        dst[m * dst_cols * dst_rows + (size_t)(dst_y + y) * dst_cols + dst_x + x] = src[i];
    }
}

int check_block(unsigned threads) {
    if (threads == 0 || threads > 1024) return fail(ERR_INVALID_ARGUMENT, "Invalid number of threads per block: %u (1-1024)", threads);
    return OK;
}

unsigned grid_for(size_t items, unsigned threads, unsigned items_per_thread) {
    if (items_per_thread == 0) items_per_thread = 1;
    size_t per_block = (size_t)threads * items_per_thread;
    size_t blocks = (items + per_block - 1) / per_block;
    if (blocks == 0) blocks = 1;
    if (blocks > 0x7fffffffu) blocks = 0x7fffffffu;
    return (unsigned)blocks;
}

template <typename C>
int hadamard_original(const void *ref, void *deformed, unsigned fft_cols, unsigned fft_rows, unsigned per_pic, unsigned batch,
                      unsigned threads, void *stream) {
    if (!ref || !deformed) return fail(ERR_INVALID_ARGUMENT, "null device pointer");
    if (int rc = check_block(threads)) return rc;
    const size_t strip = (size_t)fft_cols * fft_rows * per_pic;
    if (strip == 0 || batch == 0) return fail(ERR_INVALID_ARGUMENT, "empty hadamard product");
    // enough threads to fill the device: the batch is spread over blockIdx.y until about half a million threads exist
    size_t over_batch = ((size_t)1 << 19) / strip;
    if (over_batch < 1) over_batch = 1;
    if (over_batch > batch) over_batch = batch;
    if (over_batch > 65535) over_batch = 65535;
    const dim3 grid(grid_for(strip, threads, 1), (unsigned)over_batch);
    hadamard_original_kernel<C><<<grid, threads, 0, (hipStream_t)stream>>>((const C *)ref, (C *)deformed, strip, batch);
    HIP_CALL(hipGetLastError());
    return OK;
}

template <typename C, bool OVER_RIGHT>
int hadamard_n_to_m(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows, unsigned n_left,
                    unsigned n_right, unsigned threads, unsigned items, void *stream) {
    if (!left || !right || !out) return fail(ERR_INVALID_ARGUMENT, "null device pointer");
    if (int rc = check_block(threads)) return rc;
    const size_t len = (size_t)fft_cols * fft_rows;
    if (len == 0 || n_left == 0 || n_right == 0) return fail(ERR_INVALID_ARGUMENT, "empty hadamard product");
    if (OVER_RIGHT)
        hadamard_over_right_kernel<C><<<grid_for(len * n_right, threads, items), threads, 0, (hipStream_t)stream>>>(
            (const C *)left, (const C *)right, (C *)out, len, n_left, n_right);
    else
        hadamard_over_output_kernel<C><<<grid_for(len * n_right * n_left, threads, items), threads, 0, (hipStream_t)stream>>>(
            (const C *)left, (const C *)right, (C *)out, len, n_left, n_right);
    HIP_CALL(hipGetLastError());
    return OK;
}

template <typename T>
int scatter(const T *src, T *dst, unsigned src_cols, unsigned src_rows, unsigned n, unsigned dst_cols, unsigned dst_rows, unsigned dst_x,
            unsigned dst_y, unsigned threads, unsigned items, void *stream) {
    if (!src || !dst) return fail(ERR_INVALID_ARGUMENT, "null device pointer");
    if (int rc = check_block(threads)) return rc;
    if (dst_x + src_cols > dst_cols || dst_y + src_rows > dst_rows)
        return fail(ERR_INVALID_ARGUMENT, "scatter: %ux%u at (%u,%u) does not fit %ux%u", src_cols, src_rows, dst_x, dst_y, dst_cols, dst_rows);
    const size_t total = (size_t)src_cols * src_rows * n;
    if (total == 0) return fail(ERR_INVALID_ARGUMENT, "empty scatter");
    scatter_kernel<T><<<grid_for(total, threads, items), threads, 0, (hipStream_t)stream>>>(src, dst, src_cols, src_rows, total, dst_cols,
                                                                                        dst_rows, dst_x, dst_y);
    HIP_CALL(hipGetLastError());
    return OK;
}

} // namespace

extern "C" {

const char *xcorr_fft_last_error(void) { return error_text; }

int xcorr_fft_plan_forward(void **plan, unsigned rows, unsigned cols, unsigned batch, unsigned elem_bytes) {
    return make_plan(plan, rows, cols, batch, elem_bytes, true);
}
int xcorr_fft_plan_inverse(void **plan, unsigned rows, unsigned cols, unsigned batch, unsigned elem_bytes) {
    return make_plan(plan, rows, cols, batch, elem_bytes, false);
}
int xcorr_fft_plan_set_stream(void *plan, void *stream) {
    if (!plan) return fail(ERR_INVALID_ARGUMENT, "null plan");
    FFT_CALL(hipfftSetStream(static_cast<Plan *>(plan)->handle, (hipStream_t)stream));
    return OK;
}
int xcorr_fft_exec_forward(void *plan, const void *real_in, void *complex_out) {
    Plan *p = static_cast<Plan *>(plan);
    if (!p || !p->forward || !real_in || !complex_out) return fail(ERR_INVALID_ARGUMENT, "forward transform needs a forward plan and two buffers");
    if (p->elem_bytes == 4)
        FFT_CALL(hipfftExecR2C(p->handle, (hipfftReal *)const_cast<void *>(real_in), (hipfftComplex *)complex_out));
    else
        FFT_CALL(hipfftExecD2Z(p->handle, (hipfftDoubleReal *)const_cast<void *>(real_in), (hipfftDoubleComplex *)complex_out));
    return OK;
}
int xcorr_fft_exec_inverse(void *plan, void *complex_in, void *real_out) {
    Plan *p = static_cast<Plan *>(plan);
    if (!p || p->forward || !complex_in || !real_out) return fail(ERR_INVALID_ARGUMENT, "inverse transform needs an inverse plan and two buffers");
    if (p->elem_bytes == 4)
        FFT_CALL(hipfftExecC2R(p->handle, (hipfftComplex *)complex_in, (hipfftReal *)real_out));
    else
        FFT_CALL(hipfftExecZ2D(p->handle, (hipfftDoubleComplex *)complex_in, (hipfftDoubleReal *)real_out));
    return OK;
}
int xcorr_fft_plan_destroy(void *plan) {
    Plan *p = static_cast<Plan *>(plan);
    if (!p) return OK;
    hipfftResult r = hipfftDestroy(p->handle);
    delete p;
    if (r != HIPFFT_SUCCESS) return fail(ERR_RUNTIME, "hipFFT error %d: %s in hipfftDestroy", (int)r, fft_status_name(r));
    return OK;
}

int xcorr_hadamard_original_f32(const void *ref, void *deformed, unsigned fft_cols, unsigned fft_rows, unsigned subregions_per_pic,
                                unsigned batch, unsigned threads_per_block, void *stream) {
    return hadamard_original<float2>(ref, deformed, fft_cols, fft_rows, subregions_per_pic, batch, threads_per_block, stream);
}
int xcorr_hadamard_original_f64(const void *ref, void *deformed, unsigned fft_cols, unsigned fft_rows, unsigned subregions_per_pic,
                                unsigned batch, unsigned threads_per_block, void *stream) {
    return hadamard_original<double2>(ref, deformed, fft_cols, fft_rows, subregions_per_pic, batch, threads_per_block, stream);
}
int xcorr_hadamard_n_to_m_over_right_f32(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                         unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                         void *stream) {
    return hadamard_n_to_m<float2, true>(left, right, out, fft_cols, fft_rows, n_left, n_right, threads_per_block, items_per_thread, stream);
}
int xcorr_hadamard_n_to_m_over_right_f64(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                         unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                         void *stream) {
    return hadamard_n_to_m<double2, true>(left, right, out, fft_cols, fft_rows, n_left, n_right, threads_per_block, items_per_thread, stream);
}
int xcorr_hadamard_n_to_m_over_output_f32(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                          unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                          void *stream) {
    return hadamard_n_to_m<float2, false>(left, right, out, fft_cols, fft_rows, n_left, n_right, threads_per_block, items_per_thread, stream);
}
int xcorr_hadamard_n_to_m_over_output_f64(const void *left, const void *right, void *out, unsigned fft_cols, unsigned fft_rows,
                                          unsigned n_left, unsigned n_right, unsigned threads_per_block, unsigned items_per_thread,
                                          void *stream) {
    return hadamard_n_to_m<double2, false>(left, right, out, fft_cols, fft_rows, n_left, n_right, threads_per_block, items_per_thread, stream);
}
int xcorr_scatter_f32(const float *src, float *dst, unsigned src_cols, unsigned src_rows, unsigned n, unsigned dst_cols,
                      unsigned dst_rows, unsigned dst_x, unsigned dst_y, unsigned threads_per_block, unsigned items_per_thread,
                      void *stream) {
    return scatter<float>(src, dst, src_cols, src_rows, n, dst_cols, dst_rows, dst_x, dst_y, threads_per_block, items_per_thread, stream);
}
int xcorr_scatter_f64(const double *src, double *dst, unsigned src_cols, unsigned src_rows, unsigned n, unsigned dst_cols,
                      unsigned dst_rows, unsigned dst_x, unsigned dst_y, unsigned threads_per_block, unsigned items_per_thread,
                      void *stream) {
    return scatter<double>(src, dst, src_cols, src_rows, n, dst_cols, dst_rows, dst_x, dst_y, threads_per_block, items_per_thread, stream);
}

} // extern "C"
