// A sub-layer boundary of a block that norms a branch's output before adding it: for a row of
// the 32-bit residual stream h and the branch output y,
//     h += post(y)          (post: a layer norm, an RMS norm, or nothing but the addition)
//     out = pre(h)          (pre: the next sub-layer's norm; or no output at all)
// in one pass over the row, with every statistic and sum in 32-bit.  Either half may be absent,
// so the same kernel is a plain layer norm (with a gather of rows for the output head), the
// addition alone, or both.
//
// Layer norm: (x - mean) / sqrt(var + eps) * w + b with var the mean of the squared deviations
// from the mean (two passes over the row, which is staged in LDS).  RMS norm:
// x / sqrt(mean(x^2) + eps) * w.  The bias is optional in both.  "Dynamic tanh": tanh(alpha * x) * w + b
// with one number alpha, no statistic of the row at all.  A norm's `gain` multiplies what it gives
// as a whole (a block that adds m * post(y)).
#include "common.h"

#include "norm_params.h"

namespace {

// one value through a norm whose statistics are (shift, factor)
__device__ __forceinline__ float normed_value(float x, const CelegNorm& n, float shift, float factor, float w, float b) {
    const float v = n.mode == CELEG_NORM_TANH ? tanhf(n.alpha * x) : (x - shift) * factor;
    return (v * w + b) * n.gain;
}

// the statistics of `row` (LDS, width floats) for a norm of this mode: (shift, factor) such that
// the normalised value is (x - shift) * factor
__device__ __forceinline__ void row_stats(const float* row, int width, int mode, float eps, float* scratch, float& shift,
                                          float& factor) {
    shift = 0.f;
    factor = 1.f;
    if (mode == CELEG_NORM_LAYER) {
        float s = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) s += row[i];
        shift = block_sum(s, scratch) / static_cast<float>(width);
    }
    if (mode == CELEG_NORM_LAYER || mode == CELEG_NORM_RMS) {
        float s = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            const float d = row[i] - shift;
            s += d * d;
        }
        factor = 1.0f / sqrtf(block_sum(s, scratch) / static_cast<float>(width) + eps);
    }
}

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void norm_step_kernel(float* __restrict__ h, const TY* __restrict__ y, CelegNorm post,
                                                        CelegNorm pre, TO* __restrict__ out, const int* __restrict__ rows,
                                                        int width, int write_back) {
    extern __shared__ float row[];     // width floats
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
    if (y) {
        for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = to_float(y[src + i]);
        __syncthreads();
        float shift, factor;
        row_stats(row, width, post.mode, post.eps, scratch, shift, factor);
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float v = normed_value(row[i], post, shift, factor, post.w ? post.w[i] : 1.f, post.b ? post.b[i] : 0.f);
            v += h[src + i];
            row[i] = v;                 // (its own element: no other thread reads it before the barrier)
            if (write_back) h[src + i] = v;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = h[src + i];
    }
    if (!out) return;
    __syncthreads();
    float shift, factor;
    row_stats(row, width, pre.mode, pre.eps, scratch, shift, factor);
    TO* dst = out + static_cast<size_t>(r) * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        dst[i] = from_float<TO>(normed_value(row[i], pre, shift, factor, pre.w ? pre.w[i] : 1.f, pre.b ? pre.b[i] : 0.f));
    }
}

// The same for rows of up to 256 * NV values, with the row in registers and everything a thread reads
// (branch output, stream, both norms' weights and biases) asked for at once: three trips to memory
// one after the other become one, which is what a step of few rows waits for.
template <int NV>
__device__ __forceinline__ void reg_stats(const float (&v)[NV], const bool (&in)[NV], int width, int mode, float eps, float* scratch,
                                          float& shift, float& factor) {
    shift = 0.f;
    factor = 1.f;
    if (mode == CELEG_NORM_LAYER) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) s += in[k] ? v[k] : 0.f;
        shift = block_sum(s, scratch) / static_cast<float>(width);
    }
    if (mode == CELEG_NORM_LAYER || mode == CELEG_NORM_RMS) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const float d = in[k] ? v[k] - shift : 0.f;
            s += d * d;
        }
        factor = 1.0f / sqrtf(block_sum(s, scratch) / static_cast<float>(width) + eps);
    }
}

template <typename TY, typename TO, int NV>
__global__ __launch_bounds__(256) void norm_step_reg_kernel(float* __restrict__ h, const TY* __restrict__ y, CelegNorm post,
                                                            CelegNorm pre, TO* __restrict__ out, const int* __restrict__ rows,
                                                            int width, int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
    float yv[NV], hv[NV], pw[NV], pb[NV], nw[NV], nb[NV];
    bool in[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = threadIdx.x + 256 * k;
        in[k] = i < width;
        const int ii = in[k] ? i : 0;
        hv[k] = h[src + ii];
        yv[k] = y ? to_float(y[src + ii]) : 0.f;
        pw[k] = y && post.w ? post.w[ii] : 1.f;
        pb[k] = y && post.b ? post.b[ii] : 0.f;
        nw[k] = out && pre.w ? pre.w[ii] : 1.f;
        nb[k] = out && pre.b ? pre.b[ii] : 0.f;
    }
    if (y) {
        float shift, factor;
        reg_stats<NV>(yv, in, width, post.mode, post.eps, scratch, shift, factor);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            hv[k] = normed_value(yv[k], post, shift, factor, pw[k], pb[k]) + hv[k];
            if (write_back && in[k]) h[src + threadIdx.x + 256 * k] = hv[k];
        }
    }
    if (!out) return;
    float shift, factor;
    reg_stats<NV>(hv, in, width, pre.mode, pre.eps, scratch, shift, factor);
    TO* dst = out + static_cast<size_t>(r) * width;
#pragma unroll
    for (int k = 0; k < NV; ++k)
        if (in[k]) dst[threadIdx.x + 256 * k] = from_float<TO>(normed_value(hv[k], pre, shift, factor, nw[k], nb[k]));
}

template <typename TO>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, TO* __restrict__ out, size_t rows,
                                   int width) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= rows * 2 * width) return;
    const size_t r = idx / (2 * width);
    const int c = static_cast<int>(idx % (2 * width));
    out[idx] = from_float<TO>(c < width ? a[r * width + c] : b[r * width + c - width]);
}

}  // namespace

extern "C" int celeg_norm_step(float* h, const void* y, int y_dtype, CelegNorm post, CelegNorm pre, void* out, int out_dtype,
                               const int* rows, int n_rows, int width, int write_back, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const size_t lds = static_cast<size_t>(width) * sizeof(float);
    if (lds > 60 * 1024) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_rows), block(256);
#define CELEG_NORM_STEP(TY, TO)                                                                                            \
    if (width <= 1024)                                                                                                     \
        hipLaunchKernelGGL((norm_step_reg_kernel<TY, TO, 4>), grid, block, 0, stream, h, static_cast<const TY*>(y), post, pre, \
                           static_cast<TO*>(out), rows, width, write_back);                                               \
    else if (width <= 2048)                                                                                                \
        hipLaunchKernelGGL((norm_step_reg_kernel<TY, TO, 8>), grid, block, 0, stream, h, static_cast<const TY*>(y), post, pre, \
                           static_cast<TO*>(out), rows, width, write_back);                                               \
    else                                                                                                                   \
        hipLaunchKernelGGL((norm_step_kernel<TY, TO>), grid, block, lds, stream, h, static_cast<const TY*>(y), post, pre,     \
                           static_cast<TO*>(out), rows, width, write_back)
    if (y_dtype == CELEG_F32 && out_dtype == CELEG_F32) { CELEG_NORM_STEP(float, float); }
    else if (y_dtype == CELEG_F32) { CELEG_NORM_STEP(float, bf16); }
    else if (out_dtype == CELEG_F32) { CELEG_NORM_STEP(bf16, float); }
    else { CELEG_NORM_STEP(bf16, bf16); }
#undef CELEG_NORM_STEP
    return CELEG_LAUNCH_RESULT();
}

// out [rows, 2 * width] = (a | b) row by row, both 32-bit, in the dtype of out
extern "C" int celeg_concat_rows(const float* a, const float* b, void* out, int out_dtype, int rows, int width,
                                 hipStream_t stream) {
    const size_t total = static_cast<size_t>(rows) * 2 * width;
    if (total == 0) return 0;
    dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
    if (out_dtype == CELEG_F32)
        hipLaunchKernelGGL(concat_rows_kernel<float>, grid, block, 0, stream, a, b, static_cast<float*>(out),
                           static_cast<size_t>(rows), width);
    else
        hipLaunchKernelGGL(concat_rows_kernel<bf16>, grid, block, 0, stream, a, b, static_cast<bf16*>(out),
                           static_cast<size_t>(rows), width);
    return CELEG_LAUNCH_RESULT();
}
