// What holds a layer together besides its norms: activations with a bias, sums into the 32-bit
// residual stream, a per-layer token input, the mean of several normed branches, and the
// weighted sum over the results of all earlier layers, what a stream takes in before a run of a looped
// range, and logits bent by a tanh.  All arithmetic is 32-bit; T is the
// run's dtype of the branch rows.
#include "common.h"

namespace {

__device__ __forceinline__ float lg_gelu_tanh(float z) {
    // 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
    const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    return 0.5f * z * (1.0f + tanhf(inner));
}
__device__ __forceinline__ float lg_relu2(float z) {
    const float r = fmaxf(z, 0.f);
    return r * r;
}

// out = act(x + bias); act 0: gelu (tanh form), 1: square of relu, 2: none
template <typename T>
__global__ void activation_bias_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ bias, T* __restrict__ out,
                                       int ldo, int cols, int act) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    float z = to_float(x[static_cast<size_t>(t) * ldx + c]);
    if (bias) z += bias[c];
    const float y = act == 0 ? lg_gelu_tanh(z) : act == 1 ? lg_relu2(z) : z;
    out[static_cast<size_t>(t) * ldo + c] = from_float<T>(y);
}

// h += a (+ b); copy (optional) receives the new rows in the run's dtype
template <typename T>
__global__ void residual_sum_kernel(float* __restrict__ h, const T* __restrict__ a, int lda, const T* __restrict__ b, int ldb,
                                    T* __restrict__ copy, int width) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    float add = to_float(a[static_cast<size_t>(t) * lda + c]);
    if (b) add += to_float(b[static_cast<size_t>(t) * ldb + c]);
    const float v = h[static_cast<size_t>(t) * width + c] + add;
    h[static_cast<size_t>(t) * width + c] = v;
    if (copy) copy[static_cast<size_t>(t) * width + c] = from_float<T>(v);
}

// g[t, j] = gelu(z[t, j]) * table[token[t], offset + j]
template <typename T>
__global__ void token_gate_kernel(const T* __restrict__ z, int ldz, const T* __restrict__ table, int ld_table, int offset,
                                  const int* __restrict__ token_ids, T* __restrict__ g, int dim) {
    const int t = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= dim) return;
    const float e = to_float(table[static_cast<size_t>(token_ids[t]) * ld_table + offset + j]);
    g[static_cast<size_t>(t) * dim + j] = from_float<T>(lg_gelu_tanh(to_float(z[static_cast<size_t>(t) * ldz + j])) * e);
}

// out[t] = factor * (a[t] / rms(a[t]) * wa + b[t] / rms(b[t]) * wb); one workgroup a row
template <typename T>
__global__ __launch_bounds__(256) void normed_mean_kernel(const T* __restrict__ a, int lda, const float* __restrict__ wa,
                                                          const T* __restrict__ b, int ldb, const float* __restrict__ wb, float eps,
                                                          float factor, T* __restrict__ out, int width) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const T* ar = a + static_cast<size_t>(t) * lda;
    const T* br = b + static_cast<size_t>(t) * ldb;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float x = to_float(ar[c]), y = to_float(br[c]);
        sa = fmaf(x, x, sa);
        sb = fmaf(y, y, sb);
    }
    sa = block_sum(sa, scratch);
    sb = block_sum(sb, scratch);
    const float ia = 1.0f / sqrtf(sa / static_cast<float>(width) + eps), ib = 1.0f / sqrtf(sb / static_cast<float>(width) + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x)
        out[static_cast<size_t>(t) * width + c] = from_float<T>(factor * (to_float(ar[c]) * ia * wa[c] + to_float(br[c]) * ib * wb[c]));
}

// history [n, rows_cap, width] 32-bit holds the results of the n - 1 entries before (the embedding's rows first);
// the stream's rows become entry n - 1, and the stream becomes sum_j w[j] history[j], j rising
__global__ void depth_mix_kernel(float* __restrict__ history, size_t entry_stride, float* __restrict__ h, const float* __restrict__ w,
                                 int n, int width) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const size_t at = static_cast<size_t>(t) * width + c;
    const float last = h[at];
    history[static_cast<size_t>(n - 1) * entry_stride + at] = last;
    float sum = 0.f;
    for (int j = 0; j < n - 1; ++j) sum = fmaf(w[j], history[static_cast<size_t>(j) * entry_stride + at], sum);
    h[at] = fmaf(w[n - 1], last, sum);
}

// h[t, :] += (rows[t, :] +) vec, all 32-bit: what a stream takes in before a run of a looped range
__global__ void stream_add_kernel(float* __restrict__ h, const float* __restrict__ rows, const float* __restrict__ vec, int width) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const size_t at = static_cast<size_t>(t) * width + c;
    float v = h[at];
    if (rows) v += rows[at];
    if (vec) v += vec[c];
    h[at] = v;
}

// x <- cap * tanh(x / cap), 32-bit
__global__ void softcap_kernel(float* __restrict__ x, size_t n, float cap) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

#define LG_BY_DTYPE(kernel, grid, block, ...)                                                      \
    if (dtype == CELEG_F32) {                                                                      \
        using T = float;                                                                           \
        hipLaunchKernelGGL(kernel<T>, grid, block, 0, stream, __VA_ARGS__);                        \
    } else {                                                                                       \
        using T = bf16;                                                                            \
        hipLaunchKernelGGL(kernel<T>, grid, block, 0, stream, __VA_ARGS__);                        \
    }

extern "C" int celeg_activation_bias(const void* x, int ldx, const float* bias, void* out, int ldo, int dtype, int rows, int cols,
                                     int act, hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return 0;
    dim3 grid((cols + 255) / 256, rows), block(256);
    LG_BY_DTYPE(activation_bias_kernel, grid, block, static_cast<const T*>(x), ldx, bias, static_cast<T*>(out), ldo, cols, act);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_residual_sum(float* h, const void* a, int lda, const void* b, int ldb, void* copy, int dtype, int rows,
                                  int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid((width + 255) / 256, rows), block(256);
    LG_BY_DTYPE(residual_sum_kernel, grid, block, h, static_cast<const T*>(a), lda, static_cast<const T*>(b), ldb,
                static_cast<T*>(copy), width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_token_gate(const void* z, int ldz, const void* table, int ld_table, int offset, const int* token_ids, void* g,
                                int dtype, int rows, int dim, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid((dim + 63) / 64, rows), block(64);
    LG_BY_DTYPE(token_gate_kernel, grid, block, static_cast<const T*>(z), ldz, static_cast<const T*>(table), ld_table, offset,
                token_ids, static_cast<T*>(g), dim);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_normed_mean(const void* a, int lda, const float* wa, const void* b, int ldb, const float* wb, float eps,
                                 float factor, void* out, int dtype, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid(rows), block(256);
    LG_BY_DTYPE(normed_mean_kernel, grid, block, static_cast<const T*>(a), lda, wa, static_cast<const T*>(b), ldb, wb, eps, factor,
                static_cast<T*>(out), width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_depth_mix(float* history, size_t entry_stride, float* h, const float* w, int n, int rows, int width,
                               hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    dim3 grid((width + 255) / 256, rows), block(256);
    hipLaunchKernelGGL(depth_mix_kernel, grid, block, 0, stream, history, entry_stride, h, w, n, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_stream_add(float* h, const float* rows, const float* vec, int n_rows, int width, hipStream_t stream) {
    if (n_rows <= 0 || (!rows && !vec)) return 0;
    dim3 grid((width + 255) / 256, n_rows), block(256);
    hipLaunchKernelGGL(stream_add_kernel, grid, block, 0, stream, h, rows, vec, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_softcap(float* x, size_t n, float cap, hipStream_t stream) {
    if (n == 0) return 0;
    if (!(cap > 0.f)) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(softcap_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, stream, x, n, cap);
    return CELEG_LAUNCH_RESULT();
}
