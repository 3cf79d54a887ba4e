// What lies between an attention's q/k/v product and its scores where every projected channel
// passes a short causal convolution over time first:
//     y_t[c] = sum_j w[c, j] * u_(t - taps + 1 + j)[c]        (zeros before the sequence starts)
// then the first `rotary_dim` values of every query and key head turn by the row's position (pair i
// is (i, i + rotary_dim / 2) or (2i, 2i + 1); angle = float(position) * inv_freq[i], 32-bit), the
// queries go to a buffer of their own, and keys and values to the row's place in the pages:
// K [pages, layers, kv_heads, page_tokens, head_dim], V [pages, layers, kv_heads, v_dim, page_tokens].
//
// The convolution continues from the request's saved inputs: the last taps - 1 projected rows
// [taps - 1, channels] in 32-bit, moved on afterwards by delta_conv_state (the same layout as the
// delta rule's).  Sums are 32-bit; a result is rounded once, after the rotation.
#include "common.h"

namespace {

// input i' of channel c for the row whose place in its step's portion is i (row index t): i' >= 0 lies
// in the step (row t - (i - i')), i' < 0 among the saved inputs (entry taps - 1 + i')
template <typename T>
__device__ __forceinline__ float cr_conv(const T* __restrict__ proj, int ld, int t, int i, int c, const float* __restrict__ w,
                                         const float* __restrict__ saved, int n_channels, int taps) {
    if (!w) return to_float(proj[static_cast<size_t>(t) * ld + c]);
    float y = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, ii = i - back;
        const float x = ii >= 0 ? to_float(proj[static_cast<size_t>(t - back) * ld + c])
                                : saved[static_cast<size_t>(taps - 1 + ii) * n_channels + c];
        y = fmaf(w[static_cast<size_t>(c) * taps + j], x, y);
    }
    return y;
}

// One wavefront per (row, unit): units [0, H) are query heads, [H, H + G) key heads, [H + G, H + 2G) value heads.
// proj columns: q [H * D] | k [G * D] | v [G * V]; conv_w [H * D + G * D + G * V, taps] (null: no convolution).
template <typename T>
__global__ __launch_bounds__(CELEG_WAVE) void conv_rope_store_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ conv_w, const float* __restrict__ conv_state, size_t state_stride,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ seq_start,
    const int* __restrict__ token_slot, const float* __restrict__ inv_freq, int rotary_dim, int pairing, T* __restrict__ q_out, int ldq,
    T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ table, int table_stride, int H, int G, int D, int V,
    int taps, int page_tokens, int n_layers, int layer) {
    extern __shared__ float head[];      // max(D, V) floats
    const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int n_channels = (H + G) * D + G * V;
    const int pos = positions[t];
    const int i = pos - seq_start[token_seq[t]];
    const int slot = token_slot[t];
    const float* saved = conv_state ? conv_state + static_cast<size_t>(slot) * state_stride : nullptr;
    const int page = table[static_cast<size_t>(slot) * table_stride + pos / page_tokens], in_page = pos % page_tokens;
    if (unit >= H + G) {
        const int g = unit - H - G, c0 = (H + G) * D + g * V;
        T* vd = v_pool + (((static_cast<size_t>(page) * n_layers + layer) * G + g) * V) * page_tokens + in_page;
        for (int d = lane; d < V; d += CELEG_WAVE)
            vd[static_cast<size_t>(d) * page_tokens] = from_float<T>(cr_conv(proj, ld, t, i, c0 + d, conv_w, saved, n_channels, taps));
        return;
    }
    const int c0 = unit * D;
    for (int d = lane; d < D; d += CELEG_WAVE) head[d] = cr_conv(proj, ld, t, i, c0 + d, conv_w, saved, n_channels, taps);
    __syncthreads();
    T* dst = unit < H ? q_out + static_cast<size_t>(t) * ldq + static_cast<size_t>(unit) * D
                      : k_pool + ((((static_cast<size_t>(page) * n_layers + layer) * G + (unit - H)) * page_tokens + in_page) * D);
    const int half = inv_freq ? rotary_dim / 2 : 0;
    const float p = static_cast<float>(pos);
    for (int j = lane; j < half; j += CELEG_WAVE) {
        const int a = pairing == 1 ? 2 * j : j, b = pairing == 1 ? 2 * j + 1 : j + half;
        float sn, cs;
        sincosf(p * inv_freq[j], &sn, &cs);
        const float u = head[a], v = head[b];
        dst[a] = from_float<T>(u * cs - v * sn);
        dst[b] = from_float<T>(v * cs + u * sn);
    }
    for (int d = 2 * half + lane; d < D; d += CELEG_WAVE) dst[d] = from_float<T>(head[d]);
}

}  // namespace

// proj [rows, >= (H + G) * D + G * V] (q | k | v from column 0); conv_w null: the rows pass as projected;
// inv_freq null: no rotation
extern "C" int celeg_conv_rope_store(const void* proj, int ld, int dtype, const float* conv_w, const float* conv_state,
                                     size_t state_stride, const int* positions, const int* token_seq, const int* seq_start,
                                     const int* token_slot, const float* inv_freq, int rotary_dim, int pairing, void* q_out, int ldq,
                                     void* k_pool, void* v_pool, const int* table, int table_stride, int n_tokens, int H, int G, int D,
                                     int V, int taps, int page_tokens, int n_layers, int layer, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H <= 0 || G <= 0 || D <= 0 || V <= 0 || taps <= 0 || (conv_w && taps > 1 && !conv_state) || rotary_dim % 2 || rotary_dim > D)
        return static_cast<int>(hipErrorInvalidValue);
    const size_t lds = static_cast<size_t>(D > V ? D : V) * sizeof(float);
    if (lds > 60 * 1024) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, H + 2 * G), block(CELEG_WAVE);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(conv_rope_store_kernel<float>, grid, block, lds, stream, static_cast<const float*>(proj), ld, conv_w, conv_state,
                           state_stride, positions, token_seq, seq_start, token_slot, inv_freq, rotary_dim, pairing,
                           static_cast<float*>(q_out), ldq, static_cast<float*>(k_pool), static_cast<float*>(v_pool), table, table_stride,
                           H, G, D, V, taps, page_tokens, n_layers, layer);
    else
        hipLaunchKernelGGL(conv_rope_store_kernel<bf16>, grid, block, lds, stream, static_cast<const bf16*>(proj), ld, conv_w, conv_state,
                           state_stride, positions, token_seq, seq_start, token_slot, inv_freq, rotary_dim, pairing,
                           static_cast<bf16*>(q_out), ldq, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool), table, table_stride, H,
                           G, D, V, taps, page_tokens, n_layers, layer);
    return CELEG_LAUNCH_RESULT();
}
