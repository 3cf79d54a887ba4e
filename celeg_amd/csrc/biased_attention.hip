// Softmax attention whose positions enter through the scores alone:
//     score(i, j) = (q_i . k_j) * scale * f(i) - r1[h] * ln(1 + r2[h] * (i - j))
// with a factor per query position f(i) = 1 + coef * ln(floor((i + 1) / every) + 1) (or 1) and a
// distance bias per query head (or none).  Keys at positions [first, i] of the row's request,
// first = max(0, i - window + 1) with a window, else 0; with `keep_first` the keys at positions
// [0, keep_first) stay visible after the window has passed them.  `sink_one`: the softmax's denominator
// holds a one more (a key whose score is 0 and that has no value).  Values may be wider or narrower than keys.
//
// Cache layout: K [pages, layers, kv_heads, page_tokens, head_dim],
// V [pages, layers, kv_heads, v_dim, page_tokens].
//
// kv_store writes a step's keys and values to their rows' places in the pages.  The general
// attention kernel is one wavefront per (row, query head), 64 keys a round, a lane scores one key;
// maximum, normaliser and sums are 32-bit, in an order that depends on the row's own position only.
#include "common.h"

namespace {

__device__ __forceinline__ size_t ba_k_offset(int page, int n_layers, int layer, int kv_heads, int head, int page_tokens,
                                              int in_page, int head_dim) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * page_tokens + in_page) * head_dim;
}
__device__ __forceinline__ size_t ba_v_offset(int page, int n_layers, int layer, int kv_heads, int head, int page_tokens,
                                              int v_dim) {
    return (((static_cast<size_t>(page) * n_layers + layer) * kv_heads + head) * v_dim) * page_tokens;
}

// the factor of a query at position p
__device__ __forceinline__ float ba_query_factor(int p, float coef, int every) {
    return every > 0 ? 1.0f + coef * logf(static_cast<float>((p + 1) / every) + 1.0f) : 1.0f;
}

template <typename T>
__global__ void kv_store_kernel(const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv, T* __restrict__ k_pool,
                                T* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
                                const int* __restrict__ token_slot, const int* __restrict__ positions, int kv_heads, int head_dim,
                                int v_dim, int page_tokens, int n_layers, int layer) {
    const int t = blockIdx.x, g = blockIdx.y;
    const int pos = positions[t];
    const int page = table[static_cast<size_t>(token_slot[t]) * table_stride + pos / page_tokens], in_page = pos % page_tokens;
    T* kd = k_pool + ba_k_offset(page, n_layers, layer, kv_heads, g, page_tokens, in_page, head_dim);
    const T* ks = k + static_cast<size_t>(t) * ldk + static_cast<size_t>(g) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) kd[d] = ks[d];
    T* vd = v_pool + ba_v_offset(page, n_layers, layer, kv_heads, g, page_tokens, v_dim) + in_page;
    const T* vs = v + static_cast<size_t>(t) * ldv + static_cast<size_t>(g) * v_dim;
    for (int d = threadIdx.x; d < v_dim; d += blockDim.x) vd[static_cast<size_t>(d) * page_tokens] = vs[d];
}

#define BA_MAX_V_CHUNKS 4  // v_dim <= 256

template <typename T>
__global__ __launch_bounds__(CELEG_WAVE) void biased_attention_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k_pool, const T* __restrict__ v_pool, const int* __restrict__ table,
    int table_stride, const int* __restrict__ token_slot, const int* __restrict__ positions, const float* __restrict__ r1,
    const float* __restrict__ r2, const T* __restrict__ gate, int ldg, T* __restrict__ out, int ldo, int q_heads, int kv_heads,
    int head_dim, int v_dim, int page_tokens, int n_layers, int layer, float scale, float coef, int every, int window,
    int keep_first, int sink_one) {
    extern __shared__ float lds[];  // head_dim floats of q, then 64 weights
    float* qs = lds;
    float* ps = lds + head_dim;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (q_heads / kv_heads);
    const int pos = positions[t];
    const int* pages = table + static_cast<size_t>(token_slot[t]) * table_stride;
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const float s = scale * ba_query_factor(pos, coef, every);
    const float b1 = r1 ? r1[h] : 0.f, b2 = r1 ? r2[h] : 0.f;

    const T* qrow = q + static_cast<size_t>(t) * ldq + static_cast<size_t>(h) * head_dim;
    for (int d = lane; d < head_dim; d += CELEG_WAVE) qs[d] = to_float(qrow[d]);
    __syncthreads();

    float acc[BA_MAX_V_CHUNKS];
#pragma unroll
    for (int j = 0; j < BA_MAX_V_CHUNKS; ++j) acc[j] = 0.f;
    // (the extra one of the denominator: a key of score 0 seen before all others)
    float top = sink_one ? 0.f : -INFINITY, total = sink_one ? 1.f : 0.f;

    // the kept first keys that the window has passed, then the window (or everything)
    const int kept = min(keep_first, first);
    for (int phase = kept > 0 ? 0 : 1; phase < 2; ++phase) {
        const int lo = phase == 0 ? 0 : first, hi = phase == 0 ? kept - 1 : pos;
        for (int base = lo; base <= hi; base += CELEG_WAVE) {
            const int key = base + lane;
            float score = -INFINITY;
            if (key <= hi) {
                const T* kp = k_pool + ba_k_offset(pages[key / page_tokens], n_layers, layer, kv_heads, kvh, page_tokens,
                                                   key % page_tokens, head_dim);
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_float(kp[d]), dot);
                score = dot * s;
                if (r1) score -= b1 * logf(1.0f + b2 * static_cast<float>(pos - key));
            }
            const float new_top = fmaxf(top, wave_max(score));     // (the round holds at least one visible key)
            const float p = key <= hi ? expf(score - new_top) : 0.f;
            const float keep = expf(top - new_top);                // 0 in the first round
            total = total * keep + wave_sum(p);
            top = new_top;
            ps[lane] = p;
            __syncthreads();
            const int n_keys = min(CELEG_WAVE, hi - base + 1);
#pragma unroll
            for (int j = 0; j < BA_MAX_V_CHUNKS; ++j) acc[j] *= keep;
            for (int kk = 0; kk < n_keys; ++kk) {
                const int key2 = base + kk;
                const T* vp = v_pool + ba_v_offset(pages[key2 / page_tokens], n_layers, layer, kv_heads, kvh, page_tokens, v_dim) +
                              key2 % page_tokens;
                const float pk = ps[kk];
#pragma unroll
                for (int j = 0; j < BA_MAX_V_CHUNKS; ++j) {
                    const int d = lane + j * CELEG_WAVE;
                    if (d < v_dim) acc[j] = fmaf(pk, to_float(vp[static_cast<size_t>(d) * page_tokens]), acc[j]);
                }
            }
            __syncthreads();
        }
    }
    const float inv = 1.0f / total;
    T* orow = out + static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * v_dim;
#pragma unroll
    for (int j = 0; j < BA_MAX_V_CHUNKS; ++j) {
        const int d = lane + j * CELEG_WAVE;
        if (d < v_dim) {
            float o = acc[j] * inv;
            if (gate) {
                const float z = to_float(gate[static_cast<size_t>(t) * ldg + static_cast<size_t>(h) * v_dim + d]);
                o *= 1.0f / (1.0f + expf(-z));
            }
            orow[d] = from_float<T>(o);
        }
    }
}

}  // namespace

extern "C" int celeg_kv_store(const void* k, int ldk, const void* v, int ldv, int dtype, void* k_pool, void* v_pool, const int* table,
                              int table_stride, const int* token_slot, const int* positions, int n_tokens, int kv_heads, int head_dim,
                              int v_dim, int page_tokens, int n_layers, int layer, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, kv_heads), block(CELEG_WAVE);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(kv_store_kernel<float>, grid, block, 0, stream, static_cast<const float*>(k), ldk,
                           static_cast<const float*>(v), ldv, static_cast<float*>(k_pool), static_cast<float*>(v_pool), table,
                           table_stride, token_slot, positions, kv_heads, head_dim, v_dim, page_tokens, n_layers, layer);
    else
        hipLaunchKernelGGL(kv_store_kernel<bf16>, grid, block, 0, stream, static_cast<const bf16*>(k), ldk,
                           static_cast<const bf16*>(v), ldv, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool), table,
                           table_stride, token_slot, positions, kv_heads, head_dim, v_dim, page_tokens, n_layers, layer);
    return CELEG_LAUNCH_RESULT();
}

// gate: raw gate values [rows, heads * v_dim] (the result is multiplied by their sigmoid), or null
extern "C" int celeg_biased_attention(const void* q, int ldq, int dtype, const void* k_pool, const void* v_pool, const int* table,
                                      int table_stride, const int* token_slot, const int* positions, const float* r1,
                                      const float* r2, const void* gate, int ldg, void* out, int ldo, int n_tokens, int q_heads,
                                      int kv_heads, int head_dim, int v_dim, int page_tokens, int n_layers, int layer, float scale,
                                      float coef, int every, int window, int keep_first, int sink_one, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (v_dim > BA_MAX_V_CHUNKS * CELEG_WAVE || q_heads % kv_heads) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, q_heads), block(CELEG_WAVE);
    const size_t lds = (static_cast<size_t>(head_dim) + CELEG_WAVE) * sizeof(float);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(biased_attention_kernel<float>, grid, block, lds, stream, static_cast<const float*>(q), ldq,
                           static_cast<const float*>(k_pool), static_cast<const float*>(v_pool), table, table_stride, token_slot,
                           positions, r1, r2, static_cast<const float*>(gate), ldg, static_cast<float*>(out), ldo, q_heads,
                           kv_heads, head_dim, v_dim, page_tokens, n_layers, layer, scale, coef, every, window, keep_first, sink_one);
    else
        hipLaunchKernelGGL(biased_attention_kernel<bf16>, grid, block, lds, stream, static_cast<const bf16*>(q), ldq,
                           static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool), table, table_stride, token_slot,
                           positions, r1, r2, static_cast<const bf16*>(gate), ldg, static_cast<bf16*>(out), ldo, q_heads, kv_heads,
                           head_dim, v_dim, page_tokens, n_layers, layer, scale, coef, every, window, keep_first, sink_one);
    return CELEG_LAUNCH_RESULT();
}
