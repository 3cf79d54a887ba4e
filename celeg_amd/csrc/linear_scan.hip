// Recurrent mixers whose state moves on by one linear step a token, everything in 32-bit.
//
// 1. The real-gated linear recurrent unit.  Per channel c of `width`, in `blocks` equal parts:
//        u = conv(x)                      (a short causal convolution with a bias, no activation)
//        r = sigmoid(Ra[b] u_b + ra_b),  i = sigmoid(Ri[b] u_b + ri_b)      (square matrices per part)
//        log a = -c r softplus(lam),  S <- a S + sqrt(1 - a^2) (i u),  out = S * gelu(y)
//    lru_gates does everything up to (a, sqrt(1 - a^2) i u) per row, lru_scan walks a request's
//    rows per channel from and into its slot's state.
// 2. Matrix states with a decay per key channel.  Per value head (its query/key head g), S [dim, vdim]:
//        S <- diag(decay_t) S;  u = beta (v - S^T k)  (or u = v without beta);  S <- S + k u^T;  o = S^T q
//    channel_scan keeps S in registers: P neighbouring lanes share a column of S, lane part p
//    holding rows p, p + P, ...; the two sums over dim meet by exchanges between those lanes.
//    The next row's operands are asked for while this one is computed.  A row's sums depend on
//    nothing but the rows before it, so the cut of a prompt into steps changes no bit.
//    channel_decay and gla_prepare make the decays (and 32-bit q, k, v) from the projections.
#include "common.h"

namespace {

__device__ __forceinline__ float ls_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float ls_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float ls_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------- linear recurrent unit
// One workgroup per (row, part).  x: the convolution's inputs [rows, width] (row stride ldx);
// ra_t / ri_t: [blocks, in, out] (transposed at load so that neighbouring threads read neighbouring weights).
template <typename T>
__global__ __launch_bounds__(256) void lru_gates_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ conv_w, const float* __restrict__ conv_b,
    const float* __restrict__ ra_t, const float* __restrict__ ra_b, const float* __restrict__ ri_t, const float* __restrict__ ri_b,
    const float* __restrict__ lam, const float* __restrict__ conv_state, size_t state_stride, const int* __restrict__ positions,
    const int* __restrict__ token_seq, const int* __restrict__ seq_start, const int* __restrict__ token_slot,
    float* __restrict__ decay, float* __restrict__ input, int width, int bw, int taps, float decay_scale) {
    extern __shared__ float us[];      // bw values of u
    const int t = blockIdx.x, b = blockIdx.y;
    const int i = positions[t] - seq_start[token_seq[t]];
    const float* saved = conv_state + static_cast<size_t>(token_slot[t]) * state_stride;
    for (int j = threadIdx.x; j < bw; j += blockDim.x) {
        const int c = b * bw + j;
        float u = conv_b ? conv_b[c] : 0.f;
        for (int k = 0; k < taps; ++k) {
            const int back = taps - 1 - k, ii = i - back;
            const float xv = ii >= 0 ? to_float(x[static_cast<size_t>(t - back) * ldx + c])
                                     : saved[static_cast<size_t>(taps - 1 + ii) * width + c];
            u = fmaf(conv_w[static_cast<size_t>(c) * taps + k], xv, u);
        }
        us[j] = u;
    }
    __syncthreads();
    const float* wa = ra_t + static_cast<size_t>(b) * bw * bw;
    const float* wi = ri_t + static_cast<size_t>(b) * bw * bw;
    for (int j = threadIdx.x; j < bw; j += blockDim.x) {
        const int c = b * bw + j;
        float za = ra_b[c], zi = ri_b[c];
        for (int k = 0; k < bw; ++k) {
            const float u = us[k];
            za = fmaf(wa[static_cast<size_t>(k) * bw + j], u, za);
            zi = fmaf(wi[static_cast<size_t>(k) * bw + j], u, zi);
        }
        const float log_a = -decay_scale * ls_sigmoid(za) * ls_softplus(lam[c]);
        const float a = expf(log_a);
        const float mult = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f));     // sqrt(1 - a^2)
        decay[static_cast<size_t>(t) * width + c] = a;
        input[static_cast<size_t>(t) * width + c] = mult * ls_sigmoid(zi) * us[j];
    }
}

// One thread per (request, channel): S <- a S + input, out = S * gelu(y) (y with its bias already).
template <typename T>
__global__ void lru_scan_kernel(const float* __restrict__ decay, const float* __restrict__ input, const T* __restrict__ y, int ldy,
                                float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_seqlens,
                                const int* __restrict__ seq_slot, T* __restrict__ out, int ldo, int width) {
    const int s = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + c;
    float S = *mine;
    int r = 0;
    for (; r + 4 <= n; r += 4) {
        float a[4], in[4], yv[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const size_t t = static_cast<size_t>(row0 + r + k);
            a[k] = decay[t * width + c];
            in[k] = input[t * width + c];
            yv[k] = to_float(y[t * ldy + c]);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            S = fmaf(a[k], S, in[k]);
            out[static_cast<size_t>(row0 + r + k) * ldo + c] = from_float<T>(S * ls_gelu_tanh(yv[k]));
        }
    }
    for (; r < n; ++r) {
        const size_t t = static_cast<size_t>(row0 + r);
        S = fmaf(decay[t * width + c], S, input[t * width + c]);
        out[t * ldo + c] = from_float<T>(S * ls_gelu_tanh(to_float(y[t * ldy + c])));
    }
    *mine = S;
}

// The same recurrence for long portions, a workgroup of LRU_WAVES wavefronts per (request, 64
// channels): a portion is taken in stretches of LRU_WAVES * LRU_CHUNK rows, a wavefront LRU_CHUNK
// neighbouring rows of each.  A wavefront first runs its rows from S = 0, which gives its stretch as
// a map S -> A S + L (A the product of its decays); the maps meet in LDS, every wavefront applies
// those before its own to the state the stretch started from, in their order, and runs its rows
// again from there.  (Sums taken in another order than token by token: the results agree to
// rounding, not to the bit.)
#define LRU_WAVES 16
#define LRU_CHUNK 16
template <typename T>
__global__ __launch_bounds__(LRU_WAVES * CELEG_WAVE) void lru_scan_waves_kernel(
    const float* __restrict__ decay, const float* __restrict__ input, const T* __restrict__ y, int ldy, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, T* __restrict__ out, int ldo, int width) {
    __shared__ float prod_s[LRU_WAVES][CELEG_WAVE], last_s[LRU_WAVES][CELEG_WAVE];
    const int s = blockIdx.y, lane = threadIdx.x % CELEG_WAVE, wave = threadIdx.x / CELEG_WAVE;
    const int c = blockIdx.x * CELEG_WAVE + lane;
    const bool has = c < width;
    const int cc = has ? c : width - 1;       // lanes past the last channel repeat it and store nothing
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + cc;
    float carried = *mine;
    for (int base = 0; base < n; base += LRU_WAVES * LRU_CHUNK) {
        const int first = base + wave * LRU_CHUNK, count = min(LRU_CHUNK, n - first);      // <= 0: no rows here
        float a[LRU_CHUNK], in[LRU_CHUNK], yv[LRU_CHUNK];
#pragma unroll
        for (int k = 0; k < LRU_CHUNK; ++k) {
            a[k] = 1.f;
            in[k] = 0.f;
            yv[k] = 0.f;
            if (k < count) {
                const size_t t = static_cast<size_t>(row0 + first + k);
                a[k] = decay[t * width + cc];
                in[k] = input[t * width + cc];
                yv[k] = to_float(y[t * ldy + cc]);
            }
        }
        float A = 1.f, L = 0.f;
#pragma unroll
        for (int k = 0; k < LRU_CHUNK; ++k) {
            L = fmaf(a[k], L, in[k]);
            A *= a[k];
        }
        prod_s[wave][lane] = A;
        last_s[wave][lane] = L;
        __syncthreads();
        float S = carried, after = carried;
#pragma unroll
        for (int w = 0; w < LRU_WAVES; ++w) {
            after = fmaf(prod_s[w][lane], after, last_s[w][lane]);
            if (w + 1 == wave) S = after;
        }
#pragma unroll
        for (int k = 0; k < LRU_CHUNK; ++k) {
            S = fmaf(a[k], S, in[k]);
            if (has && k < count) out[static_cast<size_t>(row0 + first + k) * ldo + c] = from_float<T>(S * ls_gelu_tanh(yv[k]));
        }
        carried = after;
        __syncthreads();
    }
    if (wave == 0 && has) *mine = carried;
}

// ---------------------------------------------------------------- decays per key channel
// decay = exp(-exp(a_log[h]) softplus(z + dt_bias)), z [rows, heads * dim]
template <typename T>
__global__ void channel_decay_kernel(const T* __restrict__ z, int ldz, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                     float* __restrict__ decay, int dim, int cols) {
    const int t = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    const float zz = to_float(z[static_cast<size_t>(t) * ldz + c]) + dt_bias[c];
    decay[static_cast<size_t>(t) * cols + c] = expf(-expf(a_log[c / dim]) * ls_softplus(zz));
}

// q, k [rows, heads * dim] and v [rows, heads * vdim] widened (q times q_scale) into qk (q | k) and
// v32; decay = sigmoid(z + bias)^(1 / tau) = exp(-softplus(-(z + bias)) / tau)
template <typename T>
__global__ void gla_prepare_kernel(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
                                   const T* __restrict__ z, int ldz, const float* __restrict__ z_bias, float inv_tau, float q_scale,
                                   float* __restrict__ qk, float* __restrict__ v32, float* __restrict__ decay, int qk_cols,
                                   int v_cols) {
    const int t = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < qk_cols) {
        qk[static_cast<size_t>(t) * 2 * qk_cols + c] = to_float(q[static_cast<size_t>(t) * ldq + c]) * q_scale;
        qk[static_cast<size_t>(t) * 2 * qk_cols + qk_cols + c] = to_float(k[static_cast<size_t>(t) * ldk + c]);
        const float zz = to_float(z[static_cast<size_t>(t) * ldz + c]) + (z_bias ? z_bias[c] : 0.f);
        decay[static_cast<size_t>(t) * qk_cols + c] = expf(-ls_softplus(-zz) * inv_tau);
    }
    if (c < v_cols) v32[static_cast<size_t>(t) * v_cols + c] = to_float(v[static_cast<size_t>(t) * ldv + c]);
}

// the sum of x over the P neighbouring lanes of a column, in all of them
template <int P>
__device__ __forceinline__ float ls_part_sum(float x) {
#pragma unroll
    for (int off = 1; off < P; off <<= 1) x += __shfl_xor(x, off, CELEG_WAVE);
    return x;
}

// One wavefront per (request, value head, 64 / P columns).  qk: [rows, 2 * G * D] (query heads, then
// key heads); v, out: [rows, H * V]; decay: [rows, H * D]; beta: value [t * ld_beta + h], or null
// (no correction: u = v); state [slots, H, D, V].
template <int P, int DPL>
__global__ __launch_bounds__(CELEG_WAVE) void channel_scan_kernel(
    const float* __restrict__ qk, const float* __restrict__ v, const float* __restrict__ decay, const float* __restrict__ beta,
    int ld_beta, float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_slot, float* __restrict__ out, int G, int H, int D, int V) {
    constexpr int CPW = CELEG_WAVE / P;
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int p = lane % P, j = blockIdx.z * CPW + lane / P;
    const bool live = j < V;
    const int g = h / (H / G);
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + static_cast<size_t>(h) * D * V;
    float S[DPL];
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
        const int d = p + P * i;
        S[i] = (live && d < D) ? mine[static_cast<size_t>(d) * V + j] : 0.f;
    }
    const size_t ldqk = static_cast<size_t>(2) * G * D, ldv = static_cast<size_t>(H) * V, ldd = static_cast<size_t>(H) * D;
    float qn[DPL], kn[DPL], an[DPL], vn, bn;
    auto fetch = [&](int r) {
        const size_t t = static_cast<size_t>(row0 + r);
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
            const int d = p + P * i;
            const bool in = d < D;
            qn[i] = in ? qk[t * ldqk + static_cast<size_t>(g) * D + d] : 0.f;
            kn[i] = in ? qk[t * ldqk + static_cast<size_t>(G + g) * D + d] : 0.f;
            an[i] = in ? decay[t * ldd + static_cast<size_t>(h) * D + d] : 1.f;
        }
        vn = live ? v[t * ldv + static_cast<size_t>(h) * V + j] : 0.f;
        bn = beta ? beta[t * ld_beta + h] : 1.f;
    };
    fetch(0);
    for (int r = 0; r < n; ++r) {
        float q[DPL], k[DPL], a[DPL];
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
            q[i] = qn[i];
            k[i] = kn[i];
            a[i] = an[i];
        }
        const float vj = vn, b = bn;
        if (r + 1 < n) fetch(r + 1);
        float u = vj;
        if (beta) {
            float kv = 0.f;
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
                S[i] *= a[i];
                kv = fmaf(k[i], S[i], kv);
            }
            u = b * (vj - ls_part_sum<P>(kv));
        } else {
#pragma unroll
            for (int i = 0; i < DPL; ++i) S[i] *= a[i];
        }
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
            S[i] = fmaf(k[i], u, S[i]);
            o = fmaf(q[i], S[i], o);
        }
        o = ls_part_sum<P>(o);
        if (live && p == 0) out[static_cast<size_t>(row0 + r) * ldv + static_cast<size_t>(h) * V + j] = o;
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
            const int d = p + P * i;
            if (d < D) mine[static_cast<size_t>(d) * V + j] = S[i];
        }
    }
}

// The same recurrence for dim = DL * DPL (DPL a multiple of 4): DL neighbouring lanes share a column
// of S, each holding DPL neighbouring values of it, so the sums over dim meet by log2(DL) exchanges
// through the vector unit's cross-lane modifiers.  A request's rows are taken in blocks of TB
// tokens whose q, k, decays and values are staged in LDS, asked for from memory while the block
// before is computed: a token's steps wait for LDS, never for memory.  A wavefront issues its
// instructions one after the other, so what a block costs besides the recurrence is kept small:
// every lane brings pieces of four numbers whose place in the block never changes (offsets worked
// out once; rows past the request's end read its last row again).
// Tokens are taken one at a time in every block, so the cut of a prompt into steps changes no bit.
template <int DL, int DPL, bool BETA>
__global__ __launch_bounds__(CELEG_WAVE) void channel_scan_block_kernel(
    const float* __restrict__ qk, const float* __restrict__ v, const float* __restrict__ decay, const float* __restrict__ beta,
    int ld_beta, float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_slot, float* __restrict__ out, int G, int H, int V) {
    constexpr int D = DL * DPL, NC = DPL / 4, CPW = CELEG_WAVE / DL, TB = D <= 64 ? 16 : 8, ROW = 3 * D;
    constexpr int D4 = D / 4, PER = TB * D4 / CELEG_WAVE, PERV = (TB * CPW + CELEG_WAVE - 1) / CELEG_WAVE;
    static_assert(TB * D4 % CELEG_WAVE == 0, "a block's pieces fill whole wavefronts");
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) float rows_s[TB * ROW];
    __shared__ float vals_s[PERV * CELEG_WAVE];
    __shared__ float beta_s[TB];
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int sub = lane % DL, col = lane / DL, j = blockIdx.z * CPW + col;
    const bool live = j < V;
    const int jj = live ? j : V - 1;          // idle lanes repeat the last column and store nothing
    const int g = h / (H / G);
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + static_cast<size_t>(h) * D * V;
    float S[DPL];
#pragma unroll
    for (int i = 0; i < DPL; ++i) S[i] = mine[static_cast<size_t>(sub * DPL + i) * V + jj];
    const int ldqk = 2 * G * D, ldv = H * V, ldd = H * D;
    const float* q_base = qk + static_cast<size_t>(row0) * ldqk + g * D;
    const float* k_base = q_base + G * D;
    const float* a_base = decay + static_cast<size_t>(row0) * ldd + h * D;
    const float* v_base = v + static_cast<size_t>(row0) * ldv + static_cast<size_t>(h) * V;
    f4 pre_q[PER], pre_k[PER], pre_a[PER];
    float pre_v[PERV], pre_b = 1.f;
    auto fetch = [&](int t0) __attribute__((always_inline)) {
        const int last = n - 1 - t0;          // the block's rows past this one read it again
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int piece = lane + CELEG_WAVE * i, tt = min(piece / D4, last), c = 4 * (piece % D4);
            const size_t t = static_cast<size_t>(t0 + tt);
            pre_q[i] = *reinterpret_cast<const f4*>(q_base + t * ldqk + c);
            pre_k[i] = *reinterpret_cast<const f4*>(k_base + t * ldqk + c);
            pre_a[i] = *reinterpret_cast<const f4*>(a_base + t * ldd + c);
        }
#pragma unroll
        for (int i = 0; i < PERV; ++i) {
            const int piece = lane + CELEG_WAVE * i, tt = min(piece / CPW, min(TB - 1, last));
            const int column = min(static_cast<int>(blockIdx.z) * CPW + piece % CPW, V - 1);
            pre_v[i] = v_base[static_cast<size_t>(t0 + tt) * ldv + column];
        }
        if (BETA && lane < TB) pre_b = beta[static_cast<size_t>(row0 + t0 + min(lane, last)) * ld_beta + h];
    };
    fetch(0);
    float* out_at = out + static_cast<size_t>(row0) * ldv + static_cast<size_t>(h) * V + jj;
    const bool stores = live && sub == 0;
    for (int t0 = 0; t0 < n; t0 += TB) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int piece = lane + CELEG_WAVE * i;
            float* at = rows_s + (piece / D4) * ROW + 4 * (piece % D4);
            *reinterpret_cast<f4*>(at) = pre_q[i];
            *reinterpret_cast<f4*>(at + D) = pre_k[i];
            *reinterpret_cast<f4*>(at + 2 * D) = pre_a[i];
        }
#pragma unroll
        for (int i = 0; i < PERV; ++i) vals_s[lane + CELEG_WAVE * i] = pre_v[i];
        if (BETA && lane < TB) beta_s[lane] = pre_b;
        __syncthreads();
        if (t0 + TB < n) fetch(t0 + TB);
        const int count = min(TB, n - t0);
        auto token = [&](int tt) __attribute__((always_inline)) {
            const float* row = rows_s + tt * ROW + sub * DPL;
            const float value = vals_s[tt * CPW + col];
            f4 q4[NC], k4[NC], a4[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                q4[c] = *reinterpret_cast<const f4*>(row + 4 * c);
                k4[c] = *reinterpret_cast<const f4*>(row + D + 4 * c);
                a4[c] = *reinterpret_cast<const f4*>(row + 2 * D + 4 * c);
            }
            float u = value;
            if (BETA) {
                float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        S[4 * c + e] *= a4[c][e];
                        part[e] = fmaf(k4[c][e], S[4 * c + e], part[e]);
                    }
                u = beta_s[tt] * (value - lanes_sum<DL>((part[0] + part[1]) + (part[2] + part[3])));
            } else {
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int e = 0; e < 4; ++e) S[4 * c + e] *= a4[c][e];
            }
            float opart[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    S[4 * c + e] = fmaf(k4[c][e], u, S[4 * c + e]);
                    opart[e] = fmaf(q4[c][e], S[4 * c + e], opart[e]);
                }
            const float o = lanes_sum<DL>((opart[0] + opart[1]) + (opart[2] + opart[3]));
            if (stores) out_at[static_cast<size_t>(t0 + tt) * ldv] = o;
        };
        if (count == TB) {
#pragma unroll
            for (int tt = 0; tt < TB; ++tt) token(tt);
        } else {
            for (int tt = 0; tt < count; ++tt) token(tt);
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DPL; ++i) mine[static_cast<size_t>(sub * DPL + i) * V + j] = S[i];
    }
}

}  // namespace

extern "C" int celeg_lru_gates(const void* x, int ldx, int dtype, const float* conv_w, const float* conv_b, const float* ra_t,
                               const float* ra_b, const float* ri_t, const float* ri_b, const float* lam, const float* conv_state,
                               size_t state_stride, const int* positions, const int* token_seq, const int* seq_start,
                               const int* token_slot, float* decay, float* input, int n_tokens, int width, int blocks, int taps,
                               float decay_scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (blocks <= 0 || width % blocks) return static_cast<int>(hipErrorInvalidValue);
    const int bw = width / blocks;
    const size_t lds = static_cast<size_t>(bw) * sizeof(float);
    if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_tokens, blocks), block(bw >= 256 ? 256 : ((bw + 63) / 64) * 64);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(lru_gates_kernel<float>, grid, block, lds, stream, static_cast<const float*>(x), ldx, conv_w, conv_b, ra_t,
                           ra_b, ri_t, ri_b, lam, conv_state, state_stride, positions, token_seq, seq_start, token_slot, decay,
                           input, width, bw, taps, decay_scale);
    else
        hipLaunchKernelGGL(lru_gates_kernel<bf16>, grid, block, lds, stream, static_cast<const bf16*>(x), ldx, conv_w, conv_b, ra_t,
                           ra_b, ri_t, ri_b, lam, conv_state, state_stride, positions, token_seq, seq_start, token_slot, decay,
                           input, width, bw, taps, decay_scale);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_lru_scan(const float* decay, const float* input, const void* y, int ldy, int dtype, float* state,
                              size_t state_stride, const int* cu_seqlens, const int* seq_slot, void* out, int ldo, int n_seqs,
                              int width, int longest, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    dim3 grid((width + 63) / 64, n_seqs), block(64);
    // `longest`: the most rows a request has in this step; long portions are shared out over wavefronts
    if (longest >= 4 * LRU_CHUNK) {
        dim3 wide(LRU_WAVES * CELEG_WAVE);
        if (dtype == CELEG_F32)
            hipLaunchKernelGGL(lru_scan_waves_kernel<float>, grid, wide, 0, stream, decay, input, static_cast<const float*>(y), ldy, state,
                               state_stride, cu_seqlens, seq_slot, static_cast<float*>(out), ldo, width);
        else
            hipLaunchKernelGGL(lru_scan_waves_kernel<bf16>, grid, wide, 0, stream, decay, input, static_cast<const bf16*>(y), ldy, state,
                               state_stride, cu_seqlens, seq_slot, static_cast<bf16*>(out), ldo, width);
        return CELEG_LAUNCH_RESULT();
    }
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(lru_scan_kernel<float>, grid, block, 0, stream, decay, input, static_cast<const float*>(y), ldy, state,
                           state_stride, cu_seqlens, seq_slot, static_cast<float*>(out), ldo, width);
    else
        hipLaunchKernelGGL(lru_scan_kernel<bf16>, grid, block, 0, stream, decay, input, static_cast<const bf16*>(y), ldy, state,
                           state_stride, cu_seqlens, seq_slot, static_cast<bf16*>(out), ldo, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_channel_decay(const void* z, int ldz, int dtype, const float* a_log, const float* dt_bias, float* decay,
                                   int n_tokens, int heads, int dim, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const int cols = heads * dim;
    dim3 grid((cols + 255) / 256, n_tokens), block(256);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(channel_decay_kernel<float>, grid, block, 0, stream, static_cast<const float*>(z), ldz, a_log, dt_bias,
                           decay, dim, cols);
    else
        hipLaunchKernelGGL(channel_decay_kernel<bf16>, grid, block, 0, stream, static_cast<const bf16*>(z), ldz, a_log, dt_bias,
                           decay, dim, cols);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_gla_prepare(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const void* z, int ldz,
                                 int dtype, const float* z_bias, float inv_tau, float q_scale, float* qk, float* v32, float* decay,
                                 int n_tokens, int qk_cols, int v_cols, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const int cols = qk_cols > v_cols ? qk_cols : v_cols;
    dim3 grid((cols + 255) / 256, n_tokens), block(256);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(gla_prepare_kernel<float>, grid, block, 0, stream, static_cast<const float*>(q), ldq,
                           static_cast<const float*>(k), ldk, static_cast<const float*>(v), ldv, static_cast<const float*>(z), ldz,
                           z_bias, inv_tau, q_scale, qk, v32, decay, qk_cols, v_cols);
    else
        hipLaunchKernelGGL(gla_prepare_kernel<bf16>, grid, block, 0, stream, static_cast<const bf16*>(q), ldq,
                           static_cast<const bf16*>(k), ldk, static_cast<const bf16*>(v), ldv, static_cast<const bf16*>(z), ldz,
                           z_bias, inv_tau, q_scale, qk, v32, decay, qk_cols, v_cols);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_channel_scan(const float* qk, const float* v, const float* decay, const float* beta, int ld_beta, float* state,
                                  size_t state_stride, const int* cu_seqlens, const int* seq_slot, float* out, int n_seqs, int G,
                                  int H, int D, int V, int general, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (G <= 0 || H % G || D <= 0 || D > 256 || V <= 0) return static_cast<int>(hipErrorInvalidValue);
#define CELEG_CHANNEL_BLOCKS(DL_, DPL_)                                                                                           \
    {                                                                                                                             \
        const int cpw = CELEG_WAVE / DL_;                                                                                         \
        dim3 grid(n_seqs, H, (V + cpw - 1) / cpw), block(CELEG_WAVE);                                                             \
        if (beta)                                                                                                                 \
            hipLaunchKernelGGL((channel_scan_block_kernel<DL_, DPL_, true>), grid, block, 0, stream, qk, v, decay, beta, ld_beta, \
                               state, state_stride, cu_seqlens, seq_slot, out, G, H, V);                                          \
        else                                                                                                                      \
            hipLaunchKernelGGL((channel_scan_block_kernel<DL_, DPL_, false>), grid, block, 0, stream, qk, v, decay, beta, ld_beta, \
                               state, state_stride, cu_seqlens, seq_slot, out, G, H, V);                                          \
        return CELEG_LAUNCH_RESULT();                                                                                             \
    }
    // dims that are DL lanes of a multiple of four values each; any other dim, and `general`, take the kernel below
    const bool by_fours = ((reinterpret_cast<uintptr_t>(qk) | reinterpret_cast<uintptr_t>(decay)) & 15) == 0;      // the block kernel reads four numbers at a time
    if (!general && by_fours) {
        if (D == 16) CELEG_CHANNEL_BLOCKS(4, 4)
        if (D == 32) CELEG_CHANNEL_BLOCKS(8, 4)
        if (D == 48) CELEG_CHANNEL_BLOCKS(4, 12)
        if (D == 64) CELEG_CHANNEL_BLOCKS(16, 4)
        if (D == 96) CELEG_CHANNEL_BLOCKS(8, 12)
        if (D == 128) CELEG_CHANNEL_BLOCKS(16, 8)
        if (D == 256) CELEG_CHANNEL_BLOCKS(16, 16)
    }
#undef CELEG_CHANNEL_BLOCKS
#define CELEG_CHANNEL_SCAN(P_, DPL_)                                                                                              \
    {                                                                                                                             \
        const int cpw = CELEG_WAVE / P_;                                                                                          \
        dim3 grid(n_seqs, H, (V + cpw - 1) / cpw), block(CELEG_WAVE);                                                             \
        hipLaunchKernelGGL((channel_scan_kernel<P_, DPL_>), grid, block, 0, stream, qk, v, decay, beta, ld_beta, state,           \
                           state_stride, cu_seqlens, seq_slot, out, G, H, D, V);                                                  \
    }
    if (D <= 16) CELEG_CHANNEL_SCAN(4, 4)
    else if (D <= 32) CELEG_CHANNEL_SCAN(8, 4)
    else if (D <= 64) CELEG_CHANNEL_SCAN(16, 4)
    else if (D <= 128) CELEG_CHANNEL_SCAN(16, 8)
    else CELEG_CHANNEL_SCAN(16, 16)
#undef CELEG_CHANNEL_SCAN
    return CELEG_LAUNCH_RESULT();
}
