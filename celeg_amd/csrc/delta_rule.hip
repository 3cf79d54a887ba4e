// The gated delta rule: a recurrent mixer whose state is a matrix per head.
//
// Per token and value head h (its query/key head g = h / (heads / kv_heads)), with unit key k,
// scaled unit query q, value v, write strength beta and decay a (all 32-bit):
//     S <- a S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          S [dim, vdim]
// The state S lives in the request's slot, in 32-bit, from token to token.
//
// Kernels:
//  * delta_prepare: from the projections' rows, the short causal convolution of the q, k and v
//    channels continuing from the request's saved inputs, silu, the unit norm of q and k per
//    head, beta = sigmoid(.), a = exp(-exp(A_log) softplus(. + dt_bias));
//  * delta_conv_state: the last taps - 1 inputs of every channel become the request's new state;
//  * delta_scan: the recurrence, one wavefront per (request, value head, 64 columns of S): a lane
//    owns a column of S, so the three sums over dim are the lane's own and no lane waits for another;
//  * delta_gated_norm: o / rms(o) * w * silu(gate), per head.
#include "common.h"

namespace {

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float dr_silu(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float dr_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// Input i' of channel c for the row whose place in its step's segment is `i` (row index t):
// i' >= 0 lies in the step (row t - (i - i')), i' < 0 in the saved inputs (entry taps - 1 + i').
template <typename T>
__device__ __forceinline__ float conv_silu(const T* __restrict__ proj, int ld, int t, int i, int c, const float* __restrict__ w,
                                           const float* __restrict__ saved, int n_channels, int taps) {
    float y = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, ii = i - back;
        const float x = ii >= 0 ? to_float(proj[static_cast<size_t>(t - back) * ld + c])
                                : saved[static_cast<size_t>(taps - 1 + ii) * n_channels + c];
        y = fmaf(w[static_cast<size_t>(c) * taps + j], x, y);
    }
    return dr_silu(y);
}

// One wavefront per (row, unit): units [0, G) are query heads, [G, 2G) key heads, [2G, 2G + H)
// value heads, the last one computes beta and the decay of every value head.
// proj columns: q [G*D] | k [G*D] | v [H*V] | (gate H*V, not read here) | b [H] at col_b | a [H] at col_a.
// conv_w [2*G*D + H*V, taps]: the q, k and v channels' taps one after the other.
template <typename T>
__global__ __launch_bounds__(CELEG_WAVE) void delta_prepare_kernel(
    const T* __restrict__ proj, int ld, int col_b, int col_a, const float* __restrict__ conv_w, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const float* __restrict__ conv_state, size_t state_stride,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ seq_start,
    const int* __restrict__ token_slot, float* __restrict__ qk, float* __restrict__ v_out, float* __restrict__ beta_decay, int G,
    int H, int D, int V, int taps) {
    const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int n_channels = 2 * G * D + H * V;
    if (unit == 2 * G + H) {
        for (int h = lane; h < H; h += CELEG_WAVE) {
            const float b = to_float(proj[static_cast<size_t>(t) * ld + col_b + h]);
            const float a = a_log ? to_float(proj[static_cast<size_t>(t) * ld + col_a + h]) : 0.f;
            beta_decay[static_cast<size_t>(t) * 2 * H + h] = dr_sigmoid(b);
            // (a_log null: the decay is made elsewhere, per key channel)
            if (a_log) beta_decay[static_cast<size_t>(t) * 2 * H + H + h] = expf(-expf(a_log[h]) * dr_softplus(a + dt_bias[h]));
        }
        return;
    }
    const int i = positions[t] - seq_start[token_seq[t]];
    const float* saved = conv_state + static_cast<size_t>(token_slot[t]) * state_stride;
    if (unit >= 2 * G) {
        const int h = unit - 2 * G;
        for (int j = lane; j < V; j += CELEG_WAVE) {
            const int c = 2 * G * D + h * V + j;
            v_out[static_cast<size_t>(t) * H * V + h * V + j] = conv_silu(proj, ld, t, i, c, conv_w, saved, n_channels, taps);
        }
        return;
    }
    // a query or key head: unit vector over D (queries also times D^-1/2)
    const int c0 = unit * D;
    float* dst = qk + static_cast<size_t>(t) * 2 * G * D + c0;
    float sum = 0.f;
    for (int d = lane; d < D; d += CELEG_WAVE) {
        const float x = conv_silu(proj, ld, t, i, c0 + d, conv_w, saved, n_channels, taps);
        dst[d] = x;
        sum += x * x;
    }
    sum = wave_sum(sum);
    float inv = 1.0f / sqrtf(sum + 1e-6f);
    if (unit < G) inv *= 1.0f / sqrtf(static_cast<float>(D));
    for (int d = lane; d < D; d += CELEG_WAVE) dst[d] *= inv;     // (a lane reads what it wrote itself)
}

// per (request of the step, channel): new saved input j is old saved input j + n, or the step's
// row j + n - (taps - 1) where that is not negative
template <typename T>
__global__ void delta_conv_state_kernel(const T* __restrict__ proj, int ld, float* __restrict__ conv_state, size_t state_stride,
                                        const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, int n_channels,
                                        int taps) {
    const int s = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_channels) return;
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* saved = conv_state + static_cast<size_t>(seq_slot[s]) * state_stride;
    for (int j = 0; j < taps - 1; ++j) {      // rising j: entry j + n is still the old one when j is written
        const int from = j + n - (taps - 1);
        saved[static_cast<size_t>(j) * n_channels + c] =
            from >= 0 ? to_float(proj[static_cast<size_t>(row0 + from) * ld + c]) : saved[static_cast<size_t>(j + n) * n_channels + c];
    }
}

// One wavefront per (request, value head, 64 columns).  S's columns of this wavefront sit in LDS
// as [D][64]; k and q of the token are staged in LDS for all lanes to read.
__global__ __launch_bounds__(CELEG_WAVE) void delta_scan_kernel(
    const float* __restrict__ qk, const float* __restrict__ v, const float* __restrict__ beta_decay, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, float* __restrict__ out, int G, int H,
    int D, int V) {
    extern __shared__ float lds[];       // S [D][64], k [D], q [D]
    float* S = lds;
    float* ks = lds + static_cast<size_t>(D) * CELEG_WAVE;
    float* qs = ks + D;
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int j = blockIdx.z * CELEG_WAVE + lane;
    const bool live = j < V;
    const int g = h / (H / G);
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + static_cast<size_t>(h) * D * V;
    for (int d = 0; d < D; ++d) S[d * CELEG_WAVE + lane] = live ? mine[static_cast<size_t>(d) * V + j] : 0.f;
    for (int r = 0; r < n; ++r) {
        const size_t t = static_cast<size_t>(row0 + r);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (int d = lane; d < D; d += CELEG_WAVE) {
            qs[d] = qk[t * 2 * G * D + static_cast<size_t>(g) * D + d];
            ks[d] = qk[t * 2 * G * D + static_cast<size_t>(G + g) * D + d];
        }
        const float beta = beta_decay[t * 2 * H + h], decay = beta_decay[t * 2 * H + H + h];
        const float vj = live ? v[t * H * V + static_cast<size_t>(h) * V + j] : 0.f;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float kv = 0.f;
        for (int d = 0; d < D; ++d) {
            const float sd = decay * S[d * CELEG_WAVE + lane];
            S[d * CELEG_WAVE + lane] = sd;
            kv = fmaf(ks[d], sd, kv);
        }
        const float u = beta * (vj - kv);
        float o = 0.f;
        for (int d = 0; d < D; ++d) {
            const float sd = fmaf(ks[d], u, S[d * CELEG_WAVE + lane]);
            S[d * CELEG_WAVE + lane] = sd;
            o = fmaf(qs[d], sd, o);
        }
        if (live) out[t * H * V + static_cast<size_t>(h) * V + j] = o;
    }
    if (live)
        for (int d = 0; d < D; ++d) mine[static_cast<size_t>(d) * V + j] = S[d * CELEG_WAVE + lane];
}

// What two neighbouring rows of a request's step need of each other when the recurrence takes them
// together: for the rows at even places of their segment (and not its last), per query/key head,
// k1.k2, k1.q1, k1.q2, k2.q2 (1: the row, 2: the next one).  One wavefront per (row, head).
__global__ __launch_bounds__(CELEG_WAVE) void delta_pairs_kernel(const float* __restrict__ qk, const int* __restrict__ token_seq,
                                                                 const int* __restrict__ cu_seqlens, float* __restrict__ pairs, int G,
                                                                 int D) {
    const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
    const int seq = token_seq[t], row0 = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (((t - row0) & 1) || t + 1 >= end) return;
    const float* q1 = qk + static_cast<size_t>(t) * 2 * G * D + static_cast<size_t>(g) * D;
    const float* k1 = q1 + static_cast<size_t>(G) * D;
    const float* q2 = q1 + static_cast<size_t>(2) * G * D;
    const float* k2 = k1 + static_cast<size_t>(2) * G * D;
    float kk = 0.f, kq1 = 0.f, kq2 = 0.f, k2q2 = 0.f;
    for (int d = lane; d < D; d += CELEG_WAVE) {
        kk = fmaf(k1[d], k2[d], kk);
        kq1 = fmaf(k1[d], q1[d], kq1);
        kq2 = fmaf(k1[d], q2[d], kq2);
        k2q2 = fmaf(k2[d], q2[d], k2q2);
    }
    kk = wave_sum(kk);
    kq1 = wave_sum(kq1);
    kq2 = wave_sum(kq2);
    k2q2 = wave_sum(k2q2);
    if (lane == 0) {
        float* dst = pairs + (static_cast<size_t>(t) * G + g) * 4;
        dst[0] = kk;
        dst[1] = kq1;
        dst[2] = kq2;
        dst[3] = k2q2;
    }
}

// The same recurrence with S in registers, for dim = DL * DPL: DL neighbouring lanes share a column
// of S, each holding DPL of its values, so a wavefront owns 64 / DL columns and the sums over dim
// meet by log2(DL) exchanges between neighbours.  (Few values a lane: a token's passes over the
// state are short, and it is their chain from token to token that the kernel's time is.)  The rows of a request are taken in blocks of TB
// tokens: a block's q, k, write strengths and decays are staged in LDS (asked for from memory while
// the block before is computed), its values sit in registers.  With u = beta (v - a (S^T k)) the
// new column is a S + k u, read out with q in the same pass.
template <int DL, int DPL>
__global__ __launch_bounds__(CELEG_WAVE) void delta_scan_reg_kernel(
    const float* __restrict__ qk, const float* __restrict__ v, const float* __restrict__ beta_decay, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, float* __restrict__ out,
    const float* __restrict__ pairs, int G, int H, int V) {
    constexpr int D = DPL * DL, NC = DPL / 4, CPW = CELEG_WAVE / DL, TB = D <= 64 ? 16 : 8, ROW = 2 * D, PER_LANE = TB * ROW / CELEG_WAVE;
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) float qk_s[TB * ROW];
    __shared__ float bd_s[TB * 2];
    __shared__ float pair_s[TB * 2];
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int sub = lane % DL, j = blockIdx.z * CPW + lane / DL;
    const bool live = j < V;
    const int jj = live ? j : V - 1;          // idle lanes repeat the last column and store nothing
    const int g = h / (H / G);
    const int row0 = cu_seqlens[s], n = cu_seqlens[s + 1] - row0;
    if (n <= 0) return;
    float* mine = state + static_cast<size_t>(seq_slot[s]) * state_stride + static_cast<size_t>(h) * D * V;
    float S[DPL];
#pragma unroll
    for (int i = 0; i < DPL; ++i) S[i] = mine[static_cast<size_t>(sub * DPL + i) * V + jj];
    const size_t ldqk = static_cast<size_t>(2) * G * D;
    float pre[PER_LANE], pre_v[TB], pre_bd = 0.f, pre_pair = 0.f;
    auto fetch = [&](int block) __attribute__((always_inline)) {
        const int t0 = block * TB;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const int e = lane + CELEG_WAVE * i, tt = e / ROW, x = e % ROW;
            const int t = min(t0 + tt, n - 1);
            pre[i] = qk[static_cast<size_t>(row0 + t) * ldqk + (x < D ? g * D + x : (G + g) * D + x - D)];
        }
#pragma unroll
        for (int tt = 0; tt < TB; ++tt) pre_v[tt] = v[static_cast<size_t>(row0 + min(t0 + tt, n - 1)) * H * V + static_cast<size_t>(h) * V + jj];
        if (lane < 2 * TB) pre_bd = beta_decay[static_cast<size_t>(row0 + min(t0 + lane / 2, n - 1)) * 2 * H + (lane & 1) * H + h];
        // (what the pairs of a whole block need; a block that is not whole goes token by token)
        if (pairs && lane < 2 * TB && t0 + TB <= n) pre_pair = pairs[(static_cast<size_t>(row0 + t0 + 2 * (lane >> 2)) * G + g) * 4 + (lane & 3)];
    };
    fetch(0);
    const int n_blocks = (n + TB - 1) / TB;
    for (int block = 0; block < n_blocks; ++block) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) qk_s[lane + CELEG_WAVE * i] = pre[i];
        if (lane < 2 * TB) {
            bd_s[lane] = pre_bd;
            pair_s[lane] = pre_pair;
        }
        float vals[TB];
#pragma unroll
        for (int tt = 0; tt < TB; ++tt) vals[tt] = pre_v[tt];
        __syncthreads();
        if (block + 1 < n_blocks) fetch(block + 1);
        const int count = min(TB, n - block * TB);
        auto token = [&](int tt, float value) __attribute__((always_inline)) {
            const float* qrow = qk_s + tt * ROW + sub * DPL;
            f4 q4[NC], k4[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                q4[c] = *reinterpret_cast<const f4*>(qrow + 4 * c);
                k4[c] = *reinterpret_cast<const f4*>(qrow + D + 4 * c);
            }
            const float beta = bd_s[2 * tt], decay = bd_s[2 * tt + 1];
            float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) part[e] = fmaf(k4[c][e], S[4 * c + e], part[e]);
            const float kv = lanes_sum<DL>((part[0] + part[1]) + (part[2] + part[3]));
            const float u = beta * (value - decay * kv);
            float opart[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float sd = fmaf(k4[c][e], u, decay * S[4 * c + e]);
                    S[4 * c + e] = sd;
                    opart[e] = fmaf(q4[c][e], sd, opart[e]);
                }
            const float o = lanes_sum<DL>((opart[0] + opart[1]) + (opart[2] + opart[3]));
            if (live && sub == 0) out[static_cast<size_t>(row0 + block * TB + tt) * H * V + static_cast<size_t>(h) * V + j] = o;
        };
        // Two tokens together: with p = S^T k and r = S^T q of both tokens against the state before
        // them (one pass over S), u1 = b1 (v1 - a1 p1), u2 = b2 (v2 - a2 (a1 p2 + u1 k1.k2)),
        // o1 = a1 r1 + u1 k1.q1, o2 = a2 (a1 r2 + u1 k1.q2) + u2 k2.q2, and the state after them is
        // a2 a1 S + a2 u1 k1 + u2 k2 (a second pass): half as many passes that wait for one another.
        struct PairOperands {
            f4 q1[NC], k1[NC], q2[NC], k2[NC];
            float b1, a1, b2, a2, k1k2, k1q1, k1q2, k2q2;
        };
        // (a pair's operands are read from LDS while the pair before is computed)
        auto read_pair = [&](int tt) __attribute__((always_inline)) {
            PairOperands p;
            const float* row1 = qk_s + tt * ROW + sub * DPL;
            const float* row2 = row1 + ROW;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                p.q1[c] = *reinterpret_cast<const f4*>(row1 + 4 * c);
                p.k1[c] = *reinterpret_cast<const f4*>(row1 + D + 4 * c);
                p.q2[c] = *reinterpret_cast<const f4*>(row2 + 4 * c);
                p.k2[c] = *reinterpret_cast<const f4*>(row2 + D + 4 * c);
            }
            p.b1 = bd_s[2 * tt];
            p.a1 = bd_s[2 * tt + 1];
            p.b2 = bd_s[2 * tt + 2];
            p.a2 = bd_s[2 * tt + 3];
            const float* ps = pair_s + 2 * tt;
            p.k1k2 = ps[0];
            p.k1q1 = ps[1];
            p.k1q2 = ps[2];
            p.k2q2 = ps[3];
            return p;
        };
        auto two_tokens = [&](int tt, const PairOperands& p, float v1, float v2) __attribute__((always_inline)) {
            const f4 (&q1)[NC] = p.q1;
            const f4 (&k1)[NC] = p.k1;
            const f4 (&q2)[NC] = p.q2;
            const f4 (&k2)[NC] = p.k2;
            const float b1 = p.b1, a1 = p.a1, b2 = p.b2, a2 = p.a2, k1k2 = p.k1k2, k1q1 = p.k1q1, k1q2 = p.k1q2, k2q2 = p.k2q2;
            float p1[2] = {0.f, 0.f}, p2[2] = {0.f, 0.f}, r1[2] = {0.f, 0.f}, r2[2] = {0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float sv = S[4 * c + e];
                    p1[e & 1] = fmaf(k1[c][e], sv, p1[e & 1]);
                    p2[e & 1] = fmaf(k2[c][e], sv, p2[e & 1]);
                    r1[e & 1] = fmaf(q1[c][e], sv, r1[e & 1]);
                    r2[e & 1] = fmaf(q2[c][e], sv, r2[e & 1]);
                }
            const float sp1 = lanes_sum<DL>(p1[0] + p1[1]), sp2 = lanes_sum<DL>(p2[0] + p2[1]);
            const float sr1 = lanes_sum<DL>(r1[0] + r1[1]), sr2 = lanes_sum<DL>(r2[0] + r2[1]);
            const float u1 = b1 * (v1 - a1 * sp1);
            const float u2 = b2 * (v2 - a2 * fmaf(u1, k1k2, a1 * sp2));
            const float o1 = fmaf(u1, k1q1, a1 * sr1);
            const float o2 = fmaf(u2, k2q2, a2 * fmaf(u1, k1q2, a1 * sr2));
            const float both = a2 * a1, first = a2 * u1;
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int e = 0; e < 4; ++e) S[4 * c + e] = fmaf(k2[c][e], u2, fmaf(k1[c][e], first, both * S[4 * c + e]));
            if (live && sub == 0) {
                float* dst = out + static_cast<size_t>(row0 + block * TB + tt) * H * V + static_cast<size_t>(h) * V + j;
                dst[0] = o1;
                dst[static_cast<size_t>(H) * V] = o2;
            }
        };
        if (count == TB && pairs) {
            // a whole block: one run of instructions, so that the next tokens' operands are read while
            // these are computed
            PairOperands now = read_pair(0);
#pragma unroll
            for (int tt = 0; tt < TB; tt += 2) {
                PairOperands next = now;
                if (tt + 2 < TB) next = read_pair(tt + 2);
                two_tokens(tt, now, vals[tt], vals[tt + 1]);
                now = next;
            }
        } else if (count == TB) {
#pragma unroll
            for (int tt = 0; tt < TB; ++tt) token(tt, vals[tt]);
        } else {
#pragma unroll
            for (int tt = 0; tt < TB; ++tt) {
                if (tt >= count) break;
                token(tt, vals[tt]);
            }
        }
    }
    if (live)
#pragma unroll
        for (int i = 0; i < DPL; ++i) mine[static_cast<size_t>(sub * DPL + i) * V + j] = S[i];
}

// one wavefront per (row, head): out = o / sqrt(mean(o^2) + eps) * w * act(gate), act silu (0) or sigmoid (1)
template <typename T>
__global__ __launch_bounds__(CELEG_WAVE) void delta_gated_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                                      const T* __restrict__ gate, int ldg, float eps,
                                                                      T* __restrict__ out, int H, int V, int act) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* row = o + (static_cast<size_t>(t) * H + h) * V;
    float sum = 0.f;
    for (int j = lane; j < V; j += CELEG_WAVE) sum += row[j] * row[j];
    sum = wave_sum(sum);
    const float inv = 1.0f / sqrtf(sum / static_cast<float>(V) + eps);
    for (int j = lane; j < V; j += CELEG_WAVE) {
        const float z = to_float(gate[static_cast<size_t>(t) * ldg + h * V + j]);
        out[(static_cast<size_t>(t) * H + h) * V + j] = from_float<T>(row[j] * inv * w[j] * (act == 1 ? dr_sigmoid(z) : dr_silu(z)));
    }
}

}  // namespace

extern "C" int celeg_delta_prepare(const void* proj, int ld, int dtype, int col_b, int col_a, const float* conv_w,
                                   const float* a_log, const float* dt_bias, const float* conv_state, size_t state_stride,
                                   const int* positions, const int* token_seq, const int* seq_start, const int* token_slot,
                                   float* qk, float* v_out, float* beta_decay, int n_tokens, int G, int H, int D, int V, int taps,
                                   hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, 2 * G + H + 1), block(CELEG_WAVE);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(delta_prepare_kernel<float>, grid, block, 0, stream, static_cast<const float*>(proj), ld, col_b, col_a,
                           conv_w, a_log, dt_bias, conv_state, state_stride, positions, token_seq, seq_start, token_slot, qk,
                           v_out, beta_decay, G, H, D, V, taps);
    else
        hipLaunchKernelGGL(delta_prepare_kernel<bf16>, grid, block, 0, stream, static_cast<const bf16*>(proj), ld, col_b, col_a,
                           conv_w, a_log, dt_bias, conv_state, state_stride, positions, token_seq, seq_start, token_slot, qk,
                           v_out, beta_decay, G, H, D, V, taps);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_delta_conv_state(const void* proj, int ld, int dtype, float* conv_state, size_t state_stride,
                                      const int* cu_seqlens, const int* seq_slot, int n_seqs, int n_channels, int taps,
                                      hipStream_t stream) {
    if (n_seqs <= 0 || taps <= 1) return 0;
    dim3 grid((n_channels + 255) / 256, n_seqs), block(256);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(delta_conv_state_kernel<float>, grid, block, 0, stream, static_cast<const float*>(proj), ld, conv_state,
                           state_stride, cu_seqlens, seq_slot, n_channels, taps);
    else
        hipLaunchKernelGGL(delta_conv_state_kernel<bf16>, grid, block, 0, stream, static_cast<const bf16*>(proj), ld, conv_state,
                           state_stride, cu_seqlens, seq_slot, n_channels, taps);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_delta_scan(const float* qk, const float* v, const float* beta_decay, float* state, size_t state_stride,
                                const int* cu_seqlens, const int* seq_slot, float* out, int n_seqs, int G, int H, int D, int V,
                                int general, const int* token_seq, float* pairs, int n_tokens, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (H % G) return static_cast<int>(hipErrorInvalidValue);
    if (!general && (D == 16 || D == 32 || D == 64 || D == 128 || D == 256)) {
        const int DL = D == 16 ? 4 : D == 32 ? 8 : 16, cpw = CELEG_WAVE / DL;
        dim3 grid(n_seqs, H, (V + cpw - 1) / cpw), block(CELEG_WAVE);
        // pairs (room for n_tokens * G * 4 floats, or null): steps with rows to pair take two tokens together
        if (pairs && n_tokens > n_seqs) {
            hipLaunchKernelGGL(delta_pairs_kernel, dim3(n_tokens, G), dim3(CELEG_WAVE), 0, stream, qk, token_seq, cu_seqlens, pairs, G, D);
        } else {
            pairs = nullptr;
        }
#define CELEG_DELTA_REG(DL_, DPL_)                                                                                                  \
    hipLaunchKernelGGL((delta_scan_reg_kernel<DL_, DPL_>), grid, block, 0, stream, qk, v, beta_decay, state, state_stride, cu_seqlens, \
                       seq_slot, out, pairs, G, H, V)
        if (D == 16) CELEG_DELTA_REG(4, 4);
        else if (D == 32) CELEG_DELTA_REG(8, 4);
        else if (D == 64) CELEG_DELTA_REG(16, 4);
        else if (D == 128) CELEG_DELTA_REG(16, 8);
        else CELEG_DELTA_REG(16, 16);
#undef CELEG_DELTA_REG
        return CELEG_LAUNCH_RESULT();
    }
    const size_t lds = (static_cast<size_t>(D) * CELEG_WAVE + 2 * static_cast<size_t>(D)) * sizeof(float);
    if (lds > 64 * 1024 || H % G) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(n_seqs, H, (V + CELEG_WAVE - 1) / CELEG_WAVE), block(CELEG_WAVE);
    hipLaunchKernelGGL(delta_scan_kernel, grid, block, lds, stream, qk, v, beta_decay, state, state_stride, cu_seqlens, seq_slot,
                       out, G, H, D, V);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_delta_gated_norm(const float* o, const float* w, const void* gate, int ldg, int dtype, float eps, void* out,
                                      int n_tokens, int H, int V, int act, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, H), block(CELEG_WAVE);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(delta_gated_norm_kernel<float>, grid, block, 0, stream, o, w, static_cast<const float*>(gate), ldg, eps,
                           static_cast<float*>(out), H, V, act);
    else
        hipLaunchKernelGGL(delta_gated_norm_kernel<bf16>, grid, block, 0, stream, o, w, static_cast<const bf16*>(gate), ldg, eps,
                           static_cast<bf16*>(out), H, V, act);
    return CELEG_LAUNCH_RESULT();
}
