// Softmax attention with a factor per query position and a distance bias per head, bfloat16, on
// the matrix cores:
//     score(i, j) = (q_i . k_j) * scale * f(i) - r1[h] * ln(1 + r2[h] * (i - j)),   weights = softmax over the visible j
// Visible: j <= i, inside the window where there is one, or among the first `keep_first` positions.  With `sink_one`
// the denominator holds a one more (a key of score 0 without a value, which the row meets before all others).
// Keys of `D` numbers, values of `V` numbers a head (both multiples of 32 up to 128).
// Cache layout: K [pages, layers, kv_heads, page_tokens, D], V [pages, layers, kv_heads, V, page_tokens].
//
// Scores are computed transposed (keys as the first operand of a 16x16x32 instruction): a lane
// holds, of row r = lane % 16, the keys 16 kt + 4 (lane / 16) + i of each of a block's four tiles.
// Two tiles' weights are the second operand of the product with the values without any exchange
// between lanes; a 32-bit weight goes into that product as two bfloat16 numbers (its rounding and
// the rest), so the weights keep sixteen bits and more where the values have eight.  The softmax runs over blocks of 64 keys with a running
// maximum and normaliser per row in 32-bit, everything in powers of two (log2 e is folded into the
// scale, and r1 ln(x) log2 e = r1 log2(x)): the four lanes of a row agree on the maximum by two
// exchanges a block and keep a sum each, which meet once at the end.
//
// Two forms.  Portions of prompts: a workgroup per (64 rows of one request's step, query head), 16
// rows a wavefront; a key block is staged once for the four wavefronts into one of two buffers in
// turn while the block before is multiplied.  Single tokens and short portions: a workgroup per
// (16 rows, query head) whose wavefronts take the key blocks in turn, each staging its own, and
// whose maxima, normalisers and sums meet in LDS at the end, in the order of the wavefronts.
#include "common.h"

namespace {

typedef __bf16 bf_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf_bf16x4 __attribute__((ext_vector_type(4)));
typedef float bf_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int bf_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int bf_u32x2 __attribute__((ext_vector_type(2)));

#define BF_WAVES 4
#define BF_KEYS 64
#define BF_LOG2E 1.44269504089f

__device__ __forceinline__ float bf_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float bf_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float bf_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float bf_query_factor(int p, float coef, int every) {
    return every > 0 ? 1.0f + coef * logf(static_cast<float>((p + 1) / every) + 1.0f) : 1.0f;
}

// what a lane carries of its row's softmax
template <int DT>
struct BfRow {
    float top = -INFINITY, sum = 0.f;        // the row's running maximum (the same in its four lanes); this lane's share of the normaliser
    bf_f32x4 acc[DT];
};

// the pieces of a key block that a thread brings from the pages: keys kb .. kb + 63 (those past
// pos_last: the last one again), values with zeros past pos_last
template <int D, int V, int THREADS>
struct BfFetch {
    static constexpr int KCH = BF_KEYS * (D / 8) / THREADS, VCH = V * (BF_KEYS / 8) / THREADS;
    bf_u32x4 k[KCH], v[VCH];
    __device__ __forceinline__ void load(int tid, int kb, int pos_last, const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                                         const int* __restrict__ pages, int page_shift, int page_mask, int page_tokens,
                                         size_t head_index_stride, int kvh, size_t layer_index) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + THREADS * i, key_in = c / (D / 8), part = c % (D / 8);
            const int key = min(kb + key_in, pos_last);
            const size_t head = (static_cast<size_t>(pages[key >> page_shift]) * head_index_stride + layer_index) + kvh;
            k[i] = *reinterpret_cast<const bf_u32x4*>(k_pool + (head * page_tokens + (key & page_mask)) * D + 8 * part);
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = tid + THREADS * i, d = c / (BF_KEYS / 8), part = c % (BF_KEYS / 8);
            const int key = kb + 8 * part;         // eight keys that lie side by side in one page
            bf_u32x4 val = {0u, 0u, 0u, 0u};
            if (key <= pos_last) {
                const size_t head = (static_cast<size_t>(pages[key >> page_shift]) * head_index_stride + layer_index) + kvh;
                val = *reinterpret_cast<const bf_u32x4*>(v_pool + (head * V + d) * page_tokens + (key & page_mask));
                const int live = pos_last - key + 1;       // keys of this piece that exist
                if (live < 8) {
                    if (live <= 6) val[3] = 0u; else val[3] &= 0x0000ffffu;
                    if (live <= 4) val[2] = 0u; else if (live == 5) val[2] &= 0x0000ffffu;
                    if (live <= 2) val[1] = 0u; else if (live == 3) val[1] &= 0x0000ffffu;
                    if (live == 1) val[0] &= 0x0000ffffu;
                }
            }
            v[i] = val;
        }
    }
    __device__ __forceinline__ void stage(int tid, __bf16* ks, __bf16* vs) const {
        constexpr int KROW = D + 8, VROW = BF_KEYS + 8;
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + THREADS * i;
            *reinterpret_cast<bf_u32x4*>(ks + (c / (D / 8)) * KROW + 8 * (c % (D / 8))) = k[i];
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = tid + THREADS * i;
            *reinterpret_cast<bf_u32x4*>(vs + (c / (BF_KEYS / 8)) * VROW + 8 * (c % (BF_KEYS / 8))) = v[i];
        }
    }
};

// one staged block of 64 keys for the 16 rows of a wavefront
template <int D, int V>
__device__ __forceinline__ void bf_block(const __bf16* ks, const __bf16* vs, const bf_bf16x8 (&qreg)[D / 32], BfRow<V / 16>& row, int kb,
                                         int my_pos, int window, int keep_first, bool kept_only, int r, int quad, float s2, float b1, float b2,
                                         bool biased) {
    constexpr int KROW = D + 8, VROW = BF_KEYS + 8, KS = D / 32, DT = V / 16;
    bf_f32x4 sacc[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
        sacc[kt] = bf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < KS; ++st) {
            const bf_bf16x8 kf = __builtin_bit_cast(bf_bf16x8, *reinterpret_cast<const bf_u32x4*>(ks + (16 * kt + r) * KROW + 32 * st + 8 * quad));
            sacc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qreg[st], sacc[kt], 0, 0, 0);
        }
    }
    float top = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kb + 16 * kt + 4 * quad + i;
            const bool seen = key <= my_pos && (kept_only ? key < keep_first : (window <= 0 || key > my_pos - window || key < keep_first));
            float x = sacc[kt][i] * s2;
            if (biased) x -= b1 * bf_log2(fmaf(b2, static_cast<float>(my_pos - key), 1.0f));
            x = seen ? x : -INFINITY;
            sacc[kt][i] = x;
            top = fmaxf(top, x);
        }
    top = fmaxf(top, __shfl_xor(top, 16, CELEG_WAVE));
    top = fmaxf(top, __shfl_xor(top, 32, CELEG_WAVE));
    const float new_top = fmaxf(row.top, top);
    const float base = new_top == -INFINITY ? 0.f : new_top;      // (a row that has seen no key yet: every weight 0)
    const float keep = bf_exp2(row.top - base);
    row.top = new_top;
    float sum = 0.f;
    bf_bf16x4 w[4], rest[4];         // a weight as two bfloat16 numbers: its rounding, and what the rounding left
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = bf_exp2(sacc[kt][i] - base);
            sum += p;
            w[kt][i] = static_cast<__bf16>(p);
            rest[kt][i] = static_cast<__bf16>(p - static_cast<float>(w[kt][i]));
        }
    row.sum = fmaf(row.sum, keep, sum);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) row.acc[dt][i] *= keep;
    // output, transposed: tile dt holds values 16 dt + 4 quad + i of row r
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
        const bf_bf16x8 pw = __builtin_shufflevector(w[2 * pair], w[2 * pair + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        const bf_bf16x8 pr = __builtin_shufflevector(rest[2 * pair], rest[2 * pair + 1], 0, 1, 2, 3, 4, 5, 6, 7);
        bf_bf16x8 vf[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const __bf16* vrow = vs + (16 * dt + r) * VROW + 32 * pair + 4 * quad;
            const bf_u32x2 lo = *reinterpret_cast<const bf_u32x2*>(vrow), hi = *reinterpret_cast<const bf_u32x2*>(vrow + 16);
            vf[dt] = __builtin_bit_cast(bf_bf16x8, bf_u32x4{lo[0], lo[1], hi[0], hi[1]});
            row.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pw, row.acc[dt], 0, 0, 0);
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) row.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pr, row.acc[dt], 0, 0, 0);
    }
}

// a finished row: divided by its normaliser, times sigmoid(gate), stored
template <int V>
__device__ __forceinline__ void bf_store(const BfRow<V / 16>& row, float total, const bf16* __restrict__ gate_row, bf16* __restrict__ out_row,
                                         int quad) {
    const float inv = 1.0f / total;
#pragma unroll
    for (int dt = 0; dt < V / 16; ++dt) {
        float g[4] = {1.f, 1.f, 1.f, 1.f};
        if (gate_row) {
            const bf_bf16x4 g4 = __builtin_bit_cast(bf_bf16x4, *reinterpret_cast<const bf_u32x2*>(gate_row + 16 * dt + 4 * quad));
#pragma unroll
            for (int i = 0; i < 4; ++i) g[i] = bf_sigmoid(static_cast<float>(g4[i]));
        }
        const bf_bf16x4 o4 = {static_cast<__bf16>(row.acc[dt][0] * inv * g[0]), static_cast<__bf16>(row.acc[dt][1] * inv * g[1]),
                              static_cast<__bf16>(row.acc[dt][2] * inv * g[2]), static_cast<__bf16>(row.acc[dt][3] * inv * g[3])};
        *reinterpret_cast<bf_bf16x4*>(out_row + 16 * dt + 4 * quad) = o4;
    }
}

struct BfArgs {
    const bf16* q;
    const bf16* k_pool;
    const bf16* v_pool;
    const int* table;
    const int* cu_seqlens;
    const int* seq_slot;
    const int* seq_start;
    const float* r1;
    const float* r2;
    const bf16* gate;
    bf16* out;
    int ldq, ldg, ldo, table_stride, n_seqs, q_heads, kv_heads, page_tokens, n_layers, layer, every, window, keep_first, sink_one;
    float scale, coef;
};

// The key blocks of a tile whose lowest position is pos0: first the blocks that hold the kept first keys
// where the window has passed them (only those keys count there), then the blocks from the window's start on.
struct BfBlocks {
    int n_kept, kb0;
    __device__ __forceinline__ BfBlocks(int pos0, int window, int keep) {
        const int key_first = window > 0 ? max(0, pos0 - window + 1) : 0;
        kb0 = key_first & ~7;
        n_kept = 0;
        if (keep > 0 && kb0 > 0) {
            if (kb0 >= keep) n_kept = (keep + BF_KEYS - 1) / BF_KEYS;
            else kb0 = 0;                 // the window begins among the kept keys: one run from the start
        }
    }
    __device__ __forceinline__ int count(int pos_last) const { return n_kept + (pos_last >= kb0 ? (pos_last - kb0) / BF_KEYS + 1 : 0); }
    __device__ __forceinline__ bool kept(int i) const { return i < n_kept; }
    __device__ __forceinline__ int start(int i) const { return i < n_kept ? i * BF_KEYS : kb0 + (i - n_kept) * BF_KEYS; }
    // the last key a block may touch: pages between the kept keys and the window may be gone
    __device__ __forceinline__ int last(int i, int pos_last, int keep) const { return i < n_kept ? keep - 1 : pos_last; }
};

// which tile of `rows` rows: tiles of all requests of the step, one after the other
__device__ __forceinline__ bool bf_find_tile(const BfArgs& a, int rows, int& tile, int& s, int& row0, int& n) {
    for (s = 0; s < a.n_seqs; ++s) {
        row0 = a.cu_seqlens[s];
        n = a.cu_seqlens[s + 1] - row0;
        const int tiles = (n + rows - 1) / rows;
        if (tile < tiles) return true;
        tile -= tiles;
    }
    return false;
}

template <int D, int V>
__global__ __launch_bounds__(BF_WAVES * CELEG_WAVE) void biased_attention_rows_kernel(const BfArgs a) {
    constexpr int KROW = D + 8, VROW = BF_KEYS + 8, KS = D / 32, DT = V / 16, BUF = BF_KEYS * KROW + V * VROW;
    constexpr int THREADS = BF_WAVES * CELEG_WAVE;
    extern __shared__ __attribute__((aligned(16))) unsigned char bf_lds[];
    __bf16* lds = reinterpret_cast<__bf16*>(bf_lds);
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE, tid = threadIdx.x;
    int tile = blockIdx.x, s, row0, n;
    if (!bf_find_tile(a, 64, tile, s, row0, n)) return;
    const int h = blockIdx.y, kvh = h / (a.q_heads / a.kv_heads);
    const int r = lane & 15, quad = lane >> 4;
    const int tile_row = tile * 64, tile_rows = min(64, n - tile_row);
    const int tile_pos0 = a.seq_start[s] + tile_row, pos_last = tile_pos0 + tile_rows - 1;
    const int first_row = tile_row + 16 * wave, rows_here = min(16, n - first_row);      // <= 0: this wavefront only stages
    const int my_row = first_row + max(0, min(r, rows_here - 1));
    const int safe_row = min(my_row, n - 1);
    const int my_pos = a.seq_start[s] + safe_row;
    const int wave_pos0 = a.seq_start[s] + first_row, wave_last = wave_pos0 + rows_here - 1;
    const int* pages = a.table + static_cast<size_t>(a.seq_slot[s]) * a.table_stride;
    const float s2 = a.scale * BF_LOG2E * bf_query_factor(my_pos, a.coef, a.every);
    const bool biased = a.r1 != nullptr;
    const float b1 = biased ? a.r1[h] : 0.f, b2 = biased ? a.r2[h] : 0.f;
    bf_bf16x8 qreg[KS];
    const bf16* qrow = a.q + static_cast<size_t>(row0 + safe_row) * a.ldq + static_cast<size_t>(h) * D;
#pragma unroll
    for (int st = 0; st < KS; ++st) qreg[st] = __builtin_bit_cast(bf_bf16x8, *reinterpret_cast<const bf_u32x4*>(qrow + 32 * st + 8 * quad));
    BfRow<DT> row;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) row.acc[dt] = bf_f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.sink_one) {
        row.top = 0.f;
        row.sum = quad == 0 ? 1.f : 0.f;
    }
    const int page_shift = 31 - __builtin_clz(a.page_tokens), page_mask = a.page_tokens - 1;
    const size_t head_index_stride = static_cast<size_t>(a.n_layers) * a.kv_heads, layer_index = static_cast<size_t>(a.layer) * a.kv_heads;
    BfFetch<D, V, THREADS> pre;
    const BfBlocks blocks(tile_pos0, a.window, a.keep_first);
    const int n_blocks = blocks.count(pos_last);
    pre.load(tid, blocks.start(0), blocks.last(0, pos_last, a.keep_first), a.k_pool, a.v_pool, pages, page_shift, page_mask, a.page_tokens,
             head_index_stride, kvh, layer_index);
    int turn = 0;
    for (int i = 0; i < n_blocks; ++i, turn ^= 1) {
        const int kb = blocks.start(i);
        __bf16* ks = lds + turn * BUF;
        __bf16* vs = ks + BF_KEYS * KROW;
        pre.stage(tid, ks, vs);
        __syncthreads();
        if (i + 1 < n_blocks)
            pre.load(tid, blocks.start(i + 1), blocks.last(i + 1, pos_last, a.keep_first), a.k_pool, a.v_pool, pages, page_shift, page_mask,
                     a.page_tokens, head_index_stride, kvh, layer_index);
        // blocks none of this wavefront's rows can see
        if (rows_here <= 0) continue;
        if (!blocks.kept(i) && (kb > wave_last || (a.window > 0 && kb >= a.keep_first && kb + BF_KEYS - 1 < wave_pos0 - a.window + 1))) continue;
        bf_block<D, V>(ks, vs, qreg, row, kb, my_pos, a.window, a.keep_first, blocks.kept(i), r, quad, s2, b1, b2, biased);
    }
    float total = row.sum;
    total += __shfl_xor(total, 16, CELEG_WAVE);
    total += __shfl_xor(total, 32, CELEG_WAVE);
    if (r >= rows_here) return;
    const size_t at = static_cast<size_t>(row0 + my_row);
    bf_store<V>(row, total, a.gate ? a.gate + at * a.ldg + static_cast<size_t>(h) * V : nullptr, a.out + at * a.ldo + static_cast<size_t>(h) * V,
                quad);
}

template <int D, int V, int WAVES>
__global__ __launch_bounds__(WAVES * CELEG_WAVE) void biased_attention_tile_kernel(const BfArgs a) {
    constexpr int KROW = D + 8, VROW = BF_KEYS + 8, KS = D / 32, DT = V / 16, BUF = BF_KEYS * KROW + V * VROW;
    extern __shared__ __attribute__((aligned(16))) unsigned char bf_lds[];
    const int wave = threadIdx.x / CELEG_WAVE, lane = threadIdx.x % CELEG_WAVE;
    __bf16* ks = reinterpret_cast<__bf16*>(bf_lds) + static_cast<size_t>(wave) * BUF;
    __bf16* vs = ks + BF_KEYS * KROW;
    int tile = blockIdx.x, s, row0, n;
    if (!bf_find_tile(a, 16, tile, s, row0, n)) return;
    const int h = blockIdx.y, kvh = h / (a.q_heads / a.kv_heads);
    const int r = lane & 15, quad = lane >> 4;
    const int first_row = tile * 16, rows_here = min(16, n - first_row);
    const int pos0 = a.seq_start[s] + first_row, pos_last = pos0 + rows_here - 1;
    const int my_row = first_row + min(r, rows_here - 1);      // rows past the end repeat the last one (not stored)
    const int my_pos = a.seq_start[s] + my_row;
    const int* pages = a.table + static_cast<size_t>(a.seq_slot[s]) * a.table_stride;
    const float s2 = a.scale * BF_LOG2E * bf_query_factor(my_pos, a.coef, a.every);
    const bool biased = a.r1 != nullptr;
    const float b1 = biased ? a.r1[h] : 0.f, b2 = biased ? a.r2[h] : 0.f;
    bf_bf16x8 qreg[KS];
    const bf16* qrow = a.q + static_cast<size_t>(row0 + my_row) * a.ldq + static_cast<size_t>(h) * D;
#pragma unroll
    for (int st = 0; st < KS; ++st) qreg[st] = __builtin_bit_cast(bf_bf16x8, *reinterpret_cast<const bf_u32x4*>(qrow + 32 * st + 8 * quad));
    BfRow<DT> row;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) row.acc[dt] = bf_f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.sink_one && wave == 0) {        // (once a row: the first wavefront's share)
        row.top = 0.f;
        row.sum = quad == 0 ? 1.f : 0.f;
    }
    const int page_shift = 31 - __builtin_clz(a.page_tokens), page_mask = a.page_tokens - 1;
    const size_t head_index_stride = static_cast<size_t>(a.n_layers) * a.kv_heads, layer_index = static_cast<size_t>(a.layer) * a.kv_heads;
    BfFetch<D, V, CELEG_WAVE> pre;
    const BfBlocks blocks(pos0, a.window, a.keep_first);
    const int n_blocks = blocks.count(pos_last);
    if (wave < n_blocks)
        pre.load(lane, blocks.start(wave), blocks.last(wave, pos_last, a.keep_first), a.k_pool, a.v_pool, pages, page_shift, page_mask,
                 a.page_tokens, head_index_stride, kvh, layer_index);
    for (int i = wave; i < n_blocks; i += WAVES) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        pre.stage(lane, ks, vs);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (i + WAVES < n_blocks)
            pre.load(lane, blocks.start(i + WAVES), blocks.last(i + WAVES, pos_last, a.keep_first), a.k_pool, a.v_pool, pages, page_shift,
                     page_mask, a.page_tokens, head_index_stride, kvh, layer_index);
        bf_block<D, V>(ks, vs, qreg, row, blocks.start(i), my_pos, a.window, a.keep_first, blocks.kept(i), r, quad, s2, b1, b2, biased);
    }
    // the wavefronts' maxima, normalisers and sums meet in LDS (every wavefront's staging area is
    // free after the barrier); the first one joins them in the order of the wavefronts and stores
    constexpr int PER = DT * 4 + 2;
    __syncthreads();
    float* parts = reinterpret_cast<float*>(bf_lds);
    if (wave > 0) {
        float* mine = parts + static_cast<size_t>(wave - 1) * PER * CELEG_WAVE;
        mine[lane] = row.top;
        mine[CELEG_WAVE + lane] = row.sum;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[(2 + dt * 4 + i) * CELEG_WAVE + lane] = row.acc[dt][i];
    }
    __syncthreads();
    if (wave > 0) return;
    float top = row.top;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) top = fmaxf(top, parts[static_cast<size_t>(w - 1) * PER * CELEG_WAVE + lane]);
    // (the row's own key is visible, so the maximum over all wavefronts is finite)
    const float mine = bf_exp2(row.top - top);
    float total = row.sum * mine;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) row.acc[dt][i] *= mine;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
        const float* theirs = parts + static_cast<size_t>(w - 1) * PER * CELEG_WAVE;
        const float f = bf_exp2(theirs[lane] - top);
        total = fmaf(theirs[CELEG_WAVE + lane], f, total);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) row.acc[dt][i] = fmaf(theirs[(2 + dt * 4 + i) * CELEG_WAVE + lane], f, row.acc[dt][i]);
    }
    total += __shfl_xor(total, 16, CELEG_WAVE);
    total += __shfl_xor(total, 32, CELEG_WAVE);
    if (r >= rows_here) return;
    const size_t at = static_cast<size_t>(row0 + my_row);
    bf_store<V>(row, total, a.gate ? a.gate + at * a.ldg + static_cast<size_t>(h) * V : nullptr, a.out + at * a.ldo + static_cast<size_t>(h) * V,
                quad);
}

constexpr int bf_block_bytes(int d, int v) { return (BF_KEYS * (d + 8) + v * (BF_KEYS + 8)) * 2; }
// single tiles: eight wavefronts share out the key blocks where their staging areas fit LDS
constexpr int bf_tile_waves(int d, int v) { return 8 * bf_block_bytes(d, v) <= 160 * 1024 ? 8 : BF_WAVES; }

template <int D, int V>
int bf_launch(int form, int max_tiles, const BfArgs& a, hipStream_t stream) {
    if (form == 1) {
        dim3 grid(max_tiles, a.q_heads), block(BF_WAVES * CELEG_WAVE);
        hipLaunchKernelGGL((biased_attention_rows_kernel<D, V>), grid, block, 2 * bf_block_bytes(D, V), stream, a);
    } else {
        constexpr int WAVES = bf_tile_waves(D, V);
        dim3 grid(max_tiles, a.q_heads), block(WAVES * CELEG_WAVE);
        hipLaunchKernelGGL((biased_attention_tile_kernel<D, V, WAVES>), grid, block, WAVES * bf_block_bytes(D, V), stream, a);
    }
    return CELEG_LAUNCH_RESULT();
}

template <int D>
int bf_launch_v(int v_dim, int form, int max_tiles, const BfArgs& a, hipStream_t stream) {
    switch (v_dim) {
        case 32: return bf_launch<D, 32>(form, max_tiles, a, stream);
        case 64: return bf_launch<D, 64>(form, max_tiles, a, stream);
        case 96: return bf_launch<D, 96>(form, max_tiles, a, stream);
        default: return bf_launch<D, 128>(form, max_tiles, a, stream);
    }
}

}  // namespace

// sizes of keys and values a head that the matrix-core kernels take
extern "C" int celeg_biased_attention_fast_ok(int head_dim, int v_dim) {
    auto ok = [](int n) { return n == 32 || n == 64 || n == 96 || n == 128; };
    return ok(head_dim) && ok(v_dim);
}

// bfloat16 on the matrix cores; form 0: tiles of 16 rows whose key blocks the wavefronts share out
// (single tokens, short portions), form 1: tiles of 64 rows that stage a key block once for four
// wavefronts (portions of prompts); max_tiles: an upper bound on the step's tiles (sum over
// requests of ceil(rows / 16 or 64)); pages of a power of two of at least 8 tokens; q, gate and out
// rows start at multiples of 16, 8 and 8 bytes
extern "C" int celeg_biased_attention_fast(int form, const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                                           int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start, int n_seqs,
                                           int max_tiles, const float* r1, const float* r2, const void* gate, int ldg, void* out, int ldo,
                                           int q_heads, int kv_heads, int head_dim, int v_dim, int page_tokens, int n_layers, int layer,
                                           float scale, float coef, int every, int window, int keep_first, int sink_one,
                                           hipStream_t stream) {
    if (max_tiles <= 0 || n_seqs <= 0) return 0;
    if (!celeg_biased_attention_fast_ok(head_dim, v_dim) || q_heads % kv_heads || page_tokens < 8 || (page_tokens & (page_tokens - 1)) ||
        ldq % 8 || ldo % 4 || (gate && ldg % 4) || (r1 == nullptr) != (r2 == nullptr))
        return static_cast<int>(hipErrorInvalidValue);
    BfArgs a;
    a.q = static_cast<const bf16*>(q);
    a.k_pool = static_cast<const bf16*>(k_pool);
    a.v_pool = static_cast<const bf16*>(v_pool);
    a.table = table;
    a.cu_seqlens = cu_seqlens;
    a.seq_slot = seq_slot;
    a.seq_start = seq_start;
    a.r1 = r1;
    a.r2 = r2;
    a.gate = static_cast<const bf16*>(gate);
    a.out = static_cast<bf16*>(out);
    a.ldq = ldq;
    a.ldg = ldg;
    a.ldo = ldo;
    a.table_stride = table_stride;
    a.n_seqs = n_seqs;
    a.q_heads = q_heads;
    a.kv_heads = kv_heads;
    a.page_tokens = page_tokens;
    a.n_layers = n_layers;
    a.layer = layer;
    a.every = every;
    a.window = window;
    a.keep_first = window > 0 ? keep_first : 0;
    a.sink_one = sink_one;
    a.scale = scale;
    a.coef = coef;
    switch (head_dim) {
        case 32: return bf_launch_v<32>(v_dim, form, max_tiles, a, stream);
        case 64: return bf_launch_v<64>(v_dim, form, max_tiles, a, stream);
        case 96: return bf_launch_v<96>(v_dim, form, max_tiles, a, stream);
        default: return bf_launch_v<128>(v_dim, form, max_tiles, a, stream);
    }
}
