// A routed feed-forward: every row goes to `top` of E expert feed-forwards.
//   route:   scores from the router's 32-bit logits, the `top` largest chosen per row;
//   plan:    rows sorted by expert (a row's place among its expert's rows is its order in the
//            batch), and the list of row tiles that the products walk;
//   gather:  the rows laid in that order, each times its weight if the weight goes on the input;
//   product: out[p] = a[p] w[expert of p]^T over the tiles;
//   combine: a row's `top` results summed (times the weight if it goes on the output).
// Nothing is planned on the host: grids are sized by bounds, so a recorded step replays.
#include "mfma_rows.h"
#include "small_gemm.h"

#define MOE_MAX_PER_LANE 8        // experts <= 512

// ---------------------------------------------------------------- route
// How a row's experts are chosen and weighted.  score 0: sigmoid of the logit; 1: softmax over all
// experts.  groups > 1: the experts form `groups` equal runs of neighbours, a run's score is the sum of
// its two largest scores, and only experts of the `keep` best runs (the lower run among equal ones) can be
// chosen.  The chosen experts' scores are the weights; with `renorm` they are divided by their sum plus
// renorm_eps; then times `scale`.
struct MoeRule {
    int experts, top, score, renorm, groups, keep;
    float renorm_eps, scale;
};

__device__ __forceinline__ float route_score(float z, int score, float zmax, float denom) {
    return score == 1 ? expf(z - zmax) / denom : 1.0f / (1.0f + expf(-z));
}

// One wavefront per row.
__device__ __forceinline__ void route_row(const float* z, const MoeRule& rule, int* ids, float* weights) {
    const int experts = rule.experts, top = rule.top, score = rule.score;
    const int lane = threadIdx.x & 63;
    float v[MOE_MAX_PER_LANE];
    float zmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
        const int e = lane + j * CELEG_WAVE;
        v[j] = e < experts ? z[e] : -INFINITY;
        zmax = fmaxf(zmax, v[j]);
    }
    float denom = 1.f;
    if (score == 1) {
        zmax = wave_max(zmax);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
            if (lane + j * CELEG_WAVE < experts) s += expf(v[j] - zmax);
        denom = wave_sum(s);
    }
    if (rule.groups > 1) {
        // every run's two largest scores (the largest logits give them), their sum in lane g of `mine`
        const int per = experts / rule.groups;
        float mine = -INFINITY;
        for (int g = 0; g < rule.groups; ++g) {
            float first = -INFINITY, second = -INFINITY;      // this lane's two largest logits of run g
#pragma unroll
            for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
                const int e = lane + j * CELEG_WAVE;
                if (e < experts && e / per == g) {
                    if (v[j] > first) { second = first; first = v[j]; }
                    else if (v[j] > second) second = v[j];
                }
            }
#pragma unroll
            for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
                const float of = __shfl_xor(first, off, CELEG_WAVE), os = __shfl_xor(second, off, CELEG_WAVE);
                const float hi = fmaxf(first, of), lo = fminf(first, of);
                second = fmaxf(lo, fmaxf(second, os));
                first = hi;
            }
            float sum = route_score(first, score, zmax, denom);
            if (per > 1) sum += route_score(second, score, zmax, denom);
            if (lane == g) mine = sum;
        }
        // the `keep` best runs stay; the experts of the others leave the choice
        unsigned long long kept = 0ull;
        for (int k = 0; k < rule.keep; ++k) {
            float best = mine;
            int best_g = lane < rule.groups ? lane : 0x7fffffff;
            if (lane >= rule.groups) best = -INFINITY;
#pragma unroll
            for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, CELEG_WAVE);
                const int og = __shfl_xor(best_g, off, CELEG_WAVE);
                if (ob > best || (ob == best && og < best_g)) { best = ob; best_g = og; }
            }
            kept |= 1ull << best_g;
            if (lane == best_g) mine = -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
            const int e = lane + j * CELEG_WAVE;
            if (e < experts && !((kept >> (e / per)) & 1ull)) v[j] = -INFINITY;
        }
    }
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        // the largest logit left, the lowest expert among equal ones
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j) {
            const int e = lane + j * CELEG_WAVE;
            if (e < experts && (v[j] > best || (v[j] == best && e < best_e))) { best = v[j]; best_e = e; }
        }
#pragma unroll
        for (int off = CELEG_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, CELEG_WAVE);
            const int oe = __shfl_xor(best_e, off, CELEG_WAVE);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; }
        }
#pragma unroll
        for (int j = 0; j < MOE_MAX_PER_LANE; ++j)
            if (lane + j * CELEG_WAVE == best_e) v[j] = -INFINITY;
        const float s = route_score(best, score, zmax, denom);
        total += s;
        if (lane == 0) {
            ids[k] = best_e;
            weights[k] = s;
        }
    }
    if (lane == 0 && (rule.renorm || rule.scale != 1.0f))
        for (int k = 0; k < top; ++k) weights[k] = (rule.renorm ? weights[k] / (total + rule.renorm_eps) : weights[k]) * rule.scale;
}

__global__ void moe_route_kernel(const float* __restrict__ logits, MoeRule rule, int* __restrict__ ids, float* __restrict__ weights) {
    const size_t t = blockIdx.x;
    route_row(logits + t * rule.experts, rule, ids + t * rule.top, weights + t * rule.top);
}

// The router's product and the choice in one kernel: a workgroup takes four rows, keeps them in LDS
// in 32-bit, its wavefronts share out the experts (a weight is read once for the four rows; a row's
// sum runs over k in an order that depends on nothing else), then each wavefront routes one row.
#define ROUTE_ROWS 4
template <typename TX>
__global__ __launch_bounds__(256) void moe_router_kernel(const TX* __restrict__ x, const float* __restrict__ w, int rows,
                                                         int width, MoeRule rule, int* __restrict__ ids, float* __restrict__ weights) {
    const int experts = rule.experts, top = rule.top;
    extern __shared__ float router_lds[];        // ROUTE_ROWS rows of width, then ROUTE_ROWS rows of logits
    float* xs = router_lds;
    float* zs = router_lds + ROUTE_ROWS * width;
    const int row0 = blockIdx.x * ROUTE_ROWS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < ROUTE_ROWS * width; i += 256) {
        const int r = i / width;
        xs[i] = row0 + r < rows ? to_float(x[static_cast<size_t>(row0) * width + i]) : 0.f;
    }
    __syncthreads();
    for (int e = wave; e < experts; e += 4) {
        const float* we = w + static_cast<size_t>(e) * width;
        float acc[ROUTE_ROWS] = {0.f, 0.f, 0.f, 0.f};
        if ((width & 3) == 0) {
            // four neighbouring weights a lane and load, several loads in flight
            typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll 4
            for (int i = 4 * lane; i < width; i += 4 * CELEG_WAVE) {
                const f32x4 wv = *reinterpret_cast<const f32x4*>(we + i);
#pragma unroll
                for (int r = 0; r < ROUTE_ROWS; ++r) {
                    const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + r * width + i);
                    acc[r] = fmaf(xv[3], wv[3], fmaf(xv[2], wv[2], fmaf(xv[1], wv[1], fmaf(xv[0], wv[0], acc[r]))));
                }
            }
        } else {
            for (int i = lane; i < width; i += CELEG_WAVE) {
                const float wv = we[i];
#pragma unroll
                for (int r = 0; r < ROUTE_ROWS; ++r) acc[r] = fmaf(xs[r * width + i], wv, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < ROUTE_ROWS; ++r) {
            const float total = wave_sum(acc[r]);
            if (lane == 0) zs[r * experts + e] = total;
        }
    }
    __syncthreads();
    const int t = row0 + wave;
    if (t < rows)
        route_row(zs + wave * experts, rule, ids + static_cast<size_t>(t) * top, weights + static_cast<size_t>(t) * top);
}

// ---------------------------------------------------------------- plan
// One workgroup.  ids [n] -> offsets [E + 1], place_of [n] (entry -> place), entry_at [n] (place ->
// entry), and the tiles of `tile_rows` rows: tile_expert, tile_row0 [max_tiles], n_tiles.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int n, int experts, int tile_rows,
                                                        int* __restrict__ offsets, int* __restrict__ place_of,
                                                        int* __restrict__ entry_at, int* __restrict__ tile_expert,
                                                        int* __restrict__ tile_row0, int* __restrict__ n_tiles) {
    extern __shared__ int plan_lds[];     // counts [E], starts [E + 1]
    int* counts = plan_lds;
    int* starts = plan_lds + experts;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    // an entry's rank among the entries of its expert, in batch order
    for (int e = wave; e < experts; e += n_waves) {
        int running = 0;
        for (int base = 0; base < n; base += CELEG_WAVE) {
            const int i = base + lane;
            const bool mine = i < n && ids[i] == e;
            const unsigned long long mask = __ballot(mine);
            if (mine) place_of[i] = running + __popcll(mask & ((1ull << lane) - 1ull));
            running += __popcll(mask);
        }
        if (lane == 0) counts[e] = running;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < experts; ++e) {
            starts[e] = at;
            offsets[e] = at;
            for (int r = 0; r < counts[e]; r += tile_rows) {
                tile_expert[tiles] = e;
                tile_row0[tiles] = at + r;
                ++tiles;
            }
            at += counts[e];
        }
        starts[experts] = at;
        offsets[experts] = at;
        n_tiles[0] = tiles;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int e = ids[i];
        const int place = (e >= 0 && e < experts ? starts[e] : 0) + place_of[i];
        place_of[i] = place;
        entry_at[place] = i;
    }
}

// ---------------------------------------------------------------- gather
// a[p, :] = x[entry_at[p] / top, :] (* weight of the entry)
template <typename T>
__global__ void moe_gather_kernel(const T* __restrict__ x, const int* __restrict__ entry_at,
                                  const float* __restrict__ weights, T* __restrict__ a, int top, int width) {
    const int p = blockIdx.x;
    const int entry = entry_at[p];
    const float wgt = weights ? weights[entry] : 1.f;
    const T* src = x + static_cast<size_t>(entry / top) * width;
    T* dst = a + static_cast<size_t>(p) * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = weights ? from_float<T>(wgt * to_float(src[i])) : src[i];
}

// ---------------------------------------------------------------- product over the tiles
// w: [E, N, K]; a: [n, K]; out: [n, N].  gated: w holds, per expert, N gate rows then N up rows, and
// out = silu(a gate^T) * (a up^T) (the two sums rounded to T first, as where they are tensors).  Not gated, with
// act 1: the square of relu of the sum (rounded to T first); act 0: the sum itself.
template <typename T>
__global__ __launch_bounds__(256) void moe_product_kernel(const T* __restrict__ a, const T* __restrict__ w,
                                                          T* __restrict__ out, int N, int K, int gated, int act,
                                                          const int* __restrict__ offsets,
                                                          const int* __restrict__ tile_expert,
                                                          const int* __restrict__ tile_row0,
                                                          const int* __restrict__ n_tiles) {
    __shared__ float as[SG_ROWS][SG_K + 1], ws[SG_COLS][SG_K + 1];
    const int tile = blockIdx.x;
    if (tile >= n_tiles[0]) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile];
    const int rows_valid = min(SG_ROWS, offsets[e + 1] - row0);
    const int col0 = blockIdx.y * SG_COLS, cols_valid = min(SG_COLS, N - col0);
    const size_t per_expert = static_cast<size_t>(gated ? 2 : 1) * N * K;
    const T* we = w + static_cast<size_t>(e) * per_expert + static_cast<size_t>(col0) * K;
    SmallTileSums sums, ups;
    small_tile_product(a + static_cast<size_t>(row0) * K, K, rows_valid, we, K, cols_valid, K, as, ws, sums);
    if (gated) small_tile_product(a + static_cast<size_t>(row0) * K, K, rows_valid, we + static_cast<size_t>(N) * K, K, cols_valid, K, as, ws, ups);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = ty + 16 * i;
        if (r >= rows_valid) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = tx + 16 * j;
            if (c >= cols_valid) continue;
            float v = sums.v[i][j];
            if (gated) {
                const float g = to_float(from_float<T>(v)), u = to_float(from_float<T>(ups.v[i][j]));
                v = (g / (1.0f + expf(-g))) * u;
            } else if (act == 1) {
                const float z = fmaxf(to_float(from_float<T>(v)), 0.f);
                v = z * z;
            }
            out[static_cast<size_t>(row0 + r) * N + col0 + c] = from_float<T>(v);
        }
    }
}

// The same on the matrix cores (bfloat16; K a multiple of 32, N of 16): tiles of 64 rows x 128 columns (256 for a
// single stream of weights), a wavefront two (four) tiles of 16 columns, where the experts' tiles hold many rows (every operand of a used twice);
// 64 columns, one tile a wavefront, where they hold few (a step of single tokens is bound by how many
// workgroups pull the weights).
template <bool GATED, int MOE_CT>
__global__ __launch_bounds__(256, 2) void moe_product_mfma_kernel(const __bf16* __restrict__ a, const __bf16* __restrict__ w,
                                                                  __bf16* __restrict__ out, int N, int K, int act,
                                                                  const int* __restrict__ offsets,
                                                                  const int* __restrict__ tile_expert,
                                                                  const int* __restrict__ tile_row0,
                                                                  const int* __restrict__ n_tiles) {
    constexpr int S = GATED ? 2 : 1;
    const int tile = blockIdx.x;
    if (tile >= n_tiles[0]) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile];
    const int rows_valid = min(MR_ROWS, offsets[e + 1] - row0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, qd = lane >> 4;
    const int col0 = blockIdx.y * (MR_COLS * MOE_CT) + wave * 16 * MOE_CT;
    if (col0 >= N) return;
    const size_t per_expert = static_cast<size_t>(S) * N * K;
    const __bf16* w_row[S][MOE_CT];
#pragma unroll
    for (int ct = 0; ct < MOE_CT; ++ct) {
        const int col = col0 + ct * 16 + c;
        w_row[0][ct] = col < N ? w + static_cast<size_t>(e) * per_expert + static_cast<size_t>(col) * K : nullptr;
        if (GATED) w_row[S - 1][ct] = col < N ? w_row[0][ct] + static_cast<size_t>(N) * K : nullptr;
    }
    const __bf16* a_row[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) a_row[rt] = rt * 16 + c < rows_valid ? a + static_cast<size_t>(row0 + rt * 16 + c) * K : nullptr;
    mr_f32x4 sums[S][MOE_CT][4];
    mfma_rows_product<S, MOE_CT>(a_row, (rows_valid + 15) / 16, w_row, K, sums);
#pragma unroll
    for (int ct = 0; ct < MOE_CT; ++ct) {
        const int col = col0 + ct * 16 + 4 * qd;
        if (col >= N) continue;
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            if (rt * 16 + c >= rows_valid) continue;
            mr_bf16x4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float x = sums[0][ct][rt][r];
                if (GATED) {
                    const float g = static_cast<float>(static_cast<__bf16>(x));
                    const float u = static_cast<float>(static_cast<__bf16>(sums[S - 1][ct][rt][r]));
                    x = (g / (1.0f + expf(-g))) * u;
                } else if (act == 1) {
                    const float z = fmaxf(static_cast<float>(static_cast<__bf16>(x)), 0.f);
                    x = z * z;
                }
                v[r] = static_cast<__bf16>(x);
            }
            *reinterpret_cast<mr_bf16x4*>(out + static_cast<size_t>(row0 + rt * 16 + c) * N + col) = v;
        }
    }
}

// ---------------------------------------------------------------- combine
// out[t, :] = (base[t, :] +) sum_k (weight of entry (t, k)) * y[place_of[t * top + k], :], summed in 32-bit
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ place_of,
                                   const float* __restrict__ weights, const T* __restrict__ base, T* __restrict__ out, int top,
                                   int width) {
    const int t = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int entry = t * top + k;
            const float v = to_float(y[static_cast<size_t>(place_of[entry]) * width + i]);
            acc += weights ? weights[entry] * v : v;
        }
        if (base) acc += to_float(base[static_cast<size_t>(t) * width + i]);
        out[static_cast<size_t>(t) * width + i] = from_float<T>(acc);
    }
}

// ---------------------------------------------------------------- entry points
// whether a rule is one the routing kernels take: groups that divide the experts evenly, at most 64 of them,
// and enough experts in the kept ones
static bool moe_rule_ok(const MoeRule& r) {
    if (r.experts <= 0 || r.experts > MOE_MAX_PER_LANE * CELEG_WAVE || r.top <= 0 || r.top > r.experts) return false;
    if (r.groups < 1 || r.groups > CELEG_WAVE || r.experts % r.groups || r.keep < 1 || r.keep > r.groups) return false;
    return r.top <= r.keep * (r.experts / r.groups);
}

extern "C" int celeg_moe_route(const float* logits, int rows, int experts, int top, int score, int renorm, int groups, int keep,
                               float renorm_eps, float scale, int* ids, float* weights, hipStream_t stream) {
    if (rows <= 0) return 0;
    const MoeRule rule{experts, top, score, renorm, groups, keep, renorm_eps, scale};
    if (!moe_rule_ok(rule)) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(moe_route_kernel, dim3(rows), dim3(CELEG_WAVE), 0, stream, logits, rule, ids, weights);
    return CELEG_LAUNCH_RESULT();
}

// rows of a tile: 64 where every product of the plan runs on the matrix cores, else 32
// x [rows, width] (32-bit or bfloat16) times the router's 32-bit matrix w [experts, width], then the choice
extern "C" int celeg_moe_router(const void* x, int x_dtype, const float* w, int rows, int width, int experts, int top,
                                int score, int renorm, int groups, int keep, float renorm_eps, float scale, int* ids,
                                float* weights, hipStream_t stream) {
    if (rows <= 0) return 0;
    const size_t lds = static_cast<size_t>(ROUTE_ROWS) * (width + experts) * sizeof(float);
    const MoeRule rule{experts, top, score, renorm, groups, keep, renorm_eps, scale};
    if (!moe_rule_ok(rule) || lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid((rows + ROUTE_ROWS - 1) / ROUTE_ROWS);
    if (x_dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_router_kernel<float>, grid, dim3(256), lds, stream, static_cast<const float*>(x), w, rows, width,
                           rule, ids, weights);
    else
        hipLaunchKernelGGL(moe_router_kernel<bf16>, grid, dim3(256), lds, stream, static_cast<const bf16*>(x), w, rows, width,
                           rule, ids, weights);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_tile_rows(int matrix_cores) { return matrix_cores ? MR_ROWS : SG_ROWS; }

extern "C" int celeg_moe_plan(const int* ids, int n, int experts, int tile_rows, int* offsets, int* place_of, int* entry_at,
                              int* tile_expert, int* tile_row0, int* n_tiles, hipStream_t stream) {
    if (n <= 0) return 0;
    const size_t lds = static_cast<size_t>(2 * experts + 1) * sizeof(int);
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), lds, stream, ids, n, experts, tile_rows, offsets, place_of,
                       entry_at, tile_expert, tile_row0, n_tiles);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_gather(const void* x, int dtype, const int* entry_at, const float* weights, void* a, int n,
                                int top, int width, hipStream_t stream) {
    if (n <= 0) return 0;
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_gather_kernel<float>, dim3(n), dim3(256), 0, stream, static_cast<const float*>(x), entry_at,
                           weights, static_cast<float*>(a), top, width);
    else
        hipLaunchKernelGGL(moe_gather_kernel<bf16>, dim3(n), dim3(256), 0, stream, static_cast<const bf16*>(x), entry_at,
                           weights, static_cast<bf16*>(a), top, width);
    return CELEG_LAUNCH_RESULT();
}

extern "C" int celeg_moe_product(const void* a, const void* w, void* out, int dtype, int N, int K, int gated, int act,
                                 const int* offsets, const int* tile_expert, const int* tile_row0, const int* n_tiles,
                                 int max_tiles, int tile_rows, int wide, hipStream_t stream) {
    if (max_tiles <= 0) return 0;
    if (tile_rows == MR_ROWS) {
        if (dtype != CELEG_BF16 || K % 32 || N % 16) return static_cast<int>(hipErrorInvalidValue);
        const int ct = wide ? (gated ? 2 : 4) : 1;     // (one stream of weights leaves registers for four column tiles)
        dim3 grid(max_tiles, (N + MR_COLS * ct - 1) / (MR_COLS * ct));
#define MOE_GO(GATED, CT)                                                                                                       \
    hipLaunchKernelGGL((moe_product_mfma_kernel<GATED, CT>), grid, dim3(256), 0, stream, static_cast<const __bf16*>(a),         \
                       static_cast<const __bf16*>(w), static_cast<__bf16*>(out), N, K, act, offsets, tile_expert, tile_row0, n_tiles)
        if (gated && wide) MOE_GO(true, 2);
        else if (gated) MOE_GO(true, 1);
        else if (wide) MOE_GO(false, 4);
        else MOE_GO(false, 1);
#undef MOE_GO
        return CELEG_LAUNCH_RESULT();
    }
    if (tile_rows != SG_ROWS) return static_cast<int>(hipErrorInvalidValue);
    dim3 grid(max_tiles, (N + SG_COLS - 1) / SG_COLS);
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_product_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(a),
                           static_cast<const float*>(w), static_cast<float*>(out), N, K, gated, act, offsets, tile_expert,
                           tile_row0, n_tiles);
    else
        hipLaunchKernelGGL(moe_product_kernel<bf16>, grid, dim3(256), 0, stream, static_cast<const bf16*>(a),
                           static_cast<const bf16*>(w), static_cast<bf16*>(out), N, K, gated, act, offsets, tile_expert,
                           tile_row0, n_tiles);
    return CELEG_LAUNCH_RESULT();
}

// base: rows [rows, width] added to the sum (what every row gets besides its experts), or null
extern "C" int celeg_moe_combine(const void* y, int dtype, const int* place_of, const float* weights, const void* base, void* out,
                                 int rows, int top, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dtype == CELEG_F32)
        hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(rows), dim3(256), 0, stream, static_cast<const float*>(y),
                           place_of, weights, static_cast<const float*>(base), static_cast<float*>(out), top, width);
    else
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, dim3(rows), dim3(256), 0, stream, static_cast<const bf16*>(y), place_of,
                           weights, static_cast<const bf16*>(base), static_cast<bf16*>(out), top, width);
    return CELEG_LAUNCH_RESULT();
}
