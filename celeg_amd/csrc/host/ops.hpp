// The kernels as host calls: shapes, dtypes, strides and limits are checked here, then the
// extern "C" entry points are called with raw device pointers and the runtime's stream (so a
// stream that is recording a graph records them too).  There is no fallback: a size a kernel
// was not written for is a KernelError that says why.
//
// Matrix products in bfloat16 of more than 64 rows go to hipBLASLt (blaslt.cpp), as the
// reference sends its products to cuBLAS (src/backend/cuda/runtime/gemm_dispatcher.cpp);
// products in 32-bit go to this library's own kernel, which uses no reduced-precision matrix
// mode.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>

#include "batch.hpp"
#include "blaslt.hpp"
#include "cache.hpp"
#include "device.hpp"
#include "weights.hpp"

namespace celeg {

enum class Epilogue : int { Store = 0, StoreF32 = 1, Residual = 2, Swiglu = 3, Conv = 4 };

// What follows a q/k/v product of many rows inside its kernel (heads of 64 columns): the norm of
// query and key heads, their rotation by the rows' positions, and the write of keys and values
// into the pages of the rows' requests; the query heads alone reach `out`.
struct QkvTail {
    int heads = 0, kv_heads = 0, head_dim = 0;
    const Tensor* q_weight = nullptr;      // [head_dim] 32-bit, or null: no norm
    const Tensor* k_weight = nullptr;
    float eps = 0.f;
    const Tensor* inv_freq = nullptr;      // [head_dim / 2], or null: no rotation
    const StepBatch* batch = nullptr;
    const KVView* kv = nullptr;
};

// A decode-only step's own keys and values as the q/k/v product left them, for an attention
// that normalises and turns q and the new keys itself and writes keys and values into the pages.
struct FreshKV {
    const Tensor* k = nullptr;             // [rows, kv_heads * head_dim]
    const Tensor* v = nullptr;
    const Tensor* q_weight = nullptr;      // [head_dim] 32-bit, or null: no norm
    const Tensor* k_weight = nullptr;
    float eps = 0.f;
    const Tensor* inv_freq = nullptr;      // [head_dim / 2], or null: no rotation
};

// The convolution epilogue's operands: one new token per request.
struct ConvOperands {
    Tensor taps;          // [N, L] 32-bit
    Tensor bias;          // optional [N]
    Tensor state;         // [slots, L, N] 32-bit, the slots a fixed number of elements apart
    const int* seq_slot = nullptr;   // [M]
};

struct FusedArgs {
    Epilogue epilogue = Epilogue::Store;
    Tensor norm_weight;           // the older form: the 32-bit stream normalised on the fly
    float eps = 0.f;
    Tensor stats;                 // partial sums of squares of the rows of the stream [rows, >= stat_blocks]
    int stat_blocks = 0;
    const int* rows = nullptr;    // picks rows of a
    int n_rows = -1;              // number of output rows (with rows: how many are picked)
    Tensor bias;
    Tensor stats_out;             // residual: partial sums of squares of the new rows
    const ConvOperands* conv = nullptr;
    Tensor out_bf16;              // residual: the bfloat16 copy of the stream
    bool packed = false;          // w is [K/32, rows, 32] (pack_weight)
    // 32-bit store of an output head: beside the logits, the best (logit, index) of every share of
    // columns [row_best_rows, row_best_ld >= parts]; Ops::last_best_parts then says how many parts
    // of every row were written
    unsigned long long* row_best = nullptr;
    int row_best_ld = 0, row_best_rows = 0;
};

// What an output head left beside its logits for greedy rows: the best (logit, index) of every
// share of a row's columns [rows, ld >= parts], for the first `rows` rows of `logits`.
struct HeadBest {
    const void* logits = nullptr;
    const unsigned long long* best = nullptr;
    int ld = 0, parts = 0, rows = 0;
    int cols = 0;        // columns a part stands for: part p is the best of columns p * cols .. + cols - 1
};

// What a step begins with, when the runner leaves it to the step's first kernel: the block-table
// updates of the (one) cache group and the rows whose token is on the device.
struct StepPrologue {
    int* table = nullptr;
    int stride = 0, n_slots = 0;
    const int* updates = nullptr;
    int capacity = 0;
    int* token_ids = nullptr;
    const int* token_slot = nullptr;
    const int* last_tokens = nullptr;
    int n = 0;
    bool pending = false;
};

// Which kernel a call was handed to (counted per Ops at the time of the launch, also while a
// graph records; a replay counts nothing): what tests and tools ask to see that a size took the
// path it was meant to take.
enum class Path : int {
    AttentionDecode = 0, AttentionDecodeFresh, AttentionRows, AttentionGeneral, AttentionSigmoid, AttentionSigmoidRows, AttentionSigmoidDecode, DeltaRule, AttentionLatent, AttentionLatentRows, AttentionLatentDecode, AttentionBiased, AttentionBiasedRows, AttentionBiasedDecode, ChannelScan, LinearRecurrentUnit, RoutedExperts, LinearF32, LinearLibrary, LinearStandIn,
    FusedSliced, FusedRows, FusedStaged, Tiled, TiledQkv, ArgmaxMerged, Count
};
const char* path_name(Path p);

class Ops {
public:
    explicit Ops(hipStream_t stream) : stream(stream) {}
    hipStream_t stream;
    long long path_count[static_cast<int>(Path::Count)] = {};
    void took(Path p) { ++path_count[static_cast<int>(p)]; }
    Json paths_json() const;
    // knobs (tests and tuning)
    int attention_decode_whole = -1;     // -1: chosen from the batch; 0 split-key kernels; 1 one workgroup per request and key/value head
    bool use_blaslt = true;
    int attention_rows_per_tile = 0, attention_rows_form = 0;
    int decode_part_thresholds[2] = {64, 256};
    bool decode_parts_fill = true;       // parts of 16 rounds where they are one workgroup a compute unit
    int decode_split_rounds(long long groups, int rounds) const;
    bool decode_whole(long long groups, int rounds) const;
    bool attention_general = false;      // always the general attention kernel
    bool delta_general = false;          // the delta rule's recurrence always by the kernel for any dim
    bool delta_pairs = true;             // the recurrence in registers takes whole blocks of rows two tokens at a time
    bool use_sigmoid_mfma = true;        // bfloat16 attention with sigmoid weights on the matrix cores
    bool use_biased_mfma = true;         // bfloat16 attention with a distance bias on the matrix cores
    int biased_rows_form = -1;           // likewise for the attention with a distance bias
    int sigmoid_rows_form = -1;          // -1: by the step's longest portion; 0 tiles of 16 rows, 1 tiles of 64 rows
    bool use_router_kernel = true;       // the router's product inside the routing kernel
    bool use_moe_mfma = true;            // bfloat16 products of routed experts and per-head matrices on the matrix cores
    bool use_latent_mfma = true;         // bfloat16 attention over a latent cache on the matrix cores
    int latent_decode_workgroups = 512, latent_decode_min_blocks = 1;  // single tokens: the keys are cut into shares until about this many workgroups run
    bool use_rope_table = true, use_argmax_parts = true, use_sliced = true, use_rows_kernel = true, use_tiles = true;
    bool use_qkv_tail = true;          // q/k/v products of many rows take norm, rotation and cache write along
    bool use_fresh_decode = true;      // decode-only steps: the attention prepares and writes the new keys and values
    bool use_head_argmax = true;       // greedy rows without a penalty: the token from what the head left beside the logits
    int rows_kernel_min_rows = 9, tiles_min_rows = 65, fused_linear_shape = 0;
    int last_stat_blocks = 0, last_best_parts = 0, last_best_cols = 0;

    // row-wise
    void embed(const Tensor& table, const int* token_ids, const Tensor& out, float scale = 1.0f);
    void scale(const Tensor& x, float factor);     // x *= factor, 32-bit x
    // several residual streams: xs [rows, streams * width] 32-bit
    void streams_spread(const Tensor& h, const Tensor& xs, int streams);
    void streams_sum(const Tensor& xs, const Tensor& h, int streams);
    // One sub-layer boundary of a row's streams: if y is given, every stream becomes
    // sum_s mix[s, to] x_s + out_w[to] y (all from the old ones); then, if in_w is given,
    // normed = the RMS norm (weight, eps) of sum_s in_w[s] x_s, or that sum itself in 32-bit if
    // weight is null.
    void hyper_step(const Tensor& xs, int streams, const Tensor* y, const Tensor* mix, const Tensor* out_w,
                    const Tensor* in_w, const Tensor* weight, float eps, const Tensor* normed);
    void rmsnorm(const Tensor& x, const Tensor& weight, float eps, const Tensor& out, const Tensor* delta = nullptr,
                 const int* rows = nullptr);
    // What a norm does to a row, for kernels that take a norm as an argument: weight and bias
    // (32-bit, either may be undefined), eps, and whether the mean is taken off first (a layer
    // norm) or not (an RMS norm); `plain`: no normalisation at all.
    // `tanh`: no statistics at all, every value becomes tanh(alpha * x) before weight and bias.
    struct NormParams {
        Tensor weight, bias;
        float eps = 0.f, alpha = 1.f;
        bool centered = false, plain = false, tanh = false;
    };
    // One sub-layer boundary on a single 32-bit stream h [rows, width]: if y is given,
    // h += gain * post(y) (post null: the plain sum); then, if out is given, out = pre(h).  With `rows`
    // only those rows of h are read, nothing is written back, and out has one row per entry.
    void norm_step(const Tensor& h, const Tensor* y, const NormParams* post, const NormParams* pre, const Tensor* out,
                   const int* rows = nullptr, float gain = 1.0f);
    // h [rows, width] += (rows_in [rows, width] +) vec [width], all 32-bit; either addend may be null
    void stream_add(const Tensor& h, const Tensor* rows_in, const Tensor* vec);
    // x <- cap * tanh(x / cap), 32-bit x
    void softcap(const Tensor& x, float cap);
    // out [rows, 2 * width] = (a | b), both 32-bit [rows, width]
    void concat_rows(const Tensor& a, const Tensor& b, const Tensor& out);
    void swiglu(const Tensor& gate_up, const Tensor& out);
    void add_bias(const Tensor& x, const Tensor& bias);
    void cast(const Tensor& src, const Tensor& dst);
    void apply_table_updates(int* table, int stride, int rows, const int* updates, int capacity);
    void step_prologue(int* table, int stride, int rows, const int* updates, int capacity, int* token_ids,
                       const int* token_slot, const int* last_tokens, int n);
    void resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n);
    // products
    void linear(const Tensor& x, const Tensor& w, const Tensor& out, const Tensor* bias, Workspace& ws);
    // cache-backed
    void short_conv(const Tensor& bcx, const Tensor& weight, const Tensor* bias, const Tensor& state, const Tensor& out,
                    const StepBatch& batch);
    void qk_norm_rope_store(const Tensor& q, const Tensor* k, const Tensor* v, const Tensor* q_weight,
                            const Tensor* k_weight, float eps, const Tensor* inv_freq, int rotary_dim, int pairing, int heads,
                            int kv_heads, int head_dim, const StepBatch& batch, const KVView& kv);
    void paged_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                         int window, const StepBatch& batch, const KVView& kv, Workspace& ws, const FreshKV* fresh = nullptr);
    // Attention with sigmoid weights: weight = sigmoid((q . k) * scale * temp[h] + bias[h]), not
    // normalised over the keys; temp and bias [heads] 32-bit or null; gate: raw gate values, the
    // head's result is multiplied by sigmoid(gate[row, h]) (a view [rows, heads] with dense rows, or null).
    void sigmoid_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window,
                           const Tensor* temp, const Tensor* bias, const Tensor* gate, const StepBatch& batch, const KVView& kv,
                           Workspace& ws);
    // The gated delta rule.  heads value heads of vdim, kv_heads query/key heads of dim.
    struct DeltaShape { int heads = 0, kv_heads = 0, dim = 0, vdim = 0, taps = 0; };
    // proj [rows, >= col_a + heads]: q | k | v channels from column 0, write strengths at col_b, decay inputs
    // at col_a.  Leaves qk [rows, 2 * kv_heads * dim] (unit keys, scaled unit queries), v [rows, heads * vdim]
    // and beta_decay [rows, 2 * heads], all 32-bit, and moves the requests' saved inputs on.
    void delta_prepare(const Tensor& proj, int col_b, int col_a, const DeltaShape& shape, const Tensor& conv_w, const Tensor& a_log,
                       const Tensor& dt_bias, const Tensor& conv_state, const Tensor& qk, const Tensor& v, const Tensor& beta_decay,
                       const StepBatch& batch);
    // the recurrence over the step's rows of every request, from and into state [slots, heads, dim, vdim]
    void delta_scan(const Tensor& qk, const Tensor& v, const Tensor& beta_decay, const Tensor& state, const Tensor& out,
                    const DeltaShape& shape, const StepBatch& batch, Workspace& ws);
    // out = o / rms(o) * weight * silu(gate) per head; o [rows, heads * vdim] 32-bit, gate a view with dense rows
    // (act: what the gate passes through, 0 silu, 1 sigmoid)
    void delta_gated_norm(const Tensor& o, const Tensor& weight, const Tensor& gate, float eps, const Tensor& out, int heads, int vdim,
                          int act = 0);
    // Matrix states with a decay per key channel, S [dim, vdim] per value head: S <- diag(decay) S;
    // u = beta (v - S^T k), or u = v where beta is null; S <- S + k u^T; o = S^T q.
    // decay = exp(-exp(a_log[head]) softplus(z + dt_bias)); z [rows, heads * dim] with dense rows, decay 32-bit
    void channel_decay(const Tensor& z, const Tensor& a_log, const Tensor& dt_bias, const Tensor& decay, int heads, int dim);
    // q, k [rows, heads * dim], v [rows, heads * vdim] and z [rows, heads * dim] (views with dense rows) -> qk (q times
    // q_scale | k), v32 and decay = sigmoid(z + z_bias)^(1 / tau), all 32-bit
    void gla_prepare(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& z, const Tensor* z_bias, float tau, float q_scale,
                     const Tensor& qk, const Tensor& v32, const Tensor& decay);
    // qk [rows, 2 * kv_heads * dim], v and out [rows, heads * vdim], decay [rows, heads * dim]; beta: entry
    // [row * beta_ld + head] of a 32-bit buffer, or null; state [slots, heads, dim, vdim] (shape.taps is not read)
    void channel_scan(const Tensor& qk, const Tensor& v, const Tensor& decay, const float* beta, int beta_ld, const Tensor& state,
                      const Tensor& out, const DeltaShape& shape, const StepBatch& batch);
    // The real-gated linear recurrent unit over `width` channels in `blocks` equal parts, a causal
    // convolution of `taps` in front.  x: the convolution's inputs [rows, width] (a view with dense rows);
    // ra_t, ri_t [blocks, in, out] 32-bit; leaves decay a and input sqrt(1 - a^2) i u [rows, width] 32-bit and
    // moves the requests' saved inputs [slots, taps - 1, width] on.
    struct LruShape { int width = 0, blocks = 0, taps = 0; float decay_scale = 8.f; };   // log a = -decay_scale r softplus(lam)
    void lru_gates(const Tensor& x, const Tensor& conv_w, const Tensor* conv_b, const Tensor& ra_t, const Tensor& ra_b,
                   const Tensor& ri_t, const Tensor& ri_b, const Tensor& lam, const Tensor& conv_state, const Tensor& decay,
                   const Tensor& input, const LruShape& shape, const StepBatch& batch);
    // S <- a S + input per channel from and into state [slots, width]; out = S * gelu_tanh(y)
    void lru_scan(const Tensor& decay, const Tensor& input, const Tensor& y, const Tensor& state, const Tensor& out,
                  const StepBatch& batch);
    // Softmax attention whose positions enter through the scores: score = (q . k) * scale * f(i) - r1[h] ln(1 + r2[h] (i - j)),
    // f(i) = 1 + coef ln(floor((i + 1) / every) + 1) (every 0: f = 1); r1, r2 [heads] 32-bit or null.  Values of kv.v_head_dim.
    // gate: raw values [rows, heads * v_dim] (a view with dense rows) whose sigmoid multiplies the result, or null.
    // With a window, `keep_first` keys at the start of the sequence stay visible however far the window has moved;
    // `sink_one`: the softmax's denominator holds a one more (a key of score 0 that has no value).
    struct ScoreShape {
        int heads = 0, kv_heads = 0, head_dim = 0, v_dim = 0, window = 0, every = 0;
        float scale = 1.f, coef = 0.f;
        int keep_first = 0;
        bool sink_one = false;
    };
    // What lies between an attention's q/k/v product and its scores where the projected channels pass a short causal
    // convolution: proj [rows, >= (heads + kv_heads) * head_dim + kv_heads * v_dim] holds q | k | v from column 0;
    // conv_w [channels, taps] 32-bit continues from conv_state [slots, taps - 1, channels] 32-bit (both null: no
    // convolution), which is moved on afterwards; q and k heads turn by the rows' positions (inv_freq null: not);
    // the queries go to q_out [rows, heads * head_dim], keys and values to the rows' places in the pages.
    void conv_rope_store(const Tensor& proj, const Tensor* conv_w, const Tensor* conv_state, int taps, const Tensor* inv_freq,
                         int rotary_dim, int pairing, const Tensor& q_out, int heads, const StepBatch& batch, const KVView& kv);
    // a step's keys [rows, kv_heads * head_dim] and values [rows, kv_heads * v_dim] to their places in the pages
    void kv_store(const Tensor& k, const Tensor& v, const StepBatch& batch, const KVView& kv);
    void biased_attention(const Tensor& q, const Tensor& out, const ScoreShape& shape, const Tensor* r1, const Tensor* r2,
                          const Tensor* gate, const StepBatch& batch, const KVView& kv, Workspace& ws);
    // layer glue (32-bit arithmetic; rows of the run's dtype)
    // out = act(x + bias): act 0 gelu (tanh form), 1 square of relu, 2 none; x and out views with dense rows
    void activation_bias(const Tensor& x, const Tensor* bias, const Tensor& out, int act);
    // h += a (+ b), h the 32-bit stream; copy (or null) receives the new rows in the run's dtype
    void residual_sum(const Tensor& h, const Tensor& a, const Tensor* b, const Tensor* copy);
    // g[t, j] = gelu_tanh(z[t, j]) * table[token[t], offset + j]
    void token_gate(const Tensor& z, const Tensor& table, int offset, const int* token_ids, const Tensor& g);
    // out = factor * (rmsnorm(a) * wa + rmsnorm(b) * wb) row by row
    void normed_mean(const Tensor& a, const Tensor& wa, const Tensor& b, const Tensor& wb, float eps, float factor, const Tensor& out);
    // history [entries, rows, width] 32-bit: entry n - 1 becomes the stream h, and h becomes sum_{j < n} w[j] history[j]
    void depth_mix(const Tensor& history, const Tensor& h, const Tensor& w, int n);
    // whether a decode-only step's attention can prepare and write the step's own keys and values itself
    bool attention_fresh_ok(int heads, int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const StepBatch& batch,
                            const KVView& kv, DType dtype) const;
    // attention over a latent cache (one cached row per token: `rank` compressed values, then `rot`
    // rotated key values shared by the heads)
    struct LatentShape { int heads = 0, dim = 0, rot = 0, rank = 0; };
    // proj [rows, ...] holds the queries [heads, dim + rot] from column q_off and (dkv) [rank + rot] from
    // column dkv_off: the queries' rotated parts are turned in place; with `write` the normed
    // compressed values and the turned key part go to the rows' places in the pages
    void latent_prepare(const Tensor& proj, int q_off, int dkv_off, const LatentShape& shape, const Tensor& norm_weight,
                        float eps, const Tensor* inv_freq, int rotary_dim, int pairing, bool write, const StepBatch& batch,
                        const KVView& kv);
    // out[t, h, :N] = w[h] x[t, h, :K] (w [heads, N, K]); `tail` further values of x's head pass unchanged
    // behind them; with gate [rows, heads * N] (a view with dense rows) the result is multiplied by
    // sigmoid(gate).  x_head / o_head: the distance between heads inside a row of x / out.
    void headwise_linear(const Tensor& x, int x_head, const Tensor& w, const Tensor& out, int o_head, int tail,
                         const Tensor* gate);
    // q_lat [rows, heads * (rank + rot)] against the pages; out [rows, heads * rank]
    void latent_attention(const Tensor& q_lat, const Tensor& out, const LatentShape& shape, float scale, const Tensor* sink,
                          const StepBatch& batch, const KVView& kv, Workspace& ws);
    // routed experts
    struct RoutePlan {
        Tensor ids, weights;                       // [rows * top]: expert and score of every (row, choice)
        Tensor offsets, place_of, entry_at;        // rows sorted by expert
        Tensor tile_expert, tile_row0, n_tiles;
        int n = 0, top = 0, experts = 0, max_tiles = 0, tile_rows = 0;
    };
    // How a row's experts are chosen and weighted: score "sigmoid" (0) or "softmax" (1); with groups > 1 the experts
    // form that many equal runs of neighbours, a run's score is the sum of its two largest scores, and only the experts
    // of the `keep` best runs can be chosen; the `top` largest scores are the weights, with `renorm` divided by their
    // sum plus renorm_eps, then times `scale`.
    struct RouteRule {
        int top = 1, score = 0;
        bool renorm = false;
        float renorm_eps = 0.f, scale = 1.f;
        int groups = 1, keep = 1;
    };
    // logits [rows, experts] 32-bit -> the plan; matrix_cores: the plan's products all run on the matrix cores
    // (moe_matrix_cores_ok for each of them)
    RoutePlan moe_route(const Tensor& logits, const RouteRule& rule, bool matrix_cores, Workspace& ws);
    // the same from the rows themselves: x [rows, width] times the router's 32-bit matrix [experts, width],
    // the product in 32-bit inside the routing kernel
    RoutePlan moe_route_rows(const Tensor& x, const Tensor& router, const RouteRule& rule, bool matrix_cores, Workspace& ws);
    // whether a product of experts [.., N, K] in this dtype runs on the matrix cores
    bool moe_matrix_cores_ok(DType dtype, long long N, long long K) const {
        return use_moe_mfma && dtype == DType::BF16 && K % 32 == 0 && N % 16 == 0;
    }
    void moe_gather(const Tensor& x, const RoutePlan& plan, bool weighted, const Tensor& a);
    // out[p] = a[p] w[expert of p]^T; w [experts * N, K], or [experts * 2N, K] if gated (silu(gate) * up)
    // (not gated, act 1: the square of relu of the product)
    void moe_product(const Tensor& a, const Tensor& w, const Tensor& out, bool gated, const RoutePlan& plan, int act = 0);
    // base: rows [rows, width] added to every row's sum (what all rows get besides their experts), or null
    void moe_combine(const Tensor& y, const RoutePlan& plan, bool weighted, const Tensor& out, const Tensor* base = nullptr);
    // sampling
    void sample(const Tensor& logits, const float* fparams, const int* iparams, uint8_t* seen,
                size_t seen_stride, int* out_tokens, int* last_tokens, bool all_greedy, Workspace& ws,
                const HeadBest* head_best = nullptr, bool penalised = false);
    // the most parts a row of an output head of n columns can have (for the caller's buffer): one
    // per 16 columns, or per 4 where the columns are few (narrow tiles, or less than a tile a workgroup)
    static int head_best_parts(long long n) { return static_cast<int>(std::max((n + 15) / 16, std::min<long long>((n + 3) / 4, 4096))); }
    void mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* token_ids, const int* token_slot, int n);
    // fused skinny products
    bool fused_linear_ok(int rows, std::initializer_list<long long> inner) const;
    bool rows_kernel_ok(int rows, std::initializer_list<long long> inner) const;
    int residual_stat_blocks(int rows, int n, int k) const;
    void stream_prepare(const Tensor& h, const Tensor& xb, const Tensor& stats);
    // (with `prologue`: the step's block-table updates and token ids from the device in the same launch)
    void embed_stream(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& xb, const Tensor& stats,
                      const StepPrologue* prologue = nullptr);
    void embed_stats(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& stats);
    void fused_linear(const Tensor& a, const Tensor& w, const Tensor& out, const FusedArgs& args);
    // fused products of many rows
    bool tiled_linear_ok(int rows, int n, std::initializer_list<long long> inner) const;
    int tiled_stat_blocks(int rows, int n, int k) const;
    void tiled_linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epilogue, float eps,
                      const Tensor* stats, int stat_blocks, const Tensor* bias, const Tensor* stats_out,
                      const Tensor* out_bf16, const QkvTail* qkv = nullptr);
    // whether the q/k/v product of many rows can take what follows it (norm, rotation, cache write) along
    bool tiled_qkv_ok(int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const KVView& kv) const;
    // weights re-laid at load time: w [rows, K] scaled by a norm's weight (or not) and, if
    // `packed`, laid as [K/32, rows, 32]
    std::shared_ptr<DeviceTensor> fold_weight(const Tensor& w, const Tensor* scale, bool packed);
    // The tables of cosines and sines are kept by the address of their frequencies, which a model's
    // position encoding owns for as long as the dispatcher lives.  A caller whose frequency tensors
    // come and go (an address may then name other frequencies later) says so here: the tables made
    // for this address are set aside (not freed: a recorded graph may still read them) and made anew.
    void forget_rope_tables(const void* inv_freq);

private:
    std::unique_ptr<BlasLt> blaslt_;
    DeviceBuffer argmax_state_;
    std::map<std::pair<const void*, int>, std::shared_ptr<DeviceTensor>> rope_tables_;
    std::vector<std::shared_ptr<DeviceTensor>> retired_rope_tables_;
    const float* rope_table(const Tensor& inv_freq, int n_positions);
    void attention_decode(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                          int window, const StepBatch& batch, const KVView& kv, int T, Workspace& ws, const FreshKV* fresh = nullptr);
    void library_product(const Tensor& x, const Tensor& w, const Tensor& out, Workspace& ws);
};

// What every part computes with: the stream, the activation dtype, the kernels, a workspace of
// reusable buffers, and what the parts of the fused path tell each other about the residual
// stream between kernels.
struct Runtime {
    Runtime(DType dtype, hipStream_t stream) : dtype(dtype), stream(stream), ops(stream) {}
    DType dtype;
    hipStream_t stream;
    Ops ops;
    Workspace ws;
    bool use_fused = true;
    // Steps of more than 64 bfloat16 rows: products that read a stream of up to this width go
    // through the tiled products with the norm, SwiGLU and residual sum folded in, wider ones
    // through the library's products with separate norm and activation kernels.  The default is
    // what was measured on whole prefills of 2,048 tokens: at a width of 1,024 the tiled path
    // takes 2.33 ms against 2.72 ms, at 2,048 the library's products run at 1.2 PFLOP/s and win
    // (5.5 against 6.2 ms and 9.3 against 11.0 ms for 16 and 30 layers).  0: always the library;
    // a large number: always the tiles.
    long long tiled_max_width = 1024;
    int fused_max_rows = -1;            // -1: by the kernels' own limits
    // how many partial sums of squares of the stream's rows are valid (0: none), and whether
    // the stream's bfloat16 copy is; whoever writes the stream another way resets them
    int stream_stat_blocks = 0;
    bool stream_has_bf16 = false;
    // the stream's rows in the run's dtype, where whoever wrote the stream last left them (undefined: nobody did)
    Tensor stream_copy;
    // the step's prologue, left by the runner for the embedding's kernel to take along
    // (defer_prologue); whoever cannot take it along calls flush_prologue() before its own work
    bool defer_prologue = true;
    // what the step's output head left for greedy rows (none: logits == nullptr); every forward
    // pass and every replay of a recorded one sets it anew
    HeadBest head_best;
    StepPrologue prologue;
    void flush_prologue() {
        if (!prologue.pending) return;
        prologue.pending = false;
        ops.step_prologue(prologue.table, prologue.stride, prologue.n_slots, prologue.updates, prologue.capacity,
                          prologue.token_ids, prologue.token_slot, prologue.last_tokens, prologue.n);
    }
    // weights re-laid for the fused path, made once per (weight, norm weight) pair
    std::map<std::pair<const void*, const void*>, std::shared_ptr<DeviceTensor>> folded_weights, folded_plain_weights;
    std::map<const void*, std::shared_ptr<DeviceTensor>> packed_weights;
    // a hook for bisecting mismatches: called after every entry of the run order with the
    // residual stream (the pending addition, if any, not yet made)
    std::function<void(int step, const Tensor& h, const Tensor* delta)> after_layer;
    // set: every step is timed phase by phase (and none is replayed from a recorded graph)
    std::unique_ptr<PhaseTimer> phases;
    void mark(const std::string& phase) {
        if (phases) phases->mark(phase);
    }
};

}  // namespace celeg
