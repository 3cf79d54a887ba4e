#include "ops.hpp"

#include <algorithm>
#include <functional>

#include "kernels.hpp"

namespace celeg {

namespace {
int dt(const Tensor& t, const char* name) {
    if (t.dtype != DType::F32 && t.dtype != DType::BF16)
        throw KernelError(std::string(name) + ": dtype " + dtype_name(t.dtype) + " is not supported (float32, bfloat16)");
    return static_cast<int>(t.dtype);
}
void need(bool ok, const std::string& message) {
    if (!ok) throw KernelError(message);
}
void dev(const Tensor& t, const char* name) {
    if (!t.defined()) throw KernelError(std::string(name) + " is missing");
}
void dev(const Tensor& t, const char* name, DType dtype, bool contiguous = true) {
    dev(t, name);
    if (t.dtype != dtype)
        throw KernelError(std::string(name) + " must be " + dtype_name(dtype) + ", got " + dtype_name(t.dtype));
    if (contiguous && !t.contiguous()) throw KernelError(std::string(name) + " must be contiguous");
}
// row stride of a 2-D tensor whose rows are dense
int rows_of(const Tensor& t, const char* name) {
    if (t.ndim != 2 || (t.shape[1] > 1 && t.stride[1] != 1))
        throw KernelError(std::string(name) + " must be 2-D with dense rows");
    return static_cast<int>(t.row_stride());
}
struct Operand {
    long long rows, width, ld, k8;
};
// (rows, width, row stride, stride of a group of 8 values) of a bfloat16 operand: [rows, width]
// with dense rows, or [rows, width/8, 8], a view of a buffer in which the rows lie side by side
// inside every group of 8 values
Operand operand(const Tensor& t, const char* name) {
    if (t.ndim == 2) return {t.shape[0], t.shape[1], rows_of(t, name), 8};
    if (t.ndim != 3 || t.shape[2] != 8 || t.stride[2] != 1)
        throw KernelError(std::string(name) + " must be [rows, width] or [rows, width/8, 8]");
    return {t.shape[0], t.shape[1] * 8, t.stride[0], t.stride[1]};
}
}  // namespace

const char* path_name(Path p) {
    switch (p) {
        case Path::AttentionDecode: return "attention_decode";
        case Path::AttentionDecodeFresh: return "attention_decode_fresh";
        case Path::AttentionRows: return "attention_rows";
        case Path::AttentionGeneral: return "attention_general";
        case Path::AttentionSigmoid: return "attention_sigmoid";
        case Path::AttentionSigmoidRows: return "attention_sigmoid_rows";
        case Path::AttentionSigmoidDecode: return "attention_sigmoid_decode";
        case Path::DeltaRule: return "delta_rule";
        case Path::AttentionLatent: return "attention_latent";
        case Path::AttentionLatentRows: return "attention_latent_rows";
        case Path::AttentionLatentDecode: return "attention_latent_decode";
        case Path::AttentionBiased: return "attention_biased";
        case Path::AttentionBiasedRows: return "attention_biased_rows";
        case Path::AttentionBiasedDecode: return "attention_biased_decode";
        case Path::ChannelScan: return "channel_scan";
        case Path::LinearRecurrentUnit: return "linear_recurrent_unit";
        case Path::RoutedExperts: return "routed_experts";
        case Path::LinearF32: return "linear_f32";
        case Path::LinearLibrary: return "linear_library";
        case Path::LinearStandIn: return "linear_stand_in";
        case Path::FusedSliced: return "fused_sliced";
        case Path::FusedRows: return "fused_rows";
        case Path::FusedStaged: return "fused_staged";
        case Path::ArgmaxMerged: return "argmax_merged";
        case Path::Tiled: return "tiled";
        case Path::TiledQkv: return "tiled_qkv";
        default: return "?";
    }
}

Json Ops::paths_json() const {
    Json out = Json::object();
    for (int i = 0; i < static_cast<int>(Path::Count); ++i) out.set(path_name(static_cast<Path>(i)), path_count[i]);
    return out;
}

// the bound on the context that a step's decode attention is launched for: the step's longest
// context, or what the step's recorded graph is good for
static int hint_of(const StepBatch& batch, const KVView& kv) {
    const int max_context = kv.table_stride * kv.page_tokens;
    const int hint = batch.context_hint();
    return hint ? std::min(hint, max_context) : max_context;
}

// ---------------------------------------------------------------------------- row-wise
void Ops::embed(const Tensor& table, const int* token_ids, const Tensor& out, float scale) {
    dev(table, "table");
    dev(out, "out", DType::F32);
    need(table.ndim == 2 && out.ndim == 2 && table.shape[1] == out.shape[1] && table.contiguous(), "embed: shapes do not fit");
    kernel_check(celeg_embed(table.data, dt(table, "table"), token_ids, out.as<float>(), static_cast<int>(out.shape[0]),
                             static_cast<int>(out.shape[1]), static_cast<int>(table.shape[0]), scale, stream), "embed");
}

void Ops::scale(const Tensor& x, float factor) {
    dev(x, "x", DType::F32);
    kernel_check(celeg_scale_f32(x.as<float>(), static_cast<size_t>(x.numel()), factor, stream), "scale");
}

// ---------------------------------------------------------------------------- several residual streams
void Ops::streams_spread(const Tensor& h, const Tensor& xs, int streams) {
    dev(h, "h", DType::F32);
    dev(xs, "xs", DType::F32);
    need(h.ndim == 2 && xs.ndim == 2 && streams > 0 && xs.shape[0] == h.shape[0] && xs.shape[1] == streams * h.shape[1],
         "streams_spread: xs must be [rows, streams * width]");
    kernel_check(celeg_streams_spread(h.as<float>(), xs.as<float>(), static_cast<int>(h.shape[0]), streams,
                                      static_cast<int>(h.shape[1]), stream), "streams_spread");
}

void Ops::streams_sum(const Tensor& xs, const Tensor& h, int streams) {
    dev(h, "h", DType::F32);
    dev(xs, "xs", DType::F32);
    need(h.ndim == 2 && xs.ndim == 2 && streams > 0 && xs.shape[0] == h.shape[0] && xs.shape[1] == streams * h.shape[1],
         "streams_sum: xs must be [rows, streams * width]");
    kernel_check(celeg_streams_sum(xs.as<float>(), h.as<float>(), static_cast<int>(h.shape[0]), streams,
                                   static_cast<int>(h.shape[1]), stream), "streams_sum");
}

void Ops::hyper_step(const Tensor& xs, int streams, const Tensor* y, const Tensor* mix, const Tensor* out_w,
                     const Tensor* in_w, const Tensor* weight, float eps, const Tensor* normed) {
    dev(xs, "xs", DType::F32);
    need(xs.ndim == 2 && streams > 0 && streams <= 8 && xs.shape[1] % streams == 0, "hyper_step: xs must be [rows, streams * width] with at most 8 streams");
    const long long rows = xs.shape[0], width = xs.shape[1] / streams;
    need(width <= 16384, "hyper_step: rows of more than 16,384 values do not fit the kernel's row buffer");
    if (y) {
        dev(*y, "y");
        need(mix && out_w, "hyper_step: a sub-layer output needs its mix and out weights");
        dev(*mix, "mix", DType::F32);
        dev(*out_w, "out", DType::F32);
        need(y->ndim == 2 && y->contiguous() && y->shape[0] == rows && y->shape[1] == width && mix->numel() == streams * streams &&
                 out_w->numel() == streams, "hyper_step: y [rows, width], mix [streams, streams], out [streams]");
    }
    if (in_w) {
        dev(*in_w, "in", DType::F32);
        need(normed != nullptr, "hyper_step: the mixture needs a place");
        dev(*normed, "normed");
        need(in_w->numel() == streams && normed->ndim == 2 && normed->contiguous() && normed->shape[0] == rows &&
                 normed->shape[1] == width, "hyper_step: in [streams], normed [rows, width]");
        if (weight) {
            dev(*weight, "weight", DType::F32);
            need(weight->numel() == width, "hyper_step: the norm's weight must have the rows' width");
        } else {
            need(normed->dtype == DType::F32, "hyper_step: a mixture that is not normalised leaves in 32-bit");
        }
    }
    kernel_check(celeg_hyper_step(xs.as<float>(), y ? y->data : nullptr, y ? dt(*y, "y") : 0, mix ? mix->as<float>() : nullptr,
                                  out_w ? out_w->as<float>() : nullptr, in_w ? in_w->as<float>() : nullptr,
                                  weight ? weight->as<float>() : nullptr, eps, normed ? normed->data : nullptr,
                                  normed ? dt(*normed, "normed") : 0, static_cast<int>(rows), streams, static_cast<int>(width),
                                  stream), "hyper_step");
}

// ---------------------------------------------------------------------------- latent attention
static void latent_cache_fits(const Ops::LatentShape& s, const KVView& kv, DType dtype, const char* who) {
    need(kv.k != nullptr && kv.kv_heads == 1 && kv.head_dim == s.rank + s.rot,
         std::string(who) + ": the cache must hold one row of rank + rot values per token");
    need(kv.dtype == dtype, std::string(who) + ": the cache and the rows differ in dtype");
}

void Ops::latent_prepare(const Tensor& proj, int q_off, int dkv_off, const LatentShape& s, const Tensor& norm_weight,
                         float eps, const Tensor* inv_freq, int rotary_dim, int pairing, bool write, const StepBatch& batch,
                         const KVView& kv) {
    dev(proj, "proj");
    dev(norm_weight, "norm_weight", DType::F32);
    const int ld = rows_of(proj, "proj");
    need(s.heads > 0 && s.dim > 0 && s.rot >= 0 && s.rank > 0, "latent_prepare: sizes must be positive");
    need(proj.shape[0] == batch.n_tokens, "latent_prepare: one row per token of the step");
    need(q_off >= 0 && q_off + static_cast<long long>(s.heads) * (s.dim + s.rot) <= proj.shape[1] && dkv_off >= 0 &&
             dkv_off + s.rank + s.rot <= proj.shape[1], "latent_prepare: the queries or the compressed part lie outside the rows");
    need(norm_weight.numel() == s.rank, "latent_prepare: the norm's weight must have `rank` entries");
    need(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= s.rot, "latent_prepare: rotary_dim must be even and at most rot");
    if (rotary_dim > 0) {
        need(inv_freq != nullptr, "latent_prepare: a rotation needs its frequencies");
        dev(*inv_freq, "inv_freq", DType::F32);
        need(inv_freq->numel() == rotary_dim / 2, "latent_prepare: one frequency per rotated pair");
    }
    latent_cache_fits(s, kv, proj.dtype, "latent_prepare");
    kernel_check(celeg_latent_prepare(proj.data, ld, dt(proj, "proj"), q_off, dkv_off, s.heads, s.dim, s.rot, s.rank,
                                      norm_weight.as<float>(), eps, inv_freq && rotary_dim > 0 ? inv_freq->as<float>() : nullptr,
                                      rotary_dim, pairing, batch.positions, batch.token_slot, kv.table, kv.table_stride, kv.k,
                                      kv.n_layers, kv.layer, kv.page_tokens, write ? 1 : 0, batch.n_tokens, stream),
                 "latent_prepare");
}

void Ops::headwise_linear(const Tensor& x, int x_head, const Tensor& w, const Tensor& out, int o_head, int tail,
                          const Tensor* gate) {
    dev(x, "x");
    dev(w, "w", x.dtype);
    dev(out, "out", x.dtype, false);
    need(w.ndim == 3, "headwise_linear: w must be [heads, N, K]");
    const long long heads = w.shape[0], N = w.shape[1], K = w.shape[2];
    const int ldx = rows_of(x, "x"), ldo = rows_of(out, "out");
    need(x.shape[0] == out.shape[0] && tail >= 0 && x_head >= K + tail && o_head >= N + tail &&
             (heads - 1) * x_head + K + tail <= x.shape[1] && (heads - 1) * o_head + N + tail <= out.shape[1],
         "headwise_linear: the heads do not fit the rows");
    int ldg = 0;
    if (gate) {
        dev(*gate, "gate", x.dtype, false);
        ldg = rows_of(*gate, "gate");
        need(gate->shape[0] == x.shape[0] && gate->shape[1] == heads * N, "headwise_linear: gate must be [rows, heads * N]");
    }
    const bool cores = moe_matrix_cores_ok(x.dtype, N, K) && ldx % 8 == 0 && x_head % 8 == 0 && ldo % 4 == 0 && o_head % 4 == 0 &&
                       reinterpret_cast<uintptr_t>(x.data) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data) % 8 == 0;
    kernel_check(celeg_headwise_linear(x.data, ldx, x_head, w.data, dt(x, "x"), static_cast<int>(heads), static_cast<int>(N),
                                       static_cast<int>(K), out.data, ldo, o_head, tail, gate ? gate->data : nullptr, ldg,
                                       static_cast<int>(x.shape[0]), cores ? 1 : 0, stream), "headwise_linear");
}

void Ops::latent_attention(const Tensor& q_lat, const Tensor& out, const LatentShape& s, float scale, const Tensor* sink,
                           const StepBatch& batch, const KVView& kv, Workspace& ws) {
    dev(q_lat, "q_lat");
    dev(out, "out", q_lat.dtype);
    const int D = s.rank + s.rot;
    need(q_lat.ndim == 2 && q_lat.contiguous() && q_lat.shape[0] == batch.n_tokens && q_lat.shape[1] == static_cast<long long>(s.heads) * D,
         "latent_attention: q_lat must be [rows, heads * (rank + rot)]");
    need(out.ndim == 2 && out.shape[0] == batch.n_tokens && out.shape[1] == static_cast<long long>(s.heads) * s.rank,
         "latent_attention: out must be [rows, heads * rank]");
    need(s.rank <= 1024, "latent_attention: a compressed row of more than 1,024 values does not fit the kernel's accumulators");
    if (sink) {
        dev(*sink, "sink", DType::F32);
        need(sink->numel() == s.heads, "latent_attention: one sink per head");
    }
    latent_cache_fits(s, kv, q_lat.dtype, "latent_attention");
    took(Path::AttentionLatent);
    if (q_lat.dtype == DType::BF16 && use_latent_mfma && !attention_general && scale > 0.f && out.contiguous() &&
        celeg_latent_attention_fast_ok(s.rank, s.rot) && (kv.page_tokens & (kv.page_tokens - 1)) == 0) {
        const int T = batch.n_tokens, n_single = std::min(batch.single_rows, T);
        const float* sink_p = sink ? sink->as<float>() : nullptr;
        if (n_single > 0) {
            // single tokens: the keys of a row in shares, so that the chip is busy whatever the batch
            const int blocks = (std::max(hint_of(batch, kv), 1) + 63) / 64;
            const int groups = n_single * ((s.heads + 15) / 16);
            // (at most 64 shares, and a share is at least latent_decode_min_blocks blocks of 64 keys where there are that many)
            int n_splits = std::clamp(latent_decode_workgroups / std::max(groups, 1), 1, std::min(64, std::max(1, blocks / std::max(latent_decode_min_blocks, 1))));
            const int per_split = (blocks + n_splits - 1) / n_splits;
            n_splits = (blocks + per_split - 1) / per_split;
            const size_t parts = static_cast<size_t>(n_single) * s.heads * n_splits;
            float* ws_o = static_cast<float*>(ws.raw("latent_parts_o", parts * s.rank * sizeof(float)));
            float* ws_ml = static_cast<float*>(ws.raw("latent_parts_ml", parts * 2 * sizeof(float)));
            took(Path::AttentionLatentDecode);
            kernel_check(celeg_latent_attention_fast(1, q_lat.data, static_cast<int>(q_lat.shape[1]), kv.k, kv.table, kv.table_stride,
                                                     batch.cu_seqlens, batch.seq_slot, batch.seq_start, batch.n_seqs, 0,
                                                     batch.token_slot, batch.positions, n_single, sink_p, out.data,
                                                     static_cast<int>(out.shape[1]), ws_o, ws_ml, n_splits, per_split, s.heads,
                                                     s.rank, s.rot, kv.page_tokens, kv.n_layers, kv.layer, scale, stream),
                         "latent_attention (single tokens)");
        }
        if (T > n_single) {
            const int max_tiles = (T - n_single) / celeg_latent_attention_tile_rows(s.rank, s.rot) + std::max(batch.n_seqs - n_single, 1);
            took(Path::AttentionLatentRows);
            kernel_check(celeg_latent_attention_fast(0, q_lat.data, static_cast<int>(q_lat.shape[1]), kv.k, kv.table, kv.table_stride,
                                                     batch.cu_seqlens, batch.seq_slot, batch.seq_start, batch.n_seqs, max_tiles,
                                                     batch.token_slot, batch.positions, 0, sink_p, out.data,
                                                     static_cast<int>(out.shape[1]), nullptr, nullptr, 1, 0, s.heads, s.rank,
                                                     s.rot, kv.page_tokens, kv.n_layers, kv.layer, scale, stream),
                         "latent_attention (rows)");
        }
        return;
    }
    kernel_check(celeg_latent_attention(q_lat.data, static_cast<int>(q_lat.shape[1]), kv.k, dt(q_lat, "q_lat"), kv.table,
                                        kv.table_stride, batch.token_slot, batch.positions, sink ? sink->as<float>() : nullptr,
                                        out.data, static_cast<int>(out.shape[1]), batch.n_tokens, s.heads, s.rank, s.rot,
                                        kv.page_tokens, kv.n_layers, kv.layer, scale, stream), "latent_attention");
}

// ---------------------------------------------------------------------------- routed experts
static Ops::RoutePlan new_route_plan(long long rows, long long experts, int top, bool matrix_cores, Workspace& ws) {
    need(experts > 0 && experts <= 512, "moe_route: between 1 and 512 experts");
    need(top > 0 && top <= experts, "moe_route: `top` must be between 1 and the number of experts");
    Ops::RoutePlan p;
    p.n = static_cast<int>(rows * top);
    p.top = top;
    p.experts = static_cast<int>(experts);
    const int tile = p.tile_rows = celeg_moe_tile_rows(matrix_cores ? 1 : 0);
    p.max_tiles = static_cast<int>(std::min<long long>(p.n, p.n / tile + experts));
    const long long n = std::max(p.n, 1), tiles = std::max(p.max_tiles, 1);
    p.ids = ws.buf("moe_ids", DType::I32, {n});
    p.weights = ws.buf("moe_weights", DType::F32, {n});
    p.offsets = ws.buf("moe_offsets", DType::I32, {experts + 1});
    p.place_of = ws.buf("moe_place_of", DType::I32, {n});
    p.entry_at = ws.buf("moe_entry_at", DType::I32, {n});
    p.tile_expert = ws.buf("moe_tile_expert", DType::I32, {tiles});
    p.tile_row0 = ws.buf("moe_tile_row0", DType::I32, {tiles});
    p.n_tiles = ws.buf("moe_n_tiles", DType::I32, {4});
    return p;
}

static void plan_of(const Ops::RoutePlan& p, hipStream_t stream) {
    kernel_check(celeg_moe_plan(p.ids.as<int>(), p.n, p.experts, p.tile_rows, p.offsets.as<int>(), p.place_of.as<int>(), p.entry_at.as<int>(),
                                p.tile_expert.as<int>(), p.tile_row0.as<int>(), p.n_tiles.as<int>(), stream), "moe_plan");
}

static void check_route_rule(const Ops::RouteRule& r, long long experts, const char* who) {
    need(r.score == 0 || r.score == 1, std::string(who) + ": score is sigmoid (0) or softmax (1)");
    need(r.groups >= 1 && r.groups <= 64 && experts % r.groups == 0 && r.keep >= 1 && r.keep <= r.groups,
         std::string(who) + ": up to 64 groups that divide the experts evenly, of which 1 to all are kept");
    need(r.top <= r.keep * (experts / r.groups), std::string(who) + ": the kept groups hold fewer experts than a row uses");
}

Ops::RoutePlan Ops::moe_route(const Tensor& logits, const RouteRule& rule, bool matrix_cores, Workspace& ws) {
    dev(logits, "logits", DType::F32);
    need(logits.ndim == 2, "moe_route: logits must be [rows, experts]");
    RoutePlan p = new_route_plan(logits.shape[0], logits.shape[1], rule.top, matrix_cores, ws);
    check_route_rule(rule, p.experts, "moe_route");
    took(Path::RoutedExperts);
    kernel_check(celeg_moe_route(logits.as<float>(), static_cast<int>(logits.shape[0]), p.experts, rule.top, rule.score, rule.renorm ? 1 : 0,
                                 rule.groups, rule.keep, rule.renorm_eps, rule.scale, p.ids.as<int>(), p.weights.as<float>(), stream),
                 "moe_route");
    plan_of(p, stream);
    return p;
}

Ops::RoutePlan Ops::moe_route_rows(const Tensor& x, const Tensor& router, const RouteRule& rule, bool matrix_cores, Workspace& ws) {
    dev(x, "x");
    dev(router, "router", DType::F32);
    need(x.ndim == 2 && x.contiguous() && router.ndim == 2 && router.shape[1] == x.shape[1], "moe_route_rows: x [rows, width], router [experts, width]");
    const long long rows = x.shape[0], width = x.shape[1], experts = router.shape[0];
    if (!use_router_kernel || 4 * (width + experts) * 4 > 64 * 1024) {
        Tensor logits = ws.buf("moe_logits", DType::F32, {rows, experts});
        linear(x, router, logits, nullptr, ws);
        return moe_route(logits, rule, matrix_cores, ws);
    }
    RoutePlan p = new_route_plan(rows, experts, rule.top, matrix_cores, ws);
    check_route_rule(rule, experts, "moe_route_rows");
    took(Path::RoutedExperts);
    kernel_check(celeg_moe_router(x.data, dt(x, "x"), router.as<float>(), static_cast<int>(rows), static_cast<int>(width), p.experts,
                                  rule.top, rule.score, rule.renorm ? 1 : 0, rule.groups, rule.keep, rule.renorm_eps, rule.scale,
                                  p.ids.as<int>(), p.weights.as<float>(), stream), "moe_router");
    plan_of(p, stream);
    return p;
}

void Ops::moe_gather(const Tensor& x, const RoutePlan& p, bool weighted, const Tensor& a) {
    dev(x, "x");
    dev(a, "a", x.dtype);
    need(x.ndim == 2 && x.contiguous() && a.ndim == 2 && a.shape[0] == p.n && a.shape[1] == x.shape[1] &&
             x.shape[0] * p.top == p.n, "moe_gather: a must be [rows * top, width]");
    kernel_check(celeg_moe_gather(x.data, dt(x, "x"), p.entry_at.as<int>(), weighted ? p.weights.as<float>() : nullptr, a.data,
                                  p.n, p.top, static_cast<int>(x.shape[1]), stream), "moe_gather");
}

void Ops::moe_product(const Tensor& a, const Tensor& w, const Tensor& out, bool gated, const RoutePlan& p, int act) {
    need(act == 0 || (act == 1 && !gated), "moe_product: act is 0, or 1 (square of relu) where the product is not gated");
    dev(a, "a");
    dev(w, "w", a.dtype);
    dev(out, "out", a.dtype);
    need(a.ndim == 2 && w.ndim == 2 && out.ndim == 2 && a.shape[0] == p.n && out.shape[0] == p.n && w.shape[1] == a.shape[1] &&
             w.shape[0] == static_cast<long long>(p.experts) * (gated ? 2 : 1) * out.shape[1],
         "moe_product: a [n, K], w [experts * N (* 2 if gated), K], out [n, N]");
    need(a.contiguous() && w.contiguous() && out.contiguous(), "moe_product: a, w and out must be contiguous");
    need(p.tile_rows == celeg_moe_tile_rows(0) || moe_matrix_cores_ok(a.dtype, out.shape[1], a.shape[1]),
         "moe_product: the plan was made for the matrix cores, which do not take this product");
    kernel_check(celeg_moe_product(a.data, w.data, out.data, dt(a, "a"), static_cast<int>(out.shape[1]),
                                   static_cast<int>(a.shape[1]), gated ? 1 : 0, act, p.offsets.as<int>(), p.tile_expert.as<int>(),
                                   p.tile_row0.as<int>(), p.n_tiles.as<int>(), p.max_tiles, p.tile_rows,
                                   p.n >= 8 * p.experts ? 1 : 0, stream), "moe_product");
}

void Ops::moe_combine(const Tensor& y, const RoutePlan& p, bool weighted, const Tensor& out, const Tensor* base) {
    dev(y, "y");
    dev(out, "out", y.dtype);
    need(y.ndim == 2 && out.ndim == 2 && y.shape[0] == p.n && out.shape[0] * p.top == p.n && y.shape[1] == out.shape[1],
         "moe_combine: y [rows * top, width], out [rows, width]");
    if (base) {
        dev(*base, "base", y.dtype);
        need(base->ndim == 2 && base->shape[0] == out.shape[0] && base->shape[1] == out.shape[1] && base->contiguous(),
             "moe_combine: base must have the shape of out");
    }
    kernel_check(celeg_moe_combine(y.data, dt(y, "y"), p.place_of.as<int>(), weighted ? p.weights.as<float>() : nullptr,
                                   base ? base->data : nullptr, out.data,
                                   static_cast<int>(out.shape[0]), p.top, static_cast<int>(y.shape[1]), stream), "moe_combine");
}

void Ops::rmsnorm(const Tensor& x, const Tensor& weight, float eps, const Tensor& out, const Tensor* delta, const int* rows) {
    dev(x, "x");
    dev(weight, "weight", DType::F32);
    dev(out, "out");
    need(x.ndim == 2 && out.ndim == 2 && x.contiguous() && out.contiguous(), "rmsnorm: x and out must be contiguous matrices");
    const long long width = x.shape[1], n_rows = out.shape[0];
    need(out.shape[1] == width && weight.numel() == width, "rmsnorm: shapes do not fit");
    if (delta) {
        dev(*delta, "delta");
        need(delta->ndim == 2 && delta->shape[0] == x.shape[0] && delta->shape[1] == width && delta->contiguous(),
             "rmsnorm: delta must have the shape of x");
    }
    if (!rows) need(n_rows == x.shape[0], "rmsnorm: out must have the rows of x");
    const int write_back = delta && !rows ? 1 : 0;
    need(!write_back || x.dtype == DType::F32, "rmsnorm: the sum can only be written back to a 32-bit x");
    kernel_check(celeg_rmsnorm(x.data, dt(x, "x"), delta ? delta->data : nullptr, delta ? dt(*delta, "delta") : 0,
                               weight.as<float>(), out.data, dt(out, "out"), rows, static_cast<int>(n_rows),
                               static_cast<int>(width), eps, write_back, stream), "rmsnorm");
}

// ---------------------------------------------------------------------------- norms as kernel arguments
static CelegNorm norm_arg(const Ops::NormParams* p, long long width, const char* who) {
    CelegNorm n{nullptr, nullptr, 0.f, CELEG_NORM_NONE, 1.f, 1.f};
    if (!p) return n;
    if (p->weight.defined()) {
        dev(p->weight, "norm weight", DType::F32);
        need(p->weight.numel() == width, std::string(who) + ": a norm weight must have the rows' width");
        n.w = p->weight.as<float>();
    }
    if (p->bias.defined()) {
        dev(p->bias, "norm bias", DType::F32);
        need(p->bias.numel() == width, std::string(who) + ": a norm bias must have the rows' width");
        n.b = p->bias.as<float>();
    }
    n.eps = p->eps;
    n.mode = p->plain ? CELEG_NORM_NONE : p->tanh ? CELEG_NORM_TANH : p->centered ? CELEG_NORM_LAYER : CELEG_NORM_RMS;
    n.alpha = p->alpha;
    return n;
}

void Ops::norm_step(const Tensor& h, const Tensor* y, const NormParams* post, const NormParams* pre, const Tensor* out,
                    const int* rows, float gain) {
    dev(h, "h", DType::F32);
    need(h.ndim == 2, "norm_step: h must be a matrix");
    const long long width = h.shape[1];
    need(width * 4 <= 60 * 1024, "norm_step: rows of more than 15,360 values are not supported");
    long long n_rows = h.shape[0];
    if (y) {
        dev(*y, "y");
        need(y->ndim == 2 && y->shape[0] == h.shape[0] && y->shape[1] == width && y->contiguous(), "norm_step: y must have the shape of h");
    }
    if (out) {
        dev(*out, "out");
        need(out->ndim == 2 && out->shape[1] == width && out->contiguous(), "norm_step: out must have the width of h");
        n_rows = out->shape[0];
        need(rows || n_rows == h.shape[0], "norm_step: out must have the rows of h");
        need(pre != nullptr, "norm_step: an output needs a norm");
    }
    need(!rows || out, "norm_step: a list of rows goes with an output");
    need(y || out, "norm_step: nothing to do");
    CelegNorm post_arg = norm_arg(y ? post : nullptr, width, "norm_step");
    post_arg.gain = gain;
    kernel_check(celeg_norm_step(h.as<float>(), y ? y->data : nullptr, y ? dt(*y, "y") : 0, post_arg,
                                 norm_arg(pre, width, "norm_step"), out ? out->data : nullptr, out ? dt(*out, "out") : 0, rows,
                                 static_cast<int>(n_rows), static_cast<int>(width), y && !rows ? 1 : 0, stream), "norm_step");
}

void Ops::concat_rows(const Tensor& a, const Tensor& b, const Tensor& out) {
    dev(a, "a", DType::F32);
    dev(b, "b", DType::F32);
    dev(out, "out");
    need(a.ndim == 2 && b.ndim == 2 && out.ndim == 2 && a.shape[0] == b.shape[0] && a.shape[1] == b.shape[1] &&
             out.shape[0] == a.shape[0] && out.shape[1] == 2 * a.shape[1] && out.contiguous(), "concat_rows: shapes do not fit");
    kernel_check(celeg_concat_rows(a.as<float>(), b.as<float>(), out.data, dt(out, "out"), static_cast<int>(a.shape[0]),
                                   static_cast<int>(a.shape[1]), stream), "concat_rows");
}

void Ops::swiglu(const Tensor& gate_up, const Tensor& out) {
    dev(gate_up, "gate_up");
    dev(out, "out", gate_up.dtype);
    need(out.ndim == 2 && gate_up.ndim == 2 && gate_up.shape[0] == out.shape[0] && gate_up.shape[1] == 2 * out.shape[1] &&
             gate_up.contiguous() && out.contiguous(), "swiglu: gate_up must be [rows, 2*ff]");
    kernel_check(celeg_swiglu(gate_up.data, out.data, dt(out, "out"), static_cast<int>(out.shape[0]),
                              static_cast<int>(out.shape[1]), stream), "swiglu");
}

void Ops::add_bias(const Tensor& x, const Tensor& bias) {
    dev(x, "x");
    dev(bias, "bias", DType::F32);
    need(x.ndim == 2 && x.contiguous() && bias.numel() == x.shape[1], "add_bias: bias must have the width of x");
    kernel_check(celeg_add_bias(x.data, dt(x, "x"), bias.as<float>(), static_cast<int>(x.shape[0]),
                                static_cast<int>(x.shape[1]), stream), "add_bias");
}

void Ops::cast(const Tensor& src, const Tensor& dst) {
    dev(src, "src");
    dev(dst, "dst");
    need(src.numel() == dst.numel() && src.contiguous() && dst.contiguous(), "cast: sizes differ");
    kernel_check(celeg_cast(src.data, dt(src, "src"), dst.data, dt(dst, "dst"), static_cast<size_t>(src.numel()), stream), "cast");
}

void Ops::apply_table_updates(int* table, int stride, int rows, const int* updates, int capacity) {
    kernel_check(celeg_table_update(table, stride, rows, updates, capacity, stream), "apply_table_updates");
}

void Ops::step_prologue(int* table, int stride, int rows, const int* updates, int capacity, int* token_ids,
                        const int* token_slot, const int* last_tokens, int n) {
    need(capacity > 0, "step_prologue: the update list is shorter than its capacity");
    kernel_check(celeg_step_prologue(table, stride, rows, updates, capacity, token_ids, token_slot, last_tokens, n, stream),
                 "step_prologue");
}

void Ops::resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n) {
    kernel_check(celeg_resolve_tokens(token_ids, token_slot, last_tokens, n, stream), "resolve_tokens");
}

// ---------------------------------------------------------------------------- products
void Ops::library_product(const Tensor& x, const Tensor& w, const Tensor& out, Workspace& ws) {
    const int M = static_cast<int>(x.shape[0]), K = static_cast<int>(x.shape[1]), N = static_cast<int>(w.shape[0]);
    if (use_blaslt) {
        if (!blaslt_) blaslt_ = std::make_unique<BlasLt>();
        if (blaslt_->matmul(x.data, rows_of(x, "x"), w.data, out.data, rows_of(out, "out"), M, N, K, stream)) {
            took(Path::LinearLibrary);
            return;
        }
    }
    // sizes the library has no kernel for: the tiled product where the sizes fit it, else the
    // 32-bit product on widened copies
    if (K % 64 == 0 && N % 4 == 0 && rows_of(x, "x") % 8 == 0 && rows_of(out, "out") % 4 == 0) {
        tiled_linear(x, w, out, Epilogue::Store, 0.f, nullptr, 0, nullptr, nullptr, nullptr);
        return;
    }
    Tensor xf = ws.buf("product_x32", DType::F32, {M, K}), wf = ws.buf("product_w32", DType::F32, {N, K});
    Tensor yf = ws.buf("product_y32", DType::F32, {M, N});
    if (x.contiguous()) {
        cast(x, xf);
    } else {
        for (int m = 0; m < M; ++m) cast(x.rows(m, 1), xf.rows(m, 1));
    }
    cast(w, wf);
    took(Path::LinearStandIn);
    kernel_check(celeg_gemm_f32(xf.as<float>(), K, wf.as<float>(), K, nullptr, yf.as<float>(), N, M, N, K, stream),
                 "linear (32-bit stand-in)");
    if (out.contiguous()) {
        cast(yf, out);
    } else {
        for (int m = 0; m < M; ++m) cast(yf.rows(m, 1), out.rows(m, 1));
    }
}

// out = x w^T (+ bias).  x [M,K] (rows may be strided), w [N,K], out [M,N] in the dtype of x or
// in 32-bit.
void Ops::linear(const Tensor& x, const Tensor& w, const Tensor& out, const Tensor* bias, Workspace& ws) {
    dev(x, "x");
    dev(w, "w");
    dev(out, "out");
    need(x.ndim == 2 && w.ndim == 2 && out.ndim == 2 && w.contiguous(), "linear: x, w and out must be matrices");
    const long long M = x.shape[0], K = x.shape[1], N = w.shape[0];
    need(w.shape[1] == K && out.shape[0] == M && out.shape[1] == N,
         "linear: shapes do not fit: x [" + std::to_string(M) + ", " + std::to_string(K) + "], w [" + std::to_string(N) +
             ", " + std::to_string(w.shape[1]) + "], out [" + std::to_string(out.shape[0]) + ", " + std::to_string(out.shape[1]) + "]");
    if (bias) {
        dev(*bias, "bias", DType::F32);
        need(bias->numel() == N, "linear: bias must have one entry per output column");
    }
    if (M == 0) return;
    if (x.dtype == DType::F32 && w.dtype == DType::F32) {
        need(out.dtype == DType::F32, "linear: a 32-bit product needs a 32-bit output");
        took(Path::LinearF32);
        kernel_check(celeg_gemm_f32(x.as<float>(), rows_of(x, "x"), w.as<float>(), static_cast<int>(K),
                                    bias ? bias->as<float>() : nullptr, out.as<float>(), rows_of(out, "out"),
                                    static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), stream), "linear (32-bit)");
        return;
    }
    if (x.dtype == DType::BF16 && w.dtype == DType::F32) {
        // a matrix stored in 32-bit stays 32-bit: widen the rows and use the 32-bit product
        Tensor xf = ws.buf("linear_x32", DType::F32, {M, K});
        if (x.contiguous()) {
            cast(x, xf);
        } else {
            for (long long m = 0; m < M; ++m) cast(x.rows(m, 1), xf.rows(m, 1));
        }
        if (out.dtype == DType::F32) {
            linear(xf, w, out, bias, ws);
        } else {
            Tensor yf = ws.buf("linear_y32", DType::F32, {M, N});
            linear(xf, w, yf, bias, ws);
            if (out.contiguous()) {
                cast(yf, out);
            } else {
                for (long long m = 0; m < M; ++m) cast(yf.rows(m, 1), out.rows(m, 1));
            }
        }
        return;
    }
    need(x.dtype == DType::BF16 && w.dtype == DType::BF16,
         std::string("linear: unsupported dtypes ") + dtype_name(x.dtype) + " x " + dtype_name(w.dtype));
    if (out.dtype == DType::BF16) {
        library_product(x, w, out, ws);
        if (bias) add_bias(out, *bias);
    } else if (out.dtype == DType::F32) {
        Tensor tmp = ws.buf("linear_bf16_out", DType::BF16, {M, N});
        library_product(x, w, tmp, ws);
        cast(tmp, out);
        if (bias) add_bias(out, *bias);
    } else {
        throw KernelError("linear: out must be bfloat16 or float32");
    }
}

// ---------------------------------------------------------------------------- short convolution
void Ops::short_conv(const Tensor& bcx, const Tensor& weight, const Tensor* bias, const Tensor& state, const Tensor& out,
                     const StepBatch& batch) {
    dev(bcx, "bcx");
    dev(weight, "weight", DType::F32);
    dev(state, "state", DType::F32, false);
    dev(out, "out", bcx.dtype);
    need(out.ndim == 2 && bcx.ndim == 2 && weight.ndim == 2 && bcx.contiguous() && out.contiguous(), "short_conv: shapes do not fit");
    const long long T = out.shape[0], width = out.shape[1], taps = weight.shape[1];
    need(bcx.shape[0] == T && bcx.shape[1] == 3 * width && weight.shape[0] == width && T == batch.n_tokens,
         "short_conv: shapes do not fit");
    need(state.ndim == 3 && state.shape[1] == taps && state.shape[2] == width && state.stride[2] == 1 && state.stride[1] == width,
         "short_conv: state must be [slots, taps, width] with dense slots");
    if (bias) dev(*bias, "bias", DType::F32);
    kernel_check(celeg_short_conv(bcx.data, static_cast<int>(3 * width), dt(bcx, "bcx"), weight.as<float>(),
                                  bias ? bias->as<float>() : nullptr, state.as<float>(), static_cast<size_t>(state.stride[0]),
                                  out.data, batch.positions, batch.token_seq, batch.seq_start, batch.seq_slot,
                                  batch.cu_seqlens, batch.n_tokens, batch.n_seqs, static_cast<int>(width),
                                  static_cast<int>(taps), stream), "short_conv");
}

// ---------------------------------------------------------------------------- attention
static void check_kv(const KVView& kv, int kv_heads, int head_dim, DType dtype) {
    need(kv.kv_heads == kv_heads && kv.head_dim == head_dim, "attention: the cache has other head sizes than the mixer");
    need(kv.v_head_dim == head_dim, "attention: these kernels take values of the keys' width only");
    need(kv.k && kv.v && kv.table, "attention: the cache has no device memory");
    need(kv.dtype == dtype, std::string("attention: the cache holds ") + dtype_name(kv.dtype) + ", the rows are " + dtype_name(dtype));
    need(kv.layer >= 0 && kv.layer < kv.n_layers, "attention: layer index outside the cache");
}

// cos and sin of position * frequency for every position a request can reach
// ([n_positions, rotary_dim/2, 2], 32-bit), made once per frequency table
const float* Ops::rope_table(const Tensor& inv_freq, int n_positions) {
    const auto key = std::make_pair(static_cast<const void*>(inv_freq.data), n_positions);
    auto it = rope_tables_.find(key);
    if (it == rope_tables_.end()) {
        auto table = device_tensor(DType::F32, {n_positions, inv_freq.numel(), 2});
        kernel_check(celeg_rope_table(inv_freq.as<float>(), static_cast<int>(inv_freq.numel()), n_positions,
                                      table->view.as<float>(), stream), "rope_table");
        it = rope_tables_.emplace(key, table).first;
    }
    return it->second->view.as<float>();
}

void Ops::forget_rope_tables(const void* inv_freq) {
    for (auto it = rope_tables_.begin(); it != rope_tables_.end();) {
        if (it->first.first == inv_freq) {
            retired_rope_tables_.push_back(it->second);
            it = rope_tables_.erase(it);
        } else {
            ++it;
        }
    }
}

void Ops::qk_norm_rope_store(const Tensor& q, const Tensor* k, const Tensor* v, const Tensor* q_weight,
                             const Tensor* k_weight, float eps, const Tensor* inv_freq, int rotary_dim, int pairing, int heads,
                             int kv_heads, int head_dim, const StepBatch& batch, const KVView& kv) {
    dev(q, "q");
    const long long T = q.shape[0];
    need(q.ndim == 2 && T == batch.n_tokens && q.shape[1] == static_cast<long long>(heads) * head_dim,
         "qk_norm_rope_store: q must be [rows, heads*head_dim]");
    need(head_dim % 2 == 0 && head_dim <= 1024,
         "qk_norm_rope_store: head_dim " + std::to_string(head_dim) + " must be even and <= 1024");
    check_kv(kv, kv_heads, head_dim, q.dtype);
    const bool store = k != nullptr;
    if (store) {
        need(v != nullptr, "qk_norm_rope_store: k without v");
        dev(*k, "k", q.dtype, false);
        dev(*v, "v", q.dtype, false);
        const long long kvw = static_cast<long long>(kv_heads) * head_dim;
        need(k->ndim == 2 && v->ndim == 2 && k->shape[0] == T && k->shape[1] == kvw && v->shape[0] == T && v->shape[1] == kvw,
             "qk_norm_rope_store: k and v must be [rows, kv_heads*head_dim]");
    }
    for (const Tensor* wt : {q_weight, k_weight})
        if (wt) {
            dev(*wt, "q/k norm weight", DType::F32);
            need(wt->numel() == head_dim, "qk_norm_rope_store: a norm weight must have head_dim entries");
        }
    if (inv_freq) {
        dev(*inv_freq, "inv_freq", DType::F32);
        need(rotary_dim % 2 == 0 && rotary_dim <= head_dim && inv_freq->numel() == rotary_dim / 2,
             "qk_norm_rope_store: rotary_dim and the frequency table disagree");
        need(pairing == 0 || pairing == 1, "qk_norm_rope_store: pairing is 0 (halves) or 1 (neighbours)");
    }
    const float* cos_sin = nullptr;
    if (inv_freq && rotary_dim > 0 && use_rope_table) cos_sin = rope_table(*inv_freq, kv.table_stride * kv.page_tokens);
    kernel_check(celeg_qk_norm_rope_store(
                     q.data, rows_of(q, "q"), store ? k->data : nullptr, store ? rows_of(*k, "k") : 0,
                     store ? v->data : nullptr, store ? rows_of(*v, "v") : 0, dt(q, "q"),
                     q_weight ? q_weight->as<float>() : nullptr, (store && k_weight) ? k_weight->as<float>() : nullptr, eps,
                     inv_freq ? inv_freq->as<float>() : nullptr, cos_sin, rotary_dim, pairing, batch.positions, batch.token_slot,
                     kv.table, kv.table_stride, kv.k, kv.v, kv.n_layers, kv.layer, kv.page_tokens, static_cast<int>(T),
                     heads, kv_heads, head_dim, store ? 1 : 0, stream), "qk_norm_rope_store");
}

// The conditions under which paged_attention hands a decode-only step to the kernels for single
// rows, and those can prepare the step's own keys and values (the rotation: none, or of the whole
// head by split halves from the table).
bool Ops::attention_fresh_ok(int heads, int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const StepBatch& batch,
                             const KVView& kv, DType dtype) const {
    if (!use_fresh_decode || dtype != DType::BF16 || kv.dtype != DType::BF16 || attention_general) return false;
    if (kv.page_tokens < 16 || (kv.page_tokens & (kv.page_tokens - 1))) return false;
    if ((head_dim != 64 && head_dim != 128) || kv.head_dim != head_dim || (kv.v_head_dim && kv.v_head_dim != head_dim)) return false;
    if (!batch.decode_only || batch.n_seqs != batch.n_tokens) return false;
    // (measured with heads of 64 only)
    if (head_dim != 64) return false;
    // Which kernel attention_decode will take: one workgroup a (request, key/value head), or parts
    // of 1, 4 or 16 rounds.  In parts of many rounds every wavefront prepares q before it asks for
    // its keys, which pays where a compute unit runs one such workgroup and costs more than the
    // kernel it saves where it runs many in turn (8 requests at 8,192 and 32,768 tokens, 2,112
    // workgroups: 1 and 5 us a layer slower; 1 request at 16,384, 136 workgroups: 4 us a layer
    // faster; 264 workgroups: 1 us a layer faster).
    const int chunks = (heads / kv.kv_heads + 15) / 16;
    const long long groups = static_cast<long long>(kv.kv_heads) * chunks * batch.n_tokens;
    const int rounds = (hint_of(batch, kv) + 63) / 64;
    const bool whole = decode_whole(groups, rounds);
    if (whole) {
        // the kernel's loop over the rounds runs 1.7 % slower in this form, which outweighs the
        // kernel saved from about 8,192 tokens for each of 64 requests on (at 32,768: 4.94 against
        // 4.86 ms a step; at 2,048: 0.906 against 0.916)
        if (static_cast<long long>(batch.n_tokens) * rounds > 4096) return false;
    } else {
        const int split_rounds = decode_split_rounds(groups, rounds);
        if (split_rounds > 1 && groups * ((rounds + split_rounds - 1) / split_rounds) > 512) return false;
    }
    return !inv_freq || (rotary_dim == head_dim && pairing == 0 && use_rope_table);
}

void Ops::paged_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                          int window, const StepBatch& batch, const KVView& kv, Workspace& ws, const FreshKV* fresh) {
    dev(q, "q");
    dev(out, "out", q.dtype);
    const long long T = q.shape[0], qw = static_cast<long long>(heads) * head_dim;
    need(q.ndim == 2 && out.ndim == 2 && T == batch.n_tokens && q.shape[1] == qw && out.shape[0] == T && out.shape[1] == qw &&
             out.contiguous(), "paged_attention: q and out must be [rows, heads*head_dim]");
    need(head_dim <= 256, "paged_attention: head_dim " + std::to_string(head_dim) + " exceeds 256");
    need(heads % kv_heads == 0, "paged_attention: heads must be a multiple of kv_heads");
    check_kv(kv, kv_heads, head_dim, q.dtype);
    const int ldq = rows_of(q, "q");
    if (q.dtype == DType::BF16 && !attention_general && kv.page_tokens >= 16 &&
        (kv.page_tokens & (kv.page_tokens - 1)) == 0 && ldq % 8 == 0) {
        const bool decode_hd = head_dim == 64 || head_dim == 128;
        if (batch.decode_only && decode_hd && batch.n_seqs == T) {
            attention_decode(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, static_cast<int>(T), ws, fresh);
            return;
        }
        need(!fresh, "paged_attention: fresh keys and values go with decode-only steps");
        if (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128) {
            // entries of one token lie first: they go to the kernel for single rows (a tile of
            // the rows kernel would hold one row), the portions to the rows kernel
            const int single = decode_hd ? batch.single_rows : 0;
            if (single) attention_decode(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, single, ws);
            if (single < batch.n_seqs) took(Path::AttentionRows);
            if (single < batch.n_seqs)
                kernel_check(celeg_attention_rows_bf16(
                                 q.data, ldq, kv.k, kv.v, kv.table, kv.table_stride, batch.cu_seqlens + single,
                                 batch.seq_slot + single, batch.seq_start + single, batch.n_seqs - single,
                                 static_cast<int>(T) - single, out.data, static_cast<int>(qw), heads, kv_heads, head_dim,
                                 kv.page_tokens, kv.n_layers, kv.layer, scale, window, attention_rows_per_tile,
                                 attention_rows_form, batch.context_hint(), stream), "attention over rows (bfloat16)");
            return;
        }
    }
    need(!fresh, "paged_attention: fresh keys and values go with the kernels for single rows");
    took(Path::AttentionGeneral);
    kernel_check(celeg_paged_attention(q.data, ldq, kv.k, kv.v, dt(q, "q"), kv.table, kv.table_stride, batch.token_slot,
                                       batch.positions, out.data, static_cast<int>(qw), static_cast<int>(T), heads,
                                       kv_heads, head_dim, kv.page_tokens, kv.n_layers, kv.layer, scale, window, stream),
                 "paged_attention");
}

// ---------------------------------------------------------------------------- attention with sigmoid weights
void Ops::sigmoid_attention(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale, int window,
                            const Tensor* temp, const Tensor* bias, const Tensor* gate, const StepBatch& batch, const KVView& kv,
                            Workspace&) {
    dev(q, "q");
    dev(out, "out", q.dtype);
    const long long T = q.shape[0], qw = static_cast<long long>(heads) * head_dim;
    need(q.ndim == 2 && out.ndim == 2 && T == batch.n_tokens && q.shape[1] == qw && out.shape[0] == T && out.shape[1] == qw &&
             out.contiguous(), "sigmoid_attention: q and out must be [rows, heads*head_dim]");
    need(head_dim <= 256, "sigmoid_attention: head_dim " + std::to_string(head_dim) + " exceeds 256");
    need(heads % kv_heads == 0, "sigmoid_attention: heads must be a multiple of kv_heads");
    check_kv(kv, kv_heads, head_dim, q.dtype);
    for (const Tensor* per_head : {temp, bias})
        if (per_head) {
            dev(*per_head, "temperature / bias", DType::F32);
            need(per_head->numel() == heads, "sigmoid_attention: one temperature and one bias per query head");
        }
    int ldg = 0;
    if (gate) {
        dev(*gate, "gate", q.dtype, false);
        need(gate->ndim == 2 && gate->shape[0] == T && gate->shape[1] == heads, "sigmoid_attention: gate must be [rows, heads]");
        ldg = rows_of(*gate, "gate");
    }
    took(Path::AttentionSigmoid);
    const int ldq = rows_of(q, "q");
    if (q.dtype == DType::BF16 && use_sigmoid_mfma && !attention_general && celeg_sigmoid_attention_fast_ok(head_dim) &&
        kv.page_tokens >= 8 && (kv.page_tokens & (kv.page_tokens - 1)) == 0 && ldq % 8 == 0 && head_dim % 8 == 0 &&
        (reinterpret_cast<uintptr_t>(q.data) & 15) == 0) {
        // portions of prompts: tiles of 64 rows that share their staged keys; single tokens and short
        // portions: tiles of 16 rows whose key blocks the wavefronts take in turn.  At most one
        // partly filled tile per request.
        const int form = sigmoid_rows_form >= 0 ? sigmoid_rows_form : (batch.max_seg_len > 16 ? 1 : 0);
        const int max_tiles = static_cast<int>(T) / (form == 1 ? 64 : 16) + batch.n_seqs;
        took(batch.decode_only ? Path::AttentionSigmoidDecode : Path::AttentionSigmoidRows);
        kernel_check(celeg_sigmoid_attention_fast(form, q.data, ldq, kv.k, kv.v, kv.table, kv.table_stride, batch.cu_seqlens, batch.seq_slot,
                                                  batch.seq_start, batch.n_seqs, max_tiles, temp ? temp->as<float>() : nullptr,
                                                  bias ? bias->as<float>() : nullptr, gate ? gate->data : nullptr, ldg, out.data,
                                                  static_cast<int>(qw), heads, kv_heads, head_dim, kv.page_tokens, kv.n_layers, kv.layer,
                                                  scale, window, stream), "sigmoid attention (bfloat16, matrix cores)");
        return;
    }
    kernel_check(celeg_sigmoid_attention(q.data, rows_of(q, "q"), kv.k, kv.v, dt(q, "q"), kv.table, kv.table_stride, batch.token_slot,
                                         batch.positions, temp ? temp->as<float>() : nullptr, bias ? bias->as<float>() : nullptr,
                                         gate ? gate->data : nullptr, ldg, out.data, static_cast<int>(qw), static_cast<int>(T), heads,
                                         kv_heads, head_dim, kv.page_tokens, kv.n_layers, kv.layer, scale, window, stream),
                 "sigmoid_attention");
}

// ---------------------------------------------------------------------------- gated delta rule
void Ops::delta_prepare(const Tensor& proj, int col_b, int col_a, const DeltaShape& s, const Tensor& conv_w, const Tensor& a_log,
                        const Tensor& dt_bias, const Tensor& conv_state, const Tensor& qk, const Tensor& v, const Tensor& beta_decay,
                        const StepBatch& batch) {
    dev(proj, "proj");
    const long long T = proj.shape[0], qkw = 2LL * s.kv_heads * s.dim, vw = static_cast<long long>(s.heads) * s.vdim, C = qkw + vw;
    need(s.heads > 0 && s.kv_heads > 0 && s.heads % s.kv_heads == 0 && s.dim > 0 && s.vdim > 0 && s.taps >= 1,
         "delta_prepare: heads must be a positive multiple of kv_heads, sizes positive");
    if (!a_log.defined()) col_a = col_b;
    need(proj.ndim == 2 && T == batch.n_tokens && col_b >= C && col_a >= C && col_b + s.heads <= proj.shape[1] &&
             col_a + s.heads <= proj.shape[1], "delta_prepare: the projections' columns do not fit");
    dev(conv_w, "conv_w", DType::F32);
    need(conv_w.numel() == C * s.taps, "delta_prepare: one row of taps per channel");
    // (a_log undefined: no decay per head is made; the second half of beta_decay is left alone)
    if (a_log.defined()) {
        dev(a_log, "a_log", DType::F32);
        dev(dt_bias, "dt_bias", DType::F32);
        need(a_log.numel() == s.heads && dt_bias.numel() == s.heads, "delta_prepare: one decay constant and bias per head");
    }
    dev(conv_state, "conv_state", DType::F32, false);
    need(conv_state.ndim == 3 && conv_state.shape[1] == std::max(s.taps - 1, 1) && conv_state.shape[2] == C &&
             conv_state.stride[2] == 1 && conv_state.stride[1] == C, "delta_prepare: saved inputs must be [slots, taps - 1, channels]");
    dev(qk, "qk", DType::F32);
    dev(v, "v", DType::F32);
    dev(beta_decay, "beta_decay", DType::F32);
    need(qk.numel() == T * qkw && v.numel() == T * vw && beta_decay.numel() == T * 2 * s.heads, "delta_prepare: outputs do not fit");
    const int ld = rows_of(proj, "proj");
    took(Path::DeltaRule);
    kernel_check(celeg_delta_prepare(proj.data, ld, dt(proj, "proj"), col_b, col_a, conv_w.as<float>(),
                                     a_log.defined() ? a_log.as<float>() : nullptr, a_log.defined() ? dt_bias.as<float>() : nullptr, conv_state.as<float>(), static_cast<size_t>(conv_state.stride[0]),
                                     batch.positions, batch.token_seq, batch.seq_start, batch.token_slot, qk.as<float>(), v.as<float>(),
                                     beta_decay.as<float>(), static_cast<int>(T), s.kv_heads, s.heads, s.dim, s.vdim, s.taps, stream),
                 "delta_prepare");
    // (after every row has read the old saved inputs)
    kernel_check(celeg_delta_conv_state(proj.data, ld, dt(proj, "proj"), conv_state.as<float>(), static_cast<size_t>(conv_state.stride[0]),
                                        batch.cu_seqlens, batch.seq_slot, batch.n_seqs, static_cast<int>(C), s.taps, stream),
                 "delta_conv_state");
}

void Ops::delta_scan(const Tensor& qk, const Tensor& v, const Tensor& beta_decay, const Tensor& state, const Tensor& out,
                     const DeltaShape& s, const StepBatch& batch, Workspace& ws) {
    dev(qk, "qk", DType::F32);
    dev(v, "v", DType::F32);
    dev(beta_decay, "beta_decay", DType::F32);
    dev(out, "out", DType::F32);
    dev(state, "state", DType::F32, false);
    const long long T = batch.n_tokens, per_slot = static_cast<long long>(s.heads) * s.dim * s.vdim;
    need(qk.numel() == T * 2 * s.kv_heads * s.dim && v.numel() == T * s.heads * s.vdim && out.numel() == v.numel() &&
             beta_decay.numel() == T * 2 * s.heads, "delta_scan: rows do not fit");
    need(state.ndim >= 2 && state.numel() / state.shape[0] == per_slot && state.stride[state.ndim - 1] == 1,
         "delta_scan: state must be [slots, heads, dim, vdim]");
    need(s.dim <= 256 && (s.dim <= 248 || s.dim == 256), "delta_scan: dim " + std::to_string(s.dim) + " exceeds 256");
    // rows that have a neighbour in their request's step are taken two at a time
    float* pairs = nullptr;
    if (delta_pairs && !delta_general && batch.n_tokens > batch.n_seqs)
        pairs = ws.buf("delta_pairs", DType::F32, {T, 4LL * s.kv_heads}).as<float>();
    kernel_check(celeg_delta_scan(qk.as<float>(), v.as<float>(), beta_decay.as<float>(), state.as<float>(),
                                  static_cast<size_t>(state.stride[0]), batch.cu_seqlens, batch.seq_slot, out.as<float>(), batch.n_seqs,
                                  s.kv_heads, s.heads, s.dim, s.vdim, delta_general ? 1 : 0, batch.token_seq, pairs, batch.n_tokens, stream),
                 "delta_scan");
}

void Ops::delta_gated_norm(const Tensor& o, const Tensor& weight, const Tensor& gate, float eps, const Tensor& out, int heads, int vdim,
                           int act) {
    need(act == 0 || act == 1, "delta_gated_norm: act is 0 (silu) or 1 (sigmoid)");
    dev(o, "o", DType::F32);
    dev(weight, "weight", DType::F32);
    dev(gate, "gate", out.dtype, false);
    dev(out, "out");
    const long long T = o.shape[0], w = static_cast<long long>(heads) * vdim;
    need(o.ndim == 2 && o.shape[1] == w && out.ndim == 2 && out.shape[0] == T && out.shape[1] == w && out.contiguous() &&
             gate.ndim == 2 && gate.shape[0] == T && gate.shape[1] == w && weight.numel() == vdim, "delta_gated_norm: shapes do not fit");
    kernel_check(celeg_delta_gated_norm(o.as<float>(), weight.as<float>(), gate.data, rows_of(gate, "gate"), dt(out, "out"), eps, out.data,
                                        static_cast<int>(T), heads, vdim, act, stream), "delta_gated_norm");
}

// ---------------------------------------------------------------------------- states with a decay per key channel
void Ops::channel_decay(const Tensor& z, const Tensor& a_log, const Tensor& dt_bias, const Tensor& decay, int heads, int dim) {
    dev(z, "z");
    dev(a_log, "a_log", DType::F32);
    dev(dt_bias, "dt_bias", DType::F32);
    dev(decay, "decay", DType::F32);
    const long long T = z.shape[0], cols = static_cast<long long>(heads) * dim;
    need(z.ndim == 2 && z.shape[1] == cols && a_log.numel() == heads && dt_bias.numel() == cols && decay.numel() == T * cols,
         "channel_decay: z [rows, heads * dim], a_log [heads], dt_bias [heads * dim]");
    kernel_check(celeg_channel_decay(z.data, rows_of(z, "z"), dt(z, "z"), a_log.as<float>(), dt_bias.as<float>(), decay.as<float>(),
                                     static_cast<int>(T), heads, dim, stream), "channel_decay");
}

void Ops::gla_prepare(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& z, const Tensor* z_bias, float tau, float q_scale,
                      const Tensor& qk, const Tensor& v32, const Tensor& decay) {
    dev(q, "q");
    dev(k, "k", q.dtype, false);
    dev(v, "v", q.dtype, false);
    dev(z, "z", q.dtype, false);
    dev(qk, "qk", DType::F32);
    dev(v32, "v32", DType::F32);
    dev(decay, "decay", DType::F32);
    const long long T = q.shape[0], qc = q.shape[1], vc = v.shape[1];
    need(q.ndim == 2 && k.ndim == 2 && v.ndim == 2 && z.ndim == 2 && k.shape[0] == T && v.shape[0] == T && z.shape[0] == T &&
             k.shape[1] == qc && z.shape[1] == qc && qk.numel() == T * 2 * qc && v32.numel() == T * vc && decay.numel() == T * qc,
         "gla_prepare: shapes do not fit");
    need(tau > 0.f, "gla_prepare: tau must be positive");
    if (z_bias) {
        dev(*z_bias, "z_bias", DType::F32);
        need(z_bias->numel() == qc, "gla_prepare: one bias per decay channel");
    }
    kernel_check(celeg_gla_prepare(q.data, rows_of(q, "q"), k.data, rows_of(k, "k"), v.data, rows_of(v, "v"), z.data, rows_of(z, "z"),
                                   dt(q, "q"), z_bias ? z_bias->as<float>() : nullptr, 1.0f / tau, q_scale, qk.as<float>(),
                                   v32.as<float>(), decay.as<float>(), static_cast<int>(T), static_cast<int>(qc), static_cast<int>(vc),
                                   stream), "gla_prepare");
}

void Ops::channel_scan(const Tensor& qk, const Tensor& v, const Tensor& decay, const float* beta, int beta_ld, const Tensor& state,
                       const Tensor& out, const DeltaShape& s, const StepBatch& batch) {
    dev(qk, "qk", DType::F32);
    dev(v, "v", DType::F32);
    dev(decay, "decay", DType::F32);
    dev(out, "out", DType::F32);
    dev(state, "state", DType::F32, false);
    need(s.heads > 0 && s.kv_heads > 0 && s.heads % s.kv_heads == 0 && s.dim > 0 && s.vdim > 0,
         "channel_scan: heads must be a positive multiple of kv_heads, sizes positive");
    const long long T = batch.n_tokens, per_slot = static_cast<long long>(s.heads) * s.dim * s.vdim;
    need(qk.numel() == T * 2 * s.kv_heads * s.dim && v.numel() == T * s.heads * s.vdim && out.numel() == v.numel() &&
             decay.numel() == T * s.heads * s.dim, "channel_scan: rows do not fit");
    need(state.ndim >= 2 && state.numel() / state.shape[0] == per_slot && state.stride[state.ndim - 1] == 1,
         "channel_scan: state must be [slots, heads, dim, vdim]");
    need(s.dim <= 256, "channel_scan: dim " + std::to_string(s.dim) + " exceeds 256");
    need(!beta || beta_ld >= s.heads, "channel_scan: a row of write strengths holds one per head");
    took(Path::ChannelScan);
    kernel_check(celeg_channel_scan(qk.as<float>(), v.as<float>(), decay.as<float>(), beta, beta_ld, state.as<float>(),
                                    static_cast<size_t>(state.stride[0]), batch.cu_seqlens, batch.seq_slot, out.as<float>(),
                                    batch.n_seqs, s.kv_heads, s.heads, s.dim, s.vdim, delta_general ? 1 : 0, stream), "channel_scan");
}

// ---------------------------------------------------------------------------- linear recurrent unit
void Ops::lru_gates(const Tensor& x, const Tensor& conv_w, const Tensor* conv_b, const Tensor& ra_t, const Tensor& ra_b,
                    const Tensor& ri_t, const Tensor& ri_b, const Tensor& lam, const Tensor& conv_state, const Tensor& decay,
                    const Tensor& input, const LruShape& s, const StepBatch& batch) {
    dev(x, "x");
    need(s.width > 0 && s.blocks > 0 && s.width % s.blocks == 0 && s.taps >= 1, "lru_gates: width must be a positive multiple of blocks");
    const long long T = x.shape[0], W = s.width, bw = W / s.blocks;
    need(x.ndim == 2 && x.shape[1] == W && T == batch.n_tokens, "lru_gates: x must be [rows, width]");
    dev(conv_w, "conv_w", DType::F32);
    need(conv_w.numel() == W * s.taps, "lru_gates: one row of taps per channel");
    if (conv_b) {
        dev(*conv_b, "conv_b", DType::F32);
        need(conv_b->numel() == W, "lru_gates: one convolution bias per channel");
    }
    for (const Tensor* m : {&ra_t, &ri_t}) {
        dev(*m, "gate matrix", DType::F32);
        need(m->numel() == s.blocks * bw * bw, "lru_gates: gate matrices are [blocks, width / blocks, width / blocks]");
    }
    for (const Tensor* b : {&ra_b, &ri_b, &lam}) {
        dev(*b, "gate vector", DType::F32);
        need(b->numel() == W, "lru_gates: gate biases and lam have one entry per channel");
    }
    dev(conv_state, "conv_state", DType::F32, false);
    need(conv_state.ndim == 3 && conv_state.shape[1] == std::max(s.taps - 1, 1) && conv_state.shape[2] == W &&
             conv_state.stride[2] == 1 && conv_state.stride[1] == W, "lru_gates: saved inputs must be [slots, taps - 1, width]");
    dev(decay, "decay", DType::F32);
    dev(input, "input", DType::F32);
    need(decay.numel() == T * W && input.numel() == T * W, "lru_gates: outputs do not fit");
    const int ld = rows_of(x, "x");
    took(Path::LinearRecurrentUnit);
    kernel_check(celeg_lru_gates(x.data, ld, dt(x, "x"), conv_w.as<float>(), conv_b ? conv_b->as<float>() : nullptr, ra_t.as<float>(),
                                 ra_b.as<float>(), ri_t.as<float>(), ri_b.as<float>(), lam.as<float>(), conv_state.as<float>(),
                                 static_cast<size_t>(conv_state.stride[0]), batch.positions, batch.token_seq, batch.seq_start,
                                 batch.token_slot, decay.as<float>(), input.as<float>(), static_cast<int>(T), s.width, s.blocks, s.taps,
                                 s.decay_scale, stream), "lru_gates");
    // (after every row has read the old saved inputs)
    kernel_check(celeg_delta_conv_state(x.data, ld, dt(x, "x"), conv_state.as<float>(), static_cast<size_t>(conv_state.stride[0]),
                                        batch.cu_seqlens, batch.seq_slot, batch.n_seqs, s.width, s.taps, stream), "lru_conv_state");
}

void Ops::lru_scan(const Tensor& decay, const Tensor& input, const Tensor& y, const Tensor& state, const Tensor& out,
                   const StepBatch& batch) {
    dev(decay, "decay", DType::F32);
    dev(input, "input", DType::F32);
    dev(y, "y");
    dev(out, "out", y.dtype, false);
    dev(state, "state", DType::F32, false);
    const long long T = batch.n_tokens, W = y.shape[1];
    need(y.ndim == 2 && out.ndim == 2 && y.shape[0] == T && out.shape[0] == T && out.shape[1] == W && decay.numel() == T * W &&
             input.numel() == T * W, "lru_scan: rows do not fit");
    need(state.ndim == 2 && state.shape[1] == W && state.stride[1] == 1, "lru_scan: state must be [slots, width]");
    kernel_check(celeg_lru_scan(decay.as<float>(), input.as<float>(), y.data, rows_of(y, "y"), dt(y, "y"), state.as<float>(),
                                static_cast<size_t>(state.stride[0]), batch.cu_seqlens, batch.seq_slot, out.data, rows_of(out, "out"),
                                batch.n_seqs, static_cast<int>(W), batch.max_seg_len, stream), "lru_scan");
}

// ---------------------------------------------------------------------------- attention with a distance bias
static void check_kv_wide(const KVView& kv, int kv_heads, int head_dim, int v_dim, DType dtype, const char* who) {
    need(kv.kv_heads == kv_heads && kv.head_dim == head_dim && kv.v_head_dim == v_dim,
         std::string(who) + ": the cache has other head sizes than the mixer");
    need(kv.k && kv.v && kv.table, std::string(who) + ": the cache has no device memory");
    need(kv.dtype == dtype, std::string(who) + ": the cache holds " + dtype_name(kv.dtype) + ", the rows are " + dtype_name(dtype));
    need(kv.layer >= 0 && kv.layer < kv.n_layers, std::string(who) + ": layer index outside the cache");
}

void Ops::kv_store(const Tensor& k, const Tensor& v, const StepBatch& batch, const KVView& kv) {
    dev(k, "k");
    dev(v, "v", k.dtype, false);
    check_kv_wide(kv, kv.kv_heads, kv.head_dim, kv.v_head_dim, k.dtype, "kv_store");
    const long long T = batch.n_tokens;
    need(k.ndim == 2 && v.ndim == 2 && k.shape[0] == T && v.shape[0] == T &&
             k.shape[1] == static_cast<long long>(kv.kv_heads) * kv.head_dim &&
             v.shape[1] == static_cast<long long>(kv.kv_heads) * kv.v_head_dim,
         "kv_store: k [rows, kv_heads * head_dim], v [rows, kv_heads * v_dim]");
    kernel_check(celeg_kv_store(k.data, rows_of(k, "k"), v.data, rows_of(v, "v"), dt(k, "k"), kv.k, kv.v, kv.table, kv.table_stride,
                                batch.token_slot, batch.positions, static_cast<int>(T), kv.kv_heads, kv.head_dim, kv.v_head_dim,
                                kv.page_tokens, kv.n_layers, kv.layer, stream), "kv_store");
}

void Ops::biased_attention(const Tensor& q, const Tensor& out, const ScoreShape& s, const Tensor* r1, const Tensor* r2,
                           const Tensor* gate, const StepBatch& batch, const KVView& kv, Workspace& ws) {
    dev(q, "q");
    dev(out, "out", q.dtype, false);
    need(s.heads > 0 && s.kv_heads > 0 && s.heads % s.kv_heads == 0 && s.head_dim > 0 && s.v_dim > 0,
         "biased_attention: heads must be a positive multiple of kv_heads, sizes positive");
    check_kv_wide(kv, s.kv_heads, s.head_dim, s.v_dim, q.dtype, "biased_attention");
    const long long T = batch.n_tokens;
    need(q.ndim == 2 && out.ndim == 2 && q.shape[0] == T && out.shape[0] == T &&
             q.shape[1] == static_cast<long long>(s.heads) * s.head_dim && out.shape[1] == static_cast<long long>(s.heads) * s.v_dim,
         "biased_attention: q [rows, heads * head_dim], out [rows, heads * v_dim]");
    need(s.v_dim <= 256 && s.head_dim <= 1024, "biased_attention: values of up to 256, keys of up to 1,024 numbers a head");
    need((r1 == nullptr) == (r2 == nullptr), "biased_attention: the distance bias needs both of its numbers per head");
    if (r1) {
        dev(*r1, "r1", DType::F32);
        dev(*r2, "r2", DType::F32);
        need(r1->numel() == s.heads && r2->numel() == s.heads, "biased_attention: one pair of bias numbers per head");
    }
    need(s.every >= 0 && s.window >= 0 && s.keep_first >= 0, "biased_attention: every, window and keep_first are not negative");
    const int keep_first = s.window > 0 ? s.keep_first : 0, sink_one = s.sink_one ? 1 : 0;
    if (gate) {
        dev(*gate, "gate", q.dtype, false);
        need(gate->ndim == 2 && gate->shape[0] == T && gate->shape[1] == out.shape[1], "biased_attention: gate [rows, heads * v_dim]");
    }
    (void)ws;
    took(Path::AttentionBiased);
    const int ldq = rows_of(q, "q"), ldo = rows_of(out, "out"), ldg = gate ? rows_of(*gate, "gate") : 0;
    auto aligned = [](const void* p, uintptr_t bytes) { return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0; };
    if (q.dtype == DType::BF16 && use_biased_mfma && !attention_general && celeg_biased_attention_fast_ok(s.head_dim, s.v_dim) &&
        kv.page_tokens >= 8 && (kv.page_tokens & (kv.page_tokens - 1)) == 0 && ldq % 8 == 0 && ldo % 4 == 0 && ldg % 4 == 0 &&
        aligned(q.data, 16) && aligned(out.data, 8) && (!gate || aligned(gate->data, 8))) {
        // portions of prompts: tiles of 64 rows that share their staged keys; single tokens and short
        // portions: tiles of 16 rows whose key blocks the wavefronts take in turn.  At most one
        // partly filled tile per request.
        const int form = biased_rows_form >= 0 ? biased_rows_form : (batch.max_seg_len > 16 ? 1 : 0);
        const int max_tiles = static_cast<int>(T) / (form == 1 ? 64 : 16) + batch.n_seqs;
        took(batch.decode_only ? Path::AttentionBiasedDecode : Path::AttentionBiasedRows);
        kernel_check(celeg_biased_attention_fast(form, q.data, ldq, kv.k, kv.v, kv.table, kv.table_stride, batch.cu_seqlens, batch.seq_slot,
                                                 batch.seq_start, batch.n_seqs, max_tiles, r1 ? r1->as<float>() : nullptr,
                                                 r2 ? r2->as<float>() : nullptr, gate ? gate->data : nullptr, ldg, out.data, ldo, s.heads,
                                                 s.kv_heads, s.head_dim, s.v_dim, kv.page_tokens, kv.n_layers, kv.layer, s.scale, s.coef,
                                                 s.every, s.window, keep_first, sink_one, stream), "biased attention (bfloat16, matrix cores)");
        return;
    }
    kernel_check(celeg_biased_attention(q.data, rows_of(q, "q"), dt(q, "q"), kv.k, kv.v, kv.table, kv.table_stride, batch.token_slot,
                                        batch.positions, r1 ? r1->as<float>() : nullptr, r2 ? r2->as<float>() : nullptr,
                                        gate ? gate->data : nullptr, gate ? rows_of(*gate, "gate") : 0, out.data, rows_of(out, "out"),
                                        static_cast<int>(T), s.heads, s.kv_heads, s.head_dim, s.v_dim, kv.page_tokens, kv.n_layers,
                                        kv.layer, s.scale, s.coef, s.every, s.window, keep_first, sink_one, stream), "biased_attention");
}

void Ops::conv_rope_store(const Tensor& proj, const Tensor* conv_w, const Tensor* conv_state, int taps, const Tensor* inv_freq,
                          int rotary_dim, int pairing, const Tensor& q_out, int heads, const StepBatch& batch, const KVView& kv) {
    dev(proj, "proj");
    dev(q_out, "q_out", proj.dtype, false);
    check_kv_wide(kv, kv.kv_heads, kv.head_dim, kv.v_head_dim, proj.dtype, "conv_rope_store");
    const long long T = batch.n_tokens, D = kv.head_dim, V = kv.v_head_dim, G = kv.kv_heads;
    const long long channels = (heads + G) * D + G * V;
    need(heads > 0 && proj.ndim == 2 && proj.shape[0] == T && proj.shape[1] >= channels, "conv_rope_store: proj holds q | k | v of every row");
    need(q_out.ndim == 2 && q_out.shape[0] == T && q_out.shape[1] == heads * D, "conv_rope_store: q_out [rows, heads * head_dim]");
    need((conv_w == nullptr) == (conv_state == nullptr), "conv_rope_store: taps and saved inputs go together");
    need(std::max(D, V) * 4 <= 60 * 1024, "conv_rope_store: heads of more than 15,360 values are not supported");
    if (conv_w) {
        dev(*conv_w, "conv_w", DType::F32);
        dev(*conv_state, "conv_state", DType::F32, false);
        need(taps >= 1 && conv_w->ndim == 2 && conv_w->shape[0] == channels && conv_w->shape[1] == taps,
             "conv_rope_store: conv_w must be [channels, taps]");
        need(conv_state->ndim == 3 && conv_state->shape[1] == std::max(taps - 1, 1) && conv_state->shape[2] == channels &&
                 conv_state->stride[2] == 1 && conv_state->stride[1] == channels,
             "conv_rope_store: the saved inputs must be [slots, taps - 1, channels]");
    } else {
        taps = 1;
    }
    if (inv_freq) {
        dev(*inv_freq, "inv_freq", DType::F32);
        need(rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= D && inv_freq->numel() == rotary_dim / 2 && (pairing == 0 || pairing == 1),
             "conv_rope_store: an even number of turned values, at most a head's, with a frequency a pair");
    }
    const size_t state_stride = conv_state ? static_cast<size_t>(conv_state->stride[0]) : 0;
    kernel_check(celeg_conv_rope_store(proj.data, rows_of(proj, "proj"), dt(proj, "proj"), conv_w ? conv_w->as<float>() : nullptr,
                                       conv_state ? conv_state->as<float>() : nullptr, state_stride, batch.positions, batch.token_seq,
                                       batch.seq_start, batch.token_slot, inv_freq ? inv_freq->as<float>() : nullptr,
                                       inv_freq ? rotary_dim : 0, pairing, q_out.data, rows_of(q_out, "q_out"), kv.k, kv.v, kv.table,
                                       kv.table_stride, static_cast<int>(T), heads, static_cast<int>(G), static_cast<int>(D),
                                       static_cast<int>(V), taps, kv.page_tokens, kv.n_layers, kv.layer, stream), "conv_rope_store");
    // (after every row has read the old saved inputs)
    if (conv_w && taps > 1)
        kernel_check(celeg_delta_conv_state(proj.data, rows_of(proj, "proj"), dt(proj, "proj"), conv_state->as<float>(), state_stride,
                                            batch.cu_seqlens, batch.seq_slot, batch.n_seqs, static_cast<int>(channels), taps, stream),
                     "conv_rope_store (saved inputs)");
}

void Ops::stream_add(const Tensor& h, const Tensor* rows_in, const Tensor* vec) {
    dev(h, "h", DType::F32);
    need(h.ndim == 2, "stream_add: h must be a matrix");
    if (rows_in) {
        dev(*rows_in, "rows", DType::F32);
        need(rows_in->ndim == 2 && rows_in->shape[0] == h.shape[0] && rows_in->shape[1] == h.shape[1], "stream_add: rows must have the shape of h");
    }
    if (vec) {
        dev(*vec, "vec", DType::F32);
        need(vec->numel() == h.shape[1], "stream_add: the vector must have the width of h");
    }
    kernel_check(celeg_stream_add(h.as<float>(), rows_in ? rows_in->as<float>() : nullptr, vec ? vec->as<float>() : nullptr,
                                  static_cast<int>(h.shape[0]), static_cast<int>(h.shape[1]), stream), "stream_add");
}

void Ops::softcap(const Tensor& x, float cap) {
    dev(x, "x", DType::F32);
    need(cap > 0.f, "softcap: the cap must be positive");
    kernel_check(celeg_softcap(x.as<float>(), static_cast<size_t>(x.numel()), cap, stream), "softcap");
}

// ---------------------------------------------------------------------------- layer glue
void Ops::activation_bias(const Tensor& x, const Tensor* bias, const Tensor& out, int act) {
    dev(x, "x");
    dev(out, "out", x.dtype, false);
    need(x.ndim == 2 && out.ndim == 2 && x.shape[0] == out.shape[0] && x.shape[1] == out.shape[1], "activation_bias: x and out differ");
    need(act >= 0 && act <= 2, "activation_bias: act is 0 (gelu), 1 (square of relu) or 2 (none)");
    if (bias) {
        dev(*bias, "bias", DType::F32);
        need(bias->numel() == x.shape[1], "activation_bias: one bias per column");
    }
    kernel_check(celeg_activation_bias(x.data, rows_of(x, "x"), bias ? bias->as<float>() : nullptr, out.data, rows_of(out, "out"),
                                       dt(x, "x"), static_cast<int>(x.shape[0]), static_cast<int>(x.shape[1]), act, stream),
                 "activation_bias");
}

void Ops::residual_sum(const Tensor& h, const Tensor& a, const Tensor* b, const Tensor* copy) {
    dev(h, "h", DType::F32);
    dev(a, "a");
    const long long T = h.shape[0], W = h.shape[1];
    need(h.ndim == 2 && a.ndim == 2 && a.shape[0] == T && a.shape[1] == W, "residual_sum: a must have the stream's shape");
    if (b) {
        dev(*b, "b", a.dtype, false);
        need(b->ndim == 2 && b->shape[0] == T && b->shape[1] == W, "residual_sum: b must have the stream's shape");
    }
    if (copy) {
        dev(*copy, "copy", a.dtype);
        need(copy->numel() == T * W, "residual_sum: copy must have the stream's shape");
    }
    kernel_check(celeg_residual_sum(h.as<float>(), a.data, rows_of(a, "a"), b ? b->data : nullptr, b ? rows_of(*b, "b") : 0,
                                    copy ? copy->data : nullptr, dt(a, "a"), static_cast<int>(T), static_cast<int>(W), stream),
                 "residual_sum");
}

void Ops::token_gate(const Tensor& z, const Tensor& table, int offset, const int* token_ids, const Tensor& g) {
    dev(z, "z");
    dev(table, "table", z.dtype);
    dev(g, "g", z.dtype);
    need(z.ndim == 2 && table.ndim == 2 && g.ndim == 2 && g.shape[0] == z.shape[0] && g.shape[1] == z.shape[1] && offset >= 0 &&
             offset + z.shape[1] <= table.shape[1], "token_gate: z and g [rows, dim], the table's rows hold columns [offset, offset + dim)");
    kernel_check(celeg_token_gate(z.data, rows_of(z, "z"), table.data, rows_of(table, "table"), offset, token_ids, g.data, dt(z, "z"),
                                  static_cast<int>(z.shape[0]), static_cast<int>(z.shape[1]), stream), "token_gate");
}

void Ops::normed_mean(const Tensor& a, const Tensor& wa, const Tensor& b, const Tensor& wb, float eps, float factor, const Tensor& out) {
    dev(a, "a");
    dev(b, "b", a.dtype, false);
    dev(out, "out", a.dtype);
    dev(wa, "wa", DType::F32);
    dev(wb, "wb", DType::F32);
    const long long T = a.shape[0], W = a.shape[1];
    need(a.ndim == 2 && b.ndim == 2 && b.shape[0] == T && b.shape[1] == W && out.numel() == T * W && wa.numel() == W && wb.numel() == W,
         "normed_mean: a, b and out [rows, width], weights [width]");
    kernel_check(celeg_normed_mean(a.data, rows_of(a, "a"), wa.as<float>(), b.data, rows_of(b, "b"), wb.as<float>(), eps, factor, out.data,
                                   dt(a, "a"), static_cast<int>(T), static_cast<int>(W), stream), "normed_mean");
}

void Ops::depth_mix(const Tensor& history, const Tensor& h, const Tensor& w, int n) {
    dev(history, "history", DType::F32);
    dev(h, "h", DType::F32);
    dev(w, "w", DType::F32);
    need(history.ndim == 3 && h.ndim == 2 && history.shape[1] == h.shape[0] && history.shape[2] == h.shape[1] && n >= 1 &&
             n <= history.shape[0] && w.numel() == n, "depth_mix: history [entries >= n, rows, width], w [n]");
    kernel_check(celeg_depth_mix(history.as<float>(), static_cast<size_t>(history.stride[0]), h.as<float>(), w.as<float>(), n,
                                 static_cast<int>(h.shape[0]), static_cast<int>(h.shape[1]), stream), "depth_mix");
}

// Where the context of few requests is cut into parts: how many wavefronts a part's workgroup has
// (1, 4 or 16: as many rounds of 64 keys does it take at a time; a request's rounds are shared out
// evenly over its parts).  Workgroups of 16 where they give every compute unit just one (8 requests
// of 8 key/value heads at up to 4,096 tokens: 0.463 against 0.475 and 0.479 ms a decode step; 2
// requests at up to 16,384: 3 % faster); else by the length, so that a long context gets longer
// parts rather than hundreds of them, and at short lengths workgroups of 4 once there are enough
// of them for half the compute units (1, 2, 4 and 16 requests at 2,048 tokens: 0.5 to 1.4 % faster
// than single wavefronts).  Measured at 1 to 16 requests, 2,048 and 8,192 tokens.
// One workgroup a (request, key/value head), its wavefronts taking the rounds in turn and no second
// kernel, once there are enough of them: 192 (24 requests of 8 key/value heads) at any length, 96 at
// contexts up to 4,096 tokens (12 and 16 requests at 2,048 tokens: 1 and 3 % of a decode step
// faster than in parts; 16 requests at 8,192: 3 % slower).
bool Ops::decode_whole(long long groups, int rounds) const {
    if (attention_decode_whole >= 0) return attention_decode_whole > 0;
    return groups >= 192 || (groups >= 96 && rounds <= 64);
}

int Ops::decode_split_rounds(long long groups, int rounds) const {
    const long long long_parts = groups * ((rounds + 15) / 16);
    if (decode_parts_fill && rounds > 16 && long_parts >= 192 && long_parts <= 256) return 16;
    if (rounds <= decode_part_thresholds[0]) return decode_parts_fill && rounds > 4 && groups * ((rounds + 3) / 4) >= 128 ? 4 : 1;
    return rounds <= decode_part_thresholds[1] ? 4 : 16;
}

// The first T rows of the step, each the one new token of its request.
void Ops::attention_decode(const Tensor& q, const Tensor& out, int heads, int kv_heads, int head_dim, float scale,
                           int window, const StepBatch& batch, const KVView& kv, int T, Workspace& ws, const FreshKV* fresh) {
    const int max_context = kv.table_stride * kv.page_tokens;
    // where the context is cut into parts (few requests): parts of 1, 4 or 16 rounds of 64 keys,
    // so that a long context gets longer parts rather than hundreds of them; the bound is the
    // step's longest context, or what the step's recorded graph is good for
    const int hint = batch.context_hint();
    const int bound = hint ? std::min(hint, max_context) : max_context;
    const int rounds = (bound + 63) / 64;
    const int chunks = (heads / kv_heads + 15) / 16;
    const int whole = decode_whole(static_cast<long long>(kv_heads) * chunks * T, rounds) ? 1 : 0;
    const int split_rounds = decode_split_rounds(static_cast<long long>(kv_heads) * chunks * T, rounds);
    const int n_parts = (rounds + split_rounds - 1) / split_rounds;
    const size_t parts = static_cast<size_t>(T) * heads * n_parts;
    float* workspace = static_cast<float*>(ws.raw("attention_decode_parts", parts * (head_dim + 2) * sizeof(float)));
    if (fresh) {
        need(fresh->k && fresh->v, "attention_decode: fresh keys and values are missing");
        const long long kvw = static_cast<long long>(kv_heads) * head_dim;
        for (const Tensor* t : {fresh->k, fresh->v}) {
            dev(*t, "fresh k/v", DType::BF16, false);
            need(t->ndim == 2 && t->shape[0] == T && t->shape[1] == kvw, "attention_decode: fresh k and v must be [rows, kv_heads*head_dim]");
        }
        for (const Tensor* wt : {fresh->q_weight, fresh->k_weight})
            if (wt) {
                dev(*wt, "q/k norm weight", DType::F32);
                need(wt->numel() == head_dim, "attention_decode: a norm weight must have head_dim entries");
            }
        const float* cos_sin = nullptr;
        if (fresh->inv_freq) {
            dev(*fresh->inv_freq, "inv_freq", DType::F32);
            need(fresh->inv_freq->numel() == head_dim / 2, "attention_decode: the frequency table must have head_dim / 2 entries");
            cos_sin = rope_table(*fresh->inv_freq, kv.table_stride * kv.page_tokens);
        }
        took(Path::AttentionDecodeFresh);
        kernel_check(celeg_attention_decode_fresh_bf16(
                         q.data, rows_of(q, "q"), fresh->k->data, rows_of(*fresh->k, "k"), fresh->v->data, rows_of(*fresh->v, "v"),
                         fresh->q_weight ? fresh->q_weight->as<float>() : nullptr, fresh->k_weight ? fresh->k_weight->as<float>() : nullptr,
                         fresh->eps, cos_sin, kv.k, kv.v, kv.table, kv.table_stride, batch.token_slot, batch.positions, workspace,
                         workspace + parts * head_dim, n_parts, out.data, heads * head_dim, T, heads, kv_heads, head_dim,
                         kv.page_tokens, kv.n_layers, kv.layer, scale, window, whole, split_rounds, n_parts, stream),
                     "attention for decode rows with fresh keys (bfloat16)");
        return;
    }
    took(Path::AttentionDecode);
    kernel_check(celeg_attention_decode_bf16(q.data, rows_of(q, "q"), kv.k, kv.v, kv.table, kv.table_stride, batch.token_slot,
                                             batch.positions, workspace, workspace + parts * head_dim, n_parts, out.data,
                                             heads * head_dim, T, heads, kv_heads, head_dim, kv.page_tokens, kv.n_layers,
                                             kv.layer, scale, window, whole, split_rounds, n_parts, stream),
                 "attention for decode rows (bfloat16)");
}

// ---------------------------------------------------------------------------- sampling
void Ops::sample(const Tensor& logits, const float* fparams, const int* iparams, uint8_t* seen, size_t seen_stride,
                 int* out_tokens, int* last_tokens, bool all_greedy, Workspace& ws, const HeadBest* head_best, bool penalised) {
    dev(logits, "logits", DType::F32, false);
    const int R = static_cast<int>(logits.shape[0]), V = static_cast<int>(logits.shape[1]);
    if (R == 0) return;
    // what the head's product left beside these very logits, if it did
    const bool left = use_head_argmax && head_best && head_best->logits == logits.data && head_best->rows >= R &&
                      head_best->parts > 0 && head_best->cols > 0;
    if (all_greedy && !penalised && left) {
        // greedy rows without a penalty (the caller's word): the head's kernel left the best of every
        // share of a row's columns, so the logits need not be read again
        took(Path::ArgmaxMerged);
        kernel_check(celeg_argmax_merge(head_best->best, head_best->ld, head_best->parts, R, iparams, out_tokens, last_tokens,
                                        stream), "argmax from the head's parts");
        return;
    }
    if (all_greedy && use_argmax_parts && R <= 16) {     // (64 rows: 23 us against 12 us, one workgroup a row)
        // per row: the best (value, index) so far and a count of the parts that have arrived;
        // zero at first, and the kernel leaves both at zero for its next launch
        if (!argmax_state_.ptr()) argmax_state_ = DeviceBuffer(64 * (sizeof(unsigned long long) + sizeof(unsigned int)), true);
        char* state = argmax_state_.as<char>();
        kernel_check(celeg_argmax_rows(logits.as<float>(), rows_of(logits, "logits"), R, V, fparams, iparams, seen,
                                       seen_stride, out_tokens, last_tokens, reinterpret_cast<unsigned long long*>(state),
                                       reinterpret_cast<unsigned int*>(state + 64 * sizeof(unsigned long long)), stream),
                     "argmax of rows");
        return;
    }
    // (A row of a sampled step cut into parts over many workgroups, the last one to arrive merging
    // the parts' lists, was measured: 21 against 23 us for one row of 65,536 logits and top_k 50,
    // slower from 8 rows on and at top_k 128: what the kernel spends lies in the ranking and the
    // sums, not in reading the logits.)
    // (sampled rows find their candidates among the columns of the parts whose best logit is large enough,
    // without reading the row, where the head left such parts)
    kernel_check(celeg_sample(logits.as<float>(), rows_of(logits, "logits"), R, V, fparams, iparams, seen, seen_stride,
                              out_tokens, last_tokens, left ? head_best->best : nullptr, left ? head_best->ld : 0,
                              left ? head_best->parts : 0, left ? head_best->cols : 0, stream), "sample");
}

void Ops::mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* token_ids, const int* token_slot, int n) {
    kernel_check(celeg_mark_seen(seen, stride, n_slots, vocab, token_ids, token_slot, n, stream), "mark_seen");
}

// ---------------------------------------------------------------------------- fused skinny products
bool Ops::fused_linear_ok(int rows, std::initializer_list<long long> inner) const {
    if (rows <= 0 || rows > 64) return false;
    for (long long k : inner)
        if (k <= 0 || k % 8) return false;
    return true;
}

bool Ops::rows_kernel_ok(int rows, std::initializer_list<long long> inner) const {
    if (!use_rows_kernel || rows < rows_kernel_min_rows || rows > 64) return false;
    for (long long k : inner)
        if (k % 32) return false;
    return true;
}

int Ops::residual_stat_blocks(int rows, int n, int k) const {
    if (rows_kernel_ok(rows, {k})) return celeg_gemm_rows_blocks(rows, n, k, static_cast<int>(Epilogue::Residual));
    if (rows <= 16 && use_sliced) return celeg_gemv_slices_blocks(rows, n, k);
    return (n + 15) / 16;
}

void Ops::stream_prepare(const Tensor& h, const Tensor& xb, const Tensor& stats) {
    dev(h, "h", DType::F32, false);
    dev(xb, "xb", DType::BF16, false);
    dev(stats, "stats", DType::F32);
    const long long rows = h.shape[0], width = h.shape[1];
    const Operand o = operand(xb, "xb");
    need(o.rows >= rows && o.width == width && stats.shape[0] >= rows, "stream_prepare: shapes do not fit");
    kernel_check(celeg_stream_prepare(h.as<float>(), rows_of(h, "h"), xb.data, static_cast<int>(o.ld), o.k8,
                                      stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                      static_cast<int>(width), stream), "stream_prepare");
}

void Ops::embed_stream(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& xb, const Tensor& stats,
                       const StepPrologue* prologue) {
    dev(table, "table", DType::BF16);
    dev(out, "out", DType::F32);
    dev(xb, "xb", DType::BF16, false);
    dev(stats, "stats", DType::F32);
    const long long rows = out.shape[0], width = out.shape[1];
    const Operand o = operand(xb, "xb");
    need(table.shape[1] == width && stats.shape[0] >= rows && o.rows == rows && o.width == width, "embed_stream: shapes do not fit");
    if (prologue) {
        need(prologue->token_ids == token_ids && prologue->n == rows && prologue->capacity > 0 && prologue->table && prologue->updates,
             "embed_stream: the step's prologue is not for these rows");
        kernel_check(celeg_embed_stream_prologue(table.data, prologue->token_ids, out.as<float>(), xb.data, static_cast<int>(o.ld), o.k8,
                                                 stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                                 static_cast<int>(width), static_cast<int>(table.shape[0]), prologue->table,
                                                 prologue->stride, prologue->n_slots, prologue->updates, prologue->capacity,
                                                 prologue->token_slot, prologue->last_tokens, stream), "embed_stream with the step's prologue");
        return;
    }
    kernel_check(celeg_embed_stream(table.data, token_ids, out.as<float>(), xb.data, static_cast<int>(o.ld), o.k8,
                                    stats.as<float>(), static_cast<int>(stats.stride[0]), static_cast<int>(rows),
                                    static_cast<int>(width), static_cast<int>(table.shape[0]), stream), "embed_stream");
}

void Ops::embed_stats(const Tensor& table, const int* token_ids, const Tensor& out, const Tensor& stats) {
    dev(table, "table", DType::BF16);
    dev(out, "out", DType::F32);
    dev(stats, "stats", DType::F32);
    const long long rows = out.shape[0], width = out.shape[1];
    need(table.shape[1] == width && stats.shape[0] >= rows, "embed_stats: shapes do not fit");
    kernel_check(celeg_embed_stats(table.data, token_ids, out.as<float>(), stats.as<float>(), static_cast<int>(stats.stride[0]),
                                   static_cast<int>(rows), static_cast<int>(width), static_cast<int>(table.shape[0]), stream),
                 "embed_stats");
}

// out = epilogue(prologue(a) w^T) for up to 64 rows, bfloat16 weights.
//
// a: bfloat16 rows [M, K], or, with norm_weight, the 32-bit residual stream, normalised on the
// fly (stats[row, :stat_blocks] holding partial sums of squares of its rows if stat_blocks > 0).
// rows picks rows of a.  Epilogues: Store (bfloat16 [M, N]), StoreF32, Residual (out is the
// stream, [M, N] 32-bit, added to in place; stats_out [>= M, residual_stat_blocks] receives
// partial sums of squares of the new rows, last_stat_blocks says how many a row), Swiglu (w is
// [2N, K]: gate rows then up rows), Conv (w is [3N, K]: B, C, x rows; one new token per request).
//
// Up to 16 bfloat16 rows go to the k-sliced kernels, and 9 to 64 rows with an inner size that
// is a multiple of 32 to the kernel that streams the weights.  Both also take the form behind a
// norm whose weight the caller has folded into w: a is then the bfloat16 copy of the stream and
// stats[row, :stat_blocks] its partial sums of squares, from which the rows' 1/rms (with eps)
// scales the sums; their Residual epilogue refreshes out_bf16, the bfloat16 copy of the stream,
// if given.  They also take w in the layout of fold_weight(packed).
void Ops::fused_linear(const Tensor& a, const Tensor& w, const Tensor& out, const FusedArgs& args) {
    dev(w, "w", DType::BF16);
    const Epilogue epi = args.epilogue;
    const int streams = epi == Epilogue::Swiglu ? 2 : epi == Epilogue::Conv ? 3 : 1;
    const bool packed = args.packed;
    need(!packed || (w.ndim == 3 && w.shape[2] == 32), "fused_linear: a packed weight is [K/32, rows, 32]");
    need(packed || w.ndim == 2, "fused_linear: w must be a matrix");
    const long long w_rows = packed ? w.shape[1] : w.shape[0], K = packed ? w.shape[0] * 32 : w.shape[1];
    need(w_rows % streams == 0, "fused_linear: weight rows do not split into the epilogue's streams");
    const long long N = w_rows / streams;
    dev(a, "a");
    const Operand ao = operand(a, "a");
    const int M = args.n_rows >= 0 ? args.n_rows : static_cast<int>(ao.rows);
    need(fused_linear_ok(M, {K}), "fused_linear: " + std::to_string(M) + " rows with inner size " + std::to_string(K) +
                                      " are not supported (1..64 rows, inner size a multiple of 8)");
    need(ao.width == K && (args.rows || ao.rows >= M), "fused_linear: a does not fit the weights");
    const bool norm = args.norm_weight.defined();
    if (norm) {
        need(a.dtype == DType::F32, "fused_linear: the normalising prologue reads a 32-bit stream");
        dev(args.norm_weight, "norm_weight", DType::F32);
        need(args.norm_weight.numel() == K, "fused_linear: norm weight must have the inner size");
        need(epi != Epilogue::Residual, "fused_linear: this combination is not built");
    } else {
        need(a.dtype == DType::BF16, "fused_linear: rows must be bfloat16 (or 32-bit with a norm weight)");
        if ((epi == Epilogue::Swiglu || epi == Epilogue::Conv || args.stat_blocks > 0) && !(M <= 16 && use_sliced) &&
            !rows_kernel_ok(M, {K}))
            throw KernelError("fused_linear: this combination is not built");
    }
    need(ao.ld % 8 == 0, "fused_linear: the row stride of a must be a multiple of 8");
    const DType out_dtype = (epi == Epilogue::StoreF32 || epi == Epilogue::Residual) ? DType::F32 : DType::BF16;
    dev(out, "out", out_dtype, false);
    const Operand oo = operand(out, "out");
    need(oo.rows >= M && oo.width == N, "fused_linear: out must be [" + std::to_string(M) + ", " + std::to_string(N) + "]");
    if (args.bias.defined()) {
        dev(args.bias, "bias", DType::F32);
        need(args.bias.numel() == streams * N, "fused_linear: bias does not fit");
    }
    GemvParams prm{};
    prm.a = a.data;
    prm.lda = static_cast<int>(ao.ld);
    prm.rows = args.rows;
    prm.norm_w = norm ? args.norm_weight.as<float>() : nullptr;
    prm.eps = args.eps;
    if (args.stat_blocks > 0) {
        dev(args.stats, "stats", DType::F32);
        need(args.stats.ndim == 2 && args.stats.shape[1] >= args.stat_blocks, "fused_linear: fewer partial sums than stat_blocks");
        prm.stats = args.stats.as<float>();
        prm.n_stat_blocks = args.stat_blocks;
        prm.stats_ld = static_cast<int>(args.stats.stride[0]);
    }
    prm.w = w.as<bf16>();
    prm.stream_rows = static_cast<int>(N);
    prm.bias = args.bias.defined() ? args.bias.as<float>() : nullptr;
    prm.M = M;
    prm.N = static_cast<int>(N);
    prm.K = static_cast<int>(K);
    prm.out = out.data;
    prm.ldo = static_cast<int>(oo.ld);
    const bool streamed = !norm && rows_kernel_ok(M, {K});
    const bool sliced = !norm && !streamed && M <= 16 && use_sliced;
    prm.a_k8_stride = ao.k8;
    prm.out_k8_stride = oo.k8;
    prm.w_q_stride = 8;
    if ((a.ndim == 3 || out.ndim == 3 || (args.out_bf16.defined() && args.out_bf16.ndim == 3)) && !streamed)
        throw KernelError("fused_linear: operands with the rows side by side go with the kernel for 9 to 64 rows");
    need(!(out.ndim == 3 && out_dtype != DType::BF16), "fused_linear: a 32-bit output has its rows one after the other");
    need(!packed || sliced || streamed || K % 32 == 0, "fused_linear: a packed weight has an inner size that is a multiple of 32");
    prm.w_row_stride = packed ? 32 : K;
    prm.w_kb_stride = packed ? w_rows * 32 : 32;
    if (args.out_bf16.defined()) {
        need((sliced || streamed) && epi == Epilogue::Residual,
             "fused_linear: out_bf16 goes with the residual epilogue of bfloat16 rows");
        dev(args.out_bf16, "out_bf16", DType::BF16, false);
        const Operand bo = operand(args.out_bf16, "out_bf16");
        need(bo.rows >= M && bo.width == N, "fused_linear: out_bf16 does not fit");
        prm.out_bf16 = args.out_bf16.data;
        prm.ld_bf16 = static_cast<int>(bo.ld);
        prm.bf16_k8_stride = bo.k8;
    }
    if (epi == Epilogue::Residual) {
        // partial sums of squares: one per workgroup and row
        last_stat_blocks = (sliced || streamed) ? residual_stat_blocks(M, static_cast<int>(N), static_cast<int>(K))
                                                : static_cast<int>((N + 15) / 16);
        if (args.stats_out.defined()) {
            dev(args.stats_out, "stats_out", DType::F32);
            need(args.stats_out.shape[1] >= last_stat_blocks && args.stats_out.shape[0] >= M,
                 "fused_linear: stats_out must be [>= rows, >= " + std::to_string(last_stat_blocks) + "]");
            prm.stats_out = args.stats_out.as<float>();
            prm.stats_ld_out = static_cast<int>(args.stats_out.stride[0]);
        }
    }
    if (epi == Epilogue::Conv) {
        need(args.conv != nullptr, "fused_linear: the convolution epilogue needs its operands");
        const ConvOperands& c = *args.conv;
        dev(c.taps, "conv taps", DType::F32);
        dev(c.state, "state", DType::F32, false);
        const long long L = c.taps.shape[1];
        need(L <= 8, "fused_linear: the convolution epilogue holds up to 8 taps, not " + std::to_string(L));
        need(c.taps.shape[0] == N && c.state.ndim == 3 && c.state.shape[1] == L && c.state.shape[2] == N &&
                 c.state.stride[1] == N && c.state.stride[2] == 1 && c.seq_slot,
             "fused_linear: convolution operands do not fit");
        prm.conv_w = c.taps.as<float>();
        prm.conv_b = c.bias.defined() ? c.bias.as<float>() : nullptr;
        prm.state = c.state.as<float>();
        prm.state_slot_stride = static_cast<size_t>(c.state.stride[0]);
        prm.seq_slot = c.seq_slot;
        prm.taps = static_cast<int>(L);
    }
    last_best_parts = 0;
    last_best_cols = 0;
    if (args.row_best) {
        need(epi == Epilogue::StoreF32, "fused_linear: row_best goes with the 32-bit store");
        last_best_parts = streamed ? celeg_gemm_rows_blocks(M, static_cast<int>(N), static_cast<int>(K), static_cast<int>(epi))
                          : sliced ? celeg_gemv_slices_blocks(M, static_cast<int>(N), static_cast<int>(K))
                                   : static_cast<int>((N + 15) / 16);
        need(args.row_best_ld >= last_best_parts && args.row_best_rows >= M,
             "fused_linear: row_best has room for " + std::to_string(args.row_best_rows) + " rows of " +
                 std::to_string(args.row_best_ld) + " parts, the kernel leaves " + std::to_string(M) + " of " + std::to_string(last_best_parts));
        last_best_cols = streamed ? celeg_gemm_rows_cols(M, static_cast<int>(N), static_cast<int>(K), static_cast<int>(epi))
                         : sliced ? celeg_gemv_slices_cols(M, static_cast<int>(N), static_cast<int>(K))
                                  : 16;
        prm.row_best = args.row_best;
        prm.row_best_ld = args.row_best_ld;
        prm.row_best_rows = args.row_best_rows;
    }
    took(sliced ? Path::FusedSliced : streamed ? Path::FusedRows : Path::FusedStaged);
    if (sliced) {
        kernel_check(celeg_gemv_slices(&prm, static_cast<int>(epi), stream), "fused_linear (k-sliced)");
    } else if (streamed) {
        kernel_check(celeg_gemm_rows(&prm, static_cast<int>(epi), stream), "fused_linear (9 to 64 rows)");
    } else {
        kernel_check(celeg_gemv_fused(&prm, norm ? 1 : 0, static_cast<int>(epi), fused_linear_shape, stream), "fused_linear");
    }
}

// ---------------------------------------------------------------------------- fused products of many rows
bool Ops::tiled_linear_ok(int rows, int n, std::initializer_list<long long> inner) const {
    if (!use_tiles || rows < tiles_min_rows || n % 4) return false;
    for (long long k : inner)
        if (k <= 0 || k % 64) return false;
    return true;
}

int Ops::tiled_stat_blocks(int rows, int n, int k) const { return celeg_gemm_tiles_blocks(rows, n, k); }

// out = epilogue(scale * (a w^T) + bias) for many bfloat16 rows (any number; made for more than
// 64), inner size a multiple of 64, columns a multiple of 4.  With stat_blocks > 0, a is the
// bfloat16 copy of the residual stream behind a norm whose weight the caller has folded into w,
// and stats[row, :stat_blocks] are partial sums of squares of its rows, from which the rows'
// 1/rms (with eps) scales the sums.  Epilogues: Store (bfloat16 [M, N]), Residual (out is the
// 32-bit stream, added to in place; out_bf16 receives its bfloat16 copy and stats_out the partial
// sums of squares of the new rows; last_stat_blocks says how many a row), Swiglu (w is [2N, K]).
bool Ops::tiled_qkv_ok(int head_dim, const Tensor* inv_freq, int rotary_dim, int pairing, const KVView& kv) const {
    if (!use_qkv_tail) return false;
    if (head_dim != 64 || kv.dtype != DType::BF16 || kv.head_dim != 64 || (kv.v_head_dim && kv.v_head_dim != 64)) return false;
    if (kv.page_tokens < 4 || (kv.page_tokens & (kv.page_tokens - 1))) return false;
    // the rotation: none, or of the whole head by split halves from the table of cosines and sines
    return !inv_freq || (rotary_dim == head_dim && pairing == 0 && use_rope_table);
}

void Ops::tiled_linear(const Tensor& a, const Tensor& w, const Tensor& out, Epilogue epi, float eps, const Tensor* stats,
                       int stat_blocks, const Tensor* bias, const Tensor* stats_out, const Tensor* out_bf16, const QkvTail* qkv) {
    need(epi == Epilogue::Store || epi == Epilogue::Residual || epi == Epilogue::Swiglu, "tiled_linear: unknown epilogue");
    need(!qkv || epi == Epilogue::Store, "tiled_linear: the q/k/v tail goes with the store epilogue");
    dev(a, "a", DType::BF16, false);
    dev(w, "w", DType::BF16);
    const int streams = epi == Epilogue::Swiglu ? 2 : 1;
    need(a.ndim == 2 && w.ndim == 2, "tiled_linear: a and w must be 2-D");
    const long long M = a.shape[0], K = a.shape[1];
    need(w.shape[1] == K && w.shape[0] % streams == 0, "tiled_linear: a and w do not fit");
    const long long N = w.shape[0] / streams;
    need(K % 64 == 0 && N % 4 == 0, "tiled_linear: inner size " + std::to_string(K) + " must be a multiple of 64 and " +
                                        std::to_string(N) + " columns a multiple of 4");
    const int lda = rows_of(a, "a");
    const DType out_dtype = epi == Epilogue::Residual ? DType::F32 : DType::BF16;
    dev(out, "out", out_dtype, false);
    const int ldo = rows_of(out, "out");
    need(out.shape[0] == M && out.shape[1] == N && lda % 8 == 0 && ldo % 4 == 0 &&
             reinterpret_cast<uintptr_t>(a.data) % 16 == 0 && reinterpret_cast<uintptr_t>(w.data) % 16 == 0 &&
             reinterpret_cast<uintptr_t>(out.data) % 16 == 0, "tiled_linear: out must be [M, N] and the rows aligned");
    TileParams prm{};
    prm.a = a.as<bf16>();
    prm.lda = lda;
    prm.w = w.as<bf16>();
    prm.ldw = static_cast<int>(K);
    prm.stream_rows = static_cast<int>(N);
    if (bias) {
        dev(*bias, "bias", DType::F32);
        need(bias->numel() == streams * N, "tiled_linear: bias does not fit");
        prm.bias = bias->as<float>();
    }
    if (stat_blocks > 0) {
        need(stats != nullptr, "tiled_linear: stats are missing");
        dev(*stats, "stats", DType::F32);
        need(stats->ndim == 2 && stats->shape[0] >= M && stats->shape[1] >= stat_blocks && stats->stride[1] == 1,
             "tiled_linear: stats must be [>= rows, >= stat_blocks]");
        prm.stats = stats->as<float>();
        prm.n_stat_blocks = stat_blocks;
        prm.stats_ld = static_cast<int>(stats->stride[0]);
    }
    prm.eps = eps;
    prm.M = static_cast<int>(M);
    prm.N = static_cast<int>(N);
    prm.K = static_cast<int>(K);
    prm.out = out.data;
    prm.ldo = ldo;
    if (epi == Epilogue::Residual) {
        last_stat_blocks = tiled_stat_blocks(static_cast<int>(M), static_cast<int>(N), static_cast<int>(K));
        if (out_bf16) {
            dev(*out_bf16, "out_bf16", DType::BF16, false);
            const int ldb = rows_of(*out_bf16, "out_bf16");
            need(out_bf16->shape[0] == M && out_bf16->shape[1] == N && ldb % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(out_bf16->data) % 8 == 0, "tiled_linear: out_bf16 does not fit");
            prm.out_bf16 = out_bf16->as<bf16>();
            prm.ld_bf16 = ldb;
        }
        if (stats_out) {
            dev(*stats_out, "stats_out", DType::F32);
            need(stats_out->ndim == 2 && stats_out->shape[0] >= M && stats_out->shape[1] >= last_stat_blocks &&
                     stats_out->stride[1] == 1, "tiled_linear: stats_out must be [>= rows, >= " + std::to_string(last_stat_blocks) + "]");
            prm.stats_out = stats_out->as<float>();
            prm.stats_ld_out = static_cast<int>(stats_out->stride[0]);
        }
    } else {
        need(!out_bf16 && !stats_out, "tiled_linear: out_bf16 and stats_out go with the residual epilogue");
    }
    int kernel_epilogue = static_cast<int>(epi);
    if (qkv) {
        need(qkv->batch && qkv->kv, "tiled_linear: the q/k/v tail needs the step and the cache");
        const KVView& kv = *qkv->kv;
        need(tiled_qkv_ok(qkv->head_dim, qkv->inv_freq, qkv->head_dim, 0, kv), "tiled_linear: the q/k/v tail does not take these sizes");
        check_kv(kv, qkv->kv_heads, qkv->head_dim, DType::BF16);
        need(N == (static_cast<long long>(qkv->heads) + 2LL * qkv->kv_heads) * qkv->head_dim && M == qkv->batch->n_tokens,
             "tiled_linear: the q/k/v tail needs all heads of every row of the step");
        for (const Tensor* wt : {qkv->q_weight, qkv->k_weight})
            if (wt) {
                dev(*wt, "q/k norm weight", DType::F32);
                need(wt->numel() == qkv->head_dim, "tiled_linear: a norm weight must have head_dim entries");
            }
        prm.positions = qkv->batch->positions;
        prm.token_slot = qkv->batch->token_slot;
        prm.table = kv.table;
        prm.table_stride = kv.table_stride;
        prm.k_pool = static_cast<bf16*>(kv.k);
        prm.v_pool = static_cast<bf16*>(kv.v);
        prm.n_layers = kv.n_layers;
        prm.layer = kv.layer;
        prm.page_tokens = kv.page_tokens;
        prm.q_heads = qkv->heads;
        prm.kv_heads = qkv->kv_heads;
        prm.q_weight = qkv->q_weight ? qkv->q_weight->as<float>() : nullptr;
        prm.k_weight = qkv->k_weight ? qkv->k_weight->as<float>() : nullptr;
        prm.qk_eps = qkv->eps;
        if (qkv->inv_freq) {
            dev(*qkv->inv_freq, "inv_freq", DType::F32);
            need(qkv->inv_freq->numel() == qkv->head_dim / 2, "tiled_linear: the frequency table must have head_dim / 2 entries");
            prm.cos_sin = rope_table(*qkv->inv_freq, kv.table_stride * kv.page_tokens);
        }
        kernel_epilogue = 5;
    }
    took(qkv ? Path::TiledQkv : Path::Tiled);
    kernel_check(celeg_gemm_tiles(&prm, kernel_epilogue, stream), "tiled_linear");
}

std::shared_ptr<DeviceTensor> Ops::fold_weight(const Tensor& w, const Tensor* scale, bool packed) {
    dev(w, "w", DType::BF16);
    need(w.ndim == 2, "fold_weight: w must be a matrix");
    const long long rows = w.shape[0], K = w.shape[1];
    need(!packed || K % 32 == 0, "fold_weight: the inner size must be a multiple of 32");
    if (scale) {
        dev(*scale, "scale", DType::F32);
        need(scale->numel() == K, "fold_weight: the scale must have the inner size");
    }
    auto out = packed ? device_tensor(DType::BF16, {K / 32, rows, 32}) : device_tensor(DType::BF16, {rows, K});
    kernel_check(celeg_fold_weight(w.data, scale ? scale->as<float>() : nullptr, out->view.data, static_cast<int>(rows),
                                   static_cast<int>(K), packed ? 1 : 0, stream), "fold_weight");
    return out;
}

}  // namespace celeg
