// The registries of parts and block arrangements, and the parts this library brings:
// RMS norm, rotary and no position encoding, grouped-query attention over the paged cache,
// attention over a latent cache, the double-gated short convolution, the SwiGLU feed-forward,
// routed experts, token embedding, tied and own output head, the pre-norm block and the block
// on several residual streams; beside them the neutral parts ("none" mixer and
// feed-forward, "identity" norm, "hidden" head) with which a test runs a single part alone
// through the step function.
#include "parts.hpp"

#include <cmath>
#include <mutex>

#include "kernels.hpp"

namespace celeg {

// ---------------------------------------------------------------------------- registries
namespace {
struct Registries {
    std::map<std::string, std::map<std::string, PartFactory>> parts{
        {"norm", {}}, {"mixer", {}}, {"ffn", {}}, {"position", {}}, {"embedding", {}}, {"head", {}}, {"link", {}}, {"reinjection", {}}};
    std::map<std::string, BlockFactory> blocks;
    std::mutex lock;
};
Registries& registries() {
    static Registries r;
    return r;
}
void register_builtin_parts();
void ensure_builtin() {
    static std::once_flag once;
    std::call_once(once, register_builtin_parts);
}
std::string names_of(const std::vector<std::string>& names) {
    std::string out = "[";
    for (size_t i = 0; i < names.size(); ++i) out += (i ? ", '" : "'") + names[i] + "'";
    return out + "]";
}
}  // namespace

void register_part(const std::string& role, const std::string& kind, PartFactory factory, bool replace) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    auto table = r.parts.find(role);
    if (table == r.parts.end()) {
        std::vector<std::string> roles;
        for (const auto& e : r.parts) roles.push_back(e.first);
        throw SpecError("unknown role '" + role + "'; roles: " + names_of(roles));
    }
    if (table->second.count(kind) && !replace) throw SpecError(role + " '" + kind + "' is already registered");
    table->second[kind] = std::move(factory);
}

void register_block(const std::string& arrangement, BlockFactory factory, bool replace) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    if (r.blocks.count(arrangement) && !replace) throw SpecError("block '" + arrangement + "' is already registered");
    r.blocks[arrangement] = std::move(factory);
}

std::vector<std::string> registered_parts(const std::string& role) {
    ensure_builtin();
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    std::vector<std::string> out;
    if (role == "block") {
        for (const auto& e : r.blocks) out.push_back(e.first);
    } else if (r.parts.count(role)) {
        for (const auto& e : r.parts[role]) out.push_back(e.first);
    }
    return out;
}

std::unique_ptr<Part> build_part(const std::string& role, const PartSpec& spec) {
    ensure_builtin();
    PartFactory factory;
    {
        Registries& r = registries();
        std::lock_guard<std::mutex> guard(r.lock);
        auto table = r.parts.find(role);
        if (table == r.parts.end()) throw SpecError("unknown role '" + role + "'");
        auto it = table->second.find(spec.kind);
        if (it != table->second.end()) factory = it->second;
    }
    if (!factory)
        throw SpecError("no " + role + " of kind '" + spec.kind + "' is registered; registered: " + names_of(registered_parts(role)));
    return factory(spec);
}

std::unique_ptr<Block> build_block(const LayerSpec& layer) {
    ensure_builtin();
    BlockFactory factory;
    {
        Registries& r = registries();
        std::lock_guard<std::mutex> guard(r.lock);
        auto it = r.blocks.find(layer.arrangement);
        if (it != r.blocks.end()) factory = it->second;
    }
    if (!factory)
        throw SpecError("no block arrangement '" + layer.arrangement + "' is registered; registered: " +
                        names_of(registered_parts("block")));
    return factory(layer);
}

namespace {

std::shared_ptr<DeviceTensor> get(const PartTensors& t, const std::string& role) {
    auto it = t.find(role);
    if (it == t.end()) throw SpecError("tensor for role '" + role + "' was not handed over");
    return it->second;
}
std::shared_ptr<DeviceTensor> maybe(const PartTensors& t, const std::string& role) {
    auto it = t.find(role);
    return it == t.end() ? nullptr : it->second;
}
WeightSpec matrix(long long rows, long long cols) { return WeightSpec{{rows, cols}, "matrix", "normal", {}}; }
WeightSpec vec(long long n, const char* init = "normal") { return WeightSpec{{n}, "vector", init, {}}; }

// ---------------------------------------------------------------------------- norms
// RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, w a plain scale
// (src/backend/cpu/kernels/elementwise.cpp:56-76; CUDA kernels/norm.cuh:1-44).  The sum of
// squares and the scaling are done in 32-bit whatever the activation dtype.
// "weight_offset" c: the stored weight lies around zero and the factor is c + w; the sum is
// made once, in 32-bit, when the weight is loaded, and everything after sees a plain scale.
class RmsNorm final : public Norm {
public:
    explicit RmsNorm(const PartSpec& s)
        : Norm(s), width_(s.params.get_int("width", 0)), eps_(s.params.get_double("eps", 0.0)),
          offset_(s.params.get_double("weight_offset", 0.0)) {
        if (width_ <= 0 || !(eps_ > 0)) throw SpecError("rmsnorm: width and eps must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override { return {{"weight", vec(width_, offset_ != 0.0 ? "normal" : "around_one")}}; }
    void load(const PartTensors& t, Runtime&) override {
        weight_ = get(t, "weight");
        if (offset_ != 0.0) {
            std::vector<float> w = to_host_floats(weight_->view);
            const float c = static_cast<float>(offset_);
            for (float& v : w) v = c + v;
            weight_ = from_host_floats(w, DType::F32, {width_});
        }
        foldable_ = Foldable{weight_->view, static_cast<float>(eps_)};
        params_.weight = weight_->view;
        params_.eps = static_cast<float>(eps_);
    }
    const Ops::NormParams* params() const override { return weight_ ? &params_ : nullptr; }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        rt.ops.rmsnorm(x, weight_->view, static_cast<float>(eps_), out, delta, rows);
    }
    const Foldable* foldable() const override { return weight_ ? &foldable_ : nullptr; }

private:
    long long width_;
    double eps_, offset_;
    std::shared_ptr<DeviceTensor> weight_;
    Foldable foldable_;
    Ops::NormParams params_;
};

// y = x (+ delta): no normalisation, no weight.  With it a test sees a part's rows as they are.
class IdentityNorm final : public Norm {
public:
    using Norm::Norm;
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        const long long n_rows = out.shape[0], width = out.shape[1];
        if (rows) {
            // listed rows: gather on the host side of the stream, row by row (a test path)
            std::vector<int> picked(static_cast<size_t>(n_rows));
            CELEG_HIP(hipMemcpyAsync(picked.data(), rows, picked.size() * sizeof(int), hipMemcpyDeviceToHost, rt.stream));
            CELEG_HIP(hipStreamSynchronize(rt.stream));
            Tensor sum = rt.ws.buf("identity_norm_sum", DType::F32, {1, width});
            for (long long r = 0; r < n_rows; ++r) {
                Tensor src = x.rows(picked[static_cast<size_t>(r)], 1);
                if (delta) {
                    rt.ops.cast(src, sum);
                    add(rt, sum, delta->rows(picked[static_cast<size_t>(r)], 1));
                    rt.ops.cast(sum, out.rows(r, 1));
                } else {
                    rt.ops.cast(src, out.rows(r, 1));
                }
            }
            return;
        }
        if (delta) add(rt, x, *delta);
        rt.ops.cast(x, out);
    }

private:
    // x += delta through the norm kernel's own addition (weight one, result discarded)
    static void add(Runtime& rt, const Tensor& x, const Tensor& delta) {
        const long long width = x.shape[1];
        Tensor ones = rt.ws.buf("identity_norm_ones", DType::F32, {width});
        std::vector<float> host(static_cast<size_t>(width), 1.0f);
        CELEG_HIP(hipMemcpyAsync(ones.data, host.data(), host.size() * 4, hipMemcpyHostToDevice, rt.stream));
        CELEG_HIP(hipStreamSynchronize(rt.stream));
        Tensor scratch = rt.ws.buf("identity_norm_scratch", DType::F32, {x.shape[0], width});
        rt.ops.rmsnorm(x, ones, 1e-6f, scratch, &delta, nullptr);
    }
};

// ---------------------------------------------------------------------------- position encodings
// rope: rotary encoding: for i < rotary_dim/2 pair i is rotated by the angle
// position * theta^(-2i/rotary_dim); the pair is (x[i], x[i + rotary_dim/2]) ("pairing":
// "halves", the default and the reference's, src/backend/cpu/kernels/rope.cpp:30-36, 95-108)
// or (x[2i], x[2i+1]) ("neighbours").  The frequencies are computed on the host
// in double (include/celeg/model/position.hpp:77-78) and handed to the kernel as a 32-bit
// table; the angle is the 32-bit product float(position) * frequency.
class Rope final : public PositionEncoding {
public:
    explicit Rope(const PartSpec& s) : PositionEncoding(s) {
        theta_ = s.params.get_double("theta", 0.0);
        head_dim_ = static_cast<int>(s.params.get_int("head_dim", 0));
        rotary_dim_ = static_cast<int>(s.params.get_int("rotary_dim", head_dim_));
        if (!(theta_ > 0)) throw SpecError("rope: theta must be positive");
        if (rotary_dim_ <= 0 || rotary_dim_ % 2 || rotary_dim_ > head_dim_)
            throw SpecError("rope: rotary_dim must be even, positive and at most head_dim");
        const std::string pairing = s.params.get_string("pairing", "halves");
        if (pairing != "halves" && pairing != "neighbours") throw SpecError("rope: pairing is 'halves' or 'neighbours', not '" + pairing + "'");
        pairing_ = pairing == "neighbours" ? 1 : 0;
        if (!s.params["scaling"].is_null()) {
            const Json& sc = s.params["scaling"];
            if (!sc.is_object()) throw SpecError("rope: scaling must be an object");
            scaled_ = true;
            factor_ = sc.get_double("factor", 1.0);
            low_ = sc.get_double("low", 1.0);
            high_ = sc.get_double("high", 1.0);
            original_ = sc.get_double("original", 0.0);
            if (!(factor_ > 0) || !(low_ > 0) || !(high_ > low_) || !(original_ > 0))
                throw SpecError("rope: scaling needs factor > 0, 0 < low < high and original > 0");
        }
    }
    bool graph_safe() const override { return true; }
    Tables tables(Runtime&) override {
        if (!table_) {
            std::vector<float> freq(static_cast<size_t>(rotary_dim_ / 2));
            for (int i = 0; i < rotary_dim_ / 2; ++i)
                freq[static_cast<size_t>(i)] = static_cast<float>(scaled(std::pow(theta_, -2.0 * i / rotary_dim_)));
            table_ = from_host_floats(freq, DType::F32, {rotary_dim_ / 2});
        }
        return Tables{table_->view, rotary_dim_, pairing_};
    }

private:
    // "scaling" {factor, low, high, original}: frequencies whose wavelength 2 pi / f is below
    // original / high stay, above original / low become f / factor, and between the two
    // (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)
    double scaled(double f) const {
        if (!scaled_) return f;
        const double wavelength = 2.0 * 3.14159265358979323846 / f;
        if (wavelength < original_ / high_) return f;
        if (wavelength > original_ / low_) return f / factor_;
        const double t = (original_ / wavelength - low_) / (high_ - low_);
        return (1.0 - t) * f / factor_ + t * f;
    }
    double theta_;
    bool scaled_ = false;
    double factor_ = 1.0, low_ = 1.0, high_ = 1.0, original_ = 0.0;
    int head_dim_, rotary_dim_, pairing_ = 0;
    std::shared_ptr<DeviceTensor> table_;
};

class NoPosition final : public PositionEncoding {
public:
    using PositionEncoding::PositionEncoding;
    bool graph_safe() const override { return true; }
    Tables tables(Runtime&) override { return Tables{}; }
};

// ---------------------------------------------------------------------------- attention
// Grouped-query attention over the paged cache.
//
// Order of work (src/backend/cpu/model_forward_token.cpp:100-120;
// src/backend/cuda/model/prefill_batched/attention/regular.cpp:23-131): q, k, v projections;
// RMSNorm of every q and k head over head_dim with one weight [head_dim] for all heads
// (src/backend/cpu/kernels/rope.cpp:84-94); position encoding of q and k; k and v of ALL rows
// of the step are written into the pages before any row attends
// (src/backend/cpu/model_forward_chunk.cpp:440-520); scores (q.k)/sqrt(head_dim) over the keys
// at positions <= the row's position (and inside the window, if there is one), softmax in
// 32-bit, weighted sum of values, output projection.  The scale is applied once
// (include/celeg/backend/cuda/attention_norm.hpp:13-23).
class GqaAttention final : public Mixer {
public:
    explicit GqaAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        heads_ = static_cast<int>(p.get_int("heads", 0));
        kv_heads_ = static_cast<int>(p.get_int("kv_heads", heads_));
        head_dim_ = static_cast<int>(p.get_int("head_dim", 0));
        qk_norm_ = p.get_bool("qk_norm", false);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        if (!p["window"].is_null()) {
            window_ = static_cast<int>(p["window"].as_int());
            if (*window_ <= 0) throw SpecError("gqa_attention: window must be positive");
        }
        if (width_ <= 0 || heads_ <= 0 || kv_heads_ <= 0 || heads_ % kv_heads_)
            throw SpecError("gqa_attention: heads must be a positive multiple of kv_heads");
        if (head_dim_ <= 0 || head_dim_ % 2) throw SpecError("gqa_attention: head_dim must be even");
        scale_ = p["scale"].is_null() ? static_cast<float>(1.0 / std::sqrt(static_cast<double>(head_dim_)))
                                      : static_cast<float>(p["scale"].as_double());
        PartSpec none;
        none.kind = "none";
        position_ = build_as<PositionEncoding>(
            "position", PartSpec::is_part(p["position"]) ? PartSpec::from_json(p["position"], "gqa_attention.position") : none);
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override { return {position_.get()}; }
    void set_reads_foreign_kv() override { own_kv_ = false; }
    std::optional<KVNeed> kv_need() const override { return KVNeed{kv_heads_, head_dim_, window_}; }
    WeightSpecs weight_specs() const override {
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        WeightSpecs specs{{"q_proj", matrix(qw, width_)}, {"out_proj", matrix(width_, qw)}};
        if (own_kv_) {
            specs.push_back({"k_proj", matrix(kvw, width_)});
            specs.push_back({"v_proj", matrix(kvw, width_)});
        }
        if (qk_norm_) {
            specs.push_back({"q_norm", vec(head_dim_, "around_one")});
            if (own_kv_) specs.push_back({"k_norm", vec(head_dim_, "around_one")});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        // q, k and v projections run as one matrix product (the reference's fused_projections,
        // src/backend/cuda/execution_plan.cpp:113)
        if (own_kv_) {
            auto q = get(t, "q_proj"), k = get(t, "k_proj"), v = get(t, "v_proj");
            if (q->view.dtype != k->view.dtype || q->view.dtype != v->view.dtype)
                throw SpecError("gqa_attention: q, k and v projections are stored in different dtypes");
            w_qkv_ = concat_rows({q, k, v});
            w_q_ = std::make_shared<DeviceTensor>();
            w_q_->view = w_qkv_->view.rows(0, static_cast<long long>(heads_) * head_dim_);
        } else {
            w_q_ = get(t, "q_proj");
        }
        w_o_ = get(t, "out_proj");
        q_norm_ = maybe(t, "q_norm");
        k_norm_ = maybe(t, "k_norm");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        Tensor attended = project_and_attend(x, nullptr, batch, cache, rt);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {x.shape[0], width_});
        rt.ops.linear(attended, w_o_->view, out, nullptr, rt.ws);
        return out;
    }
    // h += mixer(norm(h)) with the norm folded into the q/k/v product and the residual addition
    // into the output product
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const LayerCache& cache,
                       Runtime& rt) override {
        const long long qw = static_cast<long long>(heads_) * head_dim_;
        const Tensor& w_in = cache.writes_kv ? w_qkv_->view : w_q_->view;
        if (!fused::fused_rows_ok(rt, batch, {width_, qw}) || w_in.dtype != rt.dtype || w_o_->view.dtype != rt.dtype)
            return false;
        Tensor attended = project_and_attend(h, &norm, batch, cache, rt);
        fused::linear_into_stream(rt, attended, w_o_->view, h);
        return true;
    }

private:
    // norm null: x are normalised rows; else x is the residual stream and the norm is applied
    // inside the product
    Tensor project_and_attend(const Tensor& x, const Norm::Foldable* norm, const StepBatch& batch, const LayerCache& cache,
                              Runtime& rt) {
        const long long T = x.shape[0];
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        const bool writes = cache.writes_kv;
        if (!cache.kv) throw SpecError("gqa_attention: the cache has no keys and values for this layer");
        if (writes && !own_kv_)
            throw SpecError("gqa_attention: built without key/value projections but asked to write a cache");
        auto project = [&](const std::shared_ptr<DeviceTensor>& w, const Tensor& out) {
            if (norm) fused::norm_linear(rt, x, *norm, w->view, out, Epilogue::Store);
            else rt.ops.linear(x, w->view, out, nullptr, rt.ws);
        };
        const PositionEncoding::Tables tables = position_->tables(rt);
        const Tensor* inv_freq = tables.inv_freq.defined() ? &tables.inv_freq : nullptr;
        Tensor q, k, v;
        bool finished = false;      // norm, rotation and cache write made by the product's own kernel
        if (writes) {
            Tensor qkv = rt.ws.buf("attn_qkv", rt.dtype, {T, qw + 2 * kvw});
            if (norm && fused::qkv_tail_ok(rt, static_cast<int>(T), width_) && T == batch.n_tokens &&
                rt.ops.tiled_qkv_ok(head_dim_, inv_freq, tables.rotary_dim, tables.pairing, *cache.kv)) {
                QkvTail tail;
                tail.heads = heads_;
                tail.kv_heads = kv_heads_;
                tail.head_dim = head_dim_;
                tail.q_weight = q_norm_ ? &q_norm_->view : nullptr;
                tail.k_weight = k_norm_ ? &k_norm_->view : nullptr;
                tail.eps = eps_;
                tail.inv_freq = inv_freq;
                tail.batch = &batch;
                tail.kv = &*cache.kv;
                fused::LinearExtras extras;
                extras.qkv = &tail;
                fused::norm_linear(rt, x, *norm, w_qkv_->view, qkv, Epilogue::Store, extras);
                finished = true;
            } else {
                project(w_qkv_, qkv);
            }
            q = qkv.cols(0, qw);
            k = qkv.cols(qw, kvw);
            v = qkv.cols(qw + kvw, kvw);
        } else {
            q = rt.ws.buf("attn_q", rt.dtype, {T, qw});
            project(w_q_, q);
        }
        Tensor attended = rt.ws.buf("attn_out", rt.dtype, {T, qw});
        // a decode-only step: the attention kernel prepares and writes the step's own keys and values
        if (!finished && writes && T == batch.n_tokens &&
            rt.ops.attention_fresh_ok(heads_, head_dim_, inv_freq, tables.rotary_dim, tables.pairing, batch, *cache.kv, rt.dtype)) {
            FreshKV fresh;
            fresh.k = &k;
            fresh.v = &v;
            fresh.q_weight = q_norm_ ? &q_norm_->view : nullptr;
            fresh.k_weight = k_norm_ ? &k_norm_->view : nullptr;
            fresh.eps = eps_;
            fresh.inv_freq = inv_freq;
            rt.ops.paged_attention(q, attended, heads_, kv_heads_, head_dim_, scale_, window_ ? *window_ : 0, batch, *cache.kv, rt.ws,
                                   &fresh);
            return attended;
        }
        if (!finished)
            rt.ops.qk_norm_rope_store(q, writes ? &k : nullptr, writes ? &v : nullptr, q_norm_ ? &q_norm_->view : nullptr,
                                      k_norm_ ? &k_norm_->view : nullptr, eps_, inv_freq,
                                      tables.rotary_dim, tables.pairing, heads_, kv_heads_, head_dim_, batch, *cache.kv);
        rt.ops.paged_attention(q, attended, heads_, kv_heads_, head_dim_, scale_, window_ ? *window_ : 0, batch, *cache.kv, rt.ws);
        return attended;
    }

    long long width_ = 0;
    int heads_ = 0, kv_heads_ = 0, head_dim_ = 0;
    bool qk_norm_ = false, own_kv_ = true;
    float eps_ = 1e-6f, scale_ = 1.f;
    std::optional<int> window_;
    std::unique_ptr<PositionEncoding> position_;
    std::shared_ptr<DeviceTensor> w_qkv_, w_q_, w_o_, q_norm_, k_norm_;
};

// ---------------------------------------------------------------------------- latent attention
// Attention whose keys and values are expanded from one compressed row per token.
//
// From the mixer's input h: q = W_q h, head by head [dim plain | rot rotated]; W_dkv h gives
// rank + rot values: the first rank, RMS-normed with a weight of their own, are the compressed
// row c, the last rot are a key part that every head shares and that is rotated by the
// position, as the queries' rot part is.  Head i's key is (W_uk[i] c | shared part), its value
// W_uv[i] c; score = (q . k) * scale over positions 0..p; softmax, whose denominator may hold
// one more term exp(sink_i) (a learned number per head with no key and no value); the heads'
// results, optionally times sigmoid(W_g h), go through W_o.
//
// Only c and the shared part are cached: one row of rank + rot values per token, in a
// keys-only group of the cache manager.  The expansion is never made: W_uk moves to the query
// side (q_lat[i] = (W_uk[i]^T q_plain[i] | q_rot[i]), a score is q_lat . cached row), the
// weighted sum runs over c, and W_uv[i] is applied to it afterwards.
class LatentAttention final : public Mixer {
public:
    explicit LatentAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        shape_.heads = static_cast<int>(p.get_int("heads", 0));
        shape_.dim = static_cast<int>(p.get_int("dim", 0));
        shape_.rot = static_cast<int>(p.get_int("rot_dim", 0));
        shape_.rank = static_cast<int>(p.get_int("kv_rank", 0));
        vdim_ = static_cast<int>(p.get_int("vdim", shape_.dim));
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        sink_ = p.get_bool("sink", false);
        gate_ = p.get_bool("gate", false);
        if (width_ <= 0 || shape_.heads <= 0 || shape_.dim <= 0 || shape_.rot < 0 || shape_.rank <= 0 || vdim_ <= 0)
            throw SpecError("latent_attention: width, heads, dim, kv_rank and vdim must be positive");
        scale_ = p["scale"].is_null() ? static_cast<float>(1.0 / std::sqrt(static_cast<double>(shape_.dim + shape_.rot)))
                                      : static_cast<float>(p["scale"].as_double());
        PartSpec none;
        none.kind = "none";
        position_ = build_as<PositionEncoding>(
            "position", PartSpec::is_part(p["position"]) ? PartSpec::from_json(p["position"], "latent_attention.position") : none);
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override { return {position_.get()}; }
    std::optional<KVNeed> kv_need() const override {
        KVNeed need;
        need.kv_heads = 1;
        need.head_dim = shape_.rank + shape_.rot;
        need.keys_only = true;
        return need;
    }
    WeightSpecs weight_specs() const override {
        const long long H = shape_.heads, qd = shape_.dim + shape_.rot;
        WeightSpecs specs{{"q", matrix(H * qd, width_)},          {"dkv", matrix(shape_.rank + shape_.rot, width_)},
                          {"dkv_norm", vec(shape_.rank, "around_one")}, {"uk", matrix(H * shape_.dim, shape_.rank)},
                          {"uv", matrix(H * vdim_, shape_.rank)},  {"o", matrix(width_, H * vdim_)}};
        if (sink_) specs.push_back({"sink", vec(H)});
        if (gate_) specs.push_back({"g", matrix(H * vdim_, width_)});
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        // q, dkv and the gate read the same rows: one product
        std::vector<std::shared_ptr<DeviceTensor>> in{get(t, "q"), get(t, "dkv")};
        if (gate_) in.push_back(get(t, "g"));
        for (const auto& w : in)
            if (w->view.dtype != in[0]->view.dtype) throw SpecError("latent_attention: the input projections are stored in different dtypes");
        w_in_ = concat_rows(in);
        w_o_ = get(t, "o");
        dkv_norm_ = get(t, "dkv_norm");
        if (sink_) sink_w_ = get(t, "sink");
        // W_uk [heads * dim, rank] becomes [heads, rank, dim] (the query side multiplies with its transpose)
        auto uk = get(t, "uk"), uv = get(t, "uv");
        const int H = shape_.heads, dim = shape_.dim, rank = shape_.rank;
        const std::vector<float> src = to_host_floats(uk->view);
        std::vector<float> turned(src.size());
        for (int h = 0; h < H; ++h)
            for (int d = 0; d < dim; ++d)
                for (int r = 0; r < rank; ++r)
                    turned[(static_cast<size_t>(h) * rank + r) * dim + d] = src[(static_cast<size_t>(h) * dim + d) * rank + r];
        w_uk_t_ = from_host_floats(turned, uk->view.dtype, {H, rank, dim});
        w_uv_ = uv;
        uv_view_ = Tensor::make(uv->view.data, uv->view.dtype, {H, vdim_, rank});
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        if (!cache.kv) throw SpecError("latent_attention: the cache has no rows for this layer");
        if (!cache.writes_kv) throw SpecError("latent_attention: reading another entry's cache is not supported");
        const long long T = x.shape[0], H = shape_.heads;
        const long long qd = shape_.dim + shape_.rot, D = shape_.rank + shape_.rot;
        const long long q_cols = H * qd, dkv_cols = D, g_cols = gate_ ? H * vdim_ : 0;
        Tensor proj = rt.ws.buf("latent_proj", rt.dtype, {T, q_cols + dkv_cols + g_cols});
        rt.ops.linear(x, w_in_->view, proj, nullptr, rt.ws);
        const PositionEncoding::Tables tables = position_->tables(rt);
        const Tensor* inv_freq = tables.inv_freq.defined() ? &tables.inv_freq : nullptr;
        rt.ops.latent_prepare(proj, 0, static_cast<int>(q_cols), shape_, dkv_norm_->view, eps_, inv_freq,
                              inv_freq ? tables.rotary_dim : 0, tables.pairing, true, batch, *cache.kv);
        Tensor q_lat = rt.ws.buf("latent_q", rt.dtype, {T, H * D});
        rt.ops.headwise_linear(proj.cols(0, q_cols), static_cast<int>(qd), w_uk_t_->view, q_lat, static_cast<int>(D), shape_.rot, nullptr);
        Tensor o_lat = rt.ws.buf("latent_o", rt.dtype, {T, H * shape_.rank});
        rt.ops.latent_attention(q_lat, o_lat, shape_, scale_, sink_ ? &sink_w_->view : nullptr, batch, *cache.kv, rt.ws);
        Tensor heads = rt.ws.buf("latent_heads", rt.dtype, {T, H * vdim_});
        Tensor gate = gate_ ? proj.cols(q_cols + dkv_cols, g_cols) : Tensor();
        rt.ops.headwise_linear(o_lat, shape_.rank, uv_view_, heads, vdim_, 0, gate_ ? &gate : nullptr);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(heads, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0;
    Ops::LatentShape shape_;
    int vdim_ = 0;
    bool sink_ = false, gate_ = false;
    float eps_ = 1e-6f, scale_ = 1.f;
    std::unique_ptr<PositionEncoding> position_;
    std::shared_ptr<DeviceTensor> w_in_, w_o_, dkv_norm_, sink_w_, w_uk_t_, w_uv_;
    Tensor uv_view_;
};

// ---------------------------------------------------------------------------- short convolution
// Double-gated short causal convolution.
//
// bcx = x W_in^T splits into B = [0,H), C = [H,2H), x = [2H,3H)
// (src/backend/cpu/kernels/convolution.cpp:16-18); bx = B*x;
// conv[t,ch] = sum_tap w[ch,tap] * bx[t-(L-1-tap), ch], zero before position 0, so the last tap
// multiplies the current token (convolution.cpp:19-26); y = C*conv; out = y W_out^T
// (src/backend/cpu/operators/recurrent.cpp:212-240).  A step continues from the request's saved
// state wherever the previous step stopped, as the reference's ragged kernel does
// (src/backend/cuda/kernels/shortconv.cuh:34-64).
//
// State per request: the last L values of bx, [L, H] in 32-bit, entry j holding position
// (tokens seen so far) - L + j; every row of a step reads the old state, then the state is
// replaced.
//
// With bias (the reference's ShortConvolutionSpec.bias is never true,
// include/celeg/model/graph.hpp:316-320): in_proj bias [3H] is added to bcx, the convolution
// bias [H] to conv before the C gate, out_proj bias [H] to the output.
class ShortConv final : public Mixer {
public:
    explicit ShortConv(const PartSpec& s) : Mixer(s) {
        width_ = s.params.get_int("width", 0);
        taps_ = s.params.get_int("taps", 0);
        bias_ = s.params.get_bool("bias", false);
        if (width_ <= 0 || taps_ <= 0) throw SpecError("short_conv: width and taps must be positive");
    }
    bool graph_safe() const override { return true; }
    std::vector<StateNeed> state_needs() const override { return {StateNeed{"bx", {taps_, width_}, DType::F32}}; }
    WeightSpecs weight_specs() const override {
        WeightSpec conv{{width_, 1, taps_}, "vector", "normal", {{width_, taps_}}};
        WeightSpecs specs{{"in_proj", matrix(3 * width_, width_)}, {"conv", conv}, {"out_proj", matrix(width_, width_)}};
        if (bias_) {
            specs.push_back({"in_proj_bias", vec(3 * width_)});
            specs.push_back({"conv_bias", vec(width_)});
            specs.push_back({"out_proj_bias", vec(width_)});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        w_in_ = get(t, "in_proj");
        w_out_ = get(t, "out_proj");
        w_conv_ = get(t, "conv");
        taps_view_ = Tensor::make(w_conv_->view.data, DType::F32, {width_, taps_});     // [H, 1, L] and [H, L] lie alike
        if (bias_) {
            b_in_ = get(t, "in_proj_bias");
            b_conv_ = get(t, "conv_bias");
            b_out_ = get(t, "out_proj_bias");
        }
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor bcx = rt.ws.buf("conv_bcx", rt.dtype, {T, 3 * width_});
        rt.ops.linear(x, w_in_->view, bcx, b_in_ ? &b_in_->view : nullptr, rt.ws);
        Tensor y = rt.ws.buf("conv_y", rt.dtype, {T, width_});
        rt.ops.short_conv(bcx, taps_view_, b_conv_ ? &b_conv_->view : nullptr, cache.states.at("bx"), y, batch);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(y, w_out_->view, out, b_out_ ? &b_out_->view : nullptr, rt.ws);
        return out;
    }
    // h += mixer(norm(h)) with the norm, the convolution (for one new token per request) and the
    // residual addition folded into the two products
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const LayerCache& cache,
                       Runtime& rt) override {
        if (!fused::fused_rows_ok(rt, batch, {width_}) || w_in_->view.dtype != rt.dtype || w_out_->view.dtype != rt.dtype)
            return false;
        const int T = batch.n_tokens;
        fused::LinearExtras extras;
        if (b_in_) extras.bias = b_in_->view;
        Tensor y;
        if (batch.decode_only && batch.n_seqs == T && taps_ <= 8 && !fused::tiled_step(rt, T, width_)) {   // the fused form holds 8 taps
            y = fused::operand_rows(rt, "conv_y_fused", T, width_, {width_});
            ConvOperands conv;
            conv.taps = taps_view_;
            if (b_conv_) conv.bias = b_conv_->view;
            conv.state = cache.states.at("bx");
            conv.seq_slot = batch.seq_slot;
            extras.conv = &conv;
            fused::norm_linear(rt, h, norm, w_in_->view, y, Epilogue::Conv, extras);
        } else {
            y = rt.ws.buf("conv_y", rt.dtype, {T, width_});
            Tensor bcx = rt.ws.buf("conv_bcx", rt.dtype, {T, 3 * width_});
            fused::norm_linear(rt, h, norm, w_in_->view, bcx, Epilogue::Store, extras);
            rt.ops.short_conv(bcx, taps_view_, b_conv_ ? &b_conv_->view : nullptr, cache.states.at("bx"), y, batch);
        }
        fused::linear_into_stream(rt, y, w_out_->view, h, b_out_ ? &b_out_->view : nullptr);
        return true;
    }

private:
    long long width_ = 0, taps_ = 0;
    bool bias_ = false;
    std::shared_ptr<DeviceTensor> w_in_, w_conv_, w_out_, b_in_, b_conv_, b_out_;
    Tensor taps_view_;
};

// a mixer that adds nothing and keeps nothing
class NoMixer final : public Mixer {
public:
    explicit NoMixer(const PartSpec& s) : Mixer(s), width_(s.params.get_int("width", 0)) {}
    bool graph_safe() const override { return true; }
    Tensor forward(const Tensor& x, const StepBatch&, const LayerCache&, Runtime& rt) override { return zeros(rt, x.shape[0], width_ ? width_ : x.shape[1]); }
    static Tensor zeros(Runtime& rt, long long rows, long long width) {
        // (a fill kernel, not a memset: a recorded graph may hold it)
        const size_t words = (static_cast<size_t>(rows * width) * dtype_size(rt.dtype) + 3) / 4;
        void* p = rt.ws.raw("none_out", words * 4);
        kernel_check(celeg_zero_words(p, words, rt.stream), "zero fill");
        return Tensor::make(p, rt.dtype, {rows, width});
    }

private:
    long long width_;
};

// ---------------------------------------------------------------------------- feed-forward
// SwiGLU feed-forward: (silu(x W1^T) * (x W3^T)) W2^T, silu(g) = g / (1 + exp(-g))
// (src/backend/cpu/model_forward_token.cpp:163-172; kernels/elementwise.cpp:101-119).  Gate and
// up projections run as one matrix product on the concatenation [W1; W3] (rows [0,ff) gate,
// [ff,2ff) up), as the reference's w13 (src/backend/cuda/model/weight_setup.cpp:289-306).
class SwiGlu final : public FeedForward {
public:
    explicit SwiGlu(const PartSpec& s) : FeedForward(s), width_(s.params.get_int("width", 0)), ff_(s.params.get_int("ff", 0)) {
        if (width_ <= 0 || ff_ <= 0) throw SpecError("swiglu: width and ff must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        return {{"gate", matrix(ff_, width_)}, {"up", matrix(ff_, width_)}, {"down", matrix(width_, ff_)}};
    }
    void load(const PartTensors& t, Runtime&) override {
        auto gate = get(t, "gate"), up = get(t, "up");
        if (gate->view.dtype != up->view.dtype) throw SpecError("swiglu: gate and up projections are stored in different dtypes");
        w_gate_up_ = concat_rows({gate, up});
        w_down_ = get(t, "down");
    }
    Tensor forward(const Tensor& x, const StepBatch&, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor gate_up = rt.ws.buf("ffn_gate_up", rt.dtype, {T, 2 * ff_});
        rt.ops.linear(x, w_gate_up_->view, gate_up, nullptr, rt.ws);
        Tensor act = rt.ws.buf("ffn_act", rt.dtype, {T, ff_});
        rt.ops.swiglu(gate_up, act);
        Tensor out = rt.ws.buf("ffn_out", rt.dtype, {T, width_});
        rt.ops.linear(act, w_down_->view, out, nullptr, rt.ws);
        return out;
    }
    // h += ffn(norm(h)): the norm and the SwiGLU folded into the first product, the residual
    // addition into the second
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, Runtime& rt) override {
        if (!fused::fused_rows_ok(rt, batch, {width_, ff_}) || w_gate_up_->view.dtype != rt.dtype || w_down_->view.dtype != rt.dtype)
            return false;
        Tensor act = fused::operand_rows(rt, "ffn_act_fused", batch.n_tokens, ff_, {width_});
        fused::norm_linear(rt, h, norm, w_gate_up_->view, act, Epilogue::Swiglu);
        fused::linear_into_stream(rt, act, w_down_->view, h);
        return true;
    }

private:
    long long width_, ff_;
    std::shared_ptr<DeviceTensor> w_gate_up_, w_down_;
};

// Routed experts: `experts` gated feed-forwards W_down (silu(W_gate x) * (W_up x)) without
// biases, of which every row uses `top`.  Router logits z = W_router x in 32-bit (the router's
// matrix is held in 32-bit); "score": "sigmoid" (s = 1 / (1 + e^-z), every expert by itself) or
// "softmax" (over all experts); the `top` largest are chosen, their scores are the weights
// ("renormalize": divided by their sum).  "weight_on": "input" (the output is
// sum expert(w x)) or "output" (sum w expert(x)).  "gated": false makes an expert
// W_down act(W_up x) with "activation": "relu2" (the square of relu) and no gate matrix.
// "groups": {"count", "keep"}: the experts form `count` equal groups of neighbours, a group's score is the
// sum of its two largest scores, and only experts of the `keep` best groups can be chosen.  "renormalize_eps"
// is added to the sum the chosen scores are divided by; "route_scale" multiplies the weights afterwards.
// "shared": a feed-forward part that every row passes as well; its output is added to the experts'.
class RoutedExperts final : public FeedForward {
public:
    explicit RoutedExperts(const PartSpec& s) : FeedForward(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        ff_ = p.get_int("ff", 0);
        experts_ = static_cast<int>(p.get_int("experts", 0));
        top_ = static_cast<int>(p.get_int("top", 0));
        const std::string score = p.get_string("score", "sigmoid"), on = p.get_string("weight_on", "output");
        if (score != "sigmoid" && score != "softmax") throw SpecError("routed_experts: score is 'sigmoid' or 'softmax', not '" + score + "'");
        if (on != "input" && on != "output") throw SpecError("routed_experts: weight_on is 'input' or 'output', not '" + on + "'");
        score_ = score == "softmax" ? 1 : 0;
        on_input_ = on == "input";
        rule_.renorm = p.get_bool("renormalize", false);
        rule_.renorm_eps = static_cast<float>(p.get_double("renormalize_eps", 0.0));
        rule_.scale = static_cast<float>(p.get_double("route_scale", 1.0));
        if (!p["groups"].is_null()) {
            rule_.groups = static_cast<int>(p["groups"].get_int("count", 1));
            rule_.keep = static_cast<int>(p["groups"].get_int("keep", rule_.groups));
        }
        if (PartSpec::is_part(p["shared"])) shared_ = build_as<FeedForward>("ffn", PartSpec::from_json(p["shared"], "routed_experts.shared"));
        gated_ = p.get_bool("gated", true);
        const std::string act = p.get_string("activation", gated_ ? "silu" : "relu2");
        if (act != (gated_ ? "silu" : "relu2"))
            throw SpecError("routed_experts: activation is 'silu' for gated experts and 'relu2' for experts without a gate, not '" + act + "'");
        if (width_ <= 0 || ff_ <= 0 || experts_ <= 0 || top_ <= 0 || top_ > experts_)
            throw SpecError("routed_experts: width, ff and experts must be positive and top between 1 and experts");
        if (rule_.groups < 1 || rule_.groups > 64 || experts_ % rule_.groups || rule_.keep < 1 || rule_.keep > rule_.groups ||
            top_ > rule_.keep * (experts_ / rule_.groups))
            throw SpecError("routed_experts: groups.count (up to 64) must divide experts, and the groups.keep kept groups must hold at least top experts");
        rule_.top = top_;
        rule_.score = score_;
    }
    bool graph_safe() const override { return !shared_ || shared_->graph_safe(); }
    std::vector<const Part*> children() const override {
        return shared_ ? std::vector<const Part*>{shared_.get()} : std::vector<const Part*>{};
    }
    static std::string role(const char* what, int e) { return std::string(what) + "." + std::to_string(e); }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"router", WeightSpec{{experts_, width_}, "vector", "normal", {}}}};
        for (int e = 0; e < experts_; ++e) {
            if (gated_) specs.push_back({role("gate", e), matrix(ff_, width_)});
            specs.push_back({role("up", e), matrix(ff_, width_)});
            specs.push_back({role("down", e), matrix(width_, ff_)});
        }
        // the shared part's tensors travel under "shared.<its role>"; its checkpoint names are in this part's tensor map
        if (shared_)
            for (const auto& ws : shared_->weight_specs()) specs.push_back({"shared." + ws.first, ws.second});
        return specs;
    }
    void load(const PartTensors& t, Runtime& rt) override {
        router_ = get(t, "router");
        if (shared_) {
            PartTensors mine;
            for (const auto& ws : shared_->weight_specs()) mine[ws.first] = get(t, "shared." + ws.first);
            shared_->load(mine, rt);
        }
        std::vector<std::shared_ptr<DeviceTensor>> in, out;
        for (int e = 0; e < experts_; ++e) {
            if (gated_) in.push_back(get(t, role("gate", e)));
            in.push_back(get(t, role("up", e)));
            out.push_back(get(t, role("down", e)));
        }
        for (const auto& w : in)
            if (w->view.dtype != in[0]->view.dtype) throw SpecError("routed_experts: the experts are stored in different dtypes");
        w_gate_up_ = concat_rows(in);       // [experts * 2 ff, width]: per expert its gate rows, then its up rows (no gate: [experts * ff, width])
        w_down_ = concat_rows(out);         // [experts * width, ff]
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, Runtime& rt) override {
        const long long T = x.shape[0];
        // what every row gets besides its experts (good until the shared part's next call: this part's own
        // result then goes to a buffer of another name than a feed-forward's usual one)
        Tensor base;
        if (shared_) base = shared_->forward(x, batch, rt);
        const bool cores = rt.ops.moe_matrix_cores_ok(x.dtype, ff_, width_) && rt.ops.moe_matrix_cores_ok(x.dtype, width_, ff_) &&
                           w_gate_up_->view.dtype == x.dtype;
        const Ops::RoutePlan plan = rt.ops.moe_route_rows(x, router_->view, rule_, cores, rt.ws);
        Tensor a = rt.ws.buf("moe_in", rt.dtype, {T * top_, width_});
        rt.ops.moe_gather(x, plan, on_input_, a);
        Tensor act = rt.ws.buf("moe_act", rt.dtype, {T * top_, ff_});
        rt.ops.moe_product(a, w_gate_up_->view, act, gated_, plan, gated_ ? 0 : 1);
        Tensor y = rt.ws.buf("moe_y", rt.dtype, {T * top_, width_});
        rt.ops.moe_product(act, w_down_->view, y, false, plan);
        Tensor out = rt.ws.buf(shared_ ? "moe_out" : "ffn_out", rt.dtype, {T, width_});
        rt.ops.moe_combine(y, plan, !on_input_, out, shared_ ? &base : nullptr);
        return out;
    }

private:
    long long width_ = 0, ff_ = 0;
    int experts_ = 0, top_ = 0, score_ = 0;
    bool on_input_ = false, gated_ = true;
    Ops::RouteRule rule_;
    std::unique_ptr<FeedForward> shared_;
    std::shared_ptr<DeviceTensor> router_, w_gate_up_, w_down_;
};

// a layer without a feed-forward (the reference's LayerSpec may hold none,
// src/model/inference/rules.cpp:44-46)
class NoFeedForward final : public FeedForward {
public:
    explicit NoFeedForward(const PartSpec& s) : FeedForward(s) {}
    bool graph_safe() const override { return true; }
    Tensor forward(const Tensor& x, const StepBatch&, Runtime& rt) override { return NoMixer::zeros(rt, x.shape[0], x.shape[1]); }
};

// ---------------------------------------------------------------------------- embedding and heads
// h0[t] = E[token[t]], nothing added and no scaling (src/backend/cpu/model_forward_token.cpp:28-60);
// logits = x E_out^T with E_out = E when the head is tied, else lm_head
// (src/backend/cpu/model_forward_token.cpp:213-218; src/model/inference/layer_bindings.cpp:24-95).
// Logits leave in 32-bit.  "scale" on the embedding multiplies the gathered rows (in 32-bit, as
// they enter the residual stream); "scale" on a head multiplies the logits; "softcap" c > 0 bends them
// afterwards to c * tanh(logit / c).
class TokenEmbedding final : public Embedding {
public:
    explicit TokenEmbedding(const PartSpec& s)
        : Embedding(s), vocab_(s.params.get_int("vocab", 0)), width_(s.params.get_int("width", 0)),
          scale_(static_cast<float>(s.params.get_double("scale", 1.0))) {
        if (vocab_ <= 0 || width_ <= 0) throw SpecError("embedding: vocab and width must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override { return {{"table", matrix(vocab_, width_)}}; }
    void load(const PartTensors& t, Runtime&) override { table_ = get(t, "table"); }
    Tensor table() const override { return table_->view; }
    bool takes_step_prologue() const override { return true; }
    void forward(const int* token_ids, const Tensor& out, Runtime& rt, const StepBatch* batch) override {
        const int rows = static_cast<int>(out.shape[0]);
        if (scale_ != 1.0f) {
            rt.flush_prologue();
            rt.ops.embed(table_->view, token_ids, out, scale_);
            rt.stream_stat_blocks = 0;
            rt.stream_has_bf16 = false;
            return;
        }
        if (batch && table_->view.dtype == DType::BF16 && fused::fused_rows_ok(rt, *batch, {width_})) {
            // few rows: leave every row's sum of squares (and the bfloat16 copy of the stream)
            // for the first norm
            if (fused::sliced(rt, rows, width_) || fused::tiled_step(rt, rows, width_)) {
                // (the step's prologue rides along where it is for these rows)
                const bool along = rt.prologue.pending && rt.prologue.token_ids == token_ids && rt.prologue.n == rows;
                if (!along) rt.flush_prologue();
                rt.ops.embed_stream(table_->view, token_ids, out, fused::stream_bf16(rt, rows, width_),
                                    fused::stream_stats(rt, width_, rows), along ? &rt.prologue : nullptr);
                rt.prologue.pending = false;
                rt.stream_has_bf16 = true;
            } else {
                rt.flush_prologue();
                rt.ops.embed_stats(table_->view, token_ids, out, fused::stream_stats(rt, width_));
                rt.stream_has_bf16 = false;
            }
            rt.stream_stat_blocks = 1;
        } else {
            rt.flush_prologue();
            rt.ops.embed(table_->view, token_ids, out);
        }
    }

private:
    long long vocab_, width_;
    float scale_;
    std::shared_ptr<DeviceTensor> table_;
};

// final norm and output product in one kernel for few wanted rows, 32-bit logits
bool head_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                const Tensor& weight) {
    const int R = batch.n_logit_rows;
    if (!(weight.defined() && weight.dtype == DType::BF16 && fused::fused_rows_ok(rt, batch, {h.shape[1]}) && R > 0 && R <= 64 &&
          !fused::tiled_step(rt, batch.n_tokens, h.shape[1])))
        return false;
    fused::LinearExtras extras;
    extras.rows = batch.logit_rows;
    extras.n_rows = R;
    // beside the logits: the best (logit, index) of every share of a row's columns, from which a
    // greedy row's token follows without the logits being read again
    const int room = Ops::head_best_parts(weight.shape[0]);
    if (rt.ops.use_head_argmax) {
        extras.row_best = static_cast<unsigned long long*>(rt.ws.raw("head_best", static_cast<size_t>(64) * room * sizeof(unsigned long long)));
        extras.row_best_ld = room;     // the parts of a row one after the other (R <= 64 rows)
        extras.row_best_rows = 64;
    }
    fused::norm_linear(rt, h, norm, weight, out, Epilogue::StoreF32, extras);
    if (extras.row_best && rt.ops.last_best_parts > 0) {
        rt.head_best.logits = out.data;
        rt.head_best.best = extras.row_best;
        rt.head_best.ld = extras.row_best_ld;
        rt.head_best.parts = rt.ops.last_best_parts;
        rt.head_best.cols = rt.ops.last_best_cols;
        rt.head_best.rows = R;
    }
    return true;
}

// uses the embedding table; wants no tensor of its own
class TiedHead final : public Head {
public:
    explicit TiedHead(const PartSpec& s)
        : Head(s), vocab_(static_cast<int>(s.params.get_int("vocab", 0))), scale_(static_cast<float>(s.params.get_double("scale", 1.0))),
          softcap_(static_cast<float>(s.params.get_double("softcap", 0.0))) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return vocab_; }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding* embedding) override {
        rt.ops.linear(x, table_of(embedding), out, nullptr, rt.ws);
        if (scale_ != 1.0f) rt.ops.scale(out, scale_);
        if (softcap_ > 0.f) rt.ops.softcap(out, softcap_);
    }
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                       const Embedding* embedding) override {
        if (scale_ != 1.0f || softcap_ > 0.f) return false;       // (what the fused head leaves beside the logits knows no scale)
        return head_fused(h, norm, batch, out, rt, table_of(embedding));
    }

private:
    static Tensor table_of(const Embedding* embedding) {
        const Tensor t = embedding ? embedding->table() : Tensor();
        if (!t.defined()) throw SpecError("tied_head: the model's embedding has no table to share");
        return t;
    }
    int vocab_;
    float scale_, softcap_;
};

class LinearHead final : public Head {
public:
    explicit LinearHead(const PartSpec& s)
        : Head(s), vocab_(static_cast<int>(s.params.get_int("vocab", 0))), width_(s.params.get_int("width", 0)),
          scale_(static_cast<float>(s.params.get_double("scale", 1.0))), softcap_(static_cast<float>(s.params.get_double("softcap", 0.0))) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return vocab_; }
    WeightSpecs weight_specs() const override { return {{"weight", matrix(vocab_, width_)}}; }
    void load(const PartTensors& t, Runtime&) override { weight_ = get(t, "weight"); }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding*) override {
        rt.ops.linear(x, weight_->view, out, nullptr, rt.ws);
        if (scale_ != 1.0f) rt.ops.scale(out, scale_);
        if (softcap_ > 0.f) rt.ops.softcap(out, softcap_);
    }
    bool forward_fused(const Tensor& h, const Norm::Foldable& norm, const StepBatch& batch, const Tensor& out, Runtime& rt,
                       const Embedding*) override {
        if (scale_ != 1.0f || softcap_ > 0.f) return false;
        return head_fused(h, norm, batch, out, rt, weight_->view);
    }

private:
    int vocab_;
    long long width_;
    float scale_, softcap_;
    std::shared_ptr<DeviceTensor> weight_;
};

// "logits" = the (normalised) hidden rows themselves, [rows, width] in 32-bit: what a test of a
// single part reads
class HiddenHead final : public Head {
public:
    explicit HiddenHead(const PartSpec& s) : Head(s), width_(static_cast<int>(s.params.get_int("width", 0))) {}
    bool graph_safe() const override { return true; }
    int vocab() const override { return width_; }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Embedding*) override { rt.ops.cast(x, out); }

private:
    int width_;
};

// ---------------------------------------------------------------------------- the block
// pre_norm: h += mixer(norm1(h)); h += ffn(norm2(h))
// (src/backend/cpu/model_forward_token.cpp:93-172).  The residual stream h is 32-bit in every
// mode and each sum into it is made in 32-bit; an addition is carried forward as delta and made
// by the next norm's kernel, which reads h anyway.
class PreNormBlock final : public Block {
public:
    explicit PreNormBlock(const LayerSpec& layer)
        : mixer_norm_(build_as<Norm>("norm", layer.mixer_norm)), mixer_(build_as<Mixer>("mixer", layer.mixer)),
          ffn_norm_(build_as<Norm>("norm", layer.ffn_norm)), ffn_(build_as<FeedForward>("ffn", layer.ffn)) {}
    std::vector<std::pair<std::string, Part*>> parts() override {
        return {{"mixer_norm", mixer_norm_.get()}, {"mixer", mixer_.get()}, {"ffn_norm", ffn_norm_.get()}, {"ffn", ffn_.get()}};
    }
    Mixer& mixer() override { return *mixer_; }
    Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = h.shape[0], width = h.shape[1];
        Tensor normed = rt.ws.buf("normed", rt.dtype, {T, width});
        // Few rows: parts that can, take the norm in front of them and the addition behind them
        // into their own products and write the stream themselves.
        const Norm::Foldable* fold1 = mixer_norm_->foldable();
        const Norm::Foldable* fold2 = ffn_norm_->foldable();
        const bool fusable = fold1 && fold2;
        Tensor mixed;
        if (fusable && !delta.defined() && mixer_->forward_fused(h, *fold1, batch, cache, rt)) {
            // the stream holds the mixer's sum already
        } else {
            rt.stream_stat_blocks = 0;
            mixer_norm_->forward(h, normed, rt, delta.defined() ? &delta : nullptr, nullptr);
            mixed = mixer_->forward(normed, batch, cache, rt);
        }
        rt.mark("mixer " + mixer_->spec.kind);
        if (fusable && !mixed.defined() && ffn_->forward_fused(h, *fold2, batch, rt)) {
            rt.mark("ffn " + ffn_->spec.kind);
            return Tensor();
        }
        rt.stream_stat_blocks = 0;
        ffn_norm_->forward(h, normed, rt, mixed.defined() ? &mixed : nullptr, nullptr);
        Tensor out = ffn_->forward(normed, batch, rt);
        rt.mark("ffn " + ffn_->spec.kind);
        return out;
    }

private:
    std::unique_ptr<Norm> mixer_norm_;
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<Norm> ffn_norm_;
    std::unique_ptr<FeedForward> ffn_;
};

// ---------------------------------------------------------------------------- several residual streams
// How one sub-layer hangs on a row's S residual streams: it reads sum_s in[s] x_s, and its
// output y comes back as x_t <- sum_s mix[s, t] x_s + out[t] y (mix indexed [from, to]).
class HyperLink final : public Part {
public:
    explicit HyperLink(const PartSpec& s) : Part(s), streams_(static_cast<int>(s.params.get_int("streams", 0))) {
        if (streams_ <= 0 || streams_ > 8) throw SpecError("hyper_link: between 1 and 8 streams");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        return {{"in", vec(streams_, "around_one")}, {"out", vec(streams_, "around_one")},
                {"mix", WeightSpec{{streams_, streams_}, "vector", "around_identity", {}}}};
    }
    void load(const PartTensors& t, Runtime&) override {
        in = get(t, "in");
        out = get(t, "out");
        mix = get(t, "mix");
    }
    int streams() const { return streams_; }
    std::shared_ptr<DeviceTensor> in, out, mix;

private:
    int streams_;
};

// hyper_connections: the pre-norm order of work on S streams h [T, S * width].  A kernel at each
// sub-layer boundary writes the previous output back into the streams, mixes the next input and
// normalises it.  A sub-layer of kind "none" is left out altogether.
class HyperBlock final : public Block {
public:
    explicit HyperBlock(const LayerSpec& layer)
        : mixer_norm_(build_as<Norm>("norm", layer.mixer_norm)), mixer_(build_as<Mixer>("mixer", layer.mixer)),
          mixer_link_(build_as<HyperLink>("link", layer.mixer_link)), has_ffn_(layer.ffn.kind != "none") {
        if (has_ffn_) {
            ffn_norm_ = build_as<Norm>("norm", layer.ffn_norm);
            ffn_ = build_as<FeedForward>("ffn", layer.ffn);
            ffn_link_ = build_as<HyperLink>("link", layer.ffn_link);
            if (ffn_link_->streams() != mixer_link_->streams()) throw SpecError("hyper_connections: the links of a layer differ in streams");
        }
    }
    std::vector<std::pair<std::string, Part*>> parts() override {
        std::vector<std::pair<std::string, Part*>> out{{"mixer_norm", mixer_norm_.get()}, {"mixer", mixer_.get()}, {"mixer_link", mixer_link_.get()}};
        if (has_ffn_) {
            out.emplace_back("ffn_norm", ffn_norm_.get());
            out.emplace_back("ffn", ffn_.get());
            out.emplace_back("ffn_link", ffn_link_.get());
        }
        return out;
    }
    Mixer& mixer() override { return *mixer_; }
    int streams() const override { return mixer_link_->streams(); }
    Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const int S = streams();
        if (delta.defined()) throw SpecError("hyper_connections: a pending addition from a block of another arrangement");
        if (h.shape[1] % S) throw SpecError("hyper_connections: the rows do not hold a whole number of streams");
        const long long T = h.shape[0], width = h.shape[1] / S;
        rt.stream_stat_blocks = 0;
        rt.stream_has_bf16 = false;
        Tensor normed = rt.ws.buf("normed", rt.dtype, {T, width});
        read(h, S, nullptr, nullptr, *mixer_link_, *mixer_norm_, normed, rt);
        Tensor y = mixer_->forward(normed, batch, cache, rt);
        rt.mark("mixer " + mixer_->spec.kind);
        const HyperLink* pending = mixer_link_.get();
        if (has_ffn_) {
            read(h, S, &y, pending, *ffn_link_, *ffn_norm_, normed, rt);
            y = ffn_->forward(normed, batch, rt);
            rt.mark("ffn " + ffn_->spec.kind);
            pending = ffn_link_.get();
        }
        rt.ops.hyper_step(h, S, &y, &pending->mix->view, &pending->out->view, nullptr, nullptr, 0.f, nullptr);
        return Tensor();
    }

private:
    // writes y back through `from` (if given), then normed = norm(sum_s in[s] x_s)
    static void read(const Tensor& h, int S, const Tensor* y, const HyperLink* from, const HyperLink& to, Norm& norm,
                     const Tensor& normed, Runtime& rt) {
        const Norm::Foldable* fold = norm.foldable();
        const Tensor* mix = from ? &from->mix->view : nullptr;
        const Tensor* out = from ? &from->out->view : nullptr;
        if (fold) {
            rt.ops.hyper_step(h, S, y, mix, out, &to.in->view, &fold->weight, fold->eps, &normed);
            return;
        }
        // a norm that is not an RMS norm: the mixture leaves in 32-bit and the norm runs by itself
        Tensor u = rt.ws.buf("hyper_mixture", DType::F32, {normed.shape[0], normed.shape[1]});
        rt.ops.hyper_step(h, S, y, mix, out, &to.in->view, nullptr, 0.f, &u);
        norm.forward(u, normed, rt, nullptr, nullptr);
    }
    std::unique_ptr<Norm> mixer_norm_;
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<HyperLink> mixer_link_;
    bool has_ffn_;
    std::unique_ptr<Norm> ffn_norm_;
    std::unique_ptr<FeedForward> ffn_;
    std::unique_ptr<HyperLink> ffn_link_;
};

// ---------------------------------------------------------------------------- layer norm
// y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations from the
// mean, eps inside the root; statistics and scaling in 32-bit.  "bias": false leaves b out.
class LayerNorm final : public Norm {
public:
    explicit LayerNorm(const PartSpec& s)
        : Norm(s), width_(s.params.get_int("width", 0)), eps_(s.params.get_double("eps", 0.0)), bias_(s.params.get_bool("bias", true)) {
        if (width_ <= 0 || !(eps_ > 0)) throw SpecError("layernorm: width and eps must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"weight", vec(width_, "around_one")}};
        if (bias_) specs.push_back({"bias", vec(width_)});
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        weight_ = get(t, "weight");
        if (bias_) b_ = get(t, "bias");
        params_.weight = weight_->view;
        if (b_) params_.bias = b_->view;
        params_.eps = static_cast<float>(eps_);
        params_.centered = true;
    }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        if (x.dtype != DType::F32) throw SpecError("layernorm: the rows to normalise must be 32-bit");
        rt.ops.norm_step(x, delta, nullptr, &params_, &out, rows);
    }
    const Ops::NormParams* params() const override { return weight_ ? &params_ : nullptr; }

private:
    long long width_;
    double eps_;
    bool bias_;
    std::shared_ptr<DeviceTensor> weight_, b_;
    Ops::NormParams params_;
};

// ---------------------------------------------------------------------------- dynamic tanh
// y = tanh(alpha * x) * w + b: a "norm" without any statistic of the row; alpha is one learned number
// stored beside the weight.  32-bit whatever the activation dtype.  "bias": false leaves b out.
class DynamicTanh final : public Norm {
public:
    explicit DynamicTanh(const PartSpec& s) : Norm(s), width_(s.params.get_int("width", 0)), bias_(s.params.get_bool("bias", true)) {
        if (width_ <= 0) throw SpecError("dynamic_tanh: width must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"weight", vec(width_, "around_one")}, {"alpha", WeightSpec{{}, "vector", "around_one", {{1}}}}};
        if (bias_) specs.push_back({"bias", vec(width_)});
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        weight_ = get(t, "weight");
        if (bias_) b_ = get(t, "bias");
        const std::vector<float> alpha = to_host_floats(get(t, "alpha")->view);
        if (alpha.size() != 1) throw SpecError("dynamic_tanh: alpha is one number");
        params_.weight = weight_->view;
        if (b_) params_.bias = b_->view;
        params_.alpha = alpha[0];
        params_.tanh = true;
    }
    void forward(const Tensor& x, const Tensor& out, Runtime& rt, const Tensor* delta, const int* rows) override {
        if (x.dtype != DType::F32) throw SpecError("dynamic_tanh: the rows to norm must be 32-bit");
        rt.ops.norm_step(x, delta, nullptr, &params_, &out, rows);
    }
    const Ops::NormParams* params() const override { return weight_ ? &params_ : nullptr; }

private:
    long long width_;
    bool bias_;
    std::shared_ptr<DeviceTensor> weight_, b_;
    Ops::NormParams params_;
};

// ---------------------------------------------------------------------------- attention with sigmoid weights
// Grouped-query attention whose weights are sigmoids of the scores instead of a softmax over them.
//
// q = W_q h (+ b_q), k = W_k h (+ b_k); the values are the keys as projected, before norm and
// rotation ("values": "keys"; there is then no value projection), or v = W_v h ("values":
// "projected").  RMS norm of every q and k head over head_dim with one weight for all heads
// ("qk_norm"), then the position encoding of q and k.  The weight of key j for query i of head
// h, j inside the window [i - window + 1, i] (or all j <= i without one), is
//     sigmoid((q_i . k_j) * scale * temp[h] + pb[h])
// ("temperature" and "score_bias": a learned number per head each), not normalised over the
// keys.  With "head_gate" the head's result is multiplied by sigmoid(W_g h)[h], one number per
// head from the mixer's own input.  The heads, side by side, go through W_o.
class SigmoidAttention final : public Mixer {
public:
    explicit SigmoidAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        heads_ = static_cast<int>(p.get_int("heads", 0));
        kv_heads_ = static_cast<int>(p.get_int("kv_heads", heads_));
        head_dim_ = static_cast<int>(p.get_int("head_dim", 0));
        qk_norm_ = p.get_bool("qk_norm", false);
        bias_ = p.get_bool("bias", false);
        temperature_ = p.get_bool("temperature", false);
        score_bias_ = p.get_bool("score_bias", false);
        head_gate_ = p.get_bool("head_gate", false);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        const std::string values = p.get_string("values", "projected");
        if (values != "keys" && values != "projected") throw SpecError("sigmoid_attention: values is 'keys' or 'projected', not '" + values + "'");
        values_are_keys_ = values == "keys";
        if (!p["window"].is_null()) {
            window_ = static_cast<int>(p["window"].as_int());
            if (*window_ <= 0) throw SpecError("sigmoid_attention: window must be positive");
        }
        if (width_ <= 0 || heads_ <= 0 || kv_heads_ <= 0 || heads_ % kv_heads_)
            throw SpecError("sigmoid_attention: heads must be a positive multiple of kv_heads");
        if (head_dim_ <= 0 || head_dim_ % 2) throw SpecError("sigmoid_attention: head_dim must be even");
        scale_ = p["scale"].is_null() ? static_cast<float>(1.0 / std::sqrt(static_cast<double>(head_dim_)))
                                      : static_cast<float>(p["scale"].as_double());
        PartSpec none;
        none.kind = "none";
        position_ = build_as<PositionEncoding>(
            "position", PartSpec::is_part(p["position"]) ? PartSpec::from_json(p["position"], "sigmoid_attention.position") : none);
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override { return {position_.get()}; }
    std::optional<KVNeed> kv_need() const override { return KVNeed{kv_heads_, head_dim_, window_}; }
    WeightSpecs weight_specs() const override {
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        WeightSpecs specs{{"q", matrix(qw, width_)}, {"k", matrix(kvw, width_)}, {"o", matrix(width_, qw)}};
        if (!values_are_keys_) specs.push_back({"v", matrix(kvw, width_)});
        if (bias_) {
            specs.push_back({"q_bias", vec(qw)});
            specs.push_back({"k_bias", vec(kvw)});
        }
        if (qk_norm_) {
            specs.push_back({"q_norm", vec(head_dim_, "around_one")});
            specs.push_back({"k_norm", vec(head_dim_, "around_one")});
        }
        if (temperature_) specs.push_back({"temp", vec(heads_, "around_one")});
        if (score_bias_) specs.push_back({"pb", vec(heads_)});
        if (head_gate_) specs.push_back({"g", matrix(heads_, width_)});
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        // every projection of the mixer's input in one product; the gate's few rows are padded with
        // zero rows to a multiple of 16 columns
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        std::vector<std::shared_ptr<DeviceTensor>> in{get(t, "q"), get(t, "k")};
        if (!values_are_keys_) in.push_back(get(t, "v"));
        gate_col_ = qw + kvw * (values_are_keys_ ? 1 : 2);
        long long cols = gate_col_;
        if (head_gate_) {
            in.push_back(get(t, "g"));
            const long long pad = (16 - heads_ % 16) % 16;
            if (pad) in.push_back(from_host_floats(std::vector<float>(static_cast<size_t>(pad * width_), 0.f), in[0]->view.dtype, {pad, width_}));
            cols += heads_ + pad;
        }
        for (const auto& w : in)
            if (w->view.dtype != in[0]->view.dtype) throw SpecError("sigmoid_attention: the input projections are stored in different dtypes");
        w_in_ = concat_rows(in);
        if (bias_) {
            std::vector<float> b = to_host_floats(get(t, "q_bias")->view), kb = to_host_floats(get(t, "k_bias")->view);
            b.insert(b.end(), kb.begin(), kb.end());
            b.resize(static_cast<size_t>(cols), 0.f);
            b_in_ = from_host_floats(b, DType::F32, {cols});
        }
        w_o_ = get(t, "o");
        q_norm_ = maybe(t, "q_norm");
        k_norm_ = maybe(t, "k_norm");
        temp_ = maybe(t, "temp");
        pb_ = maybe(t, "pb");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        if (!cache.kv) throw SpecError("sigmoid_attention: the cache has no keys and values for this layer");
        if (!cache.writes_kv) throw SpecError("sigmoid_attention: reading another entry's cache is not supported");
        const long long T = x.shape[0];
        const long long qw = static_cast<long long>(heads_) * head_dim_, kvw = static_cast<long long>(kv_heads_) * head_dim_;
        Tensor proj = rt.ws.buf("sattn_proj", rt.dtype, {T, w_in_->view.shape[0]});
        rt.ops.linear(x, w_in_->view, proj, b_in_ ? &b_in_->view : nullptr, rt.ws);
        Tensor q = proj.cols(0, qw), k = proj.cols(qw, kvw);
        Tensor v = values_are_keys_ ? k : proj.cols(qw + kvw, kvw);
        Tensor gate = head_gate_ ? proj.cols(gate_col_, heads_) : Tensor();
        const PositionEncoding::Tables tables = position_->tables(rt);
        const Tensor* inv_freq = tables.inv_freq.defined() ? &tables.inv_freq : nullptr;
        // (q is normed and turned in place; the keys go to their pages normed and turned, the values as they are)
        rt.ops.qk_norm_rope_store(q, &k, &v, q_norm_ ? &q_norm_->view : nullptr, k_norm_ ? &k_norm_->view : nullptr, eps_, inv_freq,
                                  tables.rotary_dim, tables.pairing, heads_, kv_heads_, head_dim_, batch, *cache.kv);
        Tensor attended = rt.ws.buf("sattn_out", rt.dtype, {T, qw});
        rt.ops.sigmoid_attention(q, attended, heads_, kv_heads_, head_dim_, scale_, window_ ? *window_ : 0,
                                 temp_ ? &temp_->view : nullptr, pb_ ? &pb_->view : nullptr, head_gate_ ? &gate : nullptr, batch,
                                 *cache.kv, rt.ws);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(attended, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0, gate_col_ = 0;
    int heads_ = 0, kv_heads_ = 0, head_dim_ = 0;
    bool qk_norm_ = false, bias_ = false, temperature_ = false, score_bias_ = false, head_gate_ = false, values_are_keys_ = false;
    float eps_ = 1e-6f, scale_ = 1.f;
    std::optional<int> window_;
    std::unique_ptr<PositionEncoding> position_;
    std::shared_ptr<DeviceTensor> w_in_, b_in_, w_o_, q_norm_, k_norm_, temp_, pb_;
};

// ---------------------------------------------------------------------------- projections side by side
// The matrices of several projections of one input, one under the other, so that one product
// makes them all.  A piece that a later product reads as its input starts at a multiple of 16
// rows (zero rows in front of it); the whole is padded to a multiple of 16 rows.
struct Stacked {
    std::shared_ptr<DeviceTensor> weight;
    std::vector<long long> at;        // the first row of every piece
    long long rows = 0;
};
Stacked stack_projections(const std::vector<std::pair<std::shared_ptr<DeviceTensor>, bool>>& pieces, const char* who) {
    Stacked out;
    std::vector<std::shared_ptr<DeviceTensor>> parts;
    const DType dtype = pieces.at(0).first->view.dtype;
    const long long width = pieces.at(0).first->view.shape[1];
    auto pad_to_16 = [&]() {
        const long long pad = (16 - out.rows % 16) % 16;
        if (pad) parts.push_back(from_host_floats(std::vector<float>(static_cast<size_t>(pad * width), 0.f), dtype, {pad, width}));
        out.rows += pad;
    };
    for (const auto& piece : pieces) {
        const Tensor& v = piece.first->view;
        if (v.dtype != dtype || v.ndim != 2 || v.shape[1] != width)
            throw SpecError(std::string(who) + ": the input projections differ in dtype or inner size");
        if (piece.second) pad_to_16();
        out.at.push_back(out.rows);
        parts.push_back(piece.first);
        out.rows += v.shape[0];
    }
    pad_to_16();
    out.weight = concat_rows(parts);
    return out;
}

// ---------------------------------------------------------------------------- gated delta rule
// A recurrent mixer with a matrix of state per head.
//
// q = W_q h and k = W_k h (kv_heads heads of dim), v = W_v h (heads of vdim; value head i uses
// query/key head i / (heads / kv_heads)); each channel of q, k and v passes a short causal
// convolution over time (taps [channels, taps], the last tap the current token's, zeros before
// the sequence starts) and silu; q and k become unit vectors per head
// (x / sqrt(sum x^2 + 1e-6)), q times dim^-1/2.  beta = sigmoid(W_b h), one per value head.
// The decay is exp(-exp(A_log[head]) softplus(z + dt_bias)) with "decay": "head" (one per value
// head, z = W_a h, dt_bias [heads]) or "channel" (one per value head and key channel, acting on
// the rows of S; z and dt_bias [heads * dim]).  "decay_rank" r > 0: z = W_a2 (W_a1 h) through r
// values (tensors a1, a2 instead of a).  Per head and token
//     S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// so the read-out sees the token's own write.  o is RMS-normed per head over vdim (weight
// [vdim] shared by the heads) and multiplied by act(W_g h), "gate": "silu" or "sigmoid";
// "gate_rank" r > 0: W_g2 (W_g1 h) (tensors g1, g2 instead of g).  The heads go through W_o.
//
// State per request: S [heads, dim, vdim] and the last taps - 1 inputs of the convolutions
// [taps - 1, channels], both 32-bit.  Everything from the convolutions' sums to the gated norm
// is 32-bit in both dtypes.
class GatedDeltaRule final : public Mixer {
public:
    explicit GatedDeltaRule(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        shape_.heads = static_cast<int>(p.get_int("heads", 0));
        shape_.kv_heads = static_cast<int>(p.get_int("kv_heads", shape_.heads));
        shape_.dim = static_cast<int>(p.get_int("dim", 0));
        shape_.vdim = static_cast<int>(p.get_int("vdim", shape_.dim));
        shape_.taps = static_cast<int>(p.get_int("taps", 0));
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        const std::string decay = p.get_string("decay", "head"), gate = p.get_string("gate", "silu");
        if (decay != "head" && decay != "channel") throw SpecError("gated_delta_rule: decay is 'head' or 'channel', not '" + decay + "'");
        if (gate != "silu" && gate != "sigmoid") throw SpecError("gated_delta_rule: gate is 'silu' or 'sigmoid', not '" + gate + "'");
        per_channel_ = decay == "channel";
        gate_act_ = gate == "sigmoid" ? 1 : 0;
        decay_rank_ = p.get_int("decay_rank", 0);
        gate_rank_ = p.get_int("gate_rank", 0);
        if (width_ <= 0 || shape_.heads <= 0 || shape_.kv_heads <= 0 || shape_.heads % shape_.kv_heads)
            throw SpecError("gated_delta_rule: heads must be a positive multiple of kv_heads");
        if (shape_.dim <= 0 || shape_.vdim <= 0 || shape_.taps <= 0) throw SpecError("gated_delta_rule: dim, vdim and taps must be positive");
        if (decay_rank_ < 0 || gate_rank_ < 0) throw SpecError("gated_delta_rule: decay_rank and gate_rank are not negative");
        if (decay_rank_ > 0 && !per_channel_) throw SpecError("gated_delta_rule: decay_rank goes with decay 'channel'");
    }
    bool graph_safe() const override { return true; }
    long long qk_width() const { return static_cast<long long>(shape_.kv_heads) * shape_.dim; }
    long long v_width() const { return static_cast<long long>(shape_.heads) * shape_.vdim; }
    long long channels() const { return 2 * qk_width() + v_width(); }
    long long decay_width() const { return per_channel_ ? static_cast<long long>(shape_.heads) * shape_.dim : shape_.heads; }
    std::vector<StateNeed> state_needs() const override {
        return {StateNeed{"S", {shape_.heads, shape_.dim, shape_.vdim}, DType::F32},
                StateNeed{"conv", {std::max(shape_.taps - 1, 1), channels()}, DType::F32}};
    }
    WeightSpecs weight_specs() const override {
        auto taps = [&](long long n) { return WeightSpec{{n, shape_.taps}, "vector", "normal", {}}; };
        WeightSpecs specs{{"q", matrix(qk_width(), width_)}, {"k", matrix(qk_width(), width_)}, {"v", matrix(v_width(), width_)},
                          {"q_conv", taps(qk_width())},      {"k_conv", taps(qk_width())},      {"v_conv", taps(v_width())},
                          {"b", matrix(shape_.heads, width_)}, {"A_log", vec(shape_.heads)},    {"dt_bias", vec(decay_width())},
                          {"norm", vec(shape_.vdim, "around_one")}, {"o", matrix(width_, v_width())}};
        if (decay_rank_ > 0) {
            specs.push_back({"a1", matrix(decay_rank_, width_)});
            specs.push_back({"a2", matrix(decay_width(), decay_rank_)});
        } else {
            specs.push_back({"a", matrix(decay_width(), width_)});
        }
        if (gate_rank_ > 0) {
            specs.push_back({"g1", matrix(gate_rank_, width_)});
            specs.push_back({"g2", matrix(v_width(), gate_rank_)});
        } else {
            specs.push_back({"g", matrix(v_width(), width_)});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        // one product for everything that reads the mixer's input: q | k | v | gate | b | a (| zero rows)
        const Stacked in = stack_projections({{get(t, "q"), false}, {get(t, "k"), false}, {get(t, "v"), false},
                                              {get(t, gate_rank_ > 0 ? "g1" : "g"), gate_rank_ > 0}, {get(t, "b"), false},
                                              {get(t, decay_rank_ > 0 ? "a1" : "a"), decay_rank_ > 0}}, "gated_delta_rule");
        w_in_ = in.weight;
        col_gate_ = in.at[3];
        col_b_ = in.at[4];
        col_a_ = in.at[5];
        conv_w_ = concat_rows({get(t, "q_conv"), get(t, "k_conv"), get(t, "v_conv")});
        a_log_ = get(t, "A_log");
        dt_bias_ = get(t, "dt_bias");
        norm_ = get(t, "norm");
        w_o_ = get(t, "o");
        a2_ = maybe(t, "a2");
        g2_ = maybe(t, "g2");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor proj = rt.ws.buf("delta_proj", rt.dtype, {T, w_in_->view.shape[0]});
        rt.ops.linear(x, w_in_->view, proj, nullptr, rt.ws);
        Tensor qk = rt.ws.buf("delta_qk", DType::F32, {T, 2 * qk_width()});
        Tensor v = rt.ws.buf("delta_v", DType::F32, {T, v_width()});
        Tensor beta_decay = rt.ws.buf("delta_beta_decay", DType::F32, {T, 2LL * shape_.heads});
        Tensor o = rt.ws.buf("delta_o", DType::F32, {T, v_width()});
        if (!per_channel_) {
            rt.ops.delta_prepare(proj, static_cast<int>(col_b_), static_cast<int>(col_a_), shape_, conv_w_->view, a_log_->view,
                                 dt_bias_->view, cache.states.at("conv"), qk, v, beta_decay, batch);
            rt.ops.delta_scan(qk, v, beta_decay, cache.states.at("S"), o, shape_, batch, rt.ws);
        } else {
            Tensor z = proj.cols(col_a_, decay_width());
            if (decay_rank_ > 0) {
                z = rt.ws.buf("delta_decay_in", rt.dtype, {T, decay_width()});
                rt.ops.linear(proj.cols(col_a_, decay_rank_), a2_->view, z, nullptr, rt.ws);
            }
            Tensor decay = rt.ws.buf("delta_decay", DType::F32, {T, decay_width()});
            rt.ops.channel_decay(z, a_log_->view, dt_bias_->view, decay, shape_.heads, shape_.dim);
            rt.ops.delta_prepare(proj, static_cast<int>(col_b_), static_cast<int>(col_b_), shape_, conv_w_->view, Tensor(), Tensor(),
                                 cache.states.at("conv"), qk, v, beta_decay, batch);
            rt.ops.channel_scan(qk, v, decay, beta_decay.as<float>(), 2 * shape_.heads, cache.states.at("S"), o, shape_, batch);
        }
        Tensor gate = proj.cols(col_gate_, v_width());
        if (gate_rank_ > 0) {
            gate = rt.ws.buf("delta_gate", rt.dtype, {T, v_width()});
            rt.ops.linear(proj.cols(col_gate_, gate_rank_), g2_->view, gate, nullptr, rt.ws);
        }
        Tensor gated = rt.ws.buf("delta_gated", rt.dtype, {T, v_width()});
        rt.ops.delta_gated_norm(o, norm_->view, gate, eps_, gated, shape_.heads, shape_.vdim, gate_act_);
        Tensor out = rt.ws.buf("mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(gated, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0, col_gate_ = 0, col_b_ = 0, col_a_ = 0, decay_rank_ = 0, gate_rank_ = 0;
    Ops::DeltaShape shape_;
    float eps_ = 1e-6f;
    bool per_channel_ = false;
    int gate_act_ = 0;
    std::shared_ptr<DeviceTensor> w_in_, conv_w_, a_log_, dt_bias_, norm_, w_o_, a2_, g2_;
};

// ---------------------------------------------------------------------------- the embedding's rows, again
// linear_concat: h <- W [h ; x0], W [width, 2 * width] with the stream's columns first.
class LinearReinjection final : public Reinjection {
public:
    explicit LinearReinjection(const PartSpec& s) : Reinjection(s), width_(s.params.get_int("width", 0)) {
        if (width_ <= 0) throw SpecError("linear_concat: width must be positive");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override { return {{"weight", matrix(width_, 2 * width_)}}; }
    void load(const PartTensors& t, Runtime&) override { weight_ = get(t, "weight"); }
    void forward(const Tensor& h, const Tensor& x0, Runtime& rt, int) override {
        const long long T = h.shape[0];
        Tensor both = rt.ws.buf("reinjection_in", rt.dtype, {T, 2 * width_});
        rt.ops.concat_rows(h, x0, both);
        rt.ops.linear(both, weight_->view, h, nullptr, rt.ws);      // (h was copied: the product may write it)
    }

private:
    long long width_;
    std::shared_ptr<DeviceTensor> weight_;
};

// add_rows: before run t of the looped range, h <- h + (x0 if t >= "embedding_from") + step[t]; step
// [times, width] holds a learned vector per run ("steps": false: no such tensor).  All 32-bit.
class AdditiveReinjection final : public Reinjection {
public:
    explicit AdditiveReinjection(const PartSpec& s)
        : Reinjection(s), width_(s.params.get_int("width", 0)), times_(s.params.get_int("times", 1)),
          from_(s.params.get_int("embedding_from", 1)), steps_(s.params.get_bool("steps", true)) {
        if (width_ <= 0 || times_ <= 0 || from_ < 0) throw SpecError("add_rows: width and times must be positive, embedding_from not negative");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        if (!steps_) return {};
        return {{"step", WeightSpec{{times_, width_}, "vector", "normal", {}}}};
    }
    void load(const PartTensors& t, Runtime&) override {
        if (steps_) step_ = get(t, "step");
    }
    void forward(const Tensor& h, const Tensor& x0, Runtime& rt, int pass) override {
        if (pass < 0 || pass >= times_) throw SpecError("add_rows: run " + std::to_string(pass) + " of " + std::to_string(times_));
        Tensor vec;
        if (steps_) vec = Tensor::make(step_->view.as<float>() + static_cast<size_t>(pass) * static_cast<size_t>(width_), DType::F32, {width_});
        rt.ops.stream_add(h, pass >= from_ ? &x0 : nullptr, steps_ ? &vec : nullptr);
    }

private:
    long long width_, times_, from_;
    bool steps_;
    std::shared_ptr<DeviceTensor> step_;
};

// ---------------------------------------------------------------------------- norms before and after
// sandwich_norm: h += post1(mixer(pre1(h))); h += post2(ffn(pre2(h))).  The stream is 32-bit
// and so are the norms' statistics and the sums.  One kernel per boundary: the first norms the
// stream, the second adds the mixer's normed output and norms for the feed-forward, the third
// adds the feed-forward's normed output.  A feed-forward of kind "none" is left out with its norms.
// The layer's "residual_scale" m makes the sums h += m * post(...).
class SandwichBlock final : public Block {
public:
    explicit SandwichBlock(const LayerSpec& layer)
        : mixer_norm_(build_as<Norm>("norm", layer.mixer_norm)), mixer_(build_as<Mixer>("mixer", layer.mixer)),
          mixer_post_(build_as<Norm>("norm", layer.mixer_post_norm)), has_ffn_(layer.ffn.kind != "none"),
          gain_(static_cast<float>(layer.residual_scale)) {
        if (has_ffn_) {
            ffn_norm_ = build_as<Norm>("norm", layer.ffn_norm);
            ffn_ = build_as<FeedForward>("ffn", layer.ffn);
            ffn_post_ = build_as<Norm>("norm", layer.ffn_post_norm);
        }
    }
    std::vector<std::pair<std::string, Part*>> parts() override {
        std::vector<std::pair<std::string, Part*>> out{{"mixer_norm", mixer_norm_.get()}, {"mixer", mixer_.get()}, {"mixer_post_norm", mixer_post_.get()}};
        if (has_ffn_) {
            out.emplace_back("ffn_norm", ffn_norm_.get());
            out.emplace_back("ffn", ffn_.get());
            out.emplace_back("ffn_post_norm", ffn_post_.get());
        }
        return out;
    }
    Mixer& mixer() override { return *mixer_; }
    Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = h.shape[0], width = h.shape[1];
        rt.stream_stat_blocks = 0;
        rt.stream_has_bf16 = false;
        Tensor normed = rt.ws.buf("normed", rt.dtype, {T, width});
        rt.ops.norm_step(h, delta.defined() ? &delta : nullptr, nullptr, &of(*mixer_norm_), &normed);
        Tensor y = mixer_->forward(normed, batch, cache, rt);
        rt.mark("mixer " + mixer_->spec.kind);
        if (!has_ffn_) {
            rt.ops.norm_step(h, &y, &of(*mixer_post_), nullptr, nullptr, nullptr, gain_);
            return Tensor();
        }
        rt.ops.norm_step(h, &y, &of(*mixer_post_), &of(*ffn_norm_), &normed, nullptr, gain_);
        y = ffn_->forward(normed, batch, rt);
        rt.ops.norm_step(h, &y, &of(*ffn_post_), nullptr, nullptr, nullptr, gain_);
        rt.mark("ffn " + ffn_->spec.kind);
        return Tensor();
    }

private:
    static const Ops::NormParams& of(const Norm& norm) {
        const Ops::NormParams* p = norm.params();
        if (!p) throw SpecError("sandwich_norm: norm '" + norm.spec.kind + "' cannot be taken into the boundary kernels");
        return *p;
    }
    std::unique_ptr<Norm> mixer_norm_;
    std::unique_ptr<Mixer> mixer_;
    std::unique_ptr<Norm> mixer_post_;
    bool has_ffn_;
    float gain_ = 1.f;
    std::unique_ptr<Norm> ffn_norm_;
    std::unique_ptr<FeedForward> ffn_;
    std::unique_ptr<Norm> ffn_post_;
};

// ---------------------------------------------------------------------------- attention with a distance bias
// Grouped-query softmax attention whose options are parameters: positions enter through the scores (a factor on
// the query, a distance bias) or, with a "position" part, through a rotation of q and k.
//
// q = W_q h, k = W_k h (head_dim a head), v = W_v h ("v_dim" a head, which may differ from head_dim).
// score(i, j) = (q_i . k_j) * scale * f(i) - r1[h] ln(1 + r2[h] (i - j)) with
// f(i) = 1 + coef ln(floor((i + 1) / every) + 1) ("query_temperature": {"coef", "every"}; absent: f = 1) and,
// with "distance_bias", a learned pair (r1, r2) per query head.  Keys j <= i (inside "window" where one is
// given; with "keep_first" n the first n positions of the sequence stay visible behind the window, at their
// true positions).  "gate": "sigmoid" multiplies the heads, side by side, element by element with sigmoid(W_g h).
// "sink_one": the softmax's denominator holds a one more, p_j = exp(s_j) / (1 + sum exp(s_j)).
// "taps" n > 0: every channel of q, k and v passes a causal convolution over time of n taps right behind its
// projection (tensors q_conv, k_conv, v_conv [channels, taps], no bias; y_t = sum_j w[:, j] u_(t - n + 1 + j),
// zeros before the sequence starts); the last n - 1 projected rows are the request's state.  "position": a
// position encoding part (rope) that turns q and k heads behind the convolution.
class BiasedAttention final : public Mixer {
public:
    explicit BiasedAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        shape_.heads = static_cast<int>(p.get_int("heads", 0));
        shape_.kv_heads = static_cast<int>(p.get_int("kv_heads", shape_.heads));
        shape_.head_dim = static_cast<int>(p.get_int("head_dim", 0));
        shape_.v_dim = static_cast<int>(p.get_int("v_dim", shape_.head_dim));
        if (width_ <= 0 || shape_.heads <= 0 || shape_.kv_heads <= 0 || shape_.heads % shape_.kv_heads)
            throw SpecError("biased_attention: heads must be a positive multiple of kv_heads");
        if (shape_.head_dim <= 0 || shape_.v_dim <= 0) throw SpecError("biased_attention: head_dim and v_dim must be positive");
        shape_.scale = p["scale"].is_null() ? static_cast<float>(1.0 / std::sqrt(static_cast<double>(shape_.head_dim)))
                                            : static_cast<float>(p["scale"].as_double());
        if (!p["window"].is_null()) {
            shape_.window = static_cast<int>(p["window"].as_int());
            if (shape_.window <= 0) throw SpecError("biased_attention: window must be positive");
        }
        if (!p["query_temperature"].is_null()) {
            const Json& t = p["query_temperature"];
            shape_.coef = static_cast<float>(t.get_double("coef", 0.0));
            shape_.every = static_cast<int>(t.get_int("every", 0));
            if (shape_.every <= 0) throw SpecError("biased_attention: query_temperature.every must be positive");
        }
        if (!p["keep_first"].is_null()) {
            shape_.keep_first = static_cast<int>(p["keep_first"].as_int());
            if (shape_.keep_first < 0) throw SpecError("biased_attention: keep_first is not negative");
            if (shape_.window <= 0) shape_.keep_first = 0;       // (without a window every key is visible anyway)
        }
        shape_.sink_one = p.get_bool("sink_one", false);
        taps_ = static_cast<int>(p.get_int("taps", 0));
        if (taps_ < 0) throw SpecError("biased_attention: taps is not negative");
        if (PartSpec::is_part(p["position"]))
            position_ = build_as<PositionEncoding>("position", PartSpec::from_json(p["position"], "biased_attention.position"));
        distance_bias_ = p.get_bool("distance_bias", false);
        const std::string gate = p.get_string("gate", "none");
        if (gate != "none" && gate != "sigmoid") throw SpecError("biased_attention: gate is 'none' or 'sigmoid', not '" + gate + "'");
        gated_ = gate == "sigmoid";
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override {
        return position_ ? std::vector<const Part*>{position_.get()} : std::vector<const Part*>{};
    }
    std::optional<KVNeed> kv_need() const override {
        KVNeed need{shape_.kv_heads, shape_.head_dim, shape_.window > 0 ? std::optional<int>(shape_.window) : std::nullopt};
        need.v_head_dim = shape_.v_dim;
        need.keep_first = shape_.keep_first;
        return need;
    }
    std::vector<StateNeed> state_needs() const override {
        if (taps_ <= 0) return {};
        return {StateNeed{"conv", {std::max(taps_ - 1, 1), q_width() + k_width() + v_width()}, DType::F32}};
    }
    long long q_width() const { return static_cast<long long>(shape_.heads) * shape_.head_dim; }
    long long k_width() const { return static_cast<long long>(shape_.kv_heads) * shape_.head_dim; }
    long long v_width() const { return static_cast<long long>(shape_.kv_heads) * shape_.v_dim; }
    long long o_width() const { return static_cast<long long>(shape_.heads) * shape_.v_dim; }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"q", matrix(q_width(), width_)}, {"k", matrix(k_width(), width_)}, {"v", matrix(v_width(), width_)},
                          {"o", matrix(width_, o_width())}};
        if (distance_bias_) {
            specs.push_back({"r1", vec(shape_.heads, "around_one")});
            specs.push_back({"r2", vec(shape_.heads, "around_one")});
        }
        if (gated_) specs.push_back({"g", matrix(o_width(), width_)});
        if (taps_ > 0) {
            auto taps = [&](long long n) { return WeightSpec{{n, taps_}, "vector", "normal", {}}; };
            specs.push_back({"q_conv", taps(q_width())});
            specs.push_back({"k_conv", taps(k_width())});
            specs.push_back({"v_conv", taps(v_width())});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        if (taps_ > 0) conv_w_ = concat_rows({get(t, "q_conv"), get(t, "k_conv"), get(t, "v_conv")});
        std::vector<std::pair<std::shared_ptr<DeviceTensor>, bool>> pieces{{get(t, "q"), false}, {get(t, "k"), false}, {get(t, "v"), false}};
        if (gated_) pieces.push_back({get(t, "g"), false});
        const Stacked in = stack_projections(pieces, "biased_attention");
        w_in_ = in.weight;
        col_k_ = in.at[1];
        col_v_ = in.at[2];
        col_g_ = gated_ ? in.at[3] : 0;
        w_o_ = get(t, "o");
        r1_ = maybe(t, "r1");
        r2_ = maybe(t, "r2");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        if (!cache.kv) throw SpecError("biased_attention: the cache has no keys and values for this layer");
        if (!cache.writes_kv) throw SpecError("biased_attention: reading another entry's cache is not supported");
        const long long T = x.shape[0];
        Tensor proj = rt.ws.buf("battn_proj", rt.dtype, {T, w_in_->view.shape[0]});
        rt.ops.linear(x, w_in_->view, proj, nullptr, rt.ws);
        // every row's keys and values are in their pages before any row attends
        Tensor q = proj.cols(0, q_width());
        if (taps_ > 0 || position_) {
            // convolutions continuing from the request's saved rows, rotation, queries to a buffer of their own
            PositionEncoding::Tables tables;
            if (position_) tables = position_->tables(rt);
            const Tensor* inv_freq = tables.inv_freq.defined() ? &tables.inv_freq : nullptr;
            q = rt.ws.buf("battn_q", rt.dtype, {T, q_width()});
            const Tensor* state = taps_ > 0 ? &cache.states.at("conv") : nullptr;
            rt.ops.conv_rope_store(proj, taps_ > 0 ? &conv_w_->view : nullptr, state, taps_, inv_freq, tables.rotary_dim, tables.pairing,
                                   q, shape_.heads, batch, *cache.kv);
        } else {
            rt.ops.kv_store(proj.cols(col_k_, k_width()), proj.cols(col_v_, v_width()), batch, *cache.kv);
        }
        Tensor attended = rt.ws.buf("battn_out", rt.dtype, {T, o_width()});
        Tensor gate = gated_ ? proj.cols(col_g_, o_width()) : Tensor();
        rt.ops.biased_attention(q, attended, shape_, r1_ ? &r1_->view : nullptr, r2_ ? &r2_->view : nullptr,
                                gated_ ? &gate : nullptr, batch, *cache.kv, rt.ws);
        Tensor out = rt.ws.buf("battn_mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(attended, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0, col_k_ = 0, col_v_ = 0, col_g_ = 0;
    Ops::ScoreShape shape_;
    bool distance_bias_ = false, gated_ = false;
    int taps_ = 0;
    std::unique_ptr<PositionEncoding> position_;
    std::shared_ptr<DeviceTensor> w_in_, w_o_, r1_, r2_, conv_w_;
};

// ---------------------------------------------------------------------------- real-gated linear recurrent unit
// A recurrent block with two branches of "inner" channels from the mixer's input h:
//     y = gelu_tanh(W_y h + b_y);   u = conv(W_x h + b_x)     (a causal convolution per channel with "taps" taps
//                                                               and a bias, the last tap the current token's)
// u in "blocks" equal parts; in part b  r = sigmoid(Ra[b] u_b + ra_b), i = sigmoid(Ri[b] u_b + ri_b), square
// matrices stored [out, in].  log a = -c r softplus(lam) ("decay_scale" c, 8 unless given), a = exp(log a),
//     S <- a S + sqrt(1 - a^2) (i u)       from S = 0, the first token like every other
// and the output is W_o (S * y).  State per request: S [inner] and the last taps - 1 inputs of the
// convolution, both 32-bit; gates, decays and the recurrence are 32-bit.
class LinearRecurrentUnit final : public Mixer {
public:
    explicit LinearRecurrentUnit(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        shape_.width = static_cast<int>(p.get_int("inner", 0));
        shape_.blocks = static_cast<int>(p.get_int("blocks", 1));
        shape_.taps = static_cast<int>(p.get_int("taps", 0));
        shape_.decay_scale = static_cast<float>(p.get_double("decay_scale", 8.0));
        if (width_ <= 0 || shape_.width <= 0 || shape_.blocks <= 0 || shape_.width % shape_.blocks)
            throw SpecError("linear_recurrent_unit: inner must be a positive multiple of blocks");
        if (shape_.taps <= 0) throw SpecError("linear_recurrent_unit: taps must be positive");
    }
    bool graph_safe() const override { return true; }
    std::vector<StateNeed> state_needs() const override {
        return {StateNeed{"S", {shape_.width}, DType::F32}, StateNeed{"conv", {std::max(shape_.taps - 1, 1), shape_.width}, DType::F32}};
    }
    WeightSpecs weight_specs() const override {
        const long long I = shape_.width, bw = I / shape_.blocks;
        auto cube = [&]() { return WeightSpec{{shape_.blocks, bw, bw}, "vector", "normal", {}}; };
        auto per_block = [&]() { return WeightSpec{{shape_.blocks, bw}, "vector", "normal", {}}; };
        return {{"y", matrix(I, width_)},      {"y_bias", vec(I)},          {"x", matrix(I, width_)},  {"x_bias", vec(I)},
                {"conv", WeightSpec{{I, shape_.taps}, "vector", "normal", {}}}, {"conv_bias", vec(I)}, {"ra", cube()},
                {"ra_bias", per_block()},      {"ri", cube()},              {"ri_bias", per_block()},  {"lam", vec(I)},
                {"o", matrix(width_, I)}};
    }
    void load(const PartTensors& t, Runtime&) override {
        const Stacked in = stack_projections({{get(t, "y"), false}, {get(t, "x"), false}}, "linear_recurrent_unit");
        w_in_ = in.weight;
        col_x_ = in.at[1];
        std::vector<float> b = to_host_floats(get(t, "y_bias")->view), bx = to_host_floats(get(t, "x_bias")->view);
        b.resize(static_cast<size_t>(col_x_), 0.f);
        b.insert(b.end(), bx.begin(), bx.end());
        b.resize(static_cast<size_t>(in.rows), 0.f);
        b_in_ = from_host_floats(b, DType::F32, {in.rows});
        conv_w_ = get(t, "conv");
        conv_b_ = get(t, "conv_bias");
        // the gate matrices turned over, [blocks, in, out]: neighbouring threads read neighbouring weights
        const long long bw = shape_.width / shape_.blocks;
        auto turned = [&](const char* role) {
            const std::vector<float> w = to_host_floats(get(t, role)->view);
            std::vector<float> out(w.size());
            for (long long b2 = 0; b2 < shape_.blocks; ++b2)
                for (long long o = 0; o < bw; ++o)
                    for (long long i = 0; i < bw; ++i)
                        out[static_cast<size_t>((b2 * bw + i) * bw + o)] = w[static_cast<size_t>((b2 * bw + o) * bw + i)];
            return from_host_floats(out, DType::F32, {shape_.blocks, bw, bw});
        };
        ra_t_ = turned("ra");
        ri_t_ = turned("ri");
        ra_b_ = get(t, "ra_bias");
        ri_b_ = get(t, "ri_bias");
        lam_ = get(t, "lam");
        w_o_ = get(t, "o");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = x.shape[0], I = shape_.width;
        Tensor proj = rt.ws.buf("lru_proj", rt.dtype, {T, w_in_->view.shape[0]});
        rt.ops.linear(x, w_in_->view, proj, &b_in_->view, rt.ws);
        Tensor decay = rt.ws.buf("lru_decay", DType::F32, {T, I}), input = rt.ws.buf("lru_input", DType::F32, {T, I});
        rt.ops.lru_gates(proj.cols(col_x_, I), conv_w_->view, &conv_b_->view, ra_t_->view, ra_b_->view, ri_t_->view, ri_b_->view,
                         lam_->view, cache.states.at("conv"), decay, input, shape_, batch);
        Tensor gated = rt.ws.buf("lru_gated", rt.dtype, {T, I});
        rt.ops.lru_scan(decay, input, proj.cols(0, I), cache.states.at("S"), gated, batch);
        Tensor out = rt.ws.buf("lru_mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(gated, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0, col_x_ = 0;
    Ops::LruShape shape_;
    std::shared_ptr<DeviceTensor> w_in_, b_in_, conv_w_, conv_b_, ra_t_, ri_t_, ra_b_, ri_b_, lam_, w_o_;
};

// ---------------------------------------------------------------------------- two mixers side by side
// normed_pair: both mixers ("left" and "right", parts of their own) read the same rows; the result is
// factor * (rmsnorm(left(h)) * w_left + rmsnorm(right(h)) * w_right) with plain weights over the model
// width ("factor" 0.5 unless given: the mean).  A child's tensors are this part's, the role prefixed
// "left." or "right."; so are its states.  At most one of the two keeps keys and values in pages.
class NormedPair final : public Mixer {
public:
    explicit NormedPair(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        factor_ = static_cast<float>(p.get_double("factor", 0.5));
        if (width_ <= 0) throw SpecError("normed_pair: width must be positive");
        const char* sides[2] = {"left", "right"};
        for (int i = 0; i < 2; ++i) {
            if (!PartSpec::is_part(p[sides[i]])) throw SpecError(std::string("normed_pair: '") + sides[i] + "' must be a mixer");
            PartSpec child = PartSpec::from_json(p[sides[i]], std::string("normed_pair.") + sides[i]);
            const std::string prefix = std::string(sides[i]) + ".";
            for (const auto& t : s.tensors)
                if (t.first.rfind(prefix, 0) == 0) child.tensors.emplace_back(t.first.substr(prefix.size()), t.second);
            child_[i] = build_as<Mixer>("mixer", child);
        }
        if (child_[0]->kv_need() && child_[1]->kv_need()) throw SpecError("normed_pair: only one of the two mixers may keep keys and values");
    }
    bool graph_safe() const override { return true; }
    std::vector<const Part*> children() const override { return {child_[0].get(), child_[1].get()}; }
    std::optional<KVNeed> kv_need() const override { return child_[0]->kv_need() ? child_[0]->kv_need() : child_[1]->kv_need(); }
    std::vector<StateNeed> state_needs() const override {
        std::vector<StateNeed> out;
        for (int i = 0; i < 2; ++i)
            for (StateNeed n : child_[i]->state_needs()) {
                n.name = prefix(i) + n.name;
                out.push_back(std::move(n));
            }
        return out;
    }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"left_out", vec(width_, "around_one")}, {"right_out", vec(width_, "around_one")}};
        for (int i = 0; i < 2; ++i)
            for (const auto& ws : child_[i]->weight_specs()) specs.push_back({prefix(i) + ws.first, ws.second});
        return specs;
    }
    void load(const PartTensors& t, Runtime& rt) override {
        w_[0] = get(t, "left_out");
        w_[1] = get(t, "right_out");
        for (int i = 0; i < 2; ++i) {
            PartTensors mine;
            for (const auto& e : t)
                if (e.first.rfind(prefix(i), 0) == 0) mine[e.first.substr(prefix(i).size())] = e.second;
            child_[i]->load(mine, rt);
        }
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        Tensor result[2];
        for (int i = 0; i < 2; ++i) {
            LayerCache mine;
            if (child_[i]->kv_need()) {
                mine.kv = cache.kv;
                mine.writes_kv = cache.writes_kv;
            }
            for (const auto& e : cache.states)
                if (e.first.rfind(prefix(i), 0) == 0) mine.states[e.first.substr(prefix(i).size())] = e.second;
            result[i] = child_[i]->forward(x, batch, mine, rt);
            if (i == 1 && result[1].data == result[0].data) throw SpecError("normed_pair: both mixers answer in the same buffer");
        }
        Tensor out = rt.ws.buf("pair_out", rt.dtype, {x.shape[0], width_});
        rt.ops.normed_mean(result[0], w_[0]->view, result[1], w_[1]->view, eps_, factor_, out);
        return out;
    }

private:
    static std::string prefix(int i) { return i == 0 ? "left." : "right."; }
    long long width_ = 0;
    float eps_ = 1e-6f, factor_ = 0.5f;
    std::unique_ptr<Mixer> child_[2];
    std::shared_ptr<DeviceTensor> w_[2];
};

// ---------------------------------------------------------------------------- gated linear attention
// A recurrent mixer with a matrix of state per head and a decay per key channel:
//     q = W_q h * dim^-1/2, k = W_k h (heads x dim), v = W_v h (heads x vdim)
//     alpha = sigmoid(W_a2 (W_a1 h) + b_a2)^(1 / tau)      ("decay_rank": the width between a1 and a2)
//     S <- diag(alpha) S + k v^T;   o = S^T q              per head, alpha on the rows of S
// o is RMS-normed per head over vdim (weight [vdim] shared by the heads), the heads side by side
// are multiplied by silu(W_g h) and go through W_o.  State per request: S [heads, dim, vdim], 32-bit;
// decays, the recurrence and the norm are 32-bit.
class GatedLinearAttention final : public Mixer {
public:
    explicit GatedLinearAttention(const PartSpec& s) : Mixer(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        shape_.heads = shape_.kv_heads = static_cast<int>(p.get_int("heads", 0));
        shape_.dim = static_cast<int>(p.get_int("dim", 0));
        shape_.vdim = static_cast<int>(p.get_int("vdim", shape_.dim));
        shape_.taps = 1;
        tau_ = static_cast<float>(p.get_double("tau", 1.0));
        rank_ = p.get_int("decay_rank", 0);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        if (width_ <= 0 || shape_.heads <= 0 || shape_.dim <= 0 || shape_.vdim <= 0 || rank_ <= 0)
            throw SpecError("gated_linear_attention: width, heads, dim, vdim and decay_rank must be positive");
        if (!(tau_ > 0.f)) throw SpecError("gated_linear_attention: tau must be positive");
    }
    bool graph_safe() const override { return true; }
    long long qk_width() const { return static_cast<long long>(shape_.heads) * shape_.dim; }
    long long v_width() const { return static_cast<long long>(shape_.heads) * shape_.vdim; }
    std::vector<StateNeed> state_needs() const override { return {StateNeed{"S", {shape_.heads, shape_.dim, shape_.vdim}, DType::F32}}; }
    WeightSpecs weight_specs() const override {
        return {{"q", matrix(qk_width(), width_)}, {"k", matrix(qk_width(), width_)}, {"v", matrix(v_width(), width_)},
                {"g", matrix(v_width(), width_)},  {"a1", matrix(rank_, width_)},     {"a2", matrix(qk_width(), rank_)},
                {"a2_bias", vec(qk_width())},      {"norm", vec(shape_.vdim, "around_one")}, {"o", matrix(width_, v_width())}};
    }
    void load(const PartTensors& t, Runtime&) override {
        const Stacked in = stack_projections({{get(t, "q"), false}, {get(t, "k"), false}, {get(t, "v"), false}, {get(t, "g"), false},
                                              {get(t, "a1"), true}}, "gated_linear_attention");
        w_in_ = in.weight;
        col_k_ = in.at[1];
        col_v_ = in.at[2];
        col_g_ = in.at[3];
        col_a_ = in.at[4];
        a2_ = get(t, "a2");
        a2_b_ = get(t, "a2_bias");
        norm_ = get(t, "norm");
        w_o_ = get(t, "o");
    }
    Tensor forward(const Tensor& x, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor proj = rt.ws.buf("gla_proj", rt.dtype, {T, w_in_->view.shape[0]});
        rt.ops.linear(x, w_in_->view, proj, nullptr, rt.ws);
        Tensor z = rt.ws.buf("gla_decay_in", rt.dtype, {T, qk_width()});
        rt.ops.linear(proj.cols(col_a_, rank_), a2_->view, z, nullptr, rt.ws);
        Tensor qk = rt.ws.buf("gla_qk", DType::F32, {T, 2 * qk_width()}), v = rt.ws.buf("gla_v", DType::F32, {T, v_width()});
        Tensor decay = rt.ws.buf("gla_decay", DType::F32, {T, qk_width()});
        rt.ops.gla_prepare(proj.cols(0, qk_width()), proj.cols(col_k_, qk_width()), proj.cols(col_v_, v_width()), z, &a2_b_->view, tau_,
                           static_cast<float>(1.0 / std::sqrt(static_cast<double>(shape_.dim))), qk, v, decay);
        Tensor o = rt.ws.buf("gla_o", DType::F32, {T, v_width()});
        rt.ops.channel_scan(qk, v, decay, nullptr, 0, cache.states.at("S"), o, shape_, batch);
        Tensor gated = rt.ws.buf("gla_gated", rt.dtype, {T, v_width()});
        rt.ops.delta_gated_norm(o, norm_->view, proj.cols(col_g_, v_width()), eps_, gated, shape_.heads, shape_.vdim, 0);
        Tensor out = rt.ws.buf("gla_mixer_out", rt.dtype, {T, width_});
        rt.ops.linear(gated, w_o_->view, out, nullptr, rt.ws);
        return out;
    }

private:
    long long width_ = 0, rank_ = 0, col_k_ = 0, col_v_ = 0, col_g_ = 0, col_a_ = 0;
    Ops::DeltaShape shape_;
    float tau_ = 1.f, eps_ = 1e-6f;
    std::shared_ptr<DeviceTensor> w_in_, a2_, a2_b_, norm_, w_o_;
};

// ---------------------------------------------------------------------------- dense feed-forward with biases
// mlp: W_down act(W_up x + b_up) + b_down; "activation": "gelu_tanh" (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))))
// or "relu2" (the square of relu); "bias": false leaves both biases out.
class DenseMlp final : public FeedForward {
public:
    explicit DenseMlp(const PartSpec& s) : FeedForward(s), width_(s.params.get_int("width", 0)), ff_(s.params.get_int("ff", 0)) {
        if (width_ <= 0 || ff_ <= 0) throw SpecError("mlp: width and ff must be positive");
        const std::string act = s.params.get_string("activation", "gelu_tanh");
        if (act != "gelu_tanh" && act != "relu2") throw SpecError("mlp: activation is 'gelu_tanh' or 'relu2', not '" + act + "'");
        act_ = act == "relu2" ? 1 : 0;
        bias_ = s.params.get_bool("bias", true);
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        WeightSpecs specs{{"up", matrix(ff_, width_)}, {"down", matrix(width_, ff_)}};
        if (bias_) {
            specs.push_back({"up_bias", vec(ff_)});
            specs.push_back({"down_bias", vec(width_)});
        }
        return specs;
    }
    void load(const PartTensors& t, Runtime&) override {
        w_up_ = get(t, "up");
        w_down_ = get(t, "down");
        b_up_ = maybe(t, "up_bias");
        b_down_ = maybe(t, "down_bias");
    }
    Tensor forward(const Tensor& x, const StepBatch&, Runtime& rt) override {
        const long long T = x.shape[0];
        Tensor up = rt.ws.buf("mlp_up", rt.dtype, {T, ff_});
        rt.ops.linear(x, w_up_->view, up, nullptr, rt.ws);
        rt.ops.activation_bias(up, b_up_ ? &b_up_->view : nullptr, up, act_);
        Tensor out = rt.ws.buf("ffn_out", rt.dtype, {T, width_});
        rt.ops.linear(up, w_down_->view, out, b_down_ ? &b_down_->view : nullptr, rt.ws);
        return out;
    }

private:
    long long width_, ff_;
    int act_ = 0;
    bool bias_ = true;
    std::shared_ptr<DeviceTensor> w_up_, w_down_, b_up_, b_down_;
};

// ---------------------------------------------------------------------------- a token input per layer
// gated_table: with e = table[token][offset, offset + dim) (a table of "table_width" values a token that all
// layers share, each reading its own columns), g = gelu_tanh(W_gate x) * e, y = W_proj g, and the stream
// becomes x + y / sqrt(mean(y^2) + eps) * w with a plain weight.
class GatedTableInput final : public TokenInput {
public:
    explicit GatedTableInput(const PartSpec& s) : TokenInput(s) {
        const Json& p = s.params;
        width_ = p.get_int("width", 0);
        vocab_ = p.get_int("vocab", 0);
        dim_ = p.get_int("dim", 0);
        offset_ = p.get_int("offset", 0);
        table_width_ = p.get_int("table_width", dim_);
        eps_ = static_cast<float>(p.get_double("eps", 1e-6));
        if (width_ <= 0 || vocab_ <= 0 || dim_ <= 0 || offset_ < 0 || offset_ + dim_ > table_width_)
            throw SpecError("gated_table: width, vocab and dim must be positive and [offset, offset + dim) inside table_width");
    }
    bool graph_safe() const override { return true; }
    WeightSpecs weight_specs() const override {
        return {{"table", matrix(vocab_, table_width_)}, {"gate", matrix(dim_, width_)}, {"proj", matrix(width_, dim_)},
                {"norm", vec(width_, "around_one")}};
    }
    void load(const PartTensors& t, Runtime&) override {
        table_ = get(t, "table");
        gate_ = get(t, "gate");
        proj_ = get(t, "proj");
        norm_ = get(t, "norm");
        post_.weight = norm_->view;
        post_.eps = eps_;
    }
    void forward(const Tensor& h, const Tensor& h_copy, const StepBatch& batch, Runtime& rt) override {
        const long long T = h.shape[0];
        Tensor z = rt.ws.buf("token_input_z", rt.dtype, {T, dim_});
        rt.ops.linear(h_copy, gate_->view, z, nullptr, rt.ws);
        Tensor g = rt.ws.buf("token_input_g", rt.dtype, {T, dim_});
        rt.ops.token_gate(z, table_->view, static_cast<int>(offset_), batch.token_ids, g);
        Tensor y = rt.ws.buf("token_input_y", rt.dtype, {T, width_});
        rt.ops.linear(g, proj_->view, y, nullptr, rt.ws);
        rt.ops.norm_step(h, &y, &post_, nullptr, nullptr);
    }

private:
    long long width_ = 0, vocab_ = 0, dim_ = 0, offset_ = 0, table_width_ = 0;
    float eps_ = 1e-6f;
    std::shared_ptr<DeviceTensor> table_, gate_, proj_, norm_;
    Ops::NormParams post_;
};

// ---------------------------------------------------------------------------- a weighted sum over depth
// weighted_history: behind run-order entry i the stream becomes sum_{j <= i + 1} w[j] X_j, X_0 the embedding's
// rows and X_(j+1) the result of entry j before this mixing ("entries": how many results, i + 2).
class WeightedHistory final : public DepthMix {
public:
    explicit WeightedHistory(const PartSpec& s) : DepthMix(s), entries_(static_cast<int>(s.params.get_int("entries", 0))) {
        if (entries_ < 1) throw SpecError("weighted_history: entries must be positive");
    }
    bool graph_safe() const override { return true; }
    int entries() const override { return entries_; }
    WeightSpecs weight_specs() const override { return {{"weights", vec(entries_, "around_one")}}; }
    void load(const PartTensors& t, Runtime&) override { w_ = get(t, "weights"); }
    void forward(const Tensor& history, const Tensor& h, Runtime& rt) override { rt.ops.depth_mix(history, h, w_->view, entries_); }

private:
    int entries_;
    std::shared_ptr<DeviceTensor> w_;
};

// ---------------------------------------------------------------------------- both sub-layers from one norm
// parallel: h += mixer(norm(h)) + ffn(norm(h)): one norm, both sub-layers read its output, one sum into
// the 32-bit stream.  A feed-forward of kind "none" is left out.
class ParallelBlock final : public Block {
public:
    explicit ParallelBlock(const LayerSpec& layer)
        : norm_(build_as<Norm>("norm", layer.mixer_norm)), mixer_(build_as<Mixer>("mixer", layer.mixer)),
          has_ffn_(layer.ffn.kind != "none" && !layer.ffn.kind.empty()) {
        if (has_ffn_) ffn_ = build_as<FeedForward>("ffn", layer.ffn);
    }
    std::vector<std::pair<std::string, Part*>> parts() override {
        std::vector<std::pair<std::string, Part*>> out{{"mixer_norm", norm_.get()}, {"mixer", mixer_.get()}};
        if (has_ffn_) out.emplace_back("ffn", ffn_.get());
        return out;
    }
    Mixer& mixer() override { return *mixer_; }
    Tensor forward(const Tensor& h, const Tensor& delta, const StepBatch& batch, const LayerCache& cache, Runtime& rt) override {
        const long long T = h.shape[0], width = h.shape[1];
        rt.stream_stat_blocks = 0;
        rt.stream_has_bf16 = false;
        Tensor normed = rt.ws.buf("normed", rt.dtype, {T, width});
        norm_->forward(h, normed, rt, delta.defined() ? &delta : nullptr, nullptr);
        Tensor mixed = mixer_->forward(normed, batch, cache, rt);
        rt.mark("mixer " + mixer_->spec.kind);
        Tensor fed;
        if (has_ffn_) {
            fed = ffn_->forward(normed, batch, rt);
            rt.mark("ffn " + ffn_->spec.kind);
        }
        // the sum into the stream, and the stream's new rows in the run's dtype for whoever reads them next
        Tensor copy = rt.ws.buf("stream_copy", rt.dtype, {T, width});
        rt.ops.residual_sum(h, mixed, has_ffn_ ? &fed : nullptr, &copy);
        rt.stream_copy = copy;
        return Tensor();
    }

private:
    std::unique_ptr<Norm> norm_;
    std::unique_ptr<Mixer> mixer_;
    bool has_ffn_;
    std::unique_ptr<FeedForward> ffn_;
};

template <typename T>
PartFactory factory_of() {
    return [](const PartSpec& s) { return std::unique_ptr<Part>(new T(s)); };
}

void register_builtin_parts() {
    Registries& r = registries();
    std::lock_guard<std::mutex> guard(r.lock);
    r.parts["norm"]["rmsnorm"] = factory_of<RmsNorm>();
    r.parts["norm"]["identity"] = factory_of<IdentityNorm>();
    r.parts["norm"]["layernorm"] = factory_of<LayerNorm>();
    r.parts["norm"]["dynamic_tanh"] = factory_of<DynamicTanh>();
    r.parts["position"]["rope"] = factory_of<Rope>();
    r.parts["position"]["none"] = factory_of<NoPosition>();
    r.parts["mixer"]["gqa_attention"] = factory_of<GqaAttention>();
    r.parts["mixer"]["latent_attention"] = factory_of<LatentAttention>();
    r.parts["mixer"]["short_conv"] = factory_of<ShortConv>();
    r.parts["mixer"]["sigmoid_attention"] = factory_of<SigmoidAttention>();
    r.parts["mixer"]["gated_delta_rule"] = factory_of<GatedDeltaRule>();
    r.parts["reinjection"]["linear_concat"] = factory_of<LinearReinjection>();
    r.parts["reinjection"]["add_rows"] = factory_of<AdditiveReinjection>();
    r.parts["mixer"]["biased_attention"] = factory_of<BiasedAttention>();
    r.parts["mixer"]["linear_recurrent_unit"] = factory_of<LinearRecurrentUnit>();
    r.parts["mixer"]["normed_pair"] = factory_of<NormedPair>();
    r.parts["mixer"]["gated_linear_attention"] = factory_of<GatedLinearAttention>();
    r.parts["ffn"]["mlp"] = factory_of<DenseMlp>();
    r.parts["token_input"]["gated_table"] = factory_of<GatedTableInput>();
    r.parts["depth_mix"]["weighted_history"] = factory_of<WeightedHistory>();
    r.parts["mixer"]["none"] = factory_of<NoMixer>();
    r.parts["ffn"]["swiglu"] = factory_of<SwiGlu>();
    r.parts["ffn"]["routed_experts"] = factory_of<RoutedExperts>();
    r.parts["ffn"]["none"] = factory_of<NoFeedForward>();
    r.parts["link"]["hyper_link"] = factory_of<HyperLink>();
    r.parts["embedding"]["embedding"] = factory_of<TokenEmbedding>();
    r.parts["head"]["tied_head"] = factory_of<TiedHead>();
    r.parts["head"]["linear_head"] = factory_of<LinearHead>();
    r.parts["head"]["hidden"] = factory_of<HiddenHead>();
    r.blocks["pre_norm"] = [](const LayerSpec& layer) { return std::unique_ptr<Block>(new PreNormBlock(layer)); };
    r.blocks["parallel"] = [](const LayerSpec& layer) { return std::unique_ptr<Block>(new ParallelBlock(layer)); };
    r.blocks["sandwich_norm"] = [](const LayerSpec& layer) { return std::unique_ptr<Block>(new SandwichBlock(layer)); };
    r.blocks["hyper_connections"] = [](const LayerSpec& layer) { return std::unique_ptr<Block>(new HyperBlock(layer)); };
}

}  // namespace

}  // namespace celeg
