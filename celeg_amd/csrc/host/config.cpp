// The architecture registry, reading config.json, and the LFM2 dense configuration.
//
// The reference has no class for this architecture: it recognises the layers from tensor
// names (src/model/inference/rules.cpp:12-90 for the short convolution,
// src/model/inference/rules_attention.cpp:138-345 for attention) and reads the scalar keys
// through its metadata normaliser (src/model/inference/metadata.cpp:350-703).  Here every
// size comes from config.json; nothing about a particular checkpoint stands in code.
#include "config.hpp"

#include <cmath>
#include <fstream>
#include <mutex>
#include <set>
#include <sstream>

namespace celeg {

namespace {
std::map<std::string, Architecture>& table() {
    static std::map<std::string, Architecture> t;
    return t;
}
std::mutex& table_lock() {
    static std::mutex m;
    return m;
}
void register_builtin();
void ensure_builtin() {
    static std::once_flag once;
    std::call_once(once, register_builtin);
}
std::string list_of(const std::vector<std::string>& names) {
    std::string out = "[";
    for (size_t i = 0; i < names.size(); ++i) out += (i ? ", '" : "'") + names[i] + "'";
    return out + "]";
}
}  // namespace

void register_architecture(Architecture arch, bool replace) {
    ensure_builtin();
    std::lock_guard<std::mutex> guard(table_lock());
    std::vector<std::string> names{arch.name};
    names.insert(names.end(), arch.aliases.begin(), arch.aliases.end());
    for (const auto& n : names)
        if (table().count(n) && !replace) throw SpecError("architecture '" + n + "' is already registered");
    for (const auto& n : names) table()[n] = arch;
}

std::vector<std::string> registered_architectures() {
    ensure_builtin();
    std::lock_guard<std::mutex> guard(table_lock());
    std::vector<std::string> out;
    for (const auto& e : table()) out.push_back(e.first);
    return out;
}

std::string architecture_name(const Json& config) {
    const Json& archs = config["architectures"];
    if (archs.is_array() && archs.size() > 0 && archs[0].is_string()) return archs[0].as_string();
    if (config["model_type"].is_string()) return config["model_type"].as_string();
    if (config["architecture"].is_string()) return config["architecture"].as_string();
    throw ConfigError("config.json names no architecture: none of 'architectures', 'model_type' and 'architecture' is present");
}

const Architecture& find_architecture(const Json& config) {
    ensure_builtin();
    const std::string name = architecture_name(config);
    {
        std::lock_guard<std::mutex> guard(table_lock());
        auto it = table().find(name);
        if (it != table().end()) return it->second;
    }
    throw ConfigError("no registered architecture is called '" + name + "'; registered: " +
                      list_of(registered_architectures()));
}

static bool read_text(const std::string& path, std::string& out) {
    std::ifstream in(path, std::ios::binary);
    if (!in) return false;
    std::ostringstream ss;
    ss << in.rdbuf();
    out = ss.str();
    return true;
}

Json read_config_file(const std::string& model_dir) {
    std::string text;
    const std::string path = model_dir + "/config.json";
    if (!read_text(path, text)) throw ConfigError("config.json not found in model folder " + model_dir);
    Json config;
    try {
        config = Json::parse(text);
    } catch (const JsonError& e) {
        throw ConfigError("config.json in " + model_dir + " cannot be read: " + e.what());
    }
    if (!config.is_object()) throw ConfigError("config.json in " + model_dir + " is not an object");
    std::string gen_text;
    if (read_text(model_dir + "/generation_config.json", gen_text)) {
        try {
            const Json gen = Json::parse(gen_text);
            for (const char* key : {"bos_token_id", "eos_token_id"}) {
                const Json& v = gen[key];
                if (v.is_number()) {
                    config.set(key, Json(v.as_int()));
                } else if (v.is_array()) {
                    Json ids = Json::array();
                    for (const Json& item : v.items())
                        if (item.is_number()) ids.push(Json(item.as_int()));
                    if (ids.size() > 0) config.set(key, ids);
                }
            }
        } catch (const JsonError&) {
            // unreadable: ignored, as the reference does
        }
    }
    return config;
}

Described describe_config(const Json& config, const TensorShapes* shapes) {
    const Architecture& arch = find_architecture(config);
    Described d;
    d.config = arch.read_config(config, shapes);
    d.spec = arch.build_spec(d.config);
    d.spec.validate();
    return d;
}

// ---------------------------------------------------------------------------- LFM2 dense
namespace {

std::string repr(const Json& v) { return v.dump(); }

long long typed_int(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (v.is_int()) return v.as_int();
    if (v.kind() == Json::Float && std::floor(v.as_double()) == v.as_double()) return v.as_int();
    throw ConfigError("config.json: '" + key + "' must be an integer, got " + repr(v));
}
double typed_float(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (!v.is_number()) throw ConfigError("config.json: '" + key + "' must be a number, got " + repr(v));
    return v.as_double();
}
bool typed_bool(const Json& cfg, const std::string& key) {
    const Json& v = cfg[key];
    if (!v.is_bool()) throw ConfigError("config.json: '" + key + "' must be true or false, got " + repr(v));
    return v.as_bool();
}
bool present(const Json& cfg, const std::string& key) { return !cfg[key].is_null(); }

long long require_int(const Json& cfg, const std::string& key) {
    if (!present(cfg, key)) throw ConfigError("config.json: required key '" + key + "' is missing");
    return typed_int(cfg, key);
}

// First present alias wins; two aliases that disagree are an error, as in the reference
// (src/model/inference/metadata.cpp:350-703 raises ConflictingMetadata).
template <typename T, typename Read>
bool alias(const Json& cfg, const std::vector<std::string>& keys, Read read, T& out) {
    bool found = false;
    std::string first_key;
    for (const auto& k : keys) {
        if (!present(cfg, k)) continue;
        const T v = read(cfg, k);
        if (!found) {
            out = v;
            found = true;
            first_key = k;
        } else if (!(v == out)) {
            throw ConfigError("config.json: '" + first_key + "'=" + repr(cfg[first_key]) + " and '" + k + "'=" +
                              repr(cfg[k]) + " disagree");
        }
    }
    return found;
}

const char* const LAYER_KINDS[] = {"conv", "full_attention"};
bool known_kind(const std::string& k) { return k == LAYER_KINDS[0] || k == LAYER_KINDS[1]; }

// layer_types if given; else from full_attn_idxs; else from the tensors each layer has
// (src/model/inference/rules.cpp:18-26, rules_attention.cpp:138-160).  Whatever the source,
// tensors that say otherwise are an error.
std::vector<std::string> layer_kinds(const Json& cfg, long long layers, const TensorShapes* shapes) {
    std::vector<std::string> from_tensors;     // "" where the tensors tell nothing
    if (shapes) {
        for (long long i = 0; i < layers; ++i) {
            const std::string p = "model.layers." + std::to_string(i) + ".";
            const bool conv = shapes->count(p + "conv.in_proj.weight") > 0;
            const bool attn = shapes->count(p + "self_attn.q_proj.weight") > 0;
            from_tensors.push_back(conv && !attn ? "conv" : attn && !conv ? "full_attention" : "");
        }
    }
    std::vector<std::string> kinds;
    if (present(cfg, "layer_types")) {
        const Json& v = cfg["layer_types"];
        bool ok = v.is_array();
        if (ok)
            for (const Json& k : v.items()) ok = ok && k.is_string();
        if (!ok) throw ConfigError("config.json: 'layer_types' must be a list of strings");
        for (const Json& k : v.items()) kinds.push_back(k.as_string());
    } else if (present(cfg, "full_attn_idxs")) {
        const Json& v = cfg["full_attn_idxs"];
        bool ok = v.is_array();
        if (ok)
            for (const Json& k : v.items()) ok = ok && k.is_int();
        if (!ok) throw ConfigError("config.json: 'full_attn_idxs' must be a list of integers");
        std::set<long long> idxs;
        for (const Json& k : v.items()) {
            if (k.as_int() < 0 || k.as_int() >= layers)
                throw ConfigError("config.json: 'full_attn_idxs' names a layer outside [0, " + std::to_string(layers) + ")");
            idxs.insert(k.as_int());
        }
        for (long long i = 0; i < layers; ++i) kinds.push_back(idxs.count(i) ? "full_attention" : "conv");
    } else if (shapes) {
        std::string unknown;
        for (size_t i = 0; i < from_tensors.size(); ++i)
            if (from_tensors[i].empty()) unknown += (unknown.empty() ? "" : ", ") + std::to_string(i);
        if (!unknown.empty())
            throw ConfigError("config.json has no 'layer_types' and the tensors of layer(s) [" + unknown +
                              "] tell neither a convolution nor an attention layer");
        return from_tensors;
    } else {
        throw ConfigError("config.json: required key 'layer_types' is missing");
    }
    if (shapes && static_cast<long long>(kinds.size()) == layers) {
        for (size_t i = 0; i < kinds.size(); ++i)
            if (!from_tensors[i].empty() && known_kind(kinds[i]) && kinds[i] != from_tensors[i])
                throw ConfigError("config.json: 'layer_types'[" + std::to_string(i) + "] is '" + kinds[i] +
                                  "' but the checkpoint's tensors of layer " + std::to_string(i) + " are those of '" +
                                  from_tensors[i] + "'");
    }
    return kinds;
}

// Keys and defaults follow src/model/inference/metadata.cpp: hidden_size (353),
// intermediate_size (355-357), num_hidden_layers (358-360), num_attention_heads (364-366),
// num_key_value_heads (367-369), head_dim (370), vocab_size (399), max_position_embeddings
// (404-406), norm_eps (407-409, default 1e-6 at 643), conv_L_cache (425-426), rope_theta
// (427-429: also as rope_parameters.rope_theta; required 663-666), block_auto_adjust_ff_dim
// (512-514), tying (630-632), token ids (638-642).  The original LFM2 keys full_attn_idxs
// (the attention layers; every other layer is a convolution) and block_ff_dim
// (= intermediate_size) are read too.  With the checkpoint's tensor shapes at hand, what
// config.json leaves out is filled the way the reference does: layer kinds from the tensors
// each layer has, the feed-forward width from the rows of w1 (global_facts.cpp:127-152).
Json lfm2_read_config(const Json& raw, const TensorShapes* shapes) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json cfg = raw;
    const Json& nested = raw["rope_parameters"];
    if (nested.is_object() && !nested["rope_theta"].is_null())
        cfg.set("rope_parameters.rope_theta", nested["rope_theta"]);
    const long long vocab = require_int(cfg, "vocab_size");
    const long long hidden = require_int(cfg, "hidden_size");
    const long long layers = require_int(cfg, "num_hidden_layers");
    const long long heads = require_int(cfg, "num_attention_heads");
    long long kv_heads = heads;
    alias<long long>(cfg, {"num_key_value_heads"}, typed_int, kv_heads);
    long long head_dim = heads > 0 ? hidden / heads : 0;
    alias<long long>(cfg, {"head_dim"}, typed_int, head_dim);
    double rope_theta = 0;
    if (!alias<double>(cfg, {"rope_theta", "rope_parameters.rope_theta"}, typed_float, rope_theta))
        throw ConfigError("config.json: required key 'rope_theta' is missing");
    const long long conv_l = require_int(cfg, "conv_L_cache");
    const long long max_pos = require_int(cfg, "max_position_embeddings");
    bool auto_adjust = false;
    alias<bool>(cfg, {"block_auto_adjust_ff_dim"}, typed_bool, auto_adjust);
    long long intermediate = 0;
    const bool has_intermediate = alias<long long>(cfg, {"intermediate_size", "block_ff_dim"}, typed_int, intermediate);
    const std::vector<std::string> kinds = layer_kinds(cfg, layers, shapes);
    if (!has_intermediate) {
        const auto w1 = shapes ? shapes->find("model.layers.0.feed_forward.w1.weight") : TensorShapes::const_iterator{};
        if (!shapes || w1 == shapes->end() || w1->second.empty())
            throw ConfigError("config.json: required key 'intermediate_size' is missing");
        // the width itself: no adjustment is applied to a size read off the weights
        intermediate = w1->second[0];
        auto_adjust = false;
    }
    Json eos = Json::array();
    if (raw["eos_token_id"].is_array()) {
        for (const Json& e : raw["eos_token_id"].items()) eos.push(Json(e.as_int()));
    } else {
        eos.push(Json(raw["eos_token_id"].is_null() ? 0LL : typed_int(cfg, "eos_token_id")));
    }
    Json multiplier = Json(1.0);
    if (raw.contains("block_ffn_dim_multiplier"))
        multiplier = raw["block_ffn_dim_multiplier"].is_null() ? Json() : Json(typed_float(cfg, "block_ffn_dim_multiplier"));
    bool conv_bias = false, tie = true;
    alias<bool>(cfg, {"conv_bias"}, typed_bool, conv_bias);
    alias<bool>(cfg, {"tie_word_embeddings", "tie_embedding"}, typed_bool, tie);
    double norm_eps = 1e-6;
    alias<double>(cfg, {"norm_eps", "rms_norm_eps"}, typed_float, norm_eps);
    long long multiple_of = 256, bos = 0, pad = 1;
    alias<long long>(cfg, {"block_multiple_of"}, typed_int, multiple_of);
    alias<long long>(cfg, {"bos_token_id"}, typed_int, bos);
    alias<long long>(cfg, {"pad_token_id"}, typed_int, pad);

    Json out = Json::object();
    out.set("architectures", Json::array_of(std::vector<std::string>{"Lfm2ForCausalLM"})).set("model_type", "lfm2")
        .set("vocab_size", vocab).set("hidden_size", hidden).set("num_hidden_layers", layers)
        .set("num_attention_heads", heads).set("num_key_value_heads", kv_heads).set("head_dim", head_dim)
        .set("intermediate_size", intermediate).set("layer_types", Json::array_of(kinds))
        .set("conv_L_cache", conv_l).set("conv_bias", conv_bias).set("rope_theta", rope_theta)
        .set("norm_eps", norm_eps).set("max_position_embeddings", max_pos)
        .set("block_auto_adjust_ff_dim", auto_adjust).set("block_multiple_of", multiple_of)
        .set("block_ffn_dim_multiplier", multiplier).set("tie_word_embeddings", tie)
        .set("bos_token_id", bos).set("eos_token_id", eos).set("pad_token_id", pad);

    // GQA divisibility, even head size and kv width as in
    // src/model/inference/rules_attention.cpp:194-204; positive cache length as in
    // src/model/inference/rules.cpp:36-40.
    for (const char* key : {"vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                            "num_key_value_heads", "head_dim", "intermediate_size", "conv_L_cache",
                            "max_position_embeddings", "block_multiple_of"})
        if (out[key].as_int() <= 0)
            throw ConfigError(std::string("config.json: '") + key + "' must be positive, got " + repr(out[key]));
    if (static_cast<long long>(kinds.size()) != layers)
        throw ConfigError("config.json: 'layer_types' has " + std::to_string(kinds.size()) +
                          " entries but 'num_hidden_layers' is " + std::to_string(layers));
    for (size_t i = 0; i < kinds.size(); ++i)
        if (!known_kind(kinds[i]))
            throw ConfigError("config.json: 'layer_types'[" + std::to_string(i) + "] is '" + kinds[i] +
                              "'; known kinds are ['conv', 'full_attention']");
    if (heads % kv_heads)
        throw ConfigError("config.json: 'num_attention_heads' must be a multiple of 'num_key_value_heads'");
    if (head_dim % 2) throw ConfigError("config.json: 'head_dim' must be even");
    if (kv_heads * head_dim > hidden)
        throw ConfigError("config.json: 'num_key_value_heads' * 'head_dim' exceeds 'hidden_size'");
    if (!(rope_theta > 0)) throw ConfigError("config.json: 'rope_theta' must be positive");
    if (!(norm_eps > 0)) throw ConfigError("config.json: 'norm_eps' must be positive");
    if (!multiplier.is_null() && !(multiplier.as_double() > 0))
        throw ConfigError("config.json: 'block_ffn_dim_multiplier' must be positive");
    const double mult = multiplier.is_null() ? 0.0 : multiplier.as_double();
    out.set("ff_dim", lfm2_feed_forward_width(intermediate, auto_adjust, multiple_of, multiplier.is_null() ? nullptr : &mult));
    return out;
}

// Tensor names: embedding and head src/model/inference/global_facts.cpp:41-73 and
// layer_bindings.cpp:24-154; norms layer_bindings.cpp:276-303; short convolution
// src/model/inference/support.cpp:114-123; attention support.cpp:57-78 and
// rules_attention.cpp:72-92; feed-forward layer_bindings.cpp:439-473.
ModelSpec lfm2_build_spec(const Json& c) {
    const long long H = c["hidden_size"].as_int();
    const double eps = c["norm_eps"].as_double();
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "rmsnorm";
        p.params = Json::object().set("width", H).set("eps", eps);
        p.tensors = {{"weight", name}};
        return p;
    };
    const bool bias = c["conv_bias"].as_bool();
    ModelSpec spec;
    int i = 0;
    for (const Json& kind : c["layer_types"].items()) {
        const std::string p = "model.layers." + std::to_string(i) + ".";
        LayerSpec layer;
        if (kind.as_string() == "conv") {
            layer.mixer.kind = "short_conv";
            layer.mixer.params = Json::object().set("width", H).set("taps", c["conv_L_cache"]).set("bias", bias);
            layer.mixer.tensors = {{"in_proj", p + "conv.in_proj.weight"}, {"conv", p + "conv.conv.weight"},
                                   {"out_proj", p + "conv.out_proj.weight"}};
            if (bias) {
                layer.mixer.tensors.emplace_back("in_proj_bias", p + "conv.in_proj.bias");
                layer.mixer.tensors.emplace_back("conv_bias", p + "conv.conv.bias");
                layer.mixer.tensors.emplace_back("out_proj_bias", p + "conv.out_proj.bias");
            }
        } else {
            PartSpec rope;
            rope.kind = "rope";
            rope.params = Json::object().set("theta", c["rope_theta"]).set("rotary_dim", c["head_dim"]).set("head_dim", c["head_dim"]);
            layer.mixer.kind = "gqa_attention";
            layer.mixer.params = Json::object().set("width", H).set("heads", c["num_attention_heads"])
                                     .set("kv_heads", c["num_key_value_heads"]).set("head_dim", c["head_dim"])
                                     .set("qk_norm", true).set("eps", eps).set("window", Json())
                                     .set("position", rope.to_json());
            layer.mixer.tensors = {{"q_proj", p + "self_attn.q_proj.weight"}, {"k_proj", p + "self_attn.k_proj.weight"},
                                   {"v_proj", p + "self_attn.v_proj.weight"}, {"out_proj", p + "self_attn.out_proj.weight"},
                                   {"q_norm", p + "self_attn.q_layernorm.weight"}, {"k_norm", p + "self_attn.k_layernorm.weight"}};
        }
        layer.mixer_norm = norm(p + "operator_norm.weight");
        layer.ffn.kind = "swiglu";
        layer.ffn.params = Json::object().set("width", H).set("ff", c["ff_dim"]);
        layer.ffn.tensors = {{"gate", p + "feed_forward.w1.weight"}, {"up", p + "feed_forward.w3.weight"},
                             {"down", p + "feed_forward.w2.weight"}};
        layer.ffn_norm = norm(p + "ffn_norm.weight");
        spec.layers.push_back(std::move(layer));
        spec.order.push_back(RunStep{i, {}});
        ++i;
    }
    spec.architecture = "Lfm2ForCausalLM";
    spec.vocab_size = static_cast<int>(c["vocab_size"].as_int());
    spec.hidden_size = static_cast<int>(H);
    spec.max_context = static_cast<int>(c["max_position_embeddings"].as_int());
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab_size"]).set("width", H);
    spec.embedding.tensors = {{"table", "model.embed_tokens.weight"}};
    spec.head.params = Json::object().set("vocab", c["vocab_size"]).set("width", H);
    if (c["tie_word_embeddings"].as_bool()) {
        spec.head.kind = "tied_head";
    } else {
        spec.head.kind = "linear_head";
        spec.head.tensors = {{"weight", "lm_head.weight"}};
    }
    spec.final_norm = norm("model.embedding_norm.weight");
    for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

}  // namespace

// ---------------------------------------------------------------------------- Regipel
// A decoder whose config.json describes every layer by itself:
//   {"architecture": "Regipel", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"},
//    "logit_scale", "streams" (absent: one residual stream and plain pre-norm sums),
//    "loop": {"start", "stop", "times"} (layers start..stop-1 run `times` times in a row with the
//    same weights and a cache of their own each time), "max_context" (an engine limit; optional),
//    "layers": [{"type": "latent_attention",
//                "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot": {"base", "dims"}},
//                "mlp": null | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}}]}
// Norm weights are stored around zero (the factor is 1 + w); the output head is the embedding
// table itself, the logits multiplied by logit_scale.
// Tensors: embed, final.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o},
// l<i>.mlp.router, l<i>.mlp.e<j>.{gate,up,down}, l<i>.hc<q>.{in,out,mix} (q = 1: mixer, 2: feed-forward).
namespace {

const Json& regipel_object(const Json& parent, const std::string& key, const std::string& where) {
    const Json& v = parent[key];
    if (!v.is_object()) throw ConfigError("config.json: " + where + "'" + key + "' must be an object");
    return v;
}
long long regipel_int(const Json& parent, const std::string& key, const std::string& where, long long least = 1) {
    const Json& v = parent[key];
    if (!v.is_int()) throw ConfigError("config.json: " + where + "'" + key + "' must be an integer, got " + v.dump());
    if (v.as_int() < least)
        throw ConfigError("config.json: " + where + "'" + key + "' must be at least " + std::to_string(least) + ", got " + v.dump());
    return v.as_int();
}
double regipel_number(const Json& parent, const std::string& key, const std::string& where) {
    const Json& v = parent[key];
    if (!v.is_number()) throw ConfigError("config.json: " + where + "'" + key + "' must be a number, got " + v.dump());
    return v.as_double();
}

Json regipel_read_config(const Json& raw, const TensorShapes*) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json out = Json::object();
    out.set("architecture", "Regipel");
    out.set("vocab", regipel_int(raw, "vocab", ""));
    out.set("width", regipel_int(raw, "width", ""));
    const double eps = regipel_number(regipel_object(raw, "norm", ""), "eps", "norm.");
    if (!(eps > 0)) throw ConfigError("config.json: 'norm.eps' must be positive");
    out.set("norm", Json::object().set("eps", eps));
    double embedding_scale = 1.0, logit_scale = 1.0;
    if (!raw["embedding"].is_null()) embedding_scale = regipel_number(regipel_object(raw, "embedding", ""), "scale", "embedding.");
    if (!raw["logit_scale"].is_null()) logit_scale = regipel_number(raw, "logit_scale", "");
    out.set("embedding", Json::object().set("scale", embedding_scale)).set("logit_scale", logit_scale);
    out.set("streams", raw["streams"].is_null() ? Json() : Json(regipel_int(raw, "streams", "")));
    if (!out["streams"].is_null() && out["streams"].as_int() > 8) throw ConfigError("config.json: 'streams' may be at most 8");
    out.set("max_context", raw["max_context"].is_null() ? 131072LL : regipel_int(raw, "max_context", ""));
    if (!raw["layers"].is_array() || raw["layers"].size() == 0) throw ConfigError("config.json: 'layers' must be a list of layers");
    Json layers = Json::array();
    int i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string where = "layers[" + std::to_string(i++) + "].";
        if (!l.is_object()) throw ConfigError("config.json: " + where + " must be an object");
        const std::string type = l.get_string("type", "");
        if (type != "latent_attention")
            throw ConfigError("config.json: " + where + "'type' is '" + type + "'; known types are ['latent_attention']");
        const Json& m = regipel_object(l, "mixer", where);
        const std::string mw = where + "mixer.";
        Json mixer = Json::object();
        for (const char* key : {"heads", "dim", "vdim", "kv_rank"}) mixer.set(key, regipel_int(m, key, mw));
        const long long rot_dim = regipel_int(m, "rot_dim", mw, 0);
        mixer.set("rot_dim", rot_dim);
        mixer.set("scale", regipel_number(m, "scale", mw));
        if (rot_dim > 0) {
            const Json& rot = regipel_object(m, "rot", mw);
            const long long dims = regipel_int(rot, "dims", mw + "rot.", 0);
            const double base = regipel_number(rot, "base", mw + "rot.");
            if (dims % 2 || dims > rot_dim) throw ConfigError("config.json: " + mw + "'rot.dims' must be even and at most 'rot_dim'");
            if (!(base > 0)) throw ConfigError("config.json: " + mw + "'rot.base' must be positive");
            mixer.set("rot", Json::object().set("base", base).set("dims", dims));
        } else {
            mixer.set("rot", Json());
        }
        mixer.set("sink", m.get_bool("sink", true)).set("gate", m.get_bool("gate", true));
        Json mlp;
        if (!l["mlp"].is_null()) {
            const Json& f = regipel_object(l, "mlp", where);
            const std::string fw = where + "mlp.";
            const std::string kind = f.get_string("kind", "");
            if (kind != "moe") throw ConfigError("config.json: " + fw + "'kind' is '" + kind + "'; known kinds are ['moe']");
            const Json& router = regipel_object(f, "router", fw);
            const long long experts = regipel_int(router, "experts", fw + "router."), top = regipel_int(router, "top", fw + "router.");
            if (top > experts) throw ConfigError("config.json: " + fw + "'router.top' exceeds 'router.experts'");
            if (experts > 512) throw ConfigError("config.json: " + fw + "'router.experts' may be at most 512");
            mlp = Json::object().set("kind", kind)
                      .set("expert", Json::object().set("ff", regipel_int(regipel_object(f, "expert", fw), "ff", fw + "expert.")))
                      .set("router", Json::object().set("experts", experts).set("top", top));
        }
        layers.push(Json::object().set("type", type).set("mixer", mixer).set("mlp", mlp));
    }
    out.set("layers", layers);
    const long long n_layers = static_cast<long long>(layers.size());
    long long start = 0, stop = 0, times = 1;
    if (!raw["loop"].is_null()) {
        const Json& loop = regipel_object(raw, "loop", "");
        start = regipel_int(loop, "start", "loop.", 0);
        stop = regipel_int(loop, "stop", "loop.", 0);
        times = regipel_int(loop, "times", "loop.", 0);
        if (start > stop || stop > n_layers)
            throw ConfigError("config.json: 'loop' must satisfy 0 <= start <= stop <= " + std::to_string(n_layers));
    }
    out.set("loop", Json::object().set("start", start).set("stop", stop).set("times", times));
    for (const char* key : {"bos_token_id", "eos_token_id"})
        if (!raw[key].is_null()) out.set(key, raw[key]);
    return out;
}

ModelSpec regipel_build_spec(const Json& c) {
    const long long W = c["width"].as_int();
    const double eps = c["norm"]["eps"].as_double();
    const bool hyper = !c["streams"].is_null();
    const long long S = hyper ? c["streams"].as_int() : 1;
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "rmsnorm";
        p.params = Json::object().set("width", W).set("eps", eps).set("weight_offset", 1.0);
        p.tensors = {{"weight", name}};
        return p;
    };
    auto link = [&](const std::string& prefix) {
        PartSpec p;
        p.kind = "hyper_link";
        p.params = Json::object().set("streams", S);
        p.tensors = {{"in", prefix + ".in"}, {"out", prefix + ".out"}, {"mix", prefix + ".mix"}};
        return p;
    };
    ModelSpec spec;
    int i = 0;
    for (const Json& l : c["layers"].items()) {
        const std::string p = "l" + std::to_string(i) + ".";
        const Json& m = l["mixer"];
        LayerSpec layer;
        layer.arrangement = hyper ? "hyper_connections" : "pre_norm";
        layer.mixer.kind = "latent_attention";
        layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("dim", m["dim"])
                                 .set("rot_dim", m["rot_dim"]).set("vdim", m["vdim"]).set("kv_rank", m["kv_rank"])
                                 .set("scale", m["scale"]).set("eps", eps).set("sink", m["sink"]).set("gate", m["gate"]);
        if (!m["rot"].is_null() && m["rot"]["dims"].as_int() > 0) {
            PartSpec rope;
            rope.kind = "rope";
            rope.params = Json::object().set("theta", m["rot"]["base"]).set("rotary_dim", m["rot"]["dims"])
                              .set("head_dim", m["rot_dim"]).set("pairing", "neighbours");
            layer.mixer.params.set("position", rope.to_json());
        }
        layer.mixer.tensors = {{"q", p + "mix.q"},   {"dkv", p + "mix.dkv"}, {"dkv_norm", p + "mix.dkv.norm"},
                               {"uk", p + "mix.uk"}, {"uv", p + "mix.uv"},   {"o", p + "mix.o"}};
        if (m["sink"].as_bool()) layer.mixer.tensors.emplace_back("sink", p + "mix.sink");
        if (m["gate"].as_bool()) layer.mixer.tensors.emplace_back("g", p + "mix.g");
        layer.mixer_norm = norm(p + "norm1");
        if (hyper) layer.mixer_link = link(p + "hc1");
        if (l["mlp"].is_null()) {
            layer.ffn.kind = "none";
            layer.ffn_norm.kind = "identity";
        } else {
            const Json& f = l["mlp"];
            const long long experts = f["router"]["experts"].as_int();
            layer.ffn.kind = "routed_experts";
            layer.ffn.params = Json::object().set("width", W).set("ff", f["expert"]["ff"]).set("experts", experts)
                                   .set("top", f["router"]["top"]).set("score", "sigmoid").set("renormalize", false)
                                   .set("weight_on", "input");
            layer.ffn.tensors = {{"router", p + "mlp.router"}};
            for (long long e = 0; e < experts; ++e) {
                const std::string ep = p + "mlp.e" + std::to_string(e) + ".", n = std::to_string(e);
                layer.ffn.tensors.emplace_back("gate." + n, ep + "gate");
                layer.ffn.tensors.emplace_back("up." + n, ep + "up");
                layer.ffn.tensors.emplace_back("down." + n, ep + "down");
            }
            layer.ffn_norm = norm(p + "norm2");
            if (hyper) layer.ffn_link = link(p + "hc2");
        }
        spec.layers.push_back(std::move(layer));
        ++i;
    }
    const int n_layers = i;
    const int start = static_cast<int>(c["loop"]["start"].as_int()), stop = static_cast<int>(c["loop"]["stop"].as_int());
    const int times = static_cast<int>(c["loop"]["times"].as_int());
    for (int l = 0; l < start; ++l) spec.order.push_back(RunStep{l, {}});
    for (int pass = 0; pass < times; ++pass)
        for (int l = start; l < stop; ++l) spec.order.push_back(RunStep{l, {}});
    for (int l = stop; l < n_layers; ++l) spec.order.push_back(RunStep{l, {}});
    spec.architecture = "Regipel";
    spec.vocab_size = static_cast<int>(c["vocab"].as_int());
    spec.hidden_size = static_cast<int>(W);
    spec.max_context = static_cast<int>(c["max_context"].as_int());
    spec.streams = static_cast<int>(S);
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab"]).set("width", W).set("scale", c["embedding"]["scale"]);
    spec.embedding.tensors = {{"table", "embed"}};
    spec.head.kind = "tied_head";
    spec.head.params = Json::object().set("vocab", c["vocab"]).set("width", W).set("scale", c["logit_scale"]);
    spec.final_norm = norm("final.norm");
    if (c["eos_token_id"].is_array())
        for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    else if (c["eos_token_id"].is_int())
        spec.eos_token_ids.push_back(static_cast<int>(c["eos_token_id"].as_int()));
    if (c["bos_token_id"].is_int()) spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

}  // namespace

// ---------------------------------------------------------------------------- Kifetar
// A decoder that norms every sub-layer's input and output (layer norms with weight and bias),
// mixes by attention with sigmoid weights inside a sliding window or by a gated delta rule, and
// may run a range of its layers several times, taking the embedding's rows in again before
// every run of the range.  config.json describes every layer by itself:
//   {"architecture": "Kifetar", "vocab", "width", "norm": {"eps"},
//    "loop": {"start", "stop", "times"} (layers start..stop-1 run `times` times in a row with the
//    same weights and a cache or state of their own each time; before the first layer of every
//    such run the stream becomes W_in [stream ; embedding rows], tensor "loop.in"),
//    "max_context" (an engine limit; optional),
//    "layers": [{"type": "attention",
//                "mixer": {"heads", "kv_heads", "dim", "vdim" (= dim: the values are the keys as
//                          projected), "scale", "mask": {"size"} (absent: every earlier key),
//                          "rot": {"base", "dims", "scaling": {"factor", "low", "high", "original"}}
//                          (absent, or dims 0: no rotation; scaling optional)},
//                "mlp": null | {"kind": "dense", "ff"}},
//               {"type": "delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": ...}]}
// The output head is the embedding table.
// Tensors: embed, loop.in, final.norm(.b), l<i>.norm1|norm1b|norm2|norm2b(.b),
// attention: l<i>.mix.{q, q.b, k, k.b, q.norm, k.norm, temp, pb, g, o};
// delta: l<i>.mix.{q, q.conv, k, k.conv, v, v.conv, b, a, A_log, dt_bias, norm, g, o};
// l<i>.mlp.{gate, up, down}.
namespace {

Json kifetar_read_config(const Json& raw, const TensorShapes*) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json out = Json::object();
    out.set("architecture", "Kifetar");
    out.set("vocab", regipel_int(raw, "vocab", ""));
    const long long width = regipel_int(raw, "width", "");
    out.set("width", width);
    const double eps = regipel_number(regipel_object(raw, "norm", ""), "eps", "norm.");
    if (!(eps > 0)) throw ConfigError("config.json: 'norm.eps' must be positive");
    out.set("norm", Json::object().set("eps", eps));
    out.set("max_context", raw["max_context"].is_null() ? 131072LL : regipel_int(raw, "max_context", ""));
    if (!raw["layers"].is_array() || raw["layers"].size() == 0) throw ConfigError("config.json: 'layers' must be a list of layers");
    Json layers = Json::array();
    int i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string where = "layers[" + std::to_string(i++) + "].";
        if (!l.is_object()) throw ConfigError("config.json: " + where + " must be an object");
        const std::string type = l.get_string("type", "");
        const Json& m = regipel_object(l, "mixer", where);
        const std::string mw = where + "mixer.";
        Json mixer = Json::object();
        const long long heads = regipel_int(m, "heads", mw), kv_heads = regipel_int(m, "kv_heads", mw);
        if (heads % kv_heads) throw ConfigError("config.json: " + mw + "'heads' must be a multiple of 'kv_heads'");
        mixer.set("heads", heads).set("kv_heads", kv_heads).set("dim", regipel_int(m, "dim", mw)).set("vdim", regipel_int(m, "vdim", mw));
        if (type == "attention") {
            if (mixer["vdim"].as_int() != mixer["dim"].as_int())
                throw ConfigError("config.json: " + mw + "'vdim' must equal 'dim': the values are the keys as projected");
            if (mixer["dim"].as_int() % 2) throw ConfigError("config.json: " + mw + "'dim' must be even");
            mixer.set("scale", regipel_number(m, "scale", mw));
            mixer.set("mask", m["mask"].is_null() ? Json() : Json::object().set("size", regipel_int(regipel_object(m, "mask", mw), "size", mw + "mask.")));
            Json rot;
            if (!m["rot"].is_null()) {
                const Json& r = regipel_object(m, "rot", mw);
                const long long dims = regipel_int(r, "dims", mw + "rot.", 0);
                if (dims % 2 || dims > mixer["dim"].as_int()) throw ConfigError("config.json: " + mw + "'rot.dims' must be even and at most 'dim'");
                if (dims > 0) {
                    const double base = regipel_number(r, "base", mw + "rot.");
                    if (!(base > 0)) throw ConfigError("config.json: " + mw + "'rot.base' must be positive");
                    rot = Json::object().set("base", base).set("dims", dims);
                    if (!r["scaling"].is_null()) {
                        const Json& sc = regipel_object(r, "scaling", mw + "rot.");
                        const std::string sw = mw + "rot.scaling.";
                        Json scaling = Json::object();
                        for (const char* key : {"factor", "low", "high", "original"}) scaling.set(key, regipel_number(sc, key, sw));
                        if (!(scaling["factor"].as_double() > 0) || !(scaling["low"].as_double() > 0) ||
                            !(scaling["high"].as_double() > scaling["low"].as_double()) || !(scaling["original"].as_double() > 0))
                            throw ConfigError("config.json: " + sw + " needs factor > 0, 0 < low < high and original > 0");
                        rot.set("scaling", scaling);
                    }
                }
            }
            mixer.set("rot", rot);
        } else if (type == "delta") {
            mixer.set("conv", regipel_int(m, "conv", mw));
        } else {
            throw ConfigError("config.json: " + where + "'type' is '" + type + "'; known types are ['attention', 'delta']");
        }
        Json mlp;
        if (!l["mlp"].is_null()) {
            const Json& f = regipel_object(l, "mlp", where);
            const std::string kind = f.get_string("kind", "");
            if (kind != "dense") throw ConfigError("config.json: " + where + "mlp.'kind' is '" + kind + "'; known kinds are ['dense']");
            mlp = Json::object().set("kind", kind).set("ff", regipel_int(f, "ff", where + "mlp."));
        }
        layers.push(Json::object().set("type", type).set("mixer", mixer).set("mlp", mlp));
    }
    out.set("layers", layers);
    const long long n_layers = static_cast<long long>(layers.size());
    long long start = 0, stop = 0, times = 1;
    if (!raw["loop"].is_null()) {
        const Json& loop = regipel_object(raw, "loop", "");
        start = regipel_int(loop, "start", "loop.", 0);
        stop = regipel_int(loop, "stop", "loop.", 0);
        times = regipel_int(loop, "times", "loop.", 0);
        if (start > stop || stop > n_layers)
            throw ConfigError("config.json: 'loop' must satisfy 0 <= start <= stop <= " + std::to_string(n_layers));
    }
    out.set("loop", Json::object().set("start", start).set("stop", stop).set("times", times));
    for (const char* key : {"bos_token_id", "eos_token_id"})
        if (!raw[key].is_null()) out.set(key, raw[key]);
    return out;
}

ModelSpec kifetar_build_spec(const Json& c) {
    const long long W = c["width"].as_int();
    const double eps = c["norm"]["eps"].as_double();
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "layernorm";
        p.params = Json::object().set("width", W).set("eps", eps).set("bias", true);
        p.tensors = {{"weight", name}, {"bias", name + ".b"}};
        return p;
    };
    ModelSpec spec;
    int i = 0;
    for (const Json& l : c["layers"].items()) {
        const std::string p = "l" + std::to_string(i) + ".";
        const Json& m = l["mixer"];
        LayerSpec layer;
        layer.arrangement = "sandwich_norm";
        if (l["type"].as_string() == "attention") {
            layer.mixer.kind = "sigmoid_attention";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("kv_heads", m["kv_heads"])
                                     .set("head_dim", m["dim"]).set("scale", m["scale"]).set("eps", eps).set("qk_norm", true)
                                     .set("bias", true).set("values", "keys").set("temperature", true).set("score_bias", true)
                                     .set("head_gate", true);
            if (!m["mask"].is_null()) layer.mixer.params.set("window", m["mask"]["size"]);
            if (!m["rot"].is_null()) {
                PartSpec rope;
                rope.kind = "rope";
                rope.params = Json::object().set("theta", m["rot"]["base"]).set("rotary_dim", m["rot"]["dims"])
                                  .set("head_dim", m["dim"]).set("pairing", "halves");
                if (!m["rot"]["scaling"].is_null()) rope.params.set("scaling", m["rot"]["scaling"]);
                layer.mixer.params.set("position", rope.to_json());
            }
            layer.mixer.tensors = {{"q", p + "mix.q"},           {"k", p + "mix.k"},           {"o", p + "mix.o"},
                                   {"q_bias", p + "mix.q.b"},    {"k_bias", p + "mix.k.b"},    {"q_norm", p + "mix.q.norm"},
                                   {"k_norm", p + "mix.k.norm"}, {"temp", p + "mix.temp"},     {"pb", p + "mix.pb"},
                                   {"g", p + "mix.g"}};
        } else {
            layer.mixer.kind = "gated_delta_rule";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("kv_heads", m["kv_heads"])
                                     .set("dim", m["dim"]).set("vdim", m["vdim"]).set("taps", m["conv"]).set("eps", eps);
            layer.mixer.tensors = {{"q", p + "mix.q"},   {"k", p + "mix.k"},         {"v", p + "mix.v"},
                                   {"q_conv", p + "mix.q.conv"}, {"k_conv", p + "mix.k.conv"}, {"v_conv", p + "mix.v.conv"},
                                   {"b", p + "mix.b"},   {"a", p + "mix.a"},         {"A_log", p + "mix.A_log"},
                                   {"dt_bias", p + "mix.dt_bias"}, {"norm", p + "mix.norm"}, {"g", p + "mix.g"},
                                   {"o", p + "mix.o"}};
        }
        layer.mixer_norm = norm(p + "norm1");
        layer.mixer_post_norm = norm(p + "norm1b");
        if (l["mlp"].is_null()) {
            layer.ffn.kind = "none";
            layer.ffn_norm.kind = "identity";
        } else {
            layer.ffn.kind = "swiglu";
            layer.ffn.params = Json::object().set("width", W).set("ff", l["mlp"]["ff"]);
            layer.ffn.tensors = {{"gate", p + "mlp.gate"}, {"up", p + "mlp.up"}, {"down", p + "mlp.down"}};
            layer.ffn_norm = norm(p + "norm2");
            layer.ffn_post_norm = norm(p + "norm2b");
        }
        spec.layers.push_back(std::move(layer));
        ++i;
    }
    const int n_layers = i;
    const int start = static_cast<int>(c["loop"]["start"].as_int()), stop = static_cast<int>(c["loop"]["stop"].as_int());
    const int times = static_cast<int>(c["loop"]["times"].as_int());
    for (int l = 0; l < start; ++l) spec.order.push_back(RunStep{l, {}, false});
    bool reinjects = false;
    for (int pass = 0; pass < times; ++pass)
        for (int l = start; l < stop; ++l) {
            spec.order.push_back(RunStep{l, {}, l == start});
            reinjects = true;
        }
    for (int l = stop; l < n_layers; ++l) spec.order.push_back(RunStep{l, {}, false});
    if (reinjects) {
        spec.reinjection.kind = "linear_concat";
        spec.reinjection.params = Json::object().set("width", W);
        spec.reinjection.tensors = {{"weight", "loop.in"}};
    }
    spec.architecture = "Kifetar";
    spec.vocab_size = static_cast<int>(c["vocab"].as_int());
    spec.hidden_size = static_cast<int>(W);
    spec.max_context = static_cast<int>(c["max_context"].as_int());
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab"]).set("width", W);
    spec.embedding.tensors = {{"table", "embed"}};
    spec.head.kind = "tied_head";
    spec.head.params = Json::object().set("vocab", c["vocab"]).set("width", W);
    spec.final_norm = norm("final.norm");
    if (c["eos_token_id"].is_array())
        for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    else if (c["eos_token_id"].is_int())
        spec.eos_token_ids.push_back(static_cast<int>(c["eos_token_id"].as_int()));
    if (c["bos_token_id"].is_int()) spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

}  // namespace

// ---------------------------------------------------------------------------- Kivorax
// A decoder whose layers read one norm for both sub-layers (x += mixer(norm(x)) + ff(norm(x))),
// add a gated row of a per-layer token table behind them, and hand on a weighted sum of the
// results of all layers so far.  config.json describes every layer by itself:
//   {"architecture": "Kivorax", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"} (absent: 1),
//    "token_side": {"dim"} (absent: no token input), "max_context" (an engine limit; optional),
//    "layers": [{"type": "parallel",
//                "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "q_temp": {"coef", "every"} (optional)},
//                          "right": {"width", "blocks", "conv"}},
//                "mlp": null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}},
//               {"type": "channel_delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": ...},
//               {"type": "gla", "mixer": {"heads", "dim", "vdim", "tau"}, "mlp": ...}]}
// The widths of the two-step projections (a1/a2 of the decays, g1/g2 of the delta rule's gate) are the
// checkpoint's ("decay_rank" / "gate_rank" of a mixer where no checkpoint is at hand, else 16); a layer
// mixes over depth where the checkpoint holds its "dwa" (without a checkpoint: every layer does).
// Tensors: embed, side.embed, final.norm, head, l<i>.norm1, l<i>.dwa, l<i>.side.{gate,proj,norm},
// parallel: l<i>.mix.left.{q,k,v,r1,r2,g,o,out}, l<i>.mix.right.{y,y.b,x,x.b,conv,conv.b,ra,ra.b,ri,ri.b,lam,o,out};
// channel_delta: l<i>.mix.{q,q.conv,k,k.conv,v,v.conv,b,A_log,dt_bias,a1,a2,g1,g2,norm,o};
// gla: l<i>.mix.{q,k,v,g,a1,a2,a2.b,norm,o}; l<i>.mlp.{up,up.b,down,down.b} or l<i>.mlp.router, l<i>.mlp.e<j>.{up,down}.
namespace {

// the number of rows of a checkpoint's tensor, or of the mixer's own key, or 16
long long kivorax_rank(const TensorShapes* shapes, const std::string& tensor, const Json& mixer, const char* key,
                       const std::string& where) {
    if (shapes) {
        auto it = shapes->find(tensor);
        if (it != shapes->end() && !it->second.empty() && it->second[0] > 0) return it->second[0];
    }
    if (!mixer[key].is_null()) return regipel_int(mixer, key, where);
    return 16;
}

Json kivorax_read_config(const Json& raw, const TensorShapes* shapes) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json out = Json::object();
    out.set("architecture", "Kivorax");
    out.set("vocab", regipel_int(raw, "vocab", ""));
    const long long width = regipel_int(raw, "width", "");
    out.set("width", width);
    const double eps = regipel_number(regipel_object(raw, "norm", ""), "eps", "norm.");
    if (!(eps > 0)) throw ConfigError("config.json: 'norm.eps' must be positive");
    out.set("norm", Json::object().set("eps", eps));
    double embedding_scale = 1.0;
    if (!raw["embedding"].is_null()) embedding_scale = regipel_number(regipel_object(raw, "embedding", ""), "scale", "embedding.");
    out.set("embedding", Json::object().set("scale", embedding_scale));
    out.set("token_side", raw["token_side"].is_null()
                              ? Json()
                              : Json::object().set("dim", regipel_int(regipel_object(raw, "token_side", ""), "dim", "token_side.")));
    out.set("max_context", raw["max_context"].is_null() ? 131072LL : regipel_int(raw, "max_context", ""));
    if (!raw["layers"].is_array() || raw["layers"].size() == 0) throw ConfigError("config.json: 'layers' must be a list of layers");
    Json layers = Json::array();
    int i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string prefix = "l" + std::to_string(i) + ".";
        const std::string where = "layers[" + std::to_string(i++) + "].";
        if (!l.is_object()) throw ConfigError("config.json: " + where + " must be an object");
        const std::string type = l.get_string("type", "");
        const Json& m = regipel_object(l, "mixer", where);
        const std::string mw = where + "mixer.";
        Json mixer = Json::object();
        if (type == "parallel") {
            const Json& a = regipel_object(m, "left", mw);
            const std::string aw = mw + "left.";
            const long long heads = regipel_int(a, "heads", aw), kv_heads = regipel_int(a, "kv_heads", aw);
            if (heads % kv_heads) throw ConfigError("config.json: " + aw + "'heads' must be a multiple of 'kv_heads'");
            Json left = Json::object().set("heads", heads).set("kv_heads", kv_heads).set("dim", regipel_int(a, "dim", aw))
                            .set("vdim", regipel_int(a, "vdim", aw)).set("scale", regipel_number(a, "scale", aw));
            if (left["vdim"].as_int() > 256) throw ConfigError("config.json: " + aw + "'vdim' may be at most 256");
            Json q_temp;
            if (!a["q_temp"].is_null()) {
                const Json& qt = regipel_object(a, "q_temp", aw);
                q_temp = Json::object().set("coef", regipel_number(qt, "coef", aw + "q_temp.")).set("every", regipel_int(qt, "every", aw + "q_temp."));
            }
            left.set("q_temp", q_temp);
            const Json& r = regipel_object(m, "right", mw);
            const std::string rw = mw + "right.";
            const long long inner = regipel_int(r, "width", rw), blocks = regipel_int(r, "blocks", rw);
            if (inner % blocks) throw ConfigError("config.json: " + rw + "'width' must be a multiple of 'blocks'");
            Json right = Json::object().set("width", inner).set("blocks", blocks).set("conv", regipel_int(r, "conv", rw));
            mixer.set("left", left).set("right", right);
        } else if (type == "channel_delta") {
            const long long heads = regipel_int(m, "heads", mw), kv_heads = regipel_int(m, "kv_heads", mw);
            if (heads % kv_heads) throw ConfigError("config.json: " + mw + "'heads' must be a multiple of 'kv_heads'");
            mixer.set("heads", heads).set("kv_heads", kv_heads).set("dim", regipel_int(m, "dim", mw)).set("vdim", regipel_int(m, "vdim", mw))
                .set("conv", regipel_int(m, "conv", mw))
                .set("decay_rank", kivorax_rank(shapes, prefix + "mix.a1", m, "decay_rank", mw))
                .set("gate_rank", kivorax_rank(shapes, prefix + "mix.g1", m, "gate_rank", mw));
            if (mixer["dim"].as_int() > 256) throw ConfigError("config.json: " + mw + "'dim' may be at most 256");
        } else if (type == "gla") {
            mixer.set("heads", regipel_int(m, "heads", mw)).set("dim", regipel_int(m, "dim", mw)).set("vdim", regipel_int(m, "vdim", mw))
                .set("tau", regipel_number(m, "tau", mw)).set("decay_rank", kivorax_rank(shapes, prefix + "mix.a1", m, "decay_rank", mw));
            if (!(mixer["tau"].as_double() > 0)) throw ConfigError("config.json: " + mw + "'tau' must be positive");
            if (mixer["dim"].as_int() > 256) throw ConfigError("config.json: " + mw + "'dim' may be at most 256");
        } else {
            throw ConfigError("config.json: " + where + "'type' is '" + type + "'; known types are ['parallel', 'channel_delta', 'gla']");
        }
        Json mlp;
        if (!l["mlp"].is_null()) {
            const Json& f = regipel_object(l, "mlp", where);
            const std::string fw = where + "mlp.";
            const std::string kind = f.get_string("kind", "");
            if (kind == "dense") {
                mlp = Json::object().set("kind", kind).set("ff", regipel_int(f, "ff", fw));
            } else if (kind == "moe") {
                const Json& router = regipel_object(f, "router", fw);
                const long long experts = regipel_int(router, "experts", fw + "router."), top = regipel_int(router, "top", fw + "router.");
                if (top > experts) throw ConfigError("config.json: " + fw + "'router.top' exceeds 'router.experts'");
                if (experts > 512) throw ConfigError("config.json: " + fw + "'router.experts' may be at most 512");
                mlp = Json::object().set("kind", kind)
                          .set("expert", Json::object().set("ff", regipel_int(regipel_object(f, "expert", fw), "ff", fw + "expert.")))
                          .set("router", Json::object().set("experts", experts).set("top", top));
            } else {
                throw ConfigError("config.json: " + fw + "'kind' is '" + kind + "'; known kinds are ['dense', 'moe']");
            }
        }
        const bool depth = shapes ? shapes->count(prefix + "dwa") > 0 : l.get_bool("depth_average", true);
        layers.push(Json::object().set("type", type).set("mixer", mixer).set("mlp", mlp).set("depth_average", depth));
    }
    out.set("layers", layers);
    for (const char* key : {"bos_token_id", "eos_token_id"})
        if (!raw[key].is_null()) out.set(key, raw[key]);
    return out;
}

ModelSpec kivorax_build_spec(const Json& c) {
    const long long W = c["width"].as_int();
    const double eps = c["norm"]["eps"].as_double();
    const long long n_layers = static_cast<long long>(c["layers"].size());
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "rmsnorm";
        p.params = Json::object().set("width", W).set("eps", eps);
        p.tensors = {{"weight", name}};
        return p;
    };
    ModelSpec spec;
    int i = 0;
    for (const Json& l : c["layers"].items()) {
        const std::string p = "l" + std::to_string(i) + ".";
        const Json& m = l["mixer"];
        const std::string type = l["type"].as_string();
        LayerSpec layer;
        layer.arrangement = "parallel";
        if (type == "parallel") {
            const Json& a = m["left"];
            const Json& r = m["right"];
            PartSpec left, right;
            left.kind = "biased_attention";
            left.params = Json::object().set("width", W).set("heads", a["heads"]).set("kv_heads", a["kv_heads"]).set("head_dim", a["dim"])
                              .set("v_dim", a["vdim"]).set("scale", a["scale"]).set("distance_bias", true).set("gate", "sigmoid");
            if (!a["q_temp"].is_null()) left.params.set("query_temperature", a["q_temp"]);
            right.kind = "linear_recurrent_unit";
            right.params = Json::object().set("width", W).set("inner", r["width"]).set("blocks", r["blocks"]).set("taps", r["conv"])
                               .set("decay_scale", 8.0);
            layer.mixer.kind = "normed_pair";
            layer.mixer.params = Json::object().set("width", W).set("eps", eps).set("factor", 0.5).set("left", left.to_json())
                                     .set("right", right.to_json());
            const std::string lp = p + "mix.left.", rp = p + "mix.right.";
            layer.mixer.tensors = {{"left_out", lp + "out"}, {"right_out", rp + "out"},
                                   {"left.q", lp + "q"},     {"left.k", lp + "k"},   {"left.v", lp + "v"},   {"left.o", lp + "o"},
                                   {"left.r1", lp + "r1"},   {"left.r2", lp + "r2"}, {"left.g", lp + "g"},
                                   {"right.y", rp + "y"},    {"right.y_bias", rp + "y.b"}, {"right.x", rp + "x"}, {"right.x_bias", rp + "x.b"},
                                   {"right.conv", rp + "conv"}, {"right.conv_bias", rp + "conv.b"}, {"right.ra", rp + "ra"},
                                   {"right.ra_bias", rp + "ra.b"}, {"right.ri", rp + "ri"}, {"right.ri_bias", rp + "ri.b"},
                                   {"right.lam", rp + "lam"}, {"right.o", rp + "o"}};
        } else if (type == "channel_delta") {
            layer.mixer.kind = "gated_delta_rule";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("kv_heads", m["kv_heads"]).set("dim", m["dim"])
                                     .set("vdim", m["vdim"]).set("taps", m["conv"]).set("eps", eps).set("decay", "channel")
                                     .set("decay_rank", m["decay_rank"]).set("gate", "sigmoid").set("gate_rank", m["gate_rank"]);
            layer.mixer.tensors = {{"q", p + "mix.q"},     {"k", p + "mix.k"},     {"v", p + "mix.v"},   {"q_conv", p + "mix.q.conv"},
                                   {"k_conv", p + "mix.k.conv"}, {"v_conv", p + "mix.v.conv"}, {"b", p + "mix.b"}, {"A_log", p + "mix.A_log"},
                                   {"dt_bias", p + "mix.dt_bias"}, {"a1", p + "mix.a1"}, {"a2", p + "mix.a2"}, {"g1", p + "mix.g1"},
                                   {"g2", p + "mix.g2"},   {"norm", p + "mix.norm"}, {"o", p + "mix.o"}};
        } else {
            layer.mixer.kind = "gated_linear_attention";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("dim", m["dim"]).set("vdim", m["vdim"])
                                     .set("tau", m["tau"]).set("decay_rank", m["decay_rank"]).set("eps", eps);
            layer.mixer.tensors = {{"q", p + "mix.q"},   {"k", p + "mix.k"},   {"v", p + "mix.v"},       {"g", p + "mix.g"},
                                   {"a1", p + "mix.a1"}, {"a2", p + "mix.a2"}, {"a2_bias", p + "mix.a2.b"}, {"norm", p + "mix.norm"},
                                   {"o", p + "mix.o"}};
        }
        layer.mixer_norm = norm(p + "norm1");
        layer.ffn_norm.kind = "identity";
        if (l["mlp"].is_null()) {
            layer.ffn.kind = "none";
        } else if (l["mlp"]["kind"].as_string() == "dense") {
            layer.ffn.kind = "mlp";
            layer.ffn.params = Json::object().set("width", W).set("ff", l["mlp"]["ff"]).set("activation", "gelu_tanh").set("bias", true);
            layer.ffn.tensors = {{"up", p + "mlp.up"}, {"up_bias", p + "mlp.up.b"}, {"down", p + "mlp.down"}, {"down_bias", p + "mlp.down.b"}};
        } else {
            const Json& f = l["mlp"];
            const long long experts = f["router"]["experts"].as_int();
            layer.ffn.kind = "routed_experts";
            layer.ffn.params = Json::object().set("width", W).set("ff", f["expert"]["ff"]).set("experts", experts)
                                   .set("top", f["router"]["top"]).set("score", "softmax").set("renormalize", false)
                                   .set("weight_on", "output").set("gated", false).set("activation", "relu2");
            layer.ffn.tensors = {{"router", p + "mlp.router"}};
            for (long long e = 0; e < experts; ++e) {
                const std::string ep = p + "mlp.e" + std::to_string(e) + ".", n = std::to_string(e);
                layer.ffn.tensors.emplace_back("up." + n, ep + "up");
                layer.ffn.tensors.emplace_back("down." + n, ep + "down");
            }
        }
        if (!c["token_side"].is_null()) {
            const long long dim = c["token_side"]["dim"].as_int();
            layer.token_input.kind = "gated_table";
            layer.token_input.params = Json::object().set("width", W).set("vocab", c["vocab"]).set("dim", dim).set("offset", dim * i)
                                           .set("table_width", dim * n_layers).set("eps", eps);
            layer.token_input.tensors = {{"table", "side.embed"}, {"gate", p + "side.gate"}, {"proj", p + "side.proj"},
                                         {"norm", p + "side.norm"}};
        }
        if (l["depth_average"].as_bool()) {
            layer.depth_mix.kind = "weighted_history";
            layer.depth_mix.params = Json::object().set("entries", static_cast<long long>(i) + 2);
            layer.depth_mix.tensors = {{"weights", p + "dwa"}};
        }
        spec.layers.push_back(std::move(layer));
        spec.order.push_back(RunStep{i, {}, false});
        ++i;
    }
    spec.architecture = "Kivorax";
    spec.vocab_size = static_cast<int>(c["vocab"].as_int());
    spec.hidden_size = static_cast<int>(W);
    spec.max_context = static_cast<int>(c["max_context"].as_int());
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab"]).set("width", W).set("scale", c["embedding"]["scale"]);
    spec.embedding.tensors = {{"table", "embed"}};
    spec.head.kind = "linear_head";
    spec.head.params = Json::object().set("vocab", c["vocab"]).set("width", W);
    spec.head.tensors = {{"weight", "head"}};
    spec.final_norm = norm("final.norm");
    if (c["eos_token_id"].is_array())
        for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    else if (c["eos_token_id"].is_int())
        spec.eos_token_ids.push_back(static_cast<int>(c["eos_token_id"].as_int()));
    if (c["bos_token_id"].is_int()) spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

}  // namespace

// ---------------------------------------------------------------------------- Vabuzen
// A decoder whose sub-layers are wrapped in "dynamic tanh" norms (tanh(alpha x) w + b, no statistics)
// before and after, their output added times a constant; two kinds of attention; dense or routed
// feed-forwards; a range of layers that may run several times, a learned vector of the run (and, from the
// second run on, the embedding's rows) added to the stream before each run; logits bent by a tanh.
// config.json describes every layer by itself:
//   {"architecture": "Vabuzen", "vocab", "width", "norm": {"eps"}, "residual_mult" (absent: 1),
//    "logit_softcap" (absent or null: none), "loop": {"start", "stop", "times"} (absent: none),
//    "max_context" (an engine limit; optional),
//    "layers": [{"type": "attention",
//                "mixer": {"heads", "kv_heads", "dim", "vdim" (absent: dim), "scale", "conv" (taps; absent or 0: none),
//                          "rot": {"base", "dims"} (absent, or dims 0: no rotation; neighbouring values pair),
//                          "mask": {"size", "keep_first" (absent: 0)} (absent: every earlier key)},
//                "mlp": null | {"kind": "dense", "ff"}
//                            | {"kind": "moe", "expert": {"ff"}, "shared": {"ff"} (absent or null: none),
//                               "router": {"experts", "top", "scale" (absent: 1), "groups": {"count", "keep"} (absent: one group)}}},
//               {"type": "latent_attention",
//                "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot": {"base", "dims"}} (the two halves
//                          of the rotated part pair), "mlp": ...}]}
// The attention's softmax has a one more in its denominator; the latent attention's is the ordinary one.
// Tensors: embed, head, loop.step [times, width], final.norm(.b, .alpha), l<i>.norm1|norm1b|norm2|norm2b(.b, .alpha),
// attention: l<i>.mix.{q, k, v, o, q.conv, k.conv, v.conv}; latent: l<i>.mix.{q, dkv, dkv.norm, uk, uv, o};
// l<i>.mlp.{up, up.b, down, down.b} or l<i>.mlp.router, l<i>.mlp.e<j>.{gate, up, down}, l<i>.mlp.shared.{gate, up, down}.
namespace {

Json vabuzen_rot(const Json& m, const std::string& mw, long long most, const char* most_name) {
    if (m["rot"].is_null()) return Json();
    const Json& r = regipel_object(m, "rot", mw);
    const long long dims = regipel_int(r, "dims", mw + "rot.", 0);
    if (dims % 2 || dims > most) throw ConfigError("config.json: " + mw + "'rot.dims' must be even and at most '" + most_name + "'");
    if (dims == 0) return Json();
    const double base = regipel_number(r, "base", mw + "rot.");
    if (!(base > 0)) throw ConfigError("config.json: " + mw + "'rot.base' must be positive");
    return Json::object().set("base", base).set("dims", dims);
}

Json vabuzen_read_config(const Json& raw, const TensorShapes*) {
    if (!raw.is_object()) throw ConfigError("config.json is not an object");
    Json out = Json::object();
    out.set("architecture", "Vabuzen");
    out.set("vocab", regipel_int(raw, "vocab", ""));
    const long long width = regipel_int(raw, "width", "");
    out.set("width", width);
    const double eps = regipel_number(regipel_object(raw, "norm", ""), "eps", "norm.");
    if (!(eps > 0)) throw ConfigError("config.json: 'norm.eps' must be positive");
    out.set("norm", Json::object().set("eps", eps));
    out.set("residual_mult", raw["residual_mult"].is_null() ? 1.0 : regipel_number(raw, "residual_mult", ""));
    if (raw["logit_softcap"].is_null()) {
        out.set("logit_softcap", Json());
    } else {
        const double cap = regipel_number(raw, "logit_softcap", "");
        if (!(cap > 0)) throw ConfigError("config.json: 'logit_softcap' must be positive");
        out.set("logit_softcap", cap);
    }
    out.set("max_context", raw["max_context"].is_null() ? 131072LL : regipel_int(raw, "max_context", ""));
    if (!raw["layers"].is_array() || raw["layers"].size() == 0) throw ConfigError("config.json: 'layers' must be a list of layers");
    Json layers = Json::array();
    int i = 0;
    for (const Json& l : raw["layers"].items()) {
        const std::string where = "layers[" + std::to_string(i++) + "].";
        if (!l.is_object()) throw ConfigError("config.json: " + where + " must be an object");
        const std::string type = l.get_string("type", "");
        const Json& m = regipel_object(l, "mixer", where);
        const std::string mw = where + "mixer.";
        Json mixer = Json::object();
        const long long heads = regipel_int(m, "heads", mw), dim = regipel_int(m, "dim", mw);
        mixer.set("heads", heads).set("dim", dim).set("scale", regipel_number(m, "scale", mw));
        if (type == "attention") {
            const long long kv_heads = m["kv_heads"].is_null() ? heads : regipel_int(m, "kv_heads", mw);
            if (heads % kv_heads) throw ConfigError("config.json: " + mw + "'heads' must be a multiple of 'kv_heads'");
            mixer.set("kv_heads", kv_heads).set("vdim", m["vdim"].is_null() ? dim : regipel_int(m, "vdim", mw));
            mixer.set("conv", m["conv"].is_null() ? 0LL : regipel_int(m, "conv", mw, 0));
            mixer.set("rot", vabuzen_rot(m, mw, dim, "dim"));
            Json mask;
            if (!m["mask"].is_null()) {
                const Json& k = regipel_object(m, "mask", mw);
                mask = Json::object().set("size", regipel_int(k, "size", mw + "mask."))
                           .set("keep_first", k["keep_first"].is_null() ? 0LL : regipel_int(k, "keep_first", mw + "mask.", 0));
            }
            mixer.set("mask", mask);
        } else if (type == "latent_attention") {
            const long long rot_dim = regipel_int(m, "rot_dim", mw, 0);
            mixer.set("rot_dim", rot_dim).set("vdim", regipel_int(m, "vdim", mw)).set("kv_rank", regipel_int(m, "kv_rank", mw));
            mixer.set("rot", rot_dim > 0 ? vabuzen_rot(m, mw, rot_dim, "rot_dim") : Json());
        } else {
            throw ConfigError("config.json: " + where + "'type' is '" + type + "'; known types are ['attention', 'latent_attention']");
        }
        Json mlp;
        if (!l["mlp"].is_null()) {
            const Json& f = regipel_object(l, "mlp", where);
            const std::string fw = where + "mlp.";
            const std::string kind = f.get_string("kind", "");
            if (kind == "dense") {
                mlp = Json::object().set("kind", kind).set("ff", regipel_int(f, "ff", fw));
            } else if (kind == "moe") {
                const Json& router = regipel_object(f, "router", fw);
                const std::string rw = fw + "router.";
                const long long experts = regipel_int(router, "experts", rw), top = regipel_int(router, "top", rw);
                if (top > experts) throw ConfigError("config.json: " + rw + "'top' exceeds 'experts'");
                if (experts > 512) throw ConfigError("config.json: " + rw + "'experts' may be at most 512");
                long long count = 1, keep = 1;
                if (!router["groups"].is_null()) {
                    const Json& g = regipel_object(router, "groups", rw);
                    count = regipel_int(g, "count", rw + "groups.");
                    keep = regipel_int(g, "keep", rw + "groups.");
                    if (count > 64 || experts % count || keep > count)
                        throw ConfigError("config.json: " + rw + "'groups.count' (at most 64) must divide 'experts', and 'groups.keep' may be at most 'groups.count'");
                    if (top > keep * (experts / count))
                        throw ConfigError("config.json: " + rw + "the kept groups hold fewer experts than 'top'");
                }
                mlp = Json::object().set("kind", kind)
                          .set("expert", Json::object().set("ff", regipel_int(regipel_object(f, "expert", fw), "ff", fw + "expert.")))
                          .set("router", Json::object().set("experts", experts).set("top", top)
                                             .set("scale", router["scale"].is_null() ? 1.0 : regipel_number(router, "scale", rw))
                                             .set("groups", Json::object().set("count", count).set("keep", keep)))
                          .set("shared", f["shared"].is_null()
                                             ? Json()
                                             : Json::object().set("ff", regipel_int(regipel_object(f, "shared", fw), "ff", fw + "shared.")));
            } else {
                throw ConfigError("config.json: " + fw + "'kind' is '" + kind + "'; known kinds are ['dense', 'moe']");
            }
        }
        layers.push(Json::object().set("type", type).set("mixer", mixer).set("mlp", mlp));
    }
    out.set("layers", layers);
    const long long n_layers = static_cast<long long>(layers.size());
    if (raw["loop"].is_null()) {
        out.set("loop", Json());
    } else {
        const Json& loop = regipel_object(raw, "loop", "");
        const long long start = regipel_int(loop, "start", "loop.", 0), stop = regipel_int(loop, "stop", "loop.", 0);
        const long long times = regipel_int(loop, "times", "loop.", 1);
        if (start > stop || stop > n_layers)
            throw ConfigError("config.json: 'loop' must satisfy 0 <= start <= stop <= " + std::to_string(n_layers));
        out.set("loop", Json::object().set("start", start).set("stop", stop).set("times", times));
    }
    for (const char* key : {"bos_token_id", "eos_token_id"})
        if (!raw[key].is_null()) out.set(key, raw[key]);
    return out;
}

ModelSpec vabuzen_build_spec(const Json& c) {
    const long long W = c["width"].as_int();
    const double eps = c["norm"]["eps"].as_double();
    auto norm = [&](const std::string& name) {
        PartSpec p;
        p.kind = "dynamic_tanh";
        p.params = Json::object().set("width", W).set("bias", true);
        p.tensors = {{"weight", name}, {"alpha", name + ".alpha"}, {"bias", name + ".b"}};
        return p;
    };
    auto rope = [&](const Json& rot, const Json& head_dim, const char* pairing) {
        PartSpec p;
        p.kind = "rope";
        p.params = Json::object().set("theta", rot["base"]).set("rotary_dim", rot["dims"]).set("head_dim", head_dim).set("pairing", pairing);
        return p.to_json();
    };
    ModelSpec spec;
    int i = 0;
    for (const Json& l : c["layers"].items()) {
        const std::string p = "l" + std::to_string(i) + ".";
        const Json& m = l["mixer"];
        LayerSpec layer;
        layer.arrangement = "sandwich_norm";
        layer.residual_scale = c["residual_mult"].as_double();
        if (l["type"].as_string() == "attention") {
            layer.mixer.kind = "biased_attention";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("kv_heads", m["kv_heads"])
                                     .set("head_dim", m["dim"]).set("v_dim", m["vdim"]).set("scale", m["scale"]).set("sink_one", true)
                                     .set("taps", m["conv"]);
            if (!m["mask"].is_null()) layer.mixer.params.set("window", m["mask"]["size"]).set("keep_first", m["mask"]["keep_first"]);
            if (!m["rot"].is_null()) layer.mixer.params.set("position", rope(m["rot"], m["dim"], "neighbours"));
            layer.mixer.tensors = {{"q", p + "mix.q"}, {"k", p + "mix.k"}, {"v", p + "mix.v"}, {"o", p + "mix.o"}};
            if (m["conv"].as_int() > 0)
                for (const char* t : {"q", "k", "v"}) layer.mixer.tensors.emplace_back(std::string(t) + "_conv", p + "mix." + t + ".conv");
        } else {
            layer.mixer.kind = "latent_attention";
            layer.mixer.params = Json::object().set("width", W).set("heads", m["heads"]).set("dim", m["dim"])
                                     .set("rot_dim", m["rot_dim"]).set("vdim", m["vdim"]).set("kv_rank", m["kv_rank"])
                                     .set("scale", m["scale"]).set("eps", eps).set("sink", false).set("gate", false);
            if (!m["rot"].is_null()) layer.mixer.params.set("position", rope(m["rot"], m["rot_dim"], "halves"));
            layer.mixer.tensors = {{"q", p + "mix.q"},   {"dkv", p + "mix.dkv"}, {"dkv_norm", p + "mix.dkv.norm"},
                                   {"uk", p + "mix.uk"}, {"uv", p + "mix.uv"},   {"o", p + "mix.o"}};
        }
        layer.mixer_norm = norm(p + "norm1");
        layer.mixer_post_norm = norm(p + "norm1b");
        if (l["mlp"].is_null()) {
            layer.ffn.kind = "none";
            layer.ffn_norm.kind = "identity";
        } else {
            const Json& f = l["mlp"];
            if (f["kind"].as_string() == "dense") {
                layer.ffn.kind = "mlp";
                layer.ffn.params = Json::object().set("width", W).set("ff", f["ff"]).set("activation", "gelu_tanh").set("bias", true);
                layer.ffn.tensors = {{"up", p + "mlp.up"}, {"up_bias", p + "mlp.up.b"}, {"down", p + "mlp.down"}, {"down_bias", p + "mlp.down.b"}};
            } else {
                const long long experts = f["router"]["experts"].as_int();
                layer.ffn.kind = "routed_experts";
                layer.ffn.params = Json::object().set("width", W).set("ff", f["expert"]["ff"]).set("experts", experts)
                                       .set("top", f["router"]["top"]).set("score", "sigmoid").set("renormalize", true)
                                       .set("renormalize_eps", 1e-20).set("route_scale", f["router"]["scale"])
                                       .set("groups", f["router"]["groups"]).set("weight_on", "output");
                layer.ffn.tensors = {{"router", p + "mlp.router"}};
                for (long long e = 0; e < experts; ++e) {
                    const std::string ep = p + "mlp.e" + std::to_string(e) + ".", n = std::to_string(e);
                    layer.ffn.tensors.emplace_back("gate." + n, ep + "gate");
                    layer.ffn.tensors.emplace_back("up." + n, ep + "up");
                    layer.ffn.tensors.emplace_back("down." + n, ep + "down");
                }
                if (!f["shared"].is_null()) {
                    PartSpec shared;
                    shared.kind = "swiglu";
                    shared.params = Json::object().set("width", W).set("ff", f["shared"]["ff"]);
                    layer.ffn.params.set("shared", shared.to_json());
                    for (const char* t : {"gate", "up", "down"})
                        layer.ffn.tensors.emplace_back(std::string("shared.") + t, p + "mlp.shared." + t);
                }
            }
            layer.ffn_norm = norm(p + "norm2");
            layer.ffn_post_norm = norm(p + "norm2b");
        }
        spec.layers.push_back(std::move(layer));
        ++i;
    }
    const int n_layers = i;
    if (c["loop"].is_null()) {
        for (int l = 0; l < n_layers; ++l) spec.order.push_back(RunStep{l, {}, false, 0});
    } else {
        const int start = static_cast<int>(c["loop"]["start"].as_int()), stop = static_cast<int>(c["loop"]["stop"].as_int());
        const int times = static_cast<int>(c["loop"]["times"].as_int());
        for (int l = 0; l < start; ++l) spec.order.push_back(RunStep{l, {}, false, 0});
        for (int pass = 0; pass < times; ++pass)
            for (int l = start; l < stop; ++l) spec.order.push_back(RunStep{l, {}, l == start, pass});
        for (int l = stop; l < n_layers; ++l) spec.order.push_back(RunStep{l, {}, false, 0});
        if (stop > start) {
            // before every run: the run's own vector; from the second run on, the embedding's rows as well
            spec.reinjection.kind = "add_rows";
            spec.reinjection.params = Json::object().set("width", W).set("times", times).set("embedding_from", 1);
            spec.reinjection.tensors = {{"step", "loop.step"}};
        }
    }
    spec.architecture = "Vabuzen";
    spec.vocab_size = static_cast<int>(c["vocab"].as_int());
    spec.hidden_size = static_cast<int>(W);
    spec.max_context = static_cast<int>(c["max_context"].as_int());
    spec.embedding.kind = "embedding";
    spec.embedding.params = Json::object().set("vocab", c["vocab"]).set("width", W);
    spec.embedding.tensors = {{"table", "embed"}};
    spec.head.kind = "linear_head";
    spec.head.params = Json::object().set("vocab", c["vocab"]).set("width", W);
    if (!c["logit_softcap"].is_null()) spec.head.params.set("softcap", c["logit_softcap"]);
    spec.head.tensors = {{"weight", "head"}};
    spec.final_norm = norm("final.norm");
    if (c["eos_token_id"].is_array())
        for (const Json& e : c["eos_token_id"].items()) spec.eos_token_ids.push_back(static_cast<int>(e.as_int()));
    else if (c["eos_token_id"].is_int())
        spec.eos_token_ids.push_back(static_cast<int>(c["eos_token_id"].as_int()));
    if (c["bos_token_id"].is_int()) spec.bos_token_id = static_cast<int>(c["bos_token_id"].as_int());
    spec.validate();
    return spec;
}

}  // namespace

namespace {
void register_builtin() {
    Architecture lfm2;
    lfm2.name = "Lfm2ForCausalLM";
    lfm2.aliases = {"lfm2"};
    lfm2.read_config = lfm2_read_config;
    lfm2.build_spec = lfm2_build_spec;
    std::lock_guard<std::mutex> guard(table_lock());
    table()["Lfm2ForCausalLM"] = lfm2;
    table()["lfm2"] = lfm2;
    Architecture regipel;
    regipel.name = "Regipel";
    regipel.aliases = {"regipel"};
    regipel.read_config = regipel_read_config;
    regipel.build_spec = regipel_build_spec;
    table()["Regipel"] = regipel;
    table()["regipel"] = regipel;
    Architecture kifetar;
    kifetar.name = "Kifetar";
    kifetar.aliases = {"kifetar"};
    kifetar.read_config = kifetar_read_config;
    kifetar.build_spec = kifetar_build_spec;
    table()["Kifetar"] = kifetar;
    table()["kifetar"] = kifetar;
    Architecture kivorax;
    kivorax.name = "Kivorax";
    kivorax.aliases = {"kivorax"};
    kivorax.read_config = kivorax_read_config;
    kivorax.build_spec = kivorax_build_spec;
    table()["Kivorax"] = kivorax;
    table()["kivorax"] = kivorax;
    Architecture vabuzen;
    vabuzen.name = "Vabuzen";
    vabuzen.aliases = {"vabuzen"};
    vabuzen.read_config = vabuzen_read_config;
    vabuzen.build_spec = vabuzen_build_spec;
    table()["Vabuzen"] = vabuzen;
    table()["vabuzen"] = vabuzen;
}

}  // namespace

long long lfm2_feed_forward_width(long long intermediate_size, bool auto_adjust, long long multiple_of,
                                  const double* multiplier) {
    if (!auto_adjust) return intermediate_size;
    long long width = static_cast<long long>(2.0 * static_cast<double>(intermediate_size) / 3.0);
    if (multiplier) width = static_cast<long long>(*multiplier * static_cast<double>(width));
    return multiple_of * ((width + multiple_of - 1) / multiple_of);
}

}  // namespace celeg
