// The description of a model as data: which parts, with which sizes, in which order.
//
// An architecture turns its typed configuration into a ModelSpec; everything below
// (weights, cache manager, step function) reads only the spec and never asks which
// architecture it came from.  The reference keeps the same separation: a LayerSpec is a
// mixer variant plus a feed-forward variant plus norms (include/celeg/model/graph.hpp:431-438)
// and back ends consume the compiled program, never names
// (src/model/program_builder.cpp:112-164).
//
// A spec also travels as JSON (an architecture defined outside this library hands its
// spec over that way):
//   part:  {"kind": .., "params": {..}, "tensors": {role: checkpoint name}}; a parameter
//          may itself be a part (an attention's "position")
//   layer: {"mixer": part, "mixer_norm": part, "ffn": part, "ffn_norm": part,
//           "arrangement": "pre_norm"}; an arrangement that joins a sub-layer to the residual
//           stream by a part of its own names them as "mixer_link" and "ffn_link"; one that norms
//           a sub-layer's output before the addition names those norms "mixer_post_norm" and
//           "ffn_post_norm"; a layer may name a "token_input" (a part that adds something made from the
//           rows' token ids to the stream after the sub-layers) and a "depth_mix" (a part that replaces
//           the stream behind the layer by a mixture of the results of all entries of the run order so
//           far, the embedding's rows first); "residual_scale" (1 if absent) multiplies what a sub-layer adds to
//           the stream, in arrangements that know it ("sandwich_norm")
//   model: {"architecture", "vocab_size", "hidden_size", "max_context", "streams" (residual
//           streams per row, 1 if absent), "embedding": part,
//           "layers": [layer], "order": [{"layer": i, "kv_from": j or null, "reinject": bool, "pass": n}],
//           "reinjection": part (how the embedding's rows come back into the stream before the
//           entries of the order that say "reinject"; absent: never),
//           "final_norm": part, "head": part, "eos_token_ids": [..], "bos_token_id"}
#pragma once
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "json.hpp"

namespace celeg {

// One message per kind of failure; the C API hands the text to the caller.
struct ConfigError : std::runtime_error { using std::runtime_error::runtime_error; };
struct SpecError : std::runtime_error { using std::runtime_error::runtime_error; };
struct KernelError : std::runtime_error { using std::runtime_error::runtime_error; };
struct PageError : std::runtime_error { using std::runtime_error::runtime_error; };
struct StepError : std::runtime_error { using std::runtime_error::runtime_error; };

struct PartSpec {
    std::string kind;
    Json params = Json::object();
    std::vector<std::pair<std::string, std::string>> tensors;   // role -> checkpoint tensor name

    const std::string* tensor(const std::string& role) const {
        for (const auto& t : tensors)
            if (t.first == role) return &t.second;
        return nullptr;
    }

    Json to_json() const {
        Json t = Json::object();
        for (const auto& p : tensors) t.set(p.first, p.second);
        return Json::object().set("kind", kind).set("params", params).set("tensors", t);
    }
    static PartSpec from_json(const Json& j, const std::string& where) {
        if (!j.is_object() || !j["kind"].is_string())
            throw SpecError(where + ": a part is an object with a \"kind\"");
        PartSpec p;
        p.kind = j["kind"].as_string();
        if (!j["params"].is_null()) {
            if (!j["params"].is_object()) throw SpecError(where + ": \"params\" must be an object");
            p.params = j["params"];
        }
        if (!j["tensors"].is_null()) {
            if (!j["tensors"].is_object()) throw SpecError(where + ": \"tensors\" must be an object");
            for (const auto& m : j["tensors"].members()) {
                if (!m.second.is_string()) throw SpecError(where + ": tensor names are strings");
                p.tensors.emplace_back(m.first, m.second.as_string());
            }
        }
        return p;
    }
    // whether a parameter value is itself a part
    static bool is_part(const Json& v) { return v.is_object() && v["kind"].is_string(); }
};

struct LayerSpec {
    PartSpec mixer, mixer_norm, ffn, ffn_norm;
    // how each sub-layer reads from and writes to the residual stream(s), for arrangements in
    // which that is a part with weights of its own (kind empty: the arrangement has none)
    PartSpec mixer_link, ffn_link;
    // norms of the sub-layers' outputs, for arrangements that norm before and after (kind empty: none)
    PartSpec mixer_post_norm, ffn_post_norm;
    // what the rows' token ids add to the stream after the sub-layers, and how the stream behind the
    // layer is mixed from the results of the entries run so far (kind empty: none)
    PartSpec token_input, depth_mix;
    std::string arrangement = "pre_norm";
    // what a sub-layer's (normed) output is multiplied by as it is added to the stream
    double residual_scale = 1.0;
};

// One entry of the run order.  `layer` indexes ModelSpec::layers (a layer may be named more
// than once: its weights are shared, its cache is not).  `kv_from` is the index of an
// EARLIER entry of the run order whose keys and values this entry's mixer reads instead of
// writing its own.
struct RunStep {
    int layer = 0;
    std::optional<int> kv_from;
    // before this entry runs, the stream is replaced by the model's reinjection part's mixture of
    // the stream and the embedding's rows
    bool reinject = false;
    // which run of a looped range of layers this entry belongs to (0 where nothing is looped): what a
    // reinjection that differs from run to run is told
    int pass = 0;
};

struct ModelSpec {
    std::string architecture;
    int vocab_size = 0, hidden_size = 0, max_context = 0;
    int streams = 1;             // residual streams a row keeps between layers
    PartSpec embedding;
    PartSpec reinjection;        // kind empty: the model has none
    std::vector<LayerSpec> layers;
    std::vector<RunStep> order;
    PartSpec final_norm, head;
    std::vector<int> eos_token_ids;
    std::optional<int> bos_token_id;

    void validate() const {
        if (vocab_size <= 0 || hidden_size <= 0 || max_context <= 0)
            throw SpecError("vocab_size, hidden_size and max_context must be positive");
        if (streams <= 0) throw SpecError("streams must be positive");
        if (order.empty()) throw SpecError("the run order is empty");
        for (size_t i = 0; i < order.size(); ++i) {
            if (order[i].layer < 0 || order[i].layer >= static_cast<int>(layers.size()))
                throw SpecError("run order entry " + std::to_string(i) + " names layer " +
                                std::to_string(order[i].layer) + ", but the model has " +
                                std::to_string(layers.size()) + " layers");
            if (order[i].reinject && reinjection.kind.empty())
                throw SpecError("run order entry " + std::to_string(i) + " asks for the embedding's rows again, but the model names no \"reinjection\" part");
            if (order[i].kv_from && (*order[i].kv_from < 0 || *order[i].kv_from >= static_cast<int>(i)))
                throw SpecError("run order entry " + std::to_string(i) + " reads the cache of entry " +
                                std::to_string(*order[i].kv_from) + ", which does not run before it");
        }
    }

    Json to_json() const {
        Json ls = Json::array();
        for (const auto& l : layers) {
            Json lj = Json::object().set("mixer", l.mixer.to_json()).set("mixer_norm", l.mixer_norm.to_json())
                          .set("ffn", l.ffn.to_json()).set("ffn_norm", l.ffn_norm.to_json())
                          .set("arrangement", l.arrangement);
            if (!l.mixer_link.kind.empty()) lj.set("mixer_link", l.mixer_link.to_json());
            if (!l.ffn_link.kind.empty()) lj.set("ffn_link", l.ffn_link.to_json());
            if (!l.mixer_post_norm.kind.empty()) lj.set("mixer_post_norm", l.mixer_post_norm.to_json());
            if (!l.ffn_post_norm.kind.empty()) lj.set("ffn_post_norm", l.ffn_post_norm.to_json());
            if (!l.token_input.kind.empty()) lj.set("token_input", l.token_input.to_json());
            if (!l.depth_mix.kind.empty()) lj.set("depth_mix", l.depth_mix.to_json());
            if (l.residual_scale != 1.0) lj.set("residual_scale", l.residual_scale);
            ls.push(lj);
        }
        Json ord = Json::array();
        for (const auto& s : order) {
            Json e = Json::object().set("layer", s.layer).set("kv_from", s.kv_from ? Json(*s.kv_from) : Json());
            if (s.reinject) e.set("reinject", true);
            if (s.pass) e.set("pass", s.pass);
            ord.push(e);
        }
        Json out = Json::object();
        if (!reinjection.kind.empty()) out.set("reinjection", reinjection.to_json());
        return out.set("architecture", architecture).set("vocab_size", vocab_size)
            .set("hidden_size", hidden_size).set("max_context", max_context).set("streams", streams)
            .set("embedding", embedding.to_json()).set("layers", ls).set("order", ord)
            .set("final_norm", final_norm.to_json()).set("head", head.to_json())
            .set("eos_token_ids", Json::array_of(eos_token_ids))
            .set("bos_token_id", bos_token_id ? Json(*bos_token_id) : Json());
    }

    static ModelSpec from_json(const Json& j) {
        if (!j.is_object()) throw SpecError("a model description is an object");
        ModelSpec m;
        m.architecture = j.get_string("architecture", "");
        m.vocab_size = static_cast<int>(j.get_int("vocab_size", 0));
        m.hidden_size = static_cast<int>(j.get_int("hidden_size", 0));
        m.max_context = static_cast<int>(j.get_int("max_context", 0));
        m.streams = static_cast<int>(j.get_int("streams", 1));
        m.embedding = PartSpec::from_json(j["embedding"], "embedding");
        if (!j["reinjection"].is_null()) m.reinjection = PartSpec::from_json(j["reinjection"], "reinjection");
        if (!j["layers"].is_array()) throw SpecError("\"layers\" must be an array");
        int n = 0;
        for (const Json& l : j["layers"].items()) {
            const std::string where = "layers[" + std::to_string(n++) + "]";
            LayerSpec ls;
            ls.mixer = PartSpec::from_json(l["mixer"], where + ".mixer");
            ls.mixer_norm = PartSpec::from_json(l["mixer_norm"], where + ".mixer_norm");
            ls.ffn = PartSpec::from_json(l["ffn"], where + ".ffn");
            ls.ffn_norm = PartSpec::from_json(l["ffn_norm"], where + ".ffn_norm");
            if (!l["mixer_link"].is_null()) ls.mixer_link = PartSpec::from_json(l["mixer_link"], where + ".mixer_link");
            if (!l["ffn_link"].is_null()) ls.ffn_link = PartSpec::from_json(l["ffn_link"], where + ".ffn_link");
            if (!l["mixer_post_norm"].is_null()) ls.mixer_post_norm = PartSpec::from_json(l["mixer_post_norm"], where + ".mixer_post_norm");
            if (!l["ffn_post_norm"].is_null()) ls.ffn_post_norm = PartSpec::from_json(l["ffn_post_norm"], where + ".ffn_post_norm");
            if (!l["token_input"].is_null()) ls.token_input = PartSpec::from_json(l["token_input"], where + ".token_input");
            if (!l["depth_mix"].is_null()) ls.depth_mix = PartSpec::from_json(l["depth_mix"], where + ".depth_mix");
            ls.arrangement = l.get_string("arrangement", "pre_norm");
            ls.residual_scale = l.get_double("residual_scale", 1.0);
            m.layers.push_back(std::move(ls));
        }
        if (j["order"].is_array()) {
            for (const Json& s : j["order"].items()) {
                RunStep step;
                step.layer = static_cast<int>(s.is_object() ? s.get_int("layer", -1) : s.as_int());
                if (s.is_object() && !s["kv_from"].is_null()) step.kv_from = static_cast<int>(s["kv_from"].as_int());
                if (s.is_object()) step.reinject = s.get_bool("reinject", false);
                if (s.is_object()) step.pass = static_cast<int>(s.get_int("pass", 0));
                m.order.push_back(step);
            }
        } else {
            for (size_t i = 0; i < m.layers.size(); ++i) m.order.push_back(RunStep{static_cast<int>(i), {}});
        }
        m.final_norm = PartSpec::from_json(j["final_norm"], "final_norm");
        m.head = PartSpec::from_json(j["head"], "head");
        if (j["eos_token_ids"].is_array())
            for (const Json& e : j["eos_token_ids"].items()) m.eos_token_ids.push_back(static_cast<int>(e.as_int()));
        if (!j["bos_token_id"].is_null()) m.bos_token_id = static_cast<int>(j["bos_token_id"].as_int());
        m.validate();
        return m;
    }
};

}  // namespace celeg
