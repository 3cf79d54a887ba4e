"""The description of a model as data, on the Python side: which parts, with which sizes, in
which order.  It mirrors the library's own description (``csrc/host/spec.hpp``) and travels to
and from it as JSON; an architecture written in Python builds one of these.

The reference keeps the same separation: a ``LayerSpec`` is a mixer variant plus a feed-forward
variant plus norms (include/celeg/model/graph.hpp:431-438) and back ends consume the compiled
program, never names (src/model/program_builder.cpp:112-164).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: its registered kind, its sizes and constants (a value may itself be a part), and
    the checkpoint tensor that fills each of its roles (role -> tensor name)."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)

    def to_json(self) -> Dict[str, Any]:
        params = {k: (v.to_json() if isinstance(v, PartSpec) else v) for k, v in self.params.items()}
        return {"kind": self.kind, "params": params, "tensors": dict(self.tensors)}

    @classmethod
    def from_json(cls, j: Dict[str, Any]) -> "PartSpec":
        params = {k: (cls.from_json(v) if isinstance(v, dict) and isinstance(v.get("kind"), str) else v)
                  for k, v in (j.get("params") or {}).items()}
        return cls(j["kind"], params, dict(j.get("tensors") or {}))


@dataclass(frozen=True)
class LayerSpec:
    """A block: how the parts are arranged, and the parts themselves."""
    mixer: PartSpec
    mixer_norm: PartSpec
    ffn: PartSpec
    ffn_norm: PartSpec
    arrangement: str = "pre_norm"
    # how each sub-layer hangs on the residual stream(s), where the arrangement makes that a
    # part with weights of its own ("hyper_connections": a "hyper_link" each)
    mixer_link: Optional[PartSpec] = None
    ffn_link: Optional[PartSpec] = None
    # norms of the sub-layers' outputs, where the arrangement norms before and after ("sandwich_norm")
    mixer_post_norm: Optional[PartSpec] = None
    ffn_post_norm: Optional[PartSpec] = None
    # what the rows' token ids add to the stream behind the sub-layers, and how the stream behind
    # the layer is mixed from the results of all entries of the run order so far
    token_input: Optional[PartSpec] = None
    depth_mix: Optional[PartSpec] = None
    # what a sub-layer's (normed) output is multiplied by as it is added to the stream ("sandwich_norm")
    residual_scale: float = 1.0

    def to_json(self) -> Dict[str, Any]:
        out = {"mixer": self.mixer.to_json(), "mixer_norm": self.mixer_norm.to_json(),
               "ffn": self.ffn.to_json(), "ffn_norm": self.ffn_norm.to_json(),
               "arrangement": self.arrangement}
        if self.mixer_link is not None:
            out["mixer_link"] = self.mixer_link.to_json()
        if self.ffn_link is not None:
            out["ffn_link"] = self.ffn_link.to_json()
        if self.mixer_post_norm is not None:
            out["mixer_post_norm"] = self.mixer_post_norm.to_json()
        if self.ffn_post_norm is not None:
            out["ffn_post_norm"] = self.ffn_post_norm.to_json()
        if self.token_input is not None:
            out["token_input"] = self.token_input.to_json()
        if self.depth_mix is not None:
            out["depth_mix"] = self.depth_mix.to_json()
        if self.residual_scale != 1.0:
            out["residual_scale"] = self.residual_scale
        return out

    @classmethod
    def from_json(cls, l: Dict[str, Any]) -> "LayerSpec":
        link = lambda key: PartSpec.from_json(l[key]) if l.get(key) else None
        return cls(PartSpec.from_json(l["mixer"]), PartSpec.from_json(l["mixer_norm"]),
                   PartSpec.from_json(l["ffn"]), PartSpec.from_json(l["ffn_norm"]),
                   l.get("arrangement", "pre_norm"), link("mixer_link"), link("ffn_link"),
                   link("mixer_post_norm"), link("ffn_post_norm"), link("token_input"), link("depth_mix"),
                   float(l.get("residual_scale", 1.0)))


@dataclass(frozen=True)
class RunStep:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    more than once: its weights are shared, its cache is not).  ``kv_from`` is the index of an
    EARLIER entry of the run order whose keys and values this entry's mixer reads instead of
    writing its own.  ``reinject``: before this entry the stream is replaced by the model's
    ``reinjection`` part's mixture of the stream and the embedding's rows.  ``pass_``: which run
    of a looped range of layers the entry belongs to ("pass" in JSON)."""
    layer: int
    kv_from: Optional[int] = None
    reinject: bool = False
    pass_: int = 0


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_context: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[RunStep, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    streams: int = 1          # residual streams a row keeps between layers
    reinjection: Optional[PartSpec] = None

    def to_json(self) -> Dict[str, Any]:
        out = {} if self.reinjection is None else {"reinjection": self.reinjection.to_json()}
        return {**out, "architecture": self.architecture, "vocab_size": self.vocab_size,
                "hidden_size": self.hidden_size, "max_context": self.max_context, "streams": self.streams,
                "embedding": self.embedding.to_json(), "layers": [l.to_json() for l in self.layers],
                "order": [{"layer": s.layer, "kv_from": s.kv_from, **({"reinject": True} if s.reinject else {}),
                           **({"pass": s.pass_} if s.pass_ else {})} for s in self.order],
                "final_norm": self.final_norm.to_json(), "head": self.head.to_json(),
                "eos_token_ids": list(self.eos_token_ids), "bos_token_id": self.bos_token_id}

    @classmethod
    def from_json(cls, j: Dict[str, Any]) -> "ModelSpec":
        layers = tuple(LayerSpec.from_json(l) for l in j["layers"])
        order = tuple(RunStep(s["layer"], s.get("kv_from"), bool(s.get("reinject")), int(s.get("pass") or 0)) for s in j["order"])
        return cls(j["architecture"], j["vocab_size"], j["hidden_size"], j["max_context"],
                   PartSpec.from_json(j["embedding"]), layers, order, PartSpec.from_json(j["final_norm"]),
                   PartSpec.from_json(j["head"]), tuple(j.get("eos_token_ids") or ()), j.get("bos_token_id"),
                   int(j.get("streams") or 1),
                   PartSpec.from_json(j["reinjection"]) if j.get("reinjection") else None)

    def tensor_names(self) -> List[str]:
        names: List[str] = []
        for part in self.all_parts():
            names.extend(part.tensors.values())
        return names

    def all_parts(self) -> List[PartSpec]:
        parts = [self.embedding] + ([self.reinjection] if self.reinjection is not None else [])
        for layer in self.layers:
            parts += [layer.mixer_norm, layer.mixer, layer.ffn_norm, layer.ffn]
            parts += [p for p in (layer.mixer_link, layer.ffn_link, layer.mixer_post_norm, layer.ffn_post_norm,
                                       layer.token_input, layer.depth_mix)
                      if p is not None]
        parts += [self.final_norm, self.head]
        return parts
