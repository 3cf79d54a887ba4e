"""Reading a Vabuzen config.json: the parts and constants of every kind of layer, the run order of a
looped range with the number of every run, the cache groups (a window that keeps first positions, a
keys-only group for the compressed rows) and the saved rows of the convolutions, what may be absent,
errors that name the key at fault, and the cache manager's bookkeeping of kept first pages.  No GPU."""
import copy

import pytest

from celeg_amd import native
from celeg_amd.config import ModelSpec

MOE = {"kind": "moe", "expert": {"ff": 24}, "shared": {"ff": 40},
       "router": {"experts": 12, "top": 3, "scale": 1.5, "groups": {"count": 4, "keep": 2}}}
ATT = {"heads": 6, "kv_heads": 3, "dim": 10, "vdim": 12, "scale": 0.3, "conv": 3, "rot": {"base": 500.0, "dims": 6},
       "mask": {"size": 21, "keep_first": 5}}
LAT = {"heads": 5, "dim": 12, "rot_dim": 8, "vdim": 14, "kv_rank": 20, "scale": 0.2, "rot": {"base": 3000.0, "dims": 8}}
CFG = {"architecture": "Vabuzen", "vocab": 99, "width": 48, "norm": {"eps": 3e-5}, "residual_mult": 0.7, "logit_softcap": 9.0,
       "loop": {"start": 1, "stop": 3, "times": 2},
       "layers": [{"type": "latent_attention", "mixer": LAT, "mlp": MOE},
                  {"type": "attention", "mixer": ATT, "mlp": {"kind": "dense", "ff": 40}},
                  {"type": "latent_attention", "mixer": LAT, "mlp": None},
                  {"type": "attention", "mixer": dict(ATT, mask={"size": 21, "keep_first": 0}), "mlp": MOE}]}


def test_parts_order_cache_and_tensors():
    d = native.describe_config(CFG)
    spec = d["spec"]
    assert [(s["layer"], bool(s.get("reinject")), s.get("pass", 0)) for s in spec["order"]] == \
        [(0, False, 0), (1, True, 0), (2, False, 0), (1, True, 1), (2, False, 1), (3, False, 0)]
    assert spec["reinjection"] == {"kind": "add_rows", "params": {"width": 48, "times": 2, "embedding_from": 1}, "tensors": {"step": "loop.step"}}
    assert spec["head"]["kind"] == "linear_head" and spec["head"]["params"]["softcap"] == 9.0 and spec["head"]["tensors"] == {"weight": "head"}
    assert spec["final_norm"] == {"kind": "dynamic_tanh", "params": {"width": 48, "bias": True},
                                  "tensors": {"weight": "final.norm", "alpha": "final.norm.alpha", "bias": "final.norm.b"}}
    lat, att, bare, att2 = spec["layers"]
    assert all(l["arrangement"] == "sandwich_norm" and l["residual_scale"] == 0.7 for l in spec["layers"])
    assert all(l["mixer_post_norm"]["kind"] == "dynamic_tanh" and l["mixer_norm"]["kind"] == "dynamic_tanh" for l in spec["layers"])
    assert lat["mixer"]["kind"] == "latent_attention"
    m = lat["mixer"]["params"]
    assert (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], m["sink"], m["gate"], m["eps"]) == \
        (5, 12, 8, 14, 20, 0.2, False, False, 3e-5)
    assert m["position"]["params"] == {"theta": 3000.0, "rotary_dim": 8, "head_dim": 8, "pairing": "halves"}
    assert att["mixer"]["kind"] == "biased_attention"
    a = att["mixer"]["params"]
    assert {k: a[k] for k in ("heads", "kv_heads", "head_dim", "v_dim", "scale", "sink_one", "taps", "window", "keep_first")} == \
        {"heads": 6, "kv_heads": 3, "head_dim": 10, "v_dim": 12, "scale": 0.3, "sink_one": True, "taps": 3, "window": 21, "keep_first": 5}
    assert a["position"]["params"] == {"theta": 500.0, "rotary_dim": 6, "head_dim": 10, "pairing": "neighbours"}
    assert att["mixer"]["tensors"]["k_conv"] == "l1.mix.k.conv"
    assert att["ffn"]["kind"] == "mlp" and att["ffn"]["params"] == {"width": 48, "ff": 40, "activation": "gelu_tanh", "bias": True}
    assert bare["ffn"]["kind"] == "none" and "ffn_post_norm" not in bare
    f = lat["ffn"]["params"]
    assert lat["ffn"]["kind"] == "routed_experts"
    assert {k: f[k] for k in ("experts", "top", "score", "renormalize", "route_scale", "weight_on", "groups")} == \
        {"experts": 12, "top": 3, "score": "sigmoid", "renormalize": True, "route_scale": 1.5, "weight_on": "output",
         "groups": {"count": 4, "keep": 2}}
    assert f["renormalize_eps"] == 1e-20 and f["shared"]["kind"] == "swiglu" and f["shared"]["params"] == {"width": 48, "ff": 40}
    assert lat["ffn"]["tensors"]["shared.down"] == "l0.mlp.shared.down"
    layout = d["cache_layout"]
    groups = [(k["kv_heads"], k["head_dim"], k["v_head_dim"], k["keys_only"], k["window"], k["keep_first"], k["layers"]) for k in layout["kv_groups"]]
    # the compressed rows of three runs, the windowed keys of two runs with kept first positions, those of one run without
    assert groups == [(1, 28, 0, True, None, 0, 3), (3, 10, 12, False, 21, 5, 2), (3, 10, 12, False, 21, 0, 1)]
    states = sorted((s["step"], s["name"], tuple(s["shape"])) for s in layout["states"])
    assert states == [(1, "conv", (2, 126)), (3, "conv", (2, 126)), (5, "conv", (2, 126))]
    names = {e["name"]: e["shape"] for e in d["expected_tensors"]}
    assert names["loop.step"] == [2, 48] and names["head"] == [99, 48] and names["final.norm.alpha"] == [] and names["l3.norm2b.b"] == [48]
    assert names["l1.mix.q"] == [60, 48] and names["l1.mix.v"] == [36, 48] and names["l1.mix.o"] == [48, 72] and names["l1.mix.v.conv"] == [36, 3]
    assert names["l0.mix.q"] == [100, 48] and names["l0.mix.dkv"] == [28, 48] and names["l0.mix.dkv.norm"] == [20]
    assert names["l0.mix.uk"] == [60, 20] and names["l0.mix.uv"] == [70, 20] and names["l0.mix.o"] == [48, 70]
    assert names["l0.mlp.router"] == [12, 48] and names["l0.mlp.e11.gate"] == [24, 48] and names["l0.mlp.shared.up"] == [40, 48]
    assert names["l1.mlp.up.b"] == [40] and names["l1.mlp.down.b"] == [48]
    assert "l2.mlp.up" not in names and "l2.norm2" not in names and "l0.mix.sink" not in names and "l0.mix.g" not in names
    again = ModelSpec.from_json(spec).to_json()
    assert again["order"] == spec["order"] and again["layers"][0]["residual_scale"] == 0.7
    assert d["graph_safe"] is True


def test_what_may_be_absent():
    cfg = copy.deepcopy(CFG)
    for key in ("loop", "residual_mult", "logit_softcap"):
        del cfg[key]
    att = cfg["layers"][1]["mixer"]
    for key in ("conv", "rot", "mask", "vdim", "kv_heads"):
        del att[key]
    moe = cfg["layers"][0]["mlp"]
    del moe["shared"], moe["router"]["groups"], moe["router"]["scale"]
    cfg["layers"][3]["mlp"] = moe
    d = native.describe_config(cfg)
    spec = d["spec"]
    assert "reinjection" not in spec and [s["layer"] for s in spec["order"]] == [0, 1, 2, 3]
    assert "softcap" not in spec["head"]["params"] and "residual_scale" not in spec["layers"][0]
    a = spec["layers"][1]["mixer"]["params"]
    assert a["taps"] == 0 and "window" not in a and "position" not in a and a["v_dim"] == 10 and a["kv_heads"] == 6
    f = spec["layers"][0]["ffn"]["params"]
    assert f["groups"] == {"count": 1, "keep": 1} and f["route_scale"] == 1.0 and "shared" not in f
    names = {e["name"] for e in d["expected_tensors"]}
    assert "loop.step" not in names and "l1.mix.q.conv" not in names and "l0.mlp.shared.up" not in names
    assert not [s for s in d["cache_layout"]["states"] if s["step"] == 1]
    # a loop over no layer at all asks for no tensor either; one run is a loop too, with its vector
    assert "reinjection" not in native.describe_config(dict(cfg, loop={"start": 2, "stop": 2, "times": 3}))["spec"]
    once = native.describe_config(dict(cfg, loop={"start": 0, "stop": 4, "times": 1}))
    assert [(s["layer"], bool(s.get("reinject"))) for s in once["spec"]["order"]] == [(0, True), (1, False), (2, False), (3, False)]
    assert {e["name"]: e["shape"] for e in once["expected_tensors"]}["loop.step"] == [1, 48]


@pytest.mark.parametrize("path,value,word", [
    (("layers", 1, "type"), "conv", "known types"),
    (("layers", 1, "mixer", "kv_heads"), 4, "multiple of 'kv_heads'"),
    (("layers", 1, "mixer", "rot", "dims"), 12, "rot.dims"),
    (("layers", 1, "mixer", "rot", "dims"), 5, "rot.dims"),
    (("layers", 0, "mixer", "rot", "dims"), 10, "rot.dims"),
    (("layers", 1, "mixer", "mask", "size"), 0, "mask.'size'"),
    (("layers", 1, "mixer", "mask", "keep_first"), -1, "keep_first"),
    (("layers", 0, "mlp", "kind"), "glu", "known kinds"),
    (("layers", 0, "mlp", "router", "top"), 13, "'top' exceeds"),
    (("layers", 0, "mlp", "router", "groups", "count"), 5, "must divide"),
    (("layers", 0, "mlp", "router", "groups", "keep"), 5, "groups.keep"),
    (("layers", 0, "mlp", "router", "top"), 7, "kept groups hold fewer"),
    (("layers", 0, "mlp", "shared", "ff"), 0, "shared.'ff'"),
    (("loop", "stop"), 5, "'loop' must satisfy"),
    (("loop", "times"), 0, "loop.'times'"),
    (("logit_softcap",), -1.0, "logit_softcap"),
    (("norm", "eps"), 0.0, "norm.eps"),
    (("residual_mult",), "half", "residual_mult"),
])
def test_errors_name_the_key(path, value, word):
    cfg = copy.deepcopy(CFG)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(native.NativeArgumentError) as err:
        native.describe_config(cfg)
    assert word in str(err.value), str(err.value)


def test_pages_of_kept_first_positions_stay():
    """The cache manager's bookkeeping alone: a window of 21 positions that keeps the first 5 on pages of 4:
    as a request grows, the pages the window has passed go back to the pool but for the first two, which
    hold positions 0..4; a group with the same window and nothing kept gives those back too."""
    layout = native.describe_config(CFG)["cache_layout"]
    cache = native.HostObject("cache", layout=layout, page_tokens=4, n_pages=[40, 40, 40], max_requests=2, max_context=160)
    slot = cache.call("open")
    at = 0
    for n in (30, 1, 1, 17, 2, 40):
        assert cache.call("prepare", slot, at, n)
        at += n
        assert cache.call("covers", slot, at - n, n)
        held = cache.call("pages_held", slot)
        first_needed = max(0, at - n - 21 + 1) // 4
        total = (at + 3) // 4
        assert len(held[0]) == total                              # every compressed row stays
        assert len(held[1]) == total - first_needed + min(2, first_needed)
        assert len(held[2]) == total - first_needed
        cache.call("check")
    assert cache.call("table", 1, slot, 0) >= 0 and cache.call("table", 1, slot, 1) >= 0 and cache.call("table", 1, slot, 2) == -1
    assert cache.call("table", 2, slot, 0) == -1
    cache.call("close", slot)
    assert cache.call("state")["free_pages"] == [40, 40, 40]
