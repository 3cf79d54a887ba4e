"""Reading a Kivorax config.json: the parts and constants of every kind of layer, the cache and
state the model asks for, sizes that only the checkpoint's shapes give, what may be absent, and
errors that name the key at fault.  No GPU."""
import copy

import pytest

from celeg_amd import native
from celeg_amd.config import ModelSpec

MOE = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 2}}
PAIR = {"left": {"heads": 6, "kv_heads": 2, "dim": 8, "vdim": 20, "scale": 0.3, "q_temp": {"coef": 0.2, "every": 7}},
        "right": {"width": 36, "blocks": 3, "conv": 3}}
CFG = {"architecture": "Kivorax", "vocab": 99, "width": 48, "norm": {"eps": 3e-5}, "embedding": {"scale": 2.5}, "token_side": {"dim": 6},
       "layers": [{"type": "gla", "mixer": {"heads": 3, "dim": 10, "vdim": 12, "tau": 8.0, "decay_rank": 5}, "mlp": MOE},
                  {"type": "parallel", "mixer": PAIR, "mlp": {"kind": "dense", "ff": 40}},
                  {"type": "channel_delta", "mixer": {"heads": 4, "kv_heads": 2, "dim": 10, "vdim": 12, "conv": 4, "decay_rank": 7,
                                                      "gate_rank": 9}, "mlp": None}]}


def test_parts_cache_and_tensors():
    d = native.describe_config(CFG)
    spec = d["spec"]
    assert [s["layer"] for s in spec["order"]] == [0, 1, 2]
    assert spec["embedding"]["params"]["scale"] == 2.5 and spec["head"]["kind"] == "linear_head" and spec["final_norm"]["kind"] == "rmsnorm"
    g, p, c = spec["layers"]
    assert all(l["arrangement"] == "parallel" and l["ffn_norm"]["kind"] == "identity" for l in spec["layers"])
    assert g["mixer"]["kind"] == "gated_linear_attention" and g["mixer"]["params"]["tau"] == 8.0 and g["mixer"]["params"]["decay_rank"] == 5
    assert g["ffn"]["kind"] == "routed_experts"
    f = g["ffn"]["params"]
    assert (f["experts"], f["top"], f["score"], f["renormalize"], f["gated"], f["activation"]) == (5, 2, "softmax", False, False, "relu2")
    assert p["mixer"]["kind"] == "normed_pair" and p["mixer"]["params"]["factor"] == 0.5 and p["mixer"]["params"]["eps"] == 3e-5
    left, right = p["mixer"]["params"]["left"], p["mixer"]["params"]["right"]
    assert left["kind"] == "biased_attention" and right["kind"] == "linear_recurrent_unit"
    assert left["params"] == {"width": 48, "heads": 6, "kv_heads": 2, "head_dim": 8, "v_dim": 20, "scale": 0.3, "distance_bias": True,
                              "gate": "sigmoid", "query_temperature": {"coef": 0.2, "every": 7}}
    assert right["params"] == {"width": 48, "inner": 36, "blocks": 3, "taps": 3, "decay_scale": 8.0}
    assert p["ffn"]["kind"] == "mlp" and p["ffn"]["params"]["activation"] == "gelu_tanh" and p["ffn"]["params"]["bias"] is True
    assert c["mixer"]["kind"] == "gated_delta_rule" and c["ffn"]["kind"] == "none"
    m = c["mixer"]["params"]
    assert (m["decay"], m["gate"], m["decay_rank"], m["gate_rank"], m["taps"], m["kv_heads"]) == ("channel", "sigmoid", 7, 9, 4, 2)
    # every layer reads its own columns of the one token table, and mixes one result more than the layer before
    assert [l["token_input"]["params"]["offset"] for l in spec["layers"]] == [0, 6, 12]
    assert all(l["token_input"]["params"]["table_width"] == 18 and l["token_input"]["tensors"]["table"] == "side.embed" for l in spec["layers"])
    assert [l["depth_mix"]["params"]["entries"] for l in spec["layers"]] == [2, 3, 4]
    layout = d["cache_layout"]
    assert [(k["kv_heads"], k["head_dim"], k["v_head_dim"], k["window"], k["layers"]) for k in layout["kv_groups"]] == [(2, 8, 20, None, 1)]
    states = sorted((s["step"], s["name"], tuple(s["shape"]), s["dtype"]) for s in layout["states"])
    assert states == [(0, "S", (3, 10, 12), "float32"), (1, "right.S", (36,), "float32"), (1, "right.conv", (2, 36), "float32"),
                      (2, "S", (4, 10, 12), "float32"), (2, "conv", (3, 88), "float32")]
    names = {e["name"]: e["shape"] for e in d["expected_tensors"]}
    assert names["side.embed"] == [99, 18] and names["head"] == [99, 48] and names["l2.dwa"] == [4]
    assert names["l1.mix.left.v"] == [40, 48] and names["l1.mix.left.g"] == [120, 48] and names["l1.mix.left.o"] == [48, 120]
    assert names["l1.mix.left.r1"] == [6] and names["l1.mix.right.ra"] == [3, 12, 12] and names["l1.mix.right.ri.b"] == [3, 12]
    assert names["l1.mix.right.conv"] == [36, 3] and names["l1.mix.right.out"] == [48] and names["l1.mlp.down.b"] == [48]
    assert names["l0.mix.a2"] == [30, 5] and names["l0.mix.a2.b"] == [30] and names["l0.mlp.e4.down"] == [48, 24] and names["l0.mlp.router"] == [5, 48]
    assert names["l2.mix.dt_bias"] == [40] and names["l2.mix.a2"] == [40, 7] and names["l2.mix.g2"] == [48, 9] and names["l2.mix.v.conv"] == [48, 4]
    assert "l2.mlp.up" not in names and "l2.mix.a" not in names and "l2.mix.g" not in names
    again = ModelSpec.from_json(spec).to_json()
    assert again["layers"][1]["token_input"]["kind"] == "gated_table" and again["layers"][2]["depth_mix"]["params"]["entries"] == 4


def test_sizes_that_the_checkpoint_gives():
    """The widths between the two steps of a decay's or gate's projection are the checkpoint's, and a
    layer mixes over depth where the checkpoint holds its weights."""
    cfg = copy.deepcopy(CFG)
    for l in cfg["layers"]:
        for key in ("decay_rank", "gate_rank"):
            l["mixer"].pop(key, None)
    plain = native.describe_config(cfg)["spec"]["layers"]
    assert plain[0]["mixer"]["params"]["decay_rank"] == 16 and plain[2]["mixer"]["params"]["gate_rank"] == 16
    shapes = {e["name"]: e["shape"] for e in native.describe_config(CFG)["expected_tensors"]}
    shapes["l0.mix.a1"], shapes["l0.mix.a2"] = [11, 48], [30, 11]
    shapes["l2.mix.g1"], shapes["l2.mix.g2"] = [3, 48], [48, 3]
    del shapes["l1.dwa"]
    layers = native.describe_config(cfg, shapes)["spec"]["layers"]
    assert layers[0]["mixer"]["params"]["decay_rank"] == 11 and layers[2]["mixer"]["params"]["gate_rank"] == 3
    assert layers[2]["mixer"]["params"]["decay_rank"] == 7
    assert "depth_mix" not in layers[1] and layers[2]["depth_mix"]["params"]["entries"] == 4


def test_what_may_be_absent():
    cfg = copy.deepcopy(CFG)
    del cfg["embedding"], cfg["token_side"]
    del cfg["layers"][1]["mixer"]["left"]["q_temp"]
    d = native.describe_config(cfg)
    spec = d["spec"]
    assert spec["embedding"]["params"]["scale"] == 1.0
    assert all("token_input" not in l for l in spec["layers"])
    assert "query_temperature" not in spec["layers"][1]["mixer"]["params"]["left"]["params"]
    names = {e["name"] for e in d["expected_tensors"]}
    assert "side.embed" not in names and "l0.side.gate" not in names


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "attention", "type"), (("layers", 1, "mixer", "left", "heads"), 5, "heads"),
    (("layers", 1, "mixer", "right", "width"), 35, "width"), (("layers", 2, "mixer", "heads"), 3, "heads"),
    (("layers", 0, "mixer", "tau"), 0.0, "tau"), (("layers", 0, "mlp", "kind"), "swiglu", "kind"),
    (("layers", 0, "mlp", "router", "top"), 6, "top"), (("norm", "eps"), 0.0, "eps"),
    (("layers", 1, "mixer", "left", "vdim"), 300, "vdim"), (("layers", 2, "mixer", "dim"), 257, "dim"),
    (("token_side", "dim"), "six", "dim")])
def test_errors_name_the_key(path, value, word):
    cfg = copy.deepcopy(CFG)
    at = cfg
    for p in path[:-1]:
        at = at[p]
    at[path[-1]] = value
    with pytest.raises(native.NativeArgumentError, match=word):
        native.describe_config(cfg)


def test_missing_key_is_named():
    cfg = copy.deepcopy(CFG)
    del cfg["layers"][1]["mixer"]["left"]["scale"]
    with pytest.raises(native.NativeArgumentError, match="scale"):
        native.describe_config(cfg)
