"""Reading a Kifetar config.json: the run order that a loop makes and where the embedding's rows
come in again, the parts and constants of every layer, the cache and state the model asks for,
what may be absent, and errors that name the key at fault.  No GPU."""
import copy

import pytest

from celeg_amd import native
from celeg_amd.config import ModelSpec


def attention(heads, kv_heads, dim, window=None, rot=None, scale=0.2):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = rot
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": 40}}


def delta(heads, kv_heads, dim, vdim, taps, mlp=True):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps},
            "mlp": {"kind": "dense", "ff": 56} if mlp else None}


ROT = {"base": 3000.0, "dims": 6, "scaling": {"factor": 8.0, "low": 1.0, "high": 2.0, "original": 64}}
CFG = {"architecture": "Kifetar", "vocab": 99, "width": 48, "norm": {"eps": 3e-5}, "loop": {"start": 1, "stop": 3, "times": 3},
       "layers": [attention(6, 2, 8, window=9, rot=ROT), delta(4, 2, 10, 12, 4), attention(3, 3, 16),
                  delta(2, 1, 8, 24, 2, mlp=False)]}


def test_run_order_parts_and_cache():
    d = native.describe_config(CFG)
    spec = d["spec"]
    assert [(s["layer"], bool(s.get("reinject"))) for s in spec["order"]] == \
        [(0, False), (1, True), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert spec["reinjection"] == {"kind": "linear_concat", "params": {"width": 48}, "tensors": {"weight": "loop.in"}}
    a, r = spec["layers"][0], spec["layers"][1]
    assert a["arrangement"] == "sandwich_norm" and a["mixer"]["kind"] == "sigmoid_attention"
    p = a["mixer"]["params"]
    assert p["window"] == 9 and p["values"] == "keys" and p["head_dim"] == 8 and p["scale"] == 0.2 and p["eps"] == 3e-5
    assert p["position"]["params"] == {"theta": 3000.0, "rotary_dim": 6, "head_dim": 8, "pairing": "halves",
                                       "scaling": {"factor": 8.0, "low": 1.0, "high": 2.0, "original": 64.0}}
    assert a["mixer_post_norm"]["kind"] == "layernorm" and a["mixer_post_norm"]["tensors"] == {"weight": "l0.norm1b", "bias": "l0.norm1b.b"}
    assert r["mixer"]["kind"] == "gated_delta_rule" and r["mixer"]["params"]["taps"] == 4
    assert "window" not in spec["layers"][2]["mixer"]["params"] and "position" not in spec["layers"][2]["mixer"]["params"]
    assert spec["layers"][3]["ffn"]["kind"] == "none" and "ffn_post_norm" not in spec["layers"][3]
    assert spec["final_norm"]["kind"] == "layernorm" and spec["head"]["kind"] == "tied_head"
    layout = d["cache_layout"]
    # every pass over a looped layer has keys and state of its own; a window and no window are two groups
    assert sorted((g["head_dim"], g["kv_heads"], g["window"], g["layers"]) for g in layout["kv_groups"]) == [(8, 2, 9, 1), (16, 3, None, 3)]
    states = sorted((s["step"], s["name"], tuple(s["shape"])) for s in layout["states"])
    assert states[:2] == [(1, "S", (4, 10, 12)), (1, "conv", (3, 88))] and (7, "conv", (1, 64)) in states and len(states) == 8
    names = {e["name"]: e["shape"] for e in d["expected_tensors"]}
    assert names["loop.in"] == [48, 96] and names["l0.mix.k"] == [16, 48] and names["l0.mix.q.b"] == [48] and names["l0.mix.g"] == [6, 48]
    assert names["l1.mix.v.conv"] == [48, 4] and names["l1.mix.A_log"] == [4] and names["l1.mix.norm"] == [12] and names["final.norm.b"] == [48]
    assert "l0.mix.v" not in names and "l3.norm2" not in names and "l3.mlp.up" not in names
    again = ModelSpec.from_json(spec).to_json()
    assert again["layers"][1]["ffn_post_norm"]["kind"] == "layernorm" and again["order"][3]["reinject"] and again["reinjection"]["kind"] == "linear_concat"


def test_what_may_be_absent():
    cfg = copy.deepcopy(CFG)
    del cfg["loop"]
    spec = native.describe_config(cfg)["spec"]
    assert [s["layer"] for s in spec["order"]] == [0, 1, 2, 3] and "reinjection" not in spec
    assert "loop.in" not in {e["name"] for e in native.describe_config(cfg)["expected_tensors"]}
    cfg["loop"] = {"start": 2, "stop": 2, "times": 5}        # an empty range: nothing runs again, nothing comes in again
    assert "reinjection" not in native.describe_config(cfg)["spec"]
    cfg["loop"] = {"start": 0, "stop": 4, "times": 1}
    order = native.describe_config(cfg)["spec"]["order"]
    assert [bool(s.get("reinject")) for s in order] == [True, False, False, False]


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "softmax", "type"), (("layers", 1, "mixer", "heads"), 3, "heads"),
    (("layers", 0, "mlp", "kind"), "moe", "kind"), (("layers", 0, "mixer", "vdim"), 12, "vdim"),
    (("loop", "stop"), 9, "loop"), (("norm", "eps"), 0.0, "eps"), (("layers", 0, "mixer", "rot", "dims"), 5, "dims"),
    (("layers", 0, "mixer", "rot", "scaling", "high"), 0.5, "scaling"), (("layers", 1, "mixer", "conv"), 0, "conv"),
    (("layers", 0, "mixer", "mask", "size"), 0, "size")])
def test_errors_name_the_key(path, value, word):
    cfg = copy.deepcopy(CFG)
    at = cfg
    for p in path[:-1]:
        at = at[p]
    at[path[-1]] = value
    with pytest.raises(native.NativeArgumentError, match=word):
        native.describe_config(cfg)
