"""Reading a Regipel config.json: the run order that a loop makes, the parts and constants of
every layer, the cache the model asks for, and the errors that name the key at fault.  No GPU."""
import copy

import pytest

from celeg_amd import native
from celeg_amd.config import ModelSpec

CFG = {"architecture": "Regipel", "vocab": 123, "width": 48, "streams": 3, "norm": {"eps": 2e-5},
       "embedding": {"scale": 4.0}, "logit_scale": 0.125, "loop": {"start": 1, "stop": 3, "times": 2},
       "layers": [{"type": "latent_attention",
                   "mixer": {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 10 + 2 * (i % 2), "scale": 0.3,
                             "rot": {"base": 777.0, "dims": 2}},
                   "mlp": None if i == 3 else {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 5, "top": 2}}}
                  for i in range(4)]}


def test_run_order_parts_and_cache():
    d = native.describe_config(CFG)
    spec = d["spec"]
    assert [s["layer"] for s in spec["order"]] == [0, 1, 2, 1, 2, 3]
    assert spec["streams"] == 3 and spec["vocab_size"] == 123 and spec["hidden_size"] == 48
    first = spec["layers"][0]
    assert first["arrangement"] == "hyper_connections" and first["mixer"]["kind"] == "latent_attention"
    assert first["mixer"]["params"]["position"]["params"] == {"theta": 777.0, "rotary_dim": 2, "head_dim": 4, "pairing": "neighbours"}
    assert first["mixer_norm"]["params"]["weight_offset"] == 1.0
    assert first["ffn"]["params"]["weight_on"] == "input" and first["ffn"]["params"]["top"] == 2
    assert spec["layers"][3]["ffn"]["kind"] == "none"
    assert spec["embedding"]["params"]["scale"] == 4.0 and spec["head"]["params"]["scale"] == 0.125
    # every pass over a looped layer has a cache of its own; rows of 14 and of 16 values are two groups
    groups = d["cache_layout"]["kv_groups"]
    assert sorted((g["head_dim"], g["layers"], g["keys_only"], g["v_head_dim"]) for g in groups) == [(14, 3, True, 0), (16, 3, True, 0)]
    names = {e["name"]: e["shape"] for e in d["expected_tensors"]}
    assert names["l1.mix.uk"] == [24, 12] and names["l0.mix.dkv"] == [14, 48] and names["l2.mlp.e4.down"] == [48, 20]
    assert names["l0.hc2.mix"] == [3, 3] and "l3.hc2.in" not in names and "l3.norm2" not in names
    assert ModelSpec.from_json(spec).to_json()["layers"][0]["mixer_link"]["kind"] == "hyper_link"


def test_what_may_be_absent():
    cfg = copy.deepcopy(CFG)
    for key in ("streams", "loop", "embedding", "logit_scale"):
        del cfg[key]
    spec = native.describe_config(cfg)["spec"]
    assert spec["streams"] == 1 and [s["layer"] for s in spec["order"]] == [0, 1, 2, 3]
    assert spec["layers"][0]["arrangement"] == "pre_norm" and "mixer_link" not in spec["layers"][0]
    assert spec["embedding"]["params"]["scale"] == 1.0 and spec["head"]["params"]["scale"] == 1.0


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "windowed", "type"), (("layers", 1, "mixer", "heads"), 0, "heads"),
    (("layers", 0, "mlp", "kind"), "dense", "kind"), (("layers", 0, "mlp", "router", "top"), 6, "top"),
    (("loop", "stop"), 9, "loop"), (("norm", "eps"), 0.0, "eps"), (("layers", 2, "mixer", "rot", "dims"), 3, "dims"),
    (("streams",), 9, "streams")])
def test_errors_name_the_key(path, value, word):
    cfg = copy.deepcopy(CFG)
    at = cfg
    for p in path[:-1]:
        at = at[p]
    at[path[-1]] = value
    with pytest.raises(native.NativeArgumentError, match=word):
        native.describe_config(cfg)
