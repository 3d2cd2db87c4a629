"""The Regipel design in the engine against the plain implementation (``plain_regipel.py``):
each mechanism alone through the step function (latent attention with sink and gate, routed
experts, several residual streams, the norm whose weight lies around zero, scaled embedding
and logits), whole models of several shapes in every way of cutting and batching, weights
made so that a far key, a sink or a lost page shows, long decoding, and greedy generation
through the engine's entry point and scheduler.  Sizes differ from model to model in every
number, and include values that make mechanisms degenerate (one stream, no streams, top = 1,
top = all experts, a layer without a feed-forward, scales of 1, a loop of one pass, a
rotation of only part of the rotated values, layers whose cached rows differ in width).
"""
import json
import os

import pytest
import torch

import plain_regipel as plain
from helpers import (EngineDriver, assert_close, assert_close_f32, mixed_schedule, peak_tokens,
                     portions_schedule, random_tokens, tail_decode_schedule, whole_schedule)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STD = 0.08


def mixer(heads, dim, rot_dim, vdim, rank, dims=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dim if dims is None else dims}
    return m


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(m, f):
    return {"type": "latent_attention", "mixer": m, "mlp": f}


# three streams, a loop of two passes over the middle layers, two experts of six a token
R1 = {"architecture": "Regipel", "vocab": 300, "width": 96, "streams": 3, "norm": {"eps": 1e-5},
      "embedding": {"scale": 3.5}, "logit_scale": 0.25, "loop": {"start": 1, "stop": 3, "times": 2},
      "layers": [layer(mixer(3, 24, 8, 16, 40, base=5000.0, scale=0.21), moe(6, 2, 48)) for _ in range(4)]}
# no streams (plain sums), no loop, scales of 1 (absent), a layer without feed-forward, one expert a
# token, a rotation of half of the rotated values, layers whose cached rows differ in width
R2 = {"architecture": "Regipel", "vocab": 211, "width": 64, "norm": {"eps": 3e-6},
      "layers": [layer(mixer(2, 16, 16, 32, 72, dims=8), moe(5, 1, 40)),
                 layer(mixer(4, 8, 8, 8, 24, base=300.0), None),
                 layer(mixer(2, 16, 16, 32, 72, dims=8), moe(5, 1, 40))]}
# one stream (with its own in, out and mix numbers), a loop of one pass, all experts chosen, no
# rotated part at all in one layer, odd sizes
R3 = {"architecture": "Regipel", "vocab": 157, "width": 80, "streams": 1, "norm": {"eps": 1e-4},
      "embedding": {"scale": 0.7}, "logit_scale": 2.0, "loop": {"start": 0, "stop": 2, "times": 1},
      "layers": [layer(mixer(5, 8, 4, 12, 20), moe(3, 3, 24)),
                 layer(mixer(5, 8, 0, 12, 20), moe(3, 3, 24))]}
# two streams and heads of another shape: 64-wide compressed rows, three passes over one layer
R4 = {"architecture": "Regipel", "vocab": 260, "width": 128, "streams": 2, "norm": {"eps": 1e-5},
      "embedding": {"scale": 2.0}, "logit_scale": 0.5, "loop": {"start": 1, "stop": 2, "times": 3},
      "layers": [layer(mixer(2, 32, 32, 64, 64, base=100000.0), moe(8, 2, 64)) for _ in range(2)]}
# compressed rows that the matrix-core attention takes (a multiple of 16 values, rows of a multiple of
# 8): 48 + 8 with five heads, and 128 + 24 with eighteen heads (two groups of heads for single tokens)
R5 = {"architecture": "Regipel", "vocab": 190, "width": 64, "streams": 2, "norm": {"eps": 1e-5},
      "embedding": {"scale": 1.3}, "logit_scale": 0.8,
      "layers": [layer(mixer(5, 16, 8, 16, 48, base=700.0), moe(4, 2, 32)) for _ in range(2)]}
R6 = {"architecture": "Regipel", "vocab": 175, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 1.5,
      "layers": [layer(mixer(18, 8, 24, 8, 128, dims=16), None), layer(mixer(18, 8, 24, 8, 128, dims=16), moe(3, 1, 32))]}
MODELS = {"R1": (R1, 11), "R2": (R2, 12), "R3": (R3, 13), "R4": (R4, 14), "R5": (R5, 15), "R6": (R6, 16)}
LENGTHS = {"R1": [40, 57, 90, 128, 65, 33], "R2": [45, 130, 64, 100, 17, 33], "R3": [70, 33, 16, 97, 48, 15],
           "R4": [31, 32, 150, 64, 49, 80], "R5": [63, 64, 65, 129, 20, 200], "R6": [70, 128, 13, 66, 191, 40]}
SCHEDULES = {"whole": whole_schedule, "tail12": lambda reqs: tail_decode_schedule(reqs, tail=12),
             "portions": portions_schedule, "mixed": mixed_schedule}


def every_expert(cfg):
    """The same model with every expert taken by every token.  In bfloat16 a router whose candidates
    lie closer than the rounding of its input may choose the other expert, which moves a row by far
    more than rounding; the bfloat16 comparisons therefore run on models whose routers have no
    choice to make (scores, weights on the input and the sum over experts stay), and the choice
    itself is compared in 32-bit."""
    out = json.loads(json.dumps(cfg))
    for l in out["layers"]:
        if l["mlp"]:
            l["mlp"]["router"]["top"] = l["mlp"]["router"]["experts"]
    return out


def config_of(name, dtype):
    cfg, seed = MODELS[name]
    return (cfg if dtype == "float32" else every_expert(cfg)), seed


def write_model(folder, cfg, seed, storage=torch.float32, std=STD, replace=None, change=None):
    """A model folder of random tensors for ``cfg``; ``replace``: name -> tensor, ``change``:
    name -> function of the drawn tensor."""
    from celeg_amd import native
    from celeg_amd.weights import random_tensors
    from celeg_amd.weights.safetensors_io import write_safetensors
    expected = native.describe_config(cfg)["expected_tensors"]
    tensors = random_tensors(expected, seed, std, torch.float32)
    for name, t in (replace or {}).items():
        assert tensors[name].shape == t.shape, name
        tensors[name] = t.float()
    for name, fn in (change or {}).items():
        tensors[name] = fn(tensors[name])
    tensors = {k: v.to(storage).contiguous() for k, v in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return str(folder)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            cfg, seed = config_of(name, dtype)
            storage = torch.float32 if dtype == "float32" else torch.bfloat16
            made[(name, dtype)] = write_model(tmp_path_factory.mktemp(f"{name}_{dtype}"), cfg, seed, storage)
        return made[(name, dtype)]
    return get


_plain = {}


def requests_of(name):
    cfg, seed = MODELS[name]
    return {f"r{i}": random_tokens(cfg["vocab"], n, seed=100 * seed + i) for i, n in enumerate(LENGTHS[name])}


def plain_logits(folder, key, requests):
    if key not in _plain:
        cfg, W = plain.load_model_folder(folder)
        _plain[key] = {rid: plain.model_logits(cfg, W, toks) for rid, toks in requests.items()}
    return _plain[key]


def load(folder, dtype, steps, max_requests=4, **kw):
    from celeg_amd.engine import load_model
    max_tokens = peak_tokens(steps)
    lm = load_model(folder, dtype=dtype, device=DEV, page_tokens=16, n_pages=max_tokens // 16, max_requests=max_requests,
                    max_context=max_tokens, max_batched_tokens=max(max_tokens, 64), **kw)
    return lm, max_tokens


@pytest.mark.parametrize("mode", list(SCHEDULES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MODELS))
def test_engine_matches_plain(folders, name, dtype, mode):
    """Whole prompts; prefill then 12 tokens one by one; portions down to two tokens (and single
    ones) that cross page borders; four live requests with pages and slots used again."""
    folder = folders(name, dtype)
    reqs = requests_of(name)
    steps = SCHEDULES[mode](reqs)
    lm, max_tokens = load(folder, dtype, steps)
    got = EngineDriver(lm).run(steps)
    ref = plain_logits(folder, (name, dtype), reqs)
    for rid in reqs:
        assert_close(got[rid], ref[rid], dtype, f"{name}/{dtype}/{mode}/{rid}")
    lm.cache.check()
    assert lm.cache.n_free_slots == 4 and lm.cache.free_pages() == [max_tokens // 16] * len(lm.cache.free_pages())
    paths = lm.paths()
    assert paths["attention_latent"] > 0
    fast = dtype == "bfloat16" and name in ("R4", "R5", "R6")
    assert (paths["attention_latent_rows"] > 0) == fast
    assert (paths["attention_latent_decode"] > 0) == (fast and mode != "whole")
    if any(l["mlp"] for l in MODELS[name][0]["layers"]):   # (every model here has some)
        assert lm.paths()["routed_experts"] > 0


def test_batches_of_unequal_requests_equal_each_alone(folders):
    """In 32-bit a row's logits are the same numbers whatever else is in the batch and however
    the prompt was cut (every kernel's order of additions depends on the row alone)."""
    folder = folders("R1", "float32")
    reqs = requests_of("R1")
    alone_steps, mixed_steps = whole_schedule(reqs), mixed_schedule(reqs, seed=3)
    lm, _ = load(folder, "float32", alone_steps)
    alone = EngineDriver(lm).run(alone_steps)
    lm2, _ = load(folder, "float32", mixed_steps)
    mixed = EngineDriver(lm2).run(mixed_steps)
    for rid in reqs:
        assert torch.equal(alone[rid], mixed[rid]), rid


# ------------------------------------------------------------------ weights made so that a fault shows
def sharp(cfg, factor):
    """Queries scaled up so that every softmax is nearly one key, which for most rows lies far back."""
    return {f"l{i}.mix.q": (lambda t, f=factor: t * f) for i in range(len(cfg["layers"]))}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dtype):
    """700 tokens, attention made sharp: a row's result is one key's value, often hundreds of
    tokens and dozens of pages back; a lost page or a key one off changes the logits wholly."""
    cfg = {"architecture": "Regipel", "vocab": 180, "width": 64, "streams": 2, "norm": {"eps": 1e-5},
           "embedding": {"scale": 1.5}, "logit_scale": 1.0,
           "layers": [layer(mixer(2, 16, 8, 16, 48, base=2000.0), None), layer(mixer(2, 16, 8, 16, 48, base=2000.0), moe(4, 1, 32))]}
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    # (in bfloat16 two keys whose scores lie within rounding of each other would trade places: less sharp there)
    cfg = cfg if dtype == "float32" else every_expert(cfg)
    folder = write_model(tmp_path / "far", cfg, 5, storage, std=0.1, change=sharp(cfg, 12.0 if dtype == "float32" else 3.0))
    c, W = plain.load_model_folder(folder)
    toks = random_tokens(cfg["vocab"], 700, seed=9)
    ref = plain.model_logits(c, W, toks)
    reqs = {"far": toks}
    for steps in (whole_schedule(reqs), tail_decode_schedule(reqs, tail=40),
                  portions_schedule(reqs, sizes=(97, 2, 130, 31, 16, 1, 64, 3))):
        lm, _ = load(folder, dtype, steps)
        got = EngineDriver(lm).run(steps)["far"]
        assert_close(got, ref, dtype, f"far/{dtype}")


def test_the_sink_shows():
    """The plain attention with and without the sink differ by far more than the tolerance when the
    sinks are large, so the comparison below cannot pass with the sink left out."""
    torch.manual_seed(0)
    m = mixer(2, 8, 4, 8, 12)
    W = {"q": torch.randn(24, 16), "dkv": torch.randn(16, 16), "dkv.norm": torch.ones(12), "uk": torch.randn(16, 12),
         "uv": torch.randn(16, 12), "sink": torch.tensor([4.0, 6.0]), "g": torch.randn(16, 16), "o": torch.randn(16, 16)}
    W = {k: v.double() for k, v in W.items()}
    h = torch.randn(9, 16, dtype=torch.float64)
    with_sink = plain.latent_attention(h, W, "", m, 1e-5)
    without = plain.latent_attention(h, W, "", dict(m, sink=False), 1e-5)
    assert float((with_sink - without).abs().max()) > 0.1 * float(with_sink.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_large_sinks(tmp_path, dtype):
    """Sinks that take most of the softmax's weight at the first tokens (few keys) and less later."""
    cfg = dict(R4, layers=[layer(mixer(4, 16, 16, 16, 32), moe(4, 2, 32)) for _ in range(2)])
    sinks = {f"l{i}.mix.sink": torch.tensor([5.0, -4.0, 2.5, 0.0]) for i in range(2)}
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    cfg = cfg if dtype == "float32" else every_expert(cfg)
    folder = write_model(tmp_path / "sink", cfg, 21, storage, replace=sinks)
    c, W = plain.load_model_folder(folder)
    reqs = {"a": random_tokens(cfg["vocab"], 50, seed=1), "b": random_tokens(cfg["vocab"], 21, seed=2)}
    steps = mixed_schedule(reqs, seed=1, decode_tail=8)
    lm, _ = load(folder, dtype, steps)
    got = EngineDriver(lm).run(steps)
    for rid, toks in reqs.items():
        assert_close(got[rid], plain.model_logits(c, W, toks), dtype, f"sink/{rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_many_pages(folders, dtype):
    """A short prompt, then 200 tokens one by one (steps replayed from a recorded graph), over a
    dozen page borders and, in bfloat16, over the borders of the blocks of 64 keys and of the
    shares that the keys of a single token are cut into."""
    folder = folders("R4", dtype)
    toks = random_tokens(R4["vocab"], 215, seed=77)
    steps = tail_decode_schedule({"long": toks}, tail=200)
    lm, _ = load(folder, dtype, steps)
    if dtype == "bfloat16":
        lm.set_knob("latent_decode_workgroups", 3)      # three shares of the keys,
        lm.set_knob("latent_decode_min_blocks", 1)      # however few the keys
    got = EngineDriver(lm).run(steps)["long"]
    c, W = plain.load_model_folder(folder)
    assert_close(got, plain.model_logits(c, W, toks), dtype, "long decoding")
    assert lm.runner.counters()["graph_replays"] > 100


def test_pages_and_slots_used_again(folders):
    """Ten requests through two slots and a pool of six pages: every page and slot serves several
    requests, and each request's logits equal the plain ones."""
    folder = folders("R1", "float32")
    reqs = {f"q{i}": random_tokens(R1["vocab"], n, seed=500 + i) for i, n in enumerate([30, 18, 33, 16, 5, 47, 31, 2, 40, 17])}
    steps = mixed_schedule(reqs, max_live=2, seed=4, decode_tail=6)
    from celeg_amd.engine import load_model
    lm = load_model(folder, dtype="float32", device=DEV, page_tokens=16, n_pages=6, max_requests=2, max_context=64,
                    max_batched_tokens=128)
    got = EngineDriver(lm).run(steps)
    c, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        assert_close_f32(got[rid], plain.model_logits(c, W, toks), rid)
    assert lm.cache.free_pages() == [6]


# ------------------------------------------------------------------ generation through the entry point
@pytest.mark.parametrize("name", ["R1", "R2"])
def test_greedy_generation_through_the_entry_point(folders, name):
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GenerationConfig
    folder = folders(name, "float32")
    cfg, W = plain.load_model_folder(folder)
    prompts = [random_tokens(cfg["vocab"], n, seed=40 + n) for n in (5, 23, 1, 37, 12)]
    engine = Engine.from_folder(folder, dtype="float32", device=DEV, max_active_requests=3, max_batched_tokens=64,
                                prefill_chunk_tokens=16, context=128, n_pages=24)
    greedy = GenerationConfig(temperature=0.0, repetition_penalty=1.0)
    outs = engine.generate(prompts, max_new_tokens=20, generation=greedy, eos_token_ids=[])
    for prompt, out in zip(prompts, outs):
        assert out == plain.greedy(cfg, W, prompt, 20)
    engine.close()


# ------------------------------------------------------------------ each mechanism alone
def alone_architecture():
    """"RegipelPartsAlone": one block put together from what the configuration spells out; the
    embedding table is the input x (tokens 0..T-1), the head gives the stream's rows back."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    if "RegipelPartsAlone" in registered_architectures():
        return

    def build(cfg, shapes):
        W, rows = cfg["width"], cfg["rows"]
        part = lambda key, neutral: PartSpec.from_json(cfg[key]) if cfg.get(key) else neutral
        link = lambda key: PartSpec.from_json(cfg[key]) if cfg.get(key) else None
        block = LayerSpec(part("mixer", PartSpec("none", {"width": W})), part("mixer_norm", PartSpec("identity")),
                          part("ffn", PartSpec("none")), part("ffn_norm", PartSpec("identity")),
                          cfg.get("arrangement", "pre_norm"), link("mixer_link"), link("ffn_link"))
        return ModelSpec("RegipelPartsAlone", rows, W, 256,
                         PartSpec("embedding", {"vocab": rows, "width": W, "scale": cfg.get("embedding_scale", 1.0)}, {"table": "x"}),
                         (block,), (RunStep(0),), part("final_norm", PartSpec("identity")), PartSpec("hidden", {"width": W}),
                         streams=cfg.get("streams", 1))
    register_architecture("RegipelPartsAlone", build)


def run_alone(tmp_path, cfg, tensors, cut=(5, 2, 9, 1, 3, 17)):
    """x + part(x) (or what the arrangement makes of it) for rows 0..T-1, in portions."""
    from celeg_amd.engine import load_model
    from celeg_amd.weights.safetensors_io import write_safetensors
    alone_architecture()
    cfg = dict(cfg, architectures=["RegipelPartsAlone"])
    os.makedirs(tmp_path, exist_ok=True)
    with open(os.path.join(tmp_path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(tmp_path, "model.safetensors"), {k: v.float().contiguous() for k, v in tensors.items()})
    steps = portions_schedule({"x": list(range(cfg["rows"]))}, sizes=cut)
    lm = load_model(str(tmp_path), dtype="float32", device=DEV, page_tokens=16, n_pages=8, max_requests=2, max_context=128,
                    max_batched_tokens=64)
    return EngineDriver(lm).run(steps)["x"].double()


def test_latent_attention_alone(tmp_path):
    torch.manual_seed(1)
    T, W_ = 37, 40
    m = mixer(3, 8, 6, 10, 14, dims=4, base=50.0, scale=0.4)
    names = {r: r for r in ("q", "dkv", "dkv_norm", "uk", "uv", "o", "sink", "g")}
    t = {"x": torch.randn(T, W_), "q": torch.randn(3 * 14, W_) * 0.3, "dkv": torch.randn(20, W_) * 0.3,
         "dkv_norm": 1 + 0.2 * torch.randn(14), "uk": torch.randn(24, 14) * 0.4, "uv": torch.randn(30, 14) * 0.4,
         "o": torch.randn(W_, 30) * 0.3, "sink": torch.tensor([1.5, -2.0, 3.0]), "g": torch.randn(30, W_) * 0.3}
    part = {"kind": "latent_attention", "tensors": names,
            "params": {"width": W_, "heads": 3, "dim": 8, "rot_dim": 6, "vdim": 10, "kv_rank": 14, "scale": 0.4, "eps": 1e-4,
                       "sink": True, "gate": True,
                       "position": {"kind": "rope", "params": {"theta": 50.0, "rotary_dim": 4, "head_dim": 6, "pairing": "neighbours"}}}}
    got = run_alone(tmp_path, {"width": W_, "rows": T, "mixer": part}, t)
    Wd = {k.replace("dkv_norm", "dkv.norm"): v.double() for k, v in t.items()}
    x = Wd["x"]
    assert_close_f32(got, x + plain.latent_attention(x, Wd, "", m, 1e-4), "latent attention alone")
    # without sink and gate the same part computes the plain softmax
    part2 = json.loads(json.dumps(part))
    part2["params"].update(sink=False, gate=False)
    part2["tensors"] = {k: v for k, v in names.items() if k not in ("sink", "g")}
    got2 = run_alone(tmp_path / "plain", {"width": W_, "rows": T, "mixer": part2}, {k: v for k, v in t.items() if k not in ("sink", "g")})
    assert_close_f32(got2, x + plain.latent_attention(x, Wd, "", dict(m, sink=False, gate=False), 1e-4), "no sink, no gate")


@pytest.mark.parametrize("experts,top", [(7, 2), (4, 1), (3, 3), (70, 5)])
def test_routed_experts_alone(tmp_path, experts, top):
    torch.manual_seed(2)
    T, W_, ff = 41, 24, 20
    t = {"x": torch.randn(T, W_), "router": torch.randn(experts, W_)}
    names = {"router": "router"}
    for e in range(experts):
        for role, shape in (("gate", (ff, W_)), ("up", (ff, W_)), ("down", (W_, ff))):
            t[f"e{e}.{role}"] = torch.randn(*shape) * 0.3
            names[f"{role}.{e}"] = f"e{e}.{role}"
    part = {"kind": "routed_experts", "tensors": names,
            "params": {"width": W_, "ff": ff, "experts": experts, "top": top, "score": "sigmoid", "weight_on": "input"}}
    got = run_alone(tmp_path, {"width": W_, "rows": T, "ffn": part}, t)
    Wd = {k: v.double() for k, v in t.items()}
    want = Wd["x"] + plain.routed_experts(Wd["x"], Wd, "", moe(experts, top, ff))
    assert_close_f32(got, want, f"routed experts alone ({experts}, {top})")


@pytest.mark.parametrize("streams", [1, 2, 4])
def test_residual_streams_alone(tmp_path, streams):
    """Two sub-layers on S streams: the mixer is absent (its output is zero, so its link only mixes
    the streams), the feed-forward is a dense gated one behind a norm whose weight lies around zero;
    the embedding's scale multiplies every stream's start."""
    torch.manual_seed(3)
    T, W_, ff, S = 29, 32, 40, streams
    t = {"x": torch.randn(T, W_), "n2": 0.3 * torch.randn(W_), "g": torch.randn(ff, W_) * 0.3, "u": torch.randn(ff, W_) * 0.3,
         "d": torch.randn(W_, ff) * 0.3}
    for q in (1, 2):
        t[f"hc{q}.in"], t[f"hc{q}.out"] = torch.randn(S), torch.randn(S)
        t[f"hc{q}.mix"] = torch.eye(S) + 0.4 * torch.randn(S, S)
    link = lambda q: {"kind": "hyper_link", "params": {"streams": S},
                      "tensors": {"in": f"hc{q}.in", "out": f"hc{q}.out", "mix": f"hc{q}.mix"}}
    cfg = {"width": W_, "rows": T, "arrangement": "hyper_connections", "streams": S, "embedding_scale": 1.7,
           "mixer_link": link(1), "ffn_link": link(2),
           "ffn": {"kind": "swiglu", "params": {"width": W_, "ff": ff}, "tensors": {"gate": "g", "up": "u", "down": "d"}},
           "ffn_norm": {"kind": "rmsnorm", "params": {"width": W_, "eps": 1e-5, "weight_offset": 1.0}, "tensors": {"weight": "n2"}}}
    got = run_alone(tmp_path, cfg, t)
    Wd = {k: v.double() for k, v in t.items()}
    xs = [Wd["x"] * 1.7 for _ in range(S)]
    xs = plain.hyper_sublayer(xs, Wd, "hc1", lambda u: torch.zeros_like(u))
    dense = lambda u: (torch.nn.functional.silu(u @ Wd["g"].T) * (u @ Wd["u"].T)) @ Wd["d"].T
    xs = plain.hyper_sublayer(xs, Wd, "hc2", lambda u: dense(plain.zero_centred_norm(u, Wd["n2"], 1e-5)))
    assert_close_f32(got, sum(xs), f"{S} streams alone")
