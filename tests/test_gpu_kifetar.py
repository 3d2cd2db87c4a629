"""The Kifetar design in the engine against the plain implementation (``plain_kifetar.py``):
each mechanism alone through the step function (attention with sigmoid weights, the gated
delta rule, norms before and after a sub-layer, the embedding's rows taken in again), whole
models of several shapes in every way of cutting and batching, weights made so that a
window that is one key off or a state that is lost shows, long decoding, pages and slots
used again, and greedy generation through the engine's entry point and scheduler.  Sizes
differ from model to model in every number and include values that make mechanisms
degenerate: one query head per key head and all query heads on one, a window of one key,
no window, no rotation, a rotation of the whole head, convolutions of one tap, value
columns that do not fill a wavefront, a layer without feed-forward, no loop, a loop from
the first layer, a loop of one pass, widths that are no multiple of 16.
"""
import json
import os

import pytest
import torch

import plain_kifetar as plain
from helpers import (EngineDriver, assert_close_f32, mixed_schedule, peak_tokens, portions_schedule, random_tokens,
                     tail_decode_schedule, whole_schedule)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STD = 0.08


def assert_close(got, ref, dtype, what=""):
    """32-bit: the shared bound (1e-4 of the largest logit).  bfloat16: relative RMS error <= 8e-2 and
    max |d| <= 1.2e-1 * max |ref|.  A norm behind every sub-layer divides the sub-layer's rounded
    output by its spread, and looped layers do so several times, so rounding alone moves these narrow
    models' logits by 1.8e-2 to 4.5e-2 relative RMS (measured; the same numbers however a prompt is
    cut); the faults these tests look for (a key, a state, a pass too many or too few) move them by
    tens of percent, and the 32-bit runs of the same schedules hold them to 1e-4."""
    if dtype in ("float32", torch.float32):
        return assert_close_f32(got, ref, what)
    got, ref = torch.as_tensor(got).double(), torch.as_tensor(ref).double()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    d = got - ref
    rel, mx = float(d.pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()), float(d.abs().max() / ref.abs().max())
    assert rel <= 8e-2 and mx <= 1.2e-1, f"{what}: rel rms {rel:.3e} (<= 8e-2), max/|ref|max {mx:.3e} (<= 1.2e-1)"


def attention(heads, kv_heads, dim, window=None, rot=None, scale=None, ff=48):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = rot
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta(heads, kv_heads, dim, vdim, taps, ff=48):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def rot(dims, base=10000.0, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


# a loop of two passes over the middle layers; frequencies on both sides of the scaling's band and inside it
K1 = {"architecture": "Kifetar", "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 2},
      "layers": [attention(6, 2, 16, window=20, rot=rot(8, 1000.0, (4.0, 1.0, 4.0, 64))), delta(4, 2, 16, 24, 4),
                 attention(3, 3, 32, rot=rot(32, 300.0)), delta(2, 1, 24, 80, 2, ff=None)]}
# no loop, a width that is no multiple of 16, one tap, a window of one key, all query heads on one key head
K2 = {"architecture": "Kifetar", "vocab": 211, "width": 72, "norm": {"eps": 3e-6},
      "layers": [delta(5, 5, 8, 8, 1, ff=40), attention(5, 1, 8, window=1, ff=None),
                 attention(2, 1, 64, window=17, rot=rot(64, 50000.0, (8.0, 1.0, 2.0, 32)), ff=56), delta(3, 1, 40, 12, 5, ff=40)]}
# the whole model runs three times: the embedding's rows come in before the very first layer too
K3 = {"architecture": "Kifetar", "vocab": 157, "width": 64, "norm": {"eps": 1e-4}, "loop": {"start": 0, "stop": 2, "times": 3},
      "layers": [delta(2, 2, 32, 32, 3, ff=32), attention(8, 2, 16, window=64, rot=rot(4, 77.0), scale=0.4, ff=32)]}
# a loop of one pass, heads of 128 and of 64 values, windows that end inside a page
K4 = {"architecture": "Kifetar", "vocab": 260, "width": 128, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 2, "times": 1},
      "layers": [attention(2, 2, 128, window=33, rot=rot(32, 5000.0)), delta(8, 2, 64, 64, 4, ff=64),
                 attention(4, 1, 32, window=5, ff=64)]}
MODELS = {"K1": (K1, 21), "K2": (K2, 22), "K3": (K3, 23), "K4": (K4, 24)}
LENGTHS = {"K1": [40, 57, 90, 128, 65, 33], "K2": [45, 130, 64, 100, 17, 33], "K3": [70, 33, 16, 97, 48, 150],
           "K4": [31, 32, 150, 64, 49, 80]}
SCHEDULES = {"whole": whole_schedule, "tail12": lambda reqs: tail_decode_schedule(reqs, tail=12),
             "portions": portions_schedule, "mixed": mixed_schedule}


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
            cfg, seed = MODELS[name]
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
        _plain[key] = {rid: plain.forward(cfg, W, toks) for rid, toks in requests.items()}
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
    ones) that cross page borders and windows; four live requests with pages and slots used again."""
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
    assert paths["attention_sigmoid"] > 0 and paths["delta_rule"] > 0


def test_batches_of_unequal_requests_equal_each_alone(folders):
    """In 32-bit a row's logits do not depend on what else is in the batch or on how the prompt was
    cut, beyond the rounding of 32-bit sums taken in another order (the delta rule takes the rows of
    a whole block two at a time, a cut block one at a time): held to 2e-5 of the largest logit."""
    folder = folders("K1", "float32")
    reqs = requests_of("K1")
    alone_steps, mixed_steps = whole_schedule(reqs), mixed_schedule(reqs, seed=3)
    lm, _ = load(folder, "float32", alone_steps)
    alone = EngineDriver(lm).run(alone_steps)
    lm2, _ = load(folder, "float32", mixed_steps)
    mixed = EngineDriver(lm2).run(mixed_steps)
    for rid in reqs:
        assert float((alone[rid] - mixed[rid]).abs().max()) <= 2e-5 * float(alone[rid].abs().max()), rid


# ------------------------------------------------------------------ weights made so that a fault shows
WINDOWS = (1, 2, 16, 17, 31, None)      # (None: every earlier key, however far)


def windows_model(windows=WINDOWS):
    return {"architecture": "Kifetar", "vocab": 120, "width": 48, "norm": {"eps": 1e-5},
            "layers": [attention(2, 1, 16, window=w, rot=rot(8, 200.0), ff=None) for w in windows]}


def sharp(cfg, factor):
    """Queries scaled up: a key's weight is close to 0 or to 1, so one key more or less in a window
    moves a head's sum by about a whole value."""
    return {f"l{i}.mix.q": (lambda t, f=factor: t * f) for i in range(len(cfg["layers"]))}


def test_a_window_one_key_off_shows():
    """The plain attention with windows one key longer or shorter differs by far more than the
    tolerance, so the comparison below cannot pass with an edge that is one key off."""
    torch.manual_seed(0)
    h = torch.randn(40, 24, dtype=torch.float64)
    t = {"q": torch.randn(32, 24) * 2, "q.b": torch.randn(32), "k": torch.randn(16, 24), "k.b": torch.randn(16), "q.norm": torch.ones(16),
         "k.norm": torch.ones(16), "temp": torch.tensor([1.0, 1.3]), "pb": torch.tensor([0.5, -0.5]), "g": torch.randn(2, 24),
         "o": torch.randn(24, 32)}
    t = {k: v.double() for k, v in t.items()}
    for w in (1, 2, 16):
        m = lambda size: {"heads": 2, "kv_heads": 1, "dim": 16, "scale": 0.25, "mask": {"size": size}}
        right = plain.sigmoid_window_attention(h, m(w), t, "", 1e-5)
        for other in (w - 1, w + 1):
            if other:
                wrong = plain.sigmoid_window_attention(h, m(other), t, "", 1e-5)
                assert float((right - wrong).abs().max()) > 0.05 * float(right.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edges_in_prompts_and_decoding(tmp_path, dtype):
    """Windows of 1, 2, 16 (a page), 17 and 31 keys and no window at all, with sharp weights, in whole
    prompts, in portions of every size and in tokens decoded one by one past every window's length."""
    cfg = windows_model()
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = write_model(tmp_path / "win", cfg, 5, storage, std=0.1, change=sharp(cfg, 6.0 if dtype == "float32" else 2.0))
    c, W = plain.load_model_folder(folder)
    reqs = {"a": random_tokens(cfg["vocab"], 100, seed=9), "b": random_tokens(cfg["vocab"], 37, seed=10)}
    ref = {rid: plain.forward(c, W, toks) for rid, toks in reqs.items()}
    for steps in (whole_schedule(reqs), tail_decode_schedule(reqs, tail=36),
                  portions_schedule(reqs, sizes=(15, 2, 17, 1, 31, 3, 16, 2)), mixed_schedule(reqs, seed=2, decode_tail=20)):
        lm, _ = load(folder, dtype, steps)
        got = EngineDriver(lm).run(steps)
        for rid in reqs:
            assert_close(got[rid], ref[rid], dtype, f"windows/{dtype}/{rid}")


@pytest.mark.parametrize("dim", [32, 64, 96, 128])
def test_matrix_core_attention_equals_the_general_kernel(tmp_path, dim):
    """bfloat16: the kernel on the matrix cores against the kernel that scores key by key, on the
    same pages, with sharp weights and windows that end before, at and behind the borders of pages
    and of the blocks of 64 keys, in whole prompts, portions and single tokens.  The two differ in
    the rounding of the weights to bfloat16 only, so they are held to a fifth of what rounding does
    to a whole model."""
    cfg = {"architecture": "Kifetar", "vocab": 150, "width": 64, "norm": {"eps": 1e-5},
           "layers": [attention(4, 2, dim, window=w, rot=rot(dim // 2, 500.0), ff=None) for w in (1, 7, 64, 65, 100, None)]}
    folder = write_model(tmp_path / "mfma", cfg, 31, torch.bfloat16, std=0.1, change=sharp(cfg, 2.0))
    reqs = {"a": random_tokens(cfg["vocab"], 300, seed=9), "b": random_tokens(cfg["vocab"], 75, seed=10), "c": random_tokens(cfg["vocab"], 16, seed=11)}
    for steps in (whole_schedule(reqs), tail_decode_schedule(reqs, tail=15), portions_schedule(reqs, sizes=(15, 2, 17, 1, 130, 3, 16, 64)),
                  mixed_schedule(reqs, seed=2, decode_tail=5)):
        got = {}
        # the kernel that scores key by key; the form chosen by the step's longest portion; tiles of 16
        # rows whose key blocks the wavefronts take in turn; tiles of 64 rows that share staged keys
        for form in ("general", -1, 0, 1):
            lm, _ = load(folder, "bfloat16", steps)
            if form == "general":
                lm.set_knob("use_sigmoid_mfma", 0)
            else:
                lm.set_knob("sigmoid_rows_form", form)
            got[form] = EngineDriver(lm).run(steps)
            assert (lm.paths()["attention_sigmoid_rows"] > 0) == (form != "general")
        for form in (-1, 0, 1):
            for rid in reqs:
                a, b = got[form][rid].double(), got["general"][rid].double()
                rel = float((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt())
                assert rel <= 1.5e-2, f"head size {dim}, form {form}, {rid}: rel rms {rel:.3e}"


def test_delta_rule_in_registers_equals_the_general_kernel(folders):
    """32-bit: the recurrence with the state in registers against the kernel for any size, same schedule."""
    folder = folders("K4", "float32")
    reqs = requests_of("K4")
    steps = mixed_schedule(reqs, seed=6)
    got = {}
    for general in (0, 1):
        lm, _ = load(folder, "float32", steps)
        lm.set_knob("delta_general", general)
        got[general] = EngineDriver(lm).run(steps)
    for rid in reqs:
        assert_close_f32(got[0][rid], got[1][rid], rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_state_that_remembers_hundreds_of_tokens(tmp_path, dtype):
    """Decays close to one: what the first tokens wrote into the state still shows 300 tokens
    later (the plain model run on the last 150 tokens alone gives other logits), so a state that
    is lost, zeroed or taken from another slot between steps cannot pass."""
    cfg = {"architecture": "Kifetar", "vocab": 140, "width": 64, "norm": {"eps": 1e-5},
           "layers": [delta(4, 2, 16, 20, 3, ff=32), delta(2, 2, 24, 16, 4, ff=None)]}
    slow = {f"l{i}.mix.A_log": torch.full((h,), -6.0) for i, h in ((0, 4), (1, 2))}
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = write_model(tmp_path / "far", cfg, 7, storage, std=0.1, replace=slow)
    c, W = plain.load_model_folder(folder)
    toks = random_tokens(cfg["vocab"], 300, seed=3)
    ref = plain.forward(c, W, toks)
    tail_alone = plain.forward(c, W, toks[150:])
    assert float((ref[-1] - tail_alone[-1]).abs().max()) > 0.02 * float(ref[-1].abs().max())
    reqs = {"far": toks, "other": random_tokens(cfg["vocab"], 90, seed=4)}
    ref = {"far": ref, "other": plain.forward(c, W, reqs["other"])}
    for steps in (tail_decode_schedule(reqs, tail=40), portions_schedule(reqs, sizes=(97, 2, 130, 31, 16, 1, 64, 3)),
                  mixed_schedule(reqs, seed=5, decode_tail=10)):
        lm, _ = load(folder, dtype, steps)
        got = EngineDriver(lm).run(steps)
        for rid in reqs:
            assert_close(got[rid], ref[rid], dtype, f"far state/{dtype}/{rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_many_pages(folders, dtype):
    """A short prompt, then 200 tokens one by one (steps replayed from a recorded graph), over a
    dozen page borders and past every window."""
    folder = folders("K4", dtype)
    toks = random_tokens(K4["vocab"], 215, seed=77)
    steps = tail_decode_schedule({"long": toks}, tail=200)
    lm, _ = load(folder, dtype, steps)
    got = EngineDriver(lm).run(steps)["long"]
    c, W = plain.load_model_folder(folder)
    assert_close(got, plain.forward(c, W, toks), dtype, "long decoding")
    assert lm.runner.counters()["graph_replays"] > 100


def test_pages_and_slots_used_again(folders):
    """Ten requests through two slots and a pool of six pages: every page and state slot serves
    several requests, and each request's logits equal the plain ones (a state that is not zeroed
    when its slot is given out again would show at the request's first token)."""
    folder = folders("K1", "float32")
    reqs = {f"q{i}": random_tokens(K1["vocab"], n, seed=500 + i) for i, n in enumerate([30, 18, 33, 16, 5, 47, 31, 2, 40, 17])}
    steps = mixed_schedule(reqs, max_live=2, seed=4, decode_tail=6)
    from celeg_amd.engine import load_model
    lm = load_model(folder, dtype="float32", device=DEV, page_tokens=16, n_pages=6, max_requests=2, max_context=64,
                    max_batched_tokens=128)
    got = EngineDriver(lm).run(steps)
    c, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        assert_close_f32(got[rid], plain.forward(c, W, toks), rid)
    assert all(n == 6 for n in lm.cache.free_pages())


# ------------------------------------------------------------------ generation through the entry point
@pytest.mark.parametrize("name", ["K1", "K2"])
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


def test_command_line(folders, tmp_path):
    """``bin/celeg-run`` on a model folder of the design: greedy tokens and the prompt's last logits."""
    import subprocess
    import sys
    import numpy as np
    folder = folders("K2", "float32")
    cfg, W = plain.load_model_folder(folder)
    prompt = random_tokens(cfg["vocab"], 19, seed=5)
    dump = str(tmp_path / "logits.f32")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "celeg-run"), "--model", folder, "--dtype", "float32", "--prompt",
                           ",".join(map(str, prompt)), "--max-new-tokens", "8", "--repetition-penalty", "1.0", "--context", "128",
                           "--runtime-tokens", "--dump-logits", dump], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    line = [l for l in proc.stdout.splitlines() if l.startswith("CELEG_GENERATED_TOKEN_IDS=")][0]
    assert json.loads(line.split("=", 1)[1]) == plain.greedy(cfg, W, prompt, 8)
    logits = np.fromfile(dump, dtype="<f4")
    assert_close_f32(torch.from_numpy(logits.copy()), plain.forward(cfg, W, prompt)[-1], "command line")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(folders, tmp_path, dtype):
    """``bin/trace_run`` in a process of its own: four schedules one after the other, a pool sized for
    the live requests only, logits read from the files it writes."""
    from helpers import TraceClient
    folder = folders("K1", dtype)
    reqs = requests_of("K1")
    ref = plain_logits(folder, ("K1", dtype), reqs)
    all_steps = []
    for tag, make in (("w", whole_schedule), ("t", tail_decode_schedule), ("p", portions_schedule), ("m", mixed_schedule)):
        for s in make({f"{tag}{rid}": toks for rid, toks in reqs.items()}):
            all_steps.append(dict(s, step=len(all_steps)))
    client = TraceClient(folder, dtype, str(tmp_path), peak_tokens(all_steps))
    got = {}
    for s in all_steps:
        logits = client.step(s["step"], s["entries"], s["end"])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(torch.as_tensor(logits[row]))
                row += 1
    assert client.close() == 0
    for rid_tagged, rows in got.items():
        assert_close(torch.stack(rows), ref[rid_tagged[1:]], dtype, f"trace/{dtype}/{rid_tagged}")


# ------------------------------------------------------------------ each mechanism alone
def alone_architecture():
    """"KifetarPartsAlone": one block put together from what the configuration spells out; the
    embedding table is the input x (tokens 0..T-1), the head gives the stream's rows back."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    if "KifetarPartsAlone" in registered_architectures():
        return

    def build(cfg, shapes):
        W, rows = cfg["width"], cfg["rows"]
        part = lambda key, neutral: PartSpec.from_json(cfg[key]) if cfg.get(key) else neutral
        maybe = lambda key: PartSpec.from_json(cfg[key]) if cfg.get(key) else None
        block = LayerSpec(part("mixer", PartSpec("none", {"width": W})), part("mixer_norm", PartSpec("identity")),
                          part("ffn", PartSpec("none")), part("ffn_norm", PartSpec("identity")),
                          cfg.get("arrangement", "pre_norm"), None, None, maybe("mixer_post_norm"), maybe("ffn_post_norm"))
        return ModelSpec("KifetarPartsAlone", rows, W, 256, PartSpec("embedding", {"vocab": rows, "width": W}, {"table": "x"}),
                         (block,), (RunStep(0, None, bool(cfg.get("reinjection"))),), PartSpec("identity"),
                         PartSpec("hidden", {"width": W}), reinjection=maybe("reinjection"))
    register_architecture("KifetarPartsAlone", build)


def run_alone(tmp_path, cfg, tensors, cut=(5, 2, 9, 1, 3, 17)):
    """What the block makes of rows 0..T-1, in portions."""
    from celeg_amd.engine import load_model
    from celeg_amd.weights.safetensors_io import write_safetensors
    alone_architecture()
    cfg = dict(cfg, architectures=["KifetarPartsAlone"])
    os.makedirs(tmp_path, exist_ok=True)
    with open(os.path.join(tmp_path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(tmp_path, "model.safetensors"), {k: v.float().contiguous() for k, v in tensors.items()})
    steps = portions_schedule({"x": list(range(cfg["rows"]))}, sizes=cut)
    lm = load_model(str(tmp_path), dtype="float32", device=DEV, page_tokens=16, n_pages=8, max_requests=2, max_context=128,
                    max_batched_tokens=64)
    return EngineDriver(lm).run(steps)["x"].double()


@pytest.mark.parametrize("window,scaling", [(None, None), (7, (4.0, 1.0, 3.0, 40)), (16, None)])
def test_sigmoid_attention_alone(tmp_path, window, scaling):
    torch.manual_seed(1)
    T, W_, H, G, D = 45, 40, 6, 3, 12
    m = attention(H, G, D, window=window, rot=rot(8, 90.0, scaling), scale=0.3)["mixer"]
    # (with this base, original and band the eight rotated values hold frequencies kept, blended and divided)
    t = {"x": torch.randn(T, W_), "q": torch.randn(H * D, W_) * 0.3, "q.b": torch.randn(H * D) * 0.3, "k": torch.randn(G * D, W_) * 0.3,
         "k.b": torch.randn(G * D) * 0.3, "q.norm": 1 + 0.2 * torch.randn(D), "k.norm": 1 + 0.2 * torch.randn(D),
         "temp": 1 + 0.5 * torch.randn(H), "pb": torch.randn(H), "g": torch.randn(H, W_) * 0.3, "o": torch.randn(W_, H * D) * 0.3}
    if scaling:
        kinds = set()
        for f in plain.rotary_frequencies(8, 90.0).tolist():
            wl = 2 * 3.141592653589793 / f
            kinds.add("kept" if wl < scaling[3] / scaling[2] else "divided" if wl > scaling[3] / scaling[1] else "blended")
        assert kinds == {"kept", "divided", "blended"}
    names = {"q": "q", "q_bias": "q.b", "k": "k", "k_bias": "k.b", "q_norm": "q.norm", "k_norm": "k.norm", "temp": "temp", "pb": "pb",
             "g": "g", "o": "o"}
    position = {"kind": "rope", "params": {"theta": 90.0, "rotary_dim": 8, "head_dim": D, "pairing": "halves"}}
    if scaling:
        position["params"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    params = {"width": W_, "heads": H, "kv_heads": G, "head_dim": D, "scale": 0.3, "eps": 1e-4, "qk_norm": True, "bias": True,
              "values": "keys", "temperature": True, "score_bias": True, "head_gate": True, "position": position}
    if window:
        params["window"] = window
    got = run_alone(tmp_path, {"width": W_, "rows": T, "mixer": {"kind": "sigmoid_attention", "tensors": names, "params": params}}, t)
    Wd = {k: v.double() for k, v in t.items()}
    assert_close_f32(got, Wd["x"] + plain.sigmoid_window_attention(Wd["x"], m, Wd, "", 1e-4), "sigmoid attention alone")


# (dims of 16, 32, 64, 128 and 256 keep the state in registers, 1, 2, 4, 8 and 16 lanes a column; the others do not)
@pytest.mark.parametrize("H,G,D,V,taps", [(4, 2, 12, 20, 3), (3, 3, 8, 70, 1), (2, 1, 40, 8, 6), (4, 2, 16, 100, 4), (2, 2, 32, 64, 2),
                                          (3, 1, 64, 48, 4), (2, 1, 128, 24, 2), (1, 1, 256, 70, 3)])
def test_gated_delta_rule_alone(tmp_path, H, G, D, V, taps):
    torch.manual_seed(2)
    T, W_ = 45, 32
    t = {"x": torch.randn(T, W_), "q": torch.randn(G * D, W_) * 0.3, "k": torch.randn(G * D, W_) * 0.3, "v": torch.randn(H * V, W_) * 0.3,
         "q.conv": torch.randn(G * D, taps) * 0.5, "k.conv": torch.randn(G * D, taps) * 0.5, "v.conv": torch.randn(H * V, taps) * 0.5,
         "b": torch.randn(H, W_) * 0.3, "a": torch.randn(H, W_) * 0.3, "A_log": torch.randn(H) - 1.0, "dt_bias": torch.randn(H),
         "norm": 1 + 0.2 * torch.randn(V), "g": torch.randn(H * V, W_) * 0.3, "o": torch.randn(W_, H * V) * 0.3}
    names = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b", "a": "a",
             "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "g": "g", "o": "o"}
    params = {"width": W_, "heads": H, "kv_heads": G, "dim": D, "vdim": V, "taps": taps, "eps": 1e-4}
    got = run_alone(tmp_path, {"width": W_, "rows": T, "mixer": {"kind": "gated_delta_rule", "tensors": names, "params": params}}, t)
    Wd = {k: v.double() for k, v in t.items()}
    m = delta(H, G, D, V, taps)["mixer"]
    assert_close_f32(got, Wd["x"] + plain.gated_delta_rule(Wd["x"], m, Wd, "", 1e-4), "gated delta rule alone")


@pytest.mark.parametrize("post,W_", [("layernorm", 36), ("rmsnorm", 36), ("layernorm", 1500), ("rmsnorm", 2304)])
def test_norms_before_and_after_alone(tmp_path, post, W_):
    """No mixer (its output is zero, whose layer norm is the norm's bias), a dense feed-forward
    between a layer norm and a norm of its output (a layer norm, or an RMS norm without bias).
    Rows of up to 1,024, up to 2,048 and of more values take three forms of the kernel."""
    torch.manual_seed(3)
    T, ff = 29, 40
    t = {"x": torch.randn(T, W_) * 3 + 1, "g": torch.randn(ff, W_) * 0.3, "u": torch.randn(ff, W_) * 0.3, "d": torch.randn(W_, ff) * 0.3}
    for n in ("n1", "n1b", "n2", "n2b"):
        t[n], t[n + ".b"] = 1 + 0.3 * torch.randn(W_), torch.randn(W_) * 0.5
    ln = lambda n: {"kind": "layernorm", "params": {"width": W_, "eps": 1e-3}, "tensors": {"weight": n, "bias": n + ".b"}}
    after = ln("n2b") if post == "layernorm" else {"kind": "rmsnorm", "params": {"width": W_, "eps": 1e-3}, "tensors": {"weight": "n2b"}}
    if post == "rmsnorm":
        del t["n2b.b"]
    cfg = {"width": W_, "rows": T, "arrangement": "sandwich_norm", "mixer_norm": ln("n1"), "mixer_post_norm": ln("n1b"),
           "ffn": {"kind": "swiglu", "params": {"width": W_, "ff": ff}, "tensors": {"gate": "g", "up": "u", "down": "d"}},
           "ffn_norm": ln("n2"), "ffn_post_norm": after}
    got = run_alone(tmp_path, cfg, t)
    Wd = {k: v.double() for k, v in t.items()}
    x = Wd["x"] + Wd["n1b.b"]
    u = plain.layer_norm(x, Wd["n2"], Wd["n2.b"], 1e-3)
    y = (torch.nn.functional.silu(u @ Wd["g"].T) * (u @ Wd["u"].T)) @ Wd["d"].T
    want = x + (plain.layer_norm(y, Wd["n2b"], Wd["n2b.b"], 1e-3) if post == "layernorm" else plain.rms_norm(y, Wd["n2b"], 1e-3))
    assert_close_f32(got, want, f"norms before and after ({post})")


def test_embedding_rows_taken_in_again_alone(tmp_path):
    torch.manual_seed(4)
    T, W_ = 21, 28
    t = {"x": torch.randn(T, W_), "w": torch.randn(W_, 2 * W_) * 0.3}
    cfg = {"width": W_, "rows": T, "reinjection": {"kind": "linear_concat", "params": {"width": W_}, "tensors": {"weight": "w"}}}
    got = run_alone(tmp_path, cfg, t)
    x = t["x"].double()
    assert_close_f32(got, torch.cat([x, x], -1) @ t["w"].double().T, "the embedding's rows, again")
