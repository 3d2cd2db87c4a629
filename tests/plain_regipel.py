"""A plain, slow implementation of the Regipel design in float64, one function per mechanism,
written from the design's equations and sharing no code with the library.  The tests compare
the engine with it.

Notation: n tokens, d model width, positions p = 0..n-1.  W[name] are the checkpoint's
tensors widened to float64 (linear weights are [out, in] and applied as W x).
"""
import json
import os

import torch

from safetensors.torch import load_file

F = torch.float64


def load_model_folder(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    W = {k: v.to(F) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, W


# ------------------------------------------------------------------ norms
def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    """RMS norm whose stored weight lies around zero: the factor is 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


# ------------------------------------------------------------------ rotation
def rotate_neighbours(x, positions, base, dims):
    """x [n, ..., r]: values 2i and 2i+1 (i < dims/2) form a pair that turns by the angle
    p * base^(-2i/dims); values from `dims` on pass unchanged."""
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(angle), torch.sin(angle)
        while c.dim() < x.dim() - 1:
            c, s = c.unsqueeze(-1), s.unsqueeze(-1)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# ------------------------------------------------------------------ latent attention
def latent_attention(h, W, prefix, m, eps, positions=None):
    """h [n, d] -> [n, d].  m: the layer's "mixer" entry of config.json."""
    n = h.shape[0]
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    p = torch.arange(n) if positions is None else positions
    q = (h @ W[prefix + "q"].T).view(n, H, dk + dr)
    q_plain, q_turn = q[..., :dk], q[..., dk:]
    down = h @ W[prefix + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * W[prefix + "dkv.norm"]        # the compressed rows (what a cache keeps)
    k_turn = down[:, rank:]                                             # one rotated key part for all heads
    if dr and m.get("rot"):
        q_turn = rotate_neighbours(q_turn, p, m["rot"]["base"], m["rot"]["dims"])
        k_turn = rotate_neighbours(k_turn, p, m["rot"]["base"], m["rot"]["dims"])
    k_plain = (c @ W[prefix + "uk"].T).view(n, H, dk)
    v = (c @ W[prefix + "uv"].T).view(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=F)
    for i in range(n):
        for a in range(H):
            s = (k_plain[: i + 1, a] @ q_plain[i, a] + k_turn[: i + 1] @ q_turn[i, a]) * m["scale"]
            e = torch.exp(s - s.max())
            denom = e.sum()
            if m.get("sink", True):
                denom = denom + torch.exp(W[prefix + "sink"][a] - s.max())    # no key, no value, not scaled, once
            out[i, a] = (e / denom) @ v[: i + 1, a]
    heads = out.reshape(n, H * dv)
    if m.get("gate", True):
        heads = heads * torch.sigmoid(h @ W[prefix + "g"].T)
    return heads @ W[prefix + "o"].T


# ------------------------------------------------------------------ routed experts
def routed_experts(h, W, prefix, f):
    """h [n, d] -> [n, d].  f: the layer's "mlp" entry.  Sigmoid scores, the `top` largest chosen,
    their scores (not renormalised) multiply the expert's INPUT."""
    E, top = f["router"]["experts"], f["router"]["top"]
    score = torch.sigmoid(h @ W[prefix + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = sorted(range(E), key=lambda e: (-float(score[t, e]), e))[:top]
        for e in chosen:
            x = score[t, e] * h[t]
            g = W[f"{prefix}e{e}.gate"] @ x
            out[t] += W[f"{prefix}e{e}.down"] @ (g * torch.sigmoid(g) * (W[f"{prefix}e{e}.up"] @ x))
    return out


# ------------------------------------------------------------------ residual streams
def hyper_sublayer(xs, W, prefix, sublayer):
    """xs: list of S streams [n, d].  The sub-layer reads sum_s in[s] x_s; its output y returns as
    x_t <- sum_s mix[s, t] x_s + out[t] y, every new stream from the old ones."""
    S = len(xs)
    w_in, w_out, mix = W[prefix + ".in"], W[prefix + ".out"], W[prefix + ".mix"]
    y = sublayer(sum(w_in[s] * xs[s] for s in range(S)))
    return [sum(mix[s, t] * xs[s] for s in range(S)) + w_out[t] * y for t in range(S)]


def run_order(cfg):
    n, loop = len(cfg["layers"]), cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    return (list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] +
            list(range(loop["stop"], n)))


# ------------------------------------------------------------------ the model
def model_hidden(cfg, W, tokens):
    """The residual stream (the sum of the streams) after every layer run: list of [n, d]."""
    eps = cfg["norm"]["eps"]
    x0 = W["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    S = cfg.get("streams")
    xs = [x0.clone() for _ in range(S or 1)]
    after = []
    for L in run_order(cfg):
        layer, p = cfg["layers"][L], f"l{L}."
        subs = [("norm1", "hc1", lambda u, L=L, layer=layer, p=p: latent_attention(u, W, p + "mix.", layer["mixer"], eps))]
        if layer.get("mlp"):
            subs.append(("norm2", "hc2", lambda u, layer=layer, p=p: routed_experts(u, W, p + "mlp.", layer["mlp"])))
        for norm, hc, fn in subs:
            normed = lambda u, norm=norm, fn=fn, p=p: fn(zero_centred_norm(u, W[p + norm], eps))
            if S:
                xs = hyper_sublayer(xs, W, p + hc, normed)
            else:
                xs = [xs[0] + normed(xs[0])]
        after.append(sum(xs))
    return after


def model_logits(cfg, W, tokens):
    x = model_hidden(cfg, W, tokens)[-1]
    x = zero_centred_norm(x, W["final.norm"], cfg["norm"]["eps"])
    return (x @ W["embed"].T * cfg.get("logit_scale", 1.0)).to(torch.float32)


def greedy(cfg, W, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(model_logits(cfg, W, tokens)[-1].argmax()))
    return tokens[len(prompt):]
