"""Kifetar in plain float64 PyTorch, one function per mechanism, whole sequences at a time.

Nothing here is shared with the library: the functions take a configuration (the dictionary
of config.json) and a dictionary of tensors by checkpoint name, and run one request's
tokens from position 0.  Slow on purpose: loops over tokens, heads and keys where the
definition has them.

The model: token embedding; layers `x += post_norm(sublayer(pre_norm(x)))` for a mixer and
a feed-forward, every norm a layer norm with weight and bias; two kinds of mixer (attention
with sigmoid weights inside a sliding window, and a gated delta rule with short
convolutions); a range of layers that runs several times, before every run of which the
stream is mixed with the embedding's rows again; final layer norm; logits from the
embedding table.
"""
import json
import math
import os

import torch
from safetensors.torch import load_file

F64 = torch.float64


def load_model_folder(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def layer_norm(x, w, b, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling` the long wavelengths are stretched:
    wavelengths below original/high keep f, above original/low get f/factor, between them a
    linear blend in original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate(x, positions, freqs):
    """x [T, heads, dim]; the first 2*len(freqs) values of a head turn, value i with value i + half."""
    half = freqs.numel()
    if half == 0:
        return x
    angle = positions.to(F64)[:, None] * freqs[None, :]          # [T, half]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


def sigmoid_window_attention(h, m, t, prefix, eps, first_pos=0):
    """h [T, width]; m the layer's "mixer" dictionary; tensors `prefix + name`."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ t[prefix + "q"].T + t[prefix + "q.b"]).view(T, H, D)
    k = (h @ t[prefix + "k"].T + t[prefix + "k.b"]).view(T, G, D)
    v = k.clone()                                  # the values are the keys as projected
    q = rms_norm(q, t[prefix + "q.norm"], eps)
    k = rms_norm(k, t[prefix + "k.norm"], eps)
    rot = m.get("rot")
    positions = torch.arange(first_pos, first_pos + T)
    if rot and rot.get("dims", 0) > 0:
        freqs = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, positions, freqs), rotate(k, positions, freqs)
    window = m["mask"]["size"] if m.get("mask") else None
    gate = torch.sigmoid(h @ t[prefix + "g"].T)    # [T, H]
    out = torch.zeros(T, H, D, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            score = (k[lo:i + 1, g] @ q[i, head]) * m["scale"] * t[prefix + "temp"][head]
            weight = torch.sigmoid(score + t[prefix + "pb"][head])
            out[i, head] = (weight[:, None] * v[lo:i + 1, g]).sum(0) * gate[i, head]
    return out.reshape(T, H * D) @ t[prefix + "o"].T


def causal_conv_silu(x, w):
    """x [T, C], w [C, taps]: the last tap is the current token's, zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        y += padded[j:j + T] * w[:, j]
    return silu(y)


def gated_delta_rule(h, m, t, prefix, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ t[prefix + "q"].T, t[prefix + "q.conv"]).view(T, G, D)
    k = causal_conv_silu(h @ t[prefix + "k"].T, t[prefix + "k.conv"]).view(T, G, D)
    v = causal_conv_silu(h @ t[prefix + "v"].T, t[prefix + "v.conv"]).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t[prefix + "b"].T)                               # [T, H]
    decay = torch.exp(-torch.exp(t[prefix + "A_log"]) *
                      torch.nn.functional.softplus(h @ t[prefix + "a"].T + t[prefix + "dt_bias"]))
    out_gate = silu(h @ t[prefix + "g"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for i in range(T):
            S = decay[i, head] * S
            u = beta[i, head] * (v[i, head] - S.T @ k[i, g])
            S = S + torch.outer(k[i, g], u)
            o[i, head] = S.T @ q[i, g]
    o = rms_norm(o, t[prefix + "norm"], eps) * out_gate
    return o.reshape(T, H * V) @ t[prefix + "o"].T


def swiglu(h, t, prefix):
    return (silu(h @ t[prefix + "gate"].T) * (h @ t[prefix + "up"].T)) @ t[prefix + "down"].T


def run_order(config):
    """[(layer, first of a pass)]: the looped range `times` times, the rest once."""
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(l, False) for l in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(l, l == loop["start"]) for l in range(loop["start"], loop["stop"])]
    return order + [(l, False) for l in range(loop["stop"], n)]


def forward(config, tensors, tokens, return_layers=False):
    """Logits [T, vocab] (float64) of one request's tokens from position 0."""
    t = {k: v.to(F64) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x0 = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    after = []
    for layer, first in run_order(config):
        spec, p = config["layers"][layer], f"l{layer}."
        if first:
            x = torch.cat([x, x0], -1) @ t["loop.in"].T
        hin = layer_norm(x, t[p + "norm1"], t[p + "norm1.b"], eps)
        if spec["type"] == "attention":
            y = sigmoid_window_attention(hin, spec["mixer"], t, p + "mix.", eps)
        elif spec["type"] == "delta":
            y = gated_delta_rule(hin, spec["mixer"], t, p + "mix.", eps)
        else:
            raise ValueError(spec["type"])
        x = x + layer_norm(y, t[p + "norm1b"], t[p + "norm1b.b"], eps)
        if spec.get("mlp"):
            y = swiglu(layer_norm(x, t[p + "norm2"], t[p + "norm2.b"], eps), t, p + "mlp.")
            x = x + layer_norm(y, t[p + "norm2b"], t[p + "norm2b.b"], eps)
        after.append(x.clone())
    logits = layer_norm(x, t["final.norm"], t["final.norm.b"], eps) @ t["embed"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy(config, tensors, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
