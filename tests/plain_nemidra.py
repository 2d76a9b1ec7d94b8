"""A plain, slow implementation of Nemidra, written from the design's equations: one function per mechanism, whole
sequences at a time, recurrences token by token, everything in the element type that it is called with (float64 in the
tests).  It shares no code with the package.

`w` maps tensor names to tensors, `cfg` is the dictionary of config.json.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    """The model's norm: the weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + weight)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def linear(w, name, x):
    y = x @ w[name].T
    if name + ".b" in w:
        y = y + w[name + ".b"]
    return y


# ---------------------------------------------------------------------------------------------- embedding
def bigram_rows(cfg, tokens):
    b = cfg["embedding"]["bigram"]
    rows = [b["buckets"]]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * b["mul_prev"] + cur * b["mul_cur"]) % b["buckets"])
    return rows


def embedding(w, cfg, tokens):
    T = len(tokens)
    x = w["embed"][torch.tensor(tokens)]
    if "bigram" in cfg.get("embedding", {}):
        x = x + w["bigram"][torch.tensor(bigram_rows(cfg, tokens))]
    if "pos" in w:
        x = x + w["pos"][:T]
    return x


# ---------------------------------------------------------------------------------------------- mixers
def window_attention(w, p, m, h):
    """Softmax attention with biases and no positions; key j is visible from i if 0 <= i - j < mask.size."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(w, p + "q", h).view(T, H, dk)
    k = linear(w, p + "k", h).view(T, G, dk)
    v = linear(w, p + "v", h).view(T, G, dv)
    i = torch.arange(T)
    seen = i[None, :] <= i[:, None]
    if m.get("mask") is not None:
        seen &= (i[:, None] - i[None, :]) < m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    return linear(w, p + "o", out.reshape(T, H * dv))


def mlstm(w, p, m, h, eps):
    """The matrix memory with exponential gates, a running maximum that starts at 0 and a normalizer."""
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh(linear(w, p + "i", h) / cap)                                   # [T, H], logarithms
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh(linear(w, p + "f", h) / cap))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for a in range(H):
        S = torch.zeros(dk, dv, dtype=h.dtype)
        n = torch.zeros(dk, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for t in range(T):
            new = torch.maximum(fg[t, a] + mx, ig[t, a])
            keep, take = torch.exp(fg[t, a] + mx - new), torch.exp(ig[t, a] - new)
            S = keep * S + take * torch.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            mx = new
            out[t, a] = (S.T @ q[t, a]) / (torch.maximum((n @ q[t, a]).abs(), torch.exp(-mx)) + 1e-6)
    y = rms_unit(out, eps).reshape(T, H * dv) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T


def parallel_mixer(w, p, m, h, eps):
    return (m["left_scale"] * window_attention(w, p + "left.", m["left"], h)
            + m["right_scale"] * mlstm(w, p + "right.", m["right"], h, eps))


def gla(w, p, m, h, eps):
    """Gated linear attention: a decay per key channel."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(T, H, dk)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for a in range(H):
        S = torch.zeros(dk, dv, dtype=h.dtype)
        for t in range(T):
            S = alpha[t, a][:, None] * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    y = (rms_unit(out, eps) * w[p + "norm"]).reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return y @ w[p + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forwards
def dense_ffn(w, p, h):
    return gelu_erf(h @ w[p + "up"].T) @ w[p + "down"].T


def expert(w, p, h):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe_ffn(w, p, mlp, h):
    r = mlp["router"]
    scores = torch.softmax((h @ w[p + "router"].T).to(torch.float64), -1).to(h.dtype)
    top = torch.topk(scores, r["top"], dim=-1)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for s, e in zip(top.values[t], top.indices[t]):
            y[t] += s * r["scale"] * expert(w, f"{p}e{int(e)}.", h[t:t + 1])[0]
    if mlp.get("shared") is not None:
        y = y + torch.sigmoid(h @ w[p + "shared.sg"].T) * expert(w, p + "shared.", h)
    return y


def feed_forward(w, p, mlp, h):
    return dense_ffn(w, p, h) if mlp["kind"] == "dense" else moe_ffn(w, p, mlp, h)


def token_side(w, cfg, i, tokens, x, eps):
    """The per-layer token input: returns what is added to x."""
    dim = cfg["token_side"]["dim"]
    e = w["side.embed"][torch.tensor(tokens)][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e) @ w[f"l{i}.side.proj"].T
    return rms_unit(y, eps) * w[f"l{i}.side.norm"]


# ---------------------------------------------------------------------------------------------- the model
def layer_order(cfg):
    """[(layer, whether the embedding output is added in front of it)]"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for rep in range(loop["times"]):
        order += [(i, rep > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def layer(w, cfg, i, tokens, x):
    L, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    h = norm_around_zero(x, w[p + "norm1"], eps)
    if L["type"] == "gla":
        y = gla(w, p + "mix.", L["mixer"], h, eps)
    else:
        y = parallel_mixer(w, p + "mix.", L["mixer"], h, eps)
    x = x + norm_around_zero(y, w[p + "norm1b"], eps)
    if L.get("mlp") is not None:
        y = feed_forward(w, p + "mlp.", L["mlp"], norm_around_zero(x, w[p + "norm2"], eps))
        x = x + norm_around_zero(y, w[p + "norm2b"], eps)
    if cfg.get("token_side") is not None:
        x = x + token_side(w, cfg, i, tokens, x, eps)
    return x


def forward(w, cfg, tokens, dtype=torch.float64, layers_out: list | None = None):
    """Logits [T, vocab] of a whole sequence.  `layers_out` collects the stream after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    tokens = [int(t) for t in tokens]
    x0 = embedding(w, cfg, tokens)
    x = x0
    for i, add in layer_order(cfg):
        if add:
            x = x + x0
        x = layer(w, cfg, i, tokens, x)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = norm_around_zero(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(w, cfg, prompt, steps, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(steps):
        tokens.append(int(forward(w, cfg, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]


def load(model_dir: str):
    """(weights by tensor name as stored, config.json as a dict)."""
    import json
    import os

    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as h:
        for name in h.keys():
            w[name] = h.get_tensor(name)
    return w, cfg
