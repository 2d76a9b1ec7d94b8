"""A plain, slow Zenuzen decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the `simply_amd` package: it reads `config.json` and `model.safetensors` itself and
computes with ordinary torch operations on the CPU in the dtype it is asked for (float64 for the tests).

The design, in this file's notation (x: residual stream [T, D]; rows of a weight are outputs):

  layer        x <- x + m * rms(mixer(x); norm1);  x <- x + m * rms(ffn(x); norm2)   (no second step without an ffn)
               the sublayers read x itself; rms(y; w) = y / sqrt(mean(y^2) + eps) * w
  attention    q, k, v, gate from x; partial rotary on q and k; q and k divided by their root mean square;
               p = softmax over (scale * q.k for the visible keys, and one more logit `sink` per head that has no
               value); values mixed with the first such layer's; heads * sigmoid(gate); output projection
  delta        q, k, v through a short causal convolution per channel and silu; q, k to unit length, q / sqrt(dim);
               per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
               o / rms(o) * w * silu(gate); output projection
  ffn          down(relu(up x)^2)
  output       head(rms(x; final.norm))
"""
from __future__ import annotations

import json
import math
import os

import torch


def load(model_dir: str):
    """(weights by tensor name as stored, config.json as a dict)."""
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as h:
        for name in h.keys():
            w[name] = h.get_tensor(name)
    return w, cfg


def _w(w, name, dtype):
    return w[name].to(dtype)


# --------------------------------------------------------------------------- small functions


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, times `weight` if there is one."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def squared_relu(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z) ** 2


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def partial_rotary(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, size]: the first `dims` entries of every head are rotated in pairs (i, i + dims / 2) by the
    angle position * base^(-2 i / dims); the others pass unchanged."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = torch.as_tensor(base, dtype=x.dtype) ** (-2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None, None] * freq[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def causal_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y[t, c] = sum_j taps[c, j] * x[t - (n - 1 - j), c], zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(n):
        y = y + padded[j:j + T] * taps[:, j][None, :]
    return y


# --------------------------------------------------------------------------- attention with a sink


def sink_softmax_attention(q, k, v, sink, scale: float) -> torch.Tensor:
    """q [T, H, dk], k [T, G, dk], v [T, G, dv], sink [H].  Causal; the softmax's denominator holds one more term
    exp(sink_h), which has no value.  Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        s = torch.cat([s, sink[h].expand(T, 1)], dim=1)
        p = torch.softmax(s, dim=-1)[:, :T]
        out[:, h] = p @ v[:, g]
    return out


def attention_mixer(x, positions, w, p: str, mc: dict, eps: float, shared: dict) -> torch.Tensor:
    """`shared` carries the first value-mixing layer's values from layer to layer."""
    dt = x.dtype
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = x.shape[0]
    q = (x @ _w(w, p + "q", dt).T).view(T, H, dk)
    k = (x @ _w(w, p + "k", dt).T).view(T, G, dk)
    v = (x @ _w(w, p + "v", dt).T).view(T, G, dv)
    rot = mc.get("rot")
    if rot:
        q = partial_rotary(q, positions, rot["dims"], rot["base"])
        k = partial_rotary(k, positions, rot["dims"], rot["base"])
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    if mc.get("v_mix"):
        if "v_first" not in shared:
            shared["v_first"] = v
        else:
            lam = _w(w, p + "vmix", dt)
            v = (1.0 - lam) * v + lam * shared["v_first"]
    o = sink_softmax_attention(q, k, v, _w(w, p + "sink", dt), mc["scale"])
    gate = torch.sigmoid(x @ _w(w, p + "g", dt).T)
    return (o.reshape(T, H * dv) * gate) @ _w(w, p + "o", dt).T


# --------------------------------------------------------------------------- gated delta rule


def delta_recurrence(q, k, v, beta, g, S0=None):
    """q, k [T, H, dk] (already unit vectors, q scaled), v [T, H, dv], beta, g [T, H].  Token by token and head by
    head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns (o [T, H, dv], final S [H, dk, dv])."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=q.dtype) if S0 is None else S0.clone()
    o = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            S[h] = g[t, h] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ k[t, h])
            S[h] = S[h] + torch.outer(k[t, h], u)
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def delta_mixer(x, w, p: str, mc: dict, eps: float) -> torch.Tensor:
    dt = x.dtype
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = x.shape[0]
    rep = H // G

    def short(name):
        return silu(causal_conv(x @ _w(w, p + name, dt).T, _w(w, p + name + ".conv", dt)))

    q, k, v = short("q").view(T, G, dk), short("k").view(T, G, dk), short("v").view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)   # head h reads q/k head h // rep
    beta = torch.sigmoid(x @ _w(w, p + "b", dt).T)
    decay = torch.exp(-torch.exp(_w(w, p + "A_log", dt)) * softplus(x @ _w(w, p + "a", dt).T + _w(w, p + "dt_bias", dt)))
    o, _ = delta_recurrence(q, k, v, beta, decay)
    o = rms_norm(o, _w(w, p + "norm", dt), eps)
    gate = silu(x @ _w(w, p + "g", dt).T).view(T, H, dv)
    return (o * gate).reshape(T, H * dv) @ _w(w, p + "o", dt).T


# --------------------------------------------------------------------------- the rest


def feed_forward(x, w, p: str, fc: dict) -> torch.Tensor:
    if fc["kind"] != "dense":
        raise ValueError(f"unknown feed-forward kind {fc['kind']!r}")
    return squared_relu(x @ _w(w, p + "up", x.dtype).T) @ _w(w, p + "down", x.dtype).T


def layer(x, positions, w, i: int, cfg: dict, shared: dict) -> torch.Tensor:
    lc = cfg["layers"][i]
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    p = f"l{i}."
    if lc["type"] == "attention":
        y = attention_mixer(x, positions, w, p + "mix.", lc["mixer"], eps, shared)
    elif lc["type"] == "delta":
        y = delta_mixer(x, w, p + "mix.", lc["mixer"], eps)
    else:
        raise ValueError(f"unknown layer type {lc['type']!r}")
    x = x + m * rms_norm(y, _w(w, p + "norm1", x.dtype), eps)
    if lc.get("mlp") is not None:
        x = x + m * rms_norm(feed_forward(x, w, p + "mlp.", lc["mlp"]), _w(w, p + "norm2", x.dtype), eps)
    return x


def forward(w: dict, cfg: dict, tokens, dtype=torch.float64, return_layers: bool = False):
    """Logits [T, vocab] for the whole sequence (and the residual stream after every layer, if asked)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = _w(w, "embed", dtype)[tokens]
    shared: dict = {}
    streams = []
    for i in range(len(cfg["layers"])):
        x = layer(x, positions, w, i, cfg, shared)
        streams.append(x)
    logits = rms_norm(x, _w(w, "final.norm", dtype), cfg["norm"]["eps"]) @ _w(w, "head", dtype).T
    return (logits, torch.stack(streams)) if return_layers else logits


def greedy(w, cfg, prompt, n: int, dtype=torch.float64) -> list[int]:
    """n tokens, each the best of the logits of everything before it; the whole sequence is run anew every time."""
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward(w, cfg, seq, dtype)[-1].argmax()))
    return seq[len(prompt):]
