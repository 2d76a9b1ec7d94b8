"""Nemidra's mechanisms one by one: each part of the framework, with weights of the test's own, against the plain
implementation's function for that mechanism (tests/plain_nemidra.py), whole and in portions.  A body takes the device
and the element type; the CPU tests run it with the kernels replaced by their plain torch references, the GPU tests
with the kernels.  Where random inputs would hide a fault (a key just inside or just outside a window, a far key among
hundreds, the token before a portion), inputs are made so that it shows."""
from __future__ import annotations

import torch

import plain_nemidra as plain
from simply_amd import parts as _parts  # noqa: F401  (registers the parts)
from simply_amd.cache import CacheManager
from simply_amd.config.spec import PartSpec
from simply_amd.registry import EMBEDDINGS, FEED_FORWARDS, MIXERS, STREAM_PARTS
from zenuzen_cases import one_request_ctx, run_mixer


def _tol(dtype):
    return 2e-5 if dtype == torch.float32 else 6e-2


def _close(got, want, dtype, what=None, scale=None):
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max() / (scale or want.abs().max()))
    assert err < _tol(dtype), (what, err)


def _draw(gen, *shape, std=0.3):
    return torch.randn(*shape, generator=gen, dtype=torch.float64) * std


def _load(part, names: dict, w: dict, dtype, device):
    """Hands `part` the tensors of the plain weights `w` (part's name -> plain name), rounded to `dtype`."""
    part.load({local: w[name].to(dtype).to(device) for local, name in names.items()})


def _rounded(w, dtype):
    return {k: v.to(dtype).double() for k, v in w.items()}


CUTS = ((61,), (1,) * 61, (29, 1, 1, 2, 17, 3, 8), (2,) * 30 + (1,))


# --------------------------------------------------------------------------- gated linear attention
def gla_part(device, dtype, heads=3, dim=12, vdim=20, rank=5, tau=8.0, width=40):
    g = torch.Generator().manual_seed(1)
    H, dk, dv, D = heads, dim, vdim, width
    w = {"p.q": _draw(g, H * dk, D), "p.k": _draw(g, H * dk, D), "p.v": _draw(g, H * dv, D), "p.g": _draw(g, H * dv, D),
         "p.o": _draw(g, D, H * dv), "p.a1": _draw(g, rank, D), "p.a2": _draw(g, H * dk, rank, std=1.0),
         "p.a2.b": _draw(g, H * dk, std=2.0), "p.norm": 1.0 + _draw(g, dv)}
    part = MIXERS.build("gated_linear_attention", hidden_size=D, num_heads=H, key_dim=dk, value_dim=dv, decay_rank=rank,
                        tau=tau, norm_eps=1e-5)
    _load(part, {"q_proj": "p.q", "k_proj": "p.k", "v_proj": "p.v", "gate_proj": "p.g", "o_proj": "p.o", "decay_in": "p.a1",
                 "decay_out": "p.a2", "decay_bias": "p.a2.b", "norm": "p.norm"}, w, dtype, device)
    x = _draw(g, 61, D, std=1.0).to(dtype)
    want = plain.gla(_rounded(w, dtype), "p.", {"heads": H, "dim": dk, "vdim": dv, "tau": tau}, x.double(), 1e-5)
    for cuts in CUTS:
        _close(run_mixer(part, x.to(device), cuts, dtype, device, page_size=4), want, dtype, ("gla", cuts))


# --------------------------------------------------------------------------- the matrix memory
def memory_part(device, dtype, heads=2, dim=8, vdim=12, cap=10.0, width=40, gate_std=3.0):
    """Gates with a wide spread: the running maximum moves, the normalizer's floor exp(-m) matters early on."""
    g = torch.Generator().manual_seed(2)
    H, dk, dv, D = heads, dim, vdim, width
    w = {"p.q": _draw(g, H * dk, D), "p.k": _draw(g, H * dk, D), "p.v": _draw(g, H * dv, D), "p.g": _draw(g, H * dv, D),
         "p.o": _draw(g, D, H * dv), "p.i": _draw(g, H, D, std=gate_std), "p.f": _draw(g, H, D, std=gate_std),
         "p.i.b": _draw(g, H, std=2.0), "p.f.b": 2.0 + _draw(g, H, std=2.0), "p.norm": 1.0 + _draw(g, H * dv)}
    part = MIXERS.build("matrix_memory", hidden_size=D, num_heads=H, key_dim=dk, value_dim=dv, gate_cap=cap, norm_eps=1e-5)
    _load(part, {"q_proj": "p.q", "k_proj": "p.k", "v_proj": "p.v", "gate_proj": "p.g", "o_proj": "p.o", "input_gate": "p.i",
                 "forget_gate": "p.f", "input_bias": "p.i.b", "forget_bias": "p.f.b", "norm": "p.norm"}, w, dtype, device)
    x = _draw(g, 61, D, std=1.0).to(dtype)
    want = plain.mlstm(_rounded(w, dtype), "p.", {"heads": H, "dim": dk, "vdim": dv, "gate_cap": cap}, x.double(), 1e-5)
    for cuts in CUTS:
        _close(run_mixer(part, x.to(device), cuts, dtype, device, page_size=4), want, dtype, ("memory", cuts))


# --------------------------------------------------------------------------- windowed attention with biases
def _attention(device, dtype, g, H, G, dk, dv, D, scale, window):
    w = {"p.q": _draw(g, H * dk, D, std=0.1), "p.k": _draw(g, G * dk, D, std=0.1), "p.v": _draw(g, G * dv, D),
         "p.o": _draw(g, D, H * dv), "p.q.b": _draw(g, H * dk, std=0.2), "p.k.b": _draw(g, G * dk, std=0.2),
         "p.v.b": _draw(g, G * dv), "p.o.b": _draw(g, D)}
    part = MIXERS.build("sink_attention", hidden_size=D, num_heads=H, num_kv_heads=G, key_dim=dk, value_dim=dv, scale=scale,
                        bias=True, window=window)
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return w, part, m


NAMES_ATTENTION = {"q_proj": "p.q", "k_proj": "p.k", "v_proj": "p.v", "o_proj": "p.o", "q_bias": "p.q.b", "k_bias": "p.k.b",
                   "v_bias": "p.v.b", "o_bias": "p.o.b"}


def window_edges(device, dtype, window=7, page_size=4, heads=4, kv_heads=2, dim=12, vdim=20, width=40, T=70):
    """One key is made to stand out for one query: its score is far above all others, so the result is that key's
    value if the key is visible and something else entirely if not.  The pair lies just inside the window
    (distance window - 1), just outside (distance window), and far away (hundreds of times the scores of the rest
    would not make up for it), at page borders, with the query in a prompt's portion and decoded alone."""
    g = torch.Generator().manual_seed(3)
    H, G, dk, dv, D = heads, kv_heads, dim, vdim, width
    w, part, m = _attention(device, dtype, g, H, G, dk, dv, D, 0.3, window)
    # the first query direction and the first key direction are read from input channels 0 and 1 alone
    w["p.q"][:, 0], w["p.k"][:, 1] = 0.0, 0.0
    w["p.q"][:, 1], w["p.k"][:, 0] = 0.0, 0.0
    for a in range(H):
        w["p.q"][a * dk, 0] = 6.0
    for b in range(G):
        w["p.k"][b * dk, 1] = 6.0
    _load(part, NAMES_ATTENTION, w, dtype, device)
    for query, distance in ((40, window - 1), (40, window), (41, window - 1), (43, window), (69, 60), (8, window - 1)):
        if distance > query:
            continue
        x = _draw(g, T, D, std=0.5)
        x[:, :2] = 0.0
        x[query, 0] = 5.0
        x[query - distance, 1] = 5.0
        x = x.to(dtype)
        want = plain.window_attention(_rounded(w, dtype), "p.", m, x.double())
        for cuts in ((T,), (query,) + (1,) * (T - query), (query - distance + 1, distance - 1, 1, T - query - 1) if distance > 1
                     else (T,), (1,) * T):
            cuts = tuple(c for c in cuts if c > 0)
            got = run_mixer(part, x.to(device), cuts, dtype, device, page_size=page_size)
            _close(got, want, dtype, ("window", query, distance, cuts))


def far_key_without_window(device, dtype, T=300, page_size=16):
    """No mask: a key hundreds of tokens back, whose score stands out, must be seen (at a page's first and last place)."""
    g = torch.Generator().manual_seed(4)
    H, G, dk, dv, D = 2, 1, 8, 8, 24
    w, part, m = _attention(device, dtype, g, H, G, dk, dv, D, 0.5, None)
    w["p.q"][:, :2], w["p.k"][:, :2] = 0.0, 0.0
    w["p.q"][0, 0] = w["p.q"][dk, 0] = w["p.k"][0, 1] = 6.0
    _load(part, NAMES_ATTENTION, w, dtype, device)
    for key in (0, 15, 16, 31):
        x = _draw(g, T, D, std=0.5)
        x[:, :2] = 0.0
        x[T - 1, 0], x[key, 1] = 4.0, 4.0
        x = x.to(dtype)
        want = plain.window_attention(_rounded(w, dtype), "p.", m, x.double())
        for cuts in ((T,), (T - 1, 1), (100, 100, 99, 1)):
            _close(run_mixer(part, x.to(device), cuts, dtype, device, page_size=page_size), want, dtype, ("far", key, cuts))


def parallel_part(device, dtype):
    """Both mixers side by side with a cache and a state of their own; the weights of the sum."""
    g = torch.Generator().manual_seed(5)
    D = 40
    wl, _, ml = _attention(device, dtype, g, 4, 2, 12, 20, D, 0.3, 9)
    H, dk, dv = 2, 8, 12
    wr = {"p.q": _draw(g, H * dk, D), "p.k": _draw(g, H * dk, D), "p.v": _draw(g, H * dv, D), "p.g": _draw(g, H * dv, D),
          "p.o": _draw(g, D, H * dv), "p.i": _draw(g, H, D), "p.f": _draw(g, H, D), "p.i.b": _draw(g, H),
          "p.f.b": _draw(g, H), "p.norm": 1.0 + _draw(g, H * dv)}
    w = {"p.left." + k[2:]: v for k, v in wl.items()} | {"p.right." + k[2:]: v for k, v in wr.items()}
    part = MIXERS.build("parallel", left_scale=1.3, right_scale=0.6,
                        left=PartSpec("sink_attention", dict(hidden_size=D, num_heads=4, num_kv_heads=2, key_dim=12,
                                                             value_dim=20, scale=0.3, bias=True, window=9)),
                        right=PartSpec("matrix_memory", dict(hidden_size=D, num_heads=H, key_dim=dk, value_dim=dv,
                                                             gate_cap=12.0, norm_eps=1e-5)))
    names = {"left." + k: "p.left." + v[2:] for k, v in NAMES_ATTENTION.items()}
    names |= {"right." + k: "p.right." + v for k, v in dict(
        q_proj="q", k_proj="k", v_proj="v", gate_proj="g", o_proj="o", input_gate="i", forget_gate="f", input_bias="i.b",
        forget_bias="f.b", norm="norm").items()}
    assert set(names) == set(part.param_specs())
    _load(part, names, w, dtype, device)
    x = _draw(g, 61, D, std=1.0).to(dtype)
    mixer = {"left": ml, "right": {"heads": H, "dim": dk, "vdim": dv, "gate_cap": 12.0}, "left_scale": 1.3, "right_scale": 0.6}
    want = plain.parallel_mixer(_rounded(w, dtype), "p.", mixer, x.double(), 1e-5)
    for cuts in CUTS:
        _close(run_mixer(part, x.to(device), cuts, dtype, device, page_size=4), want, dtype, ("parallel", cuts))


# --------------------------------------------------------------------------- feed-forwards
def routed_experts_part(device, dtype, experts=5, top=2, ff=24, shared=16, width=40, T=70):
    g = torch.Generator().manual_seed(6)
    D = width
    w = {"p.router": _draw(g, experts, D, std=1.0)}
    for e in range(experts):
        w |= {f"p.e{e}.gate": _draw(g, ff, D), f"p.e{e}.up": _draw(g, ff, D), f"p.e{e}.down": _draw(g, D, ff)}
    names = {"router": "p.router"} | {f"e{e}.{n}": f"p.e{e}.{n}" for e in range(experts) for n in ("gate", "up", "down")}
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": 1.5}, "expert": {"ff": ff}}
    if shared:
        w |= {"p.shared.gate": _draw(g, shared, D), "p.shared.up": _draw(g, shared, D), "p.shared.down": _draw(g, D, shared),
              "p.shared.sg": _draw(g, 1, D)}
        names |= {"shared.gate_proj": "p.shared.gate", "shared.up_proj": "p.shared.up", "shared.down_proj": "p.shared.down",
                  "shared.score": "p.shared.sg"}
        mlp["shared"] = {"ff": shared}
    part = FEED_FORWARDS.build("routed_experts", hidden_size=D, num_experts=experts, top=top, expert_size=ff,
                               router_scale=1.5, shared_size=shared)
    assert set(names) == set(part.param_specs())
    _load(part, names, w, dtype, device)
    x = _draw(g, T, D, std=1.0).to(dtype)
    want = plain.moe_ffn(_rounded(w, dtype), "p.", mlp, x.double())
    got = part.forward(x.to(device), None)
    rows = (got.double().cpu() - want).abs().amax(-1) / want.abs().max()
    # (a bfloat16 run may take another expert where two scores are close: a few rows at most)
    assert int((rows > _tol(dtype)).sum()) <= (0 if dtype == torch.float32 else 3), float(rows.max())
    # a row's result does not depend on the rows beside it
    alone = torch.cat([part.forward(x[t:t + 1].to(device), None) for t in (0, 1, T - 1)])
    _close(alone, got.cpu()[[0, 1, T - 1]], dtype, "rows alone", scale=float(want.abs().max()))


def dense_part(device, dtype):
    g = torch.Generator().manual_seed(7)
    w = {"p.up": _draw(g, 56, 40), "p.down": _draw(g, 40, 56)}
    part = FEED_FORWARDS.build("dense", hidden_size=40, intermediate_size=56, activation="gelu_erf")
    _load(part, {"up_proj": "p.up", "down_proj": "p.down"}, w, dtype, device)
    x = _draw(g, 33, 40, std=2.0).to(dtype)
    _close(part.forward(x.to(device)), plain.dense_ffn(_rounded(w, dtype), "p.", x.double()), dtype, "dense")


# --------------------------------------------------------------------------- embedding and the token's side input
def _step_ctx(cache, rid, tokens, start, dtype, device):
    ctx = one_request_ctx(len(tokens), start, dtype, device, cache, rid=rid)
    ctx.tokens = torch.tensor(tokens, dtype=torch.int32, device=device)
    return ctx


def embedding_part(device, dtype):
    """The pair row of a portion's first token comes from the token before the portion; a request's first token takes the
    last row; a slot that is used again starts anew; products of ids and multipliers beyond 32 bits."""
    g = torch.Generator().manual_seed(8)
    V, D, buckets = 90, 24, 53
    for mul_prev, mul_cur in ((7, 3), (1000003, 999983)):
        w = {"embed": _draw(g, V, D), "bigram": _draw(g, buckets + 1, D), "pos": _draw(g, 64, D)}
        cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}
        part = EMBEDDINGS.build("summed_embedding", vocab_size=V, dim=D, pair_buckets=buckets, mul_prev=mul_prev,
                                mul_cur=mul_cur, max_positions=64)
        _load(part, {"table": "embed", "pair": "bigram", "pos": "pos"}, w, dtype, device)
        cache = CacheManager([(part.cache_need(), None)], page_size=4, num_pages=8, num_slots=2, max_seq_len=64,
                             dtype=dtype, device=torch.device(device))
        for rid, seed in (("a", 1), ("b", 2), ("c", 3)):   # c takes the slot that a gives back
            tokens = torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(seed)).tolist()
            want = plain.embedding(_rounded(w, dtype), cfg, tokens)
            cache.admit(rid)
            at, got = 0, []
            for c in (1, 1, 5, 2, 1, 30):
                ctx = _step_ctx(cache, rid, tokens[at:at + c], at, dtype, device)
                got.append(part.forward(ctx.tokens, ctx, cache.views[0]).double().cpu())
                at += c
            _close(torch.cat(got), want, torch.float32, ("embedding", rid, mul_prev))
            if rid != "b":
                cache.free(rid)


def token_side_part(device, dtype):
    g = torch.Generator().manual_seed(9)
    V, D, dim, layers, i = 50, 40, 6, 3, 1
    w = {"side.embed": _draw(g, V, dim * layers, std=1.0), "l1.side.gate": _draw(g, dim, D), "l1.side.proj": _draw(g, D, dim),
         "l1.side.norm": _draw(g, D, std=1.0)}
    part = STREAM_PARTS.build("token_side", hidden_size=D, dim=dim, vocab_size=V, table_width=dim * layers, column=i * dim,
                              eps=1e-5)
    _load(part, {"table": "side.embed", "gate": "l1.side.gate", "proj": "l1.side.proj", "norm": "l1.side.norm"}, w, dtype,
          device)
    tokens = torch.randint(0, V, (21,), generator=g).tolist()
    x = _draw(g, 21, D, std=1.0).float()
    xin = x.to(dtype).double() if dtype != torch.float32 else x.double()
    want = x.double() + plain.token_side(_rounded(w, dtype), {"token_side": {"dim": dim}}, i, tokens, xin, 1e-5)

    class Ctx:
        pass
    ctx = Ctx()
    ctx.dtype, ctx.tokens = dtype, torch.tensor(tokens, dtype=torch.int32, device=device)
    h = x.to(device).clone()
    part.forward(h, ctx)
    _close(h, want, dtype, "token side")
