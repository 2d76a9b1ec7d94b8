"""Each mechanism of Zenuzen alone against the plain implementation's function for it (tests/plain_zenuzen.py),
as bodies that take the module of operations (`simply_amd.kernels.ops` on the GPU, `torch_ops` on the CPU) and the
device.  Inputs are made so that a fault shows: one far key whose score stands out among hundreds, a sink that
takes most of the softmax's sum, a convolution whose taps differ by an order of magnitude, a decay close to 0 and
close to 1."""
from __future__ import annotations

import torch

import plain_zenuzen as plain
from simply_amd import registry
from simply_amd.config import PartSpec
from zenuzen_cases import run_mixer


def rand(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    err = float((got - want).abs().max() / max(float(want.abs().max()), 1e-30))
    assert err <= tol, (what, err)


def tol_of(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


# --------------------------------------------------------------------------- row-wise


def residual_add_norm(o, device, dtype):
    T, D = 5, 72
    y, h, w = rand((T, D), 1, 3.0), rand((T, D), 2), rand((D,), 3)
    yd, wd = y.to(dtype), w.to(dtype)
    want = h.float().double() + 0.37 * plain.rms_norm(yd.double(), wd.double(), 1e-3)
    res = h.float().to(device)
    out = o.residual_add_norm(yd.to(device), res, weight=wd.to(device), eps=1e-3, plus_one=False, mult=0.37,
                              out_dtype=dtype)
    close(res, want, 2e-6, "residual")
    close(out, want, tol_of(dtype), "handed on")
    # nothing added: only the hand-over; and a sum without a norm
    res2 = h.float().to(device)
    close(o.residual_add_norm(None, res2, out_dtype=dtype), h, tol_of(dtype))
    o.residual_add_norm(yd.to(device), res2, mult=2.0)
    close(res2, h.float().double() + 2.0 * yd.double(), 2e-6)


def gated_heads(o, device, dtype):
    T, H, S = 4, 3, 20
    x, g, w = rand((T, H * S), 4, 2.0), rand((T, H * S + 7), 5, 2.0), rand((S,), 6)
    xd, gd, wd = x.to(dtype), g.to(dtype), w.to(dtype)
    gate = gd[:, 3:3 + H * S]     # a view with a row stride, as the mixers hand it over
    normed = plain.rms_norm(xd.double().view(T, H, S), wd.double(), 1e-4).reshape(T, H * S)
    got = o.gated_heads(xd.to(device), gd.to(device)[:, 3:3 + H * S], H, S, kind=1, weight=wd.to(device), eps=1e-4,
                        out_dtype=dtype)
    close(got, normed * plain.silu(gate.double()), tol_of(dtype), "norm and silu")
    got = o.gated_heads(xd.to(device), gd.to(device)[:, 3:3 + H * S], H, S, kind=0, out_dtype=dtype)
    close(got, xd.double() * torch.sigmoid(gate.double()), tol_of(dtype), "sigmoid")


def activation(o, device, dtype):
    x = rand((6, 37), 7, 2.0).to(dtype)
    got = o.activation_(x.clone().to(device), registry.ACTIVATIONS.get("squared_relu"))
    close(got, plain.squared_relu(x.double()), tol_of(dtype))
    got = o.activation_(x.clone().to(device), registry.ACTIVATIONS.get("gelu_tanh"))
    close(got, plain.gelu_tanh(x.double()), tol_of(dtype))


def activated_product(o, device, dtype, tiled=False):
    """relu(x W^T)^2 as one call, at row counts that the different product kernels take (a handful, a few hundred
    with the inner dimension cut over workgroups, thousands with the activation in the kernel's epilogue)."""
    from simply_amd.parts.base import as_product_weight

    K, N = 256, 384
    w = rand((N, K), 20, 0.1).to(dtype)
    wd = as_product_weight(w.to(device)) if tiled else w.to(device)
    for M in (3, 40, 300, 2100):
        x = rand((M, K), 21 + M).to(dtype)
        want = plain.squared_relu((x.double() @ w.double().T).to(dtype).double())
        got = o.gemm(x.to(device), wd, activate=registry.ACTIVATIONS.get("squared_relu"))
        close(got, want, 2e-5 if dtype == torch.float32 else 3e-2, f"{M} rows")


def partial_rotary_norm_and_pages(o, device, dtype, page_size=4):
    """Queries and keys: rotation of the first dimensions, then unit RMS; values mixed; pages written where the slot
    mapping says.  Positions far from 0 and a page's last and first place are among them."""
    import torch_ops

    T, H, K, dk, dv, rot, base, eps = 6, 4, 2, 24, 10, 8, 300.0, 1e-5
    width = (H + K) * dk + K * dv + 5
    proj = rand((T, width), 8).to(dtype)
    vf = rand((T, K * dv + 3), 9).to(dtype)
    lam = torch.tensor(0.3, dtype=dtype)
    pos = torch.tensor([0, 1, 3, 4, 1000, 40000], dtype=torch.int32)
    slots = torch.tensor([0, 1, 3, 4, 23, 9], dtype=torch.int64)   # page * page_size + offset
    inv_freq = (base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).float()
    qk = proj.double()[:, :(H + K) * dk].view(T, H + K, dk)
    # (the angle is the 32-bit product of position and frequency, as the design has it)
    ang = (pos.float()[:, None] * inv_freq[None, :]).double()[:, None, :]
    a, b = qk[..., :rot // 2], qk[..., rot // 2:rot]
    rotated = torch.cat([a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang), qk[..., rot:]], -1)
    want_qk = plain.rms_norm(rotated, None, eps)
    close(plain.partial_rotary(qk[:4], pos[:4], rot, base), rotated[:4], 1e-6, "the plain rotation itself")
    v = proj.double()[:, (H + K) * dk:(H + K) * dk + K * dv]
    want_v = (1 - lam.double()) * v + lam.double() * vf.double()[:, :K * dv]
    k_pages = torch.zeros((6, K, page_size, dk), dtype=dtype, device=device)
    v_pages = torch.zeros((6, K, dv, page_size), dtype=dtype, device=device)
    p = proj.clone().to(device)
    o.qk_norm_rope_cache_write(p, pos.to(device), inv_freq.to(device), rot, eps, H, K, dk, dv,
                               v_first=vf.to(device)[:, :K * dv], v_mix=lam.reshape(1).to(device),
                               slot_mapping=slots.to(device), k_pages=k_pages, v_pages=v_pages)
    tol = tol_of(dtype)
    close(p[:, :H * dk], want_qk[:, :H].reshape(T, H * dk), tol, "queries")
    close(p[:, H * dk:], proj[:, H * dk:], 0.0, "everything but the queries stays")
    krows = torch_ops.stored_keys_as_rows(k_pages.cpu())
    for t in range(T):
        page, off = int(slots[t]) // page_size, int(slots[t]) % page_size
        close(krows[page, :, off], want_qk[t, H:], tol, f"key {t}")
        close(v_pages[page, :, :, off], want_v[t].view(K, dv), tol, f"value {t}")
    assert int((krows.abs().sum(-1) > 0).sum()) == T * K    # nothing else was written


def sink_attention_far_key(o, device, dtype, page_size=16):
    """One key far back (at a page's last place, and at the very first position) is made to stand out among
    hundreds; the sink takes a fixed share of every sum.  Pages are scattered over the pool."""
    import torch_ops

    T, H, K, dk, dv, scale = 300, 4, 2, 24, 12, 0.6
    q, k, v = rand((T, H, dk), 10), rand((T, K, dk), 11), rand((T, K, dv), 12)
    sink = torch.tensor([2.0, -1.0, 0.5, 4.0], dtype=torch.float64)
    for far, asker, head in ((15, 299, 0), (0, 250, 3), (16, 17, 1), (63, 100, 2), (64, 31 + 64, 0)):
        k[far, head // 2] = q[asker, head] * (25.0 / (q[asker, head] ** 2).sum())   # a score of 25 * scale, far above the others
    qd, kd, vd = q.to(dtype), k.to(dtype), v.to(dtype)
    want = plain.sink_softmax_attention(qd.double(), kd.double(), vd.double(), sink.to(dtype).double(), scale)
    # without the far key the answer would be another one: the test can see it
    k2 = kd.double().clone()
    k2[15] = 0
    assert (plain.sink_softmax_attention(qd.double(), k2, vd.double(), sink.to(dtype).double(), scale)[299, 0]
            - want[299, 0]).abs().max() > 0.1
    n_pages = -(-T // page_size)
    order = torch.randperm(n_pages + 3, generator=torch.Generator().manual_seed(1))[:n_pages]
    table = torch.full((2, n_pages), -1, dtype=torch.int32)
    table[1] = order.to(torch.int32)
    krows = torch.zeros((n_pages + 3, K, page_size, dk), dtype=dtype)
    v_pages = torch.zeros((n_pages + 3, K, dv, page_size), dtype=dtype)
    for t in range(T):
        page, off = int(order[t // page_size]), t % page_size
        krows[page, :, off] = kd[t]
        v_pages[page, :, :, off] = vd[t]
    k_pages = torch_ops.rows_as_stored_keys(krows)
    rows = torch.tensor([299, 250, 17, 0, 1, 15, 16, 31, 32, 100, 95, 63, 64], dtype=torch.long)
    got = o.paged_attention_sink(qd[rows].reshape(len(rows), H * dk).contiguous().to(device), k_pages.to(device),
                                 v_pages.to(device), table.to(device), torch.ones(len(rows), dtype=torch.int32, device=device),
                                 rows.to(torch.int32).to(device), H, scale=scale, sinks=sink.to(dtype).to(device))
    close(got, want[rows].reshape(len(rows), H * dv), tol_of(dtype), "attention")
    # a sink that is left out would show: with it the first token's weights sum to less than one
    first = got[3].double().cpu().view(H, dv)
    share = 1.0 / (1.0 + torch.exp(sink.to(dtype).double() - scale * (qd[0].double() * kd[0].double().repeat_interleave(2, 0)).sum(-1)))
    close(first, vd[0].double().repeat_interleave(2, 0) * share[:, None], tol_of(dtype), "the first token and the sink")


def sink_attention_on_the_matrix_cores(device):
    """The bfloat16 MFMA kernels with sinks: single tokens (their keys cut into ranges that a second kernel merges)
    and a portion of a prompt, with far keys that stand out (at position 0, at a page's last and first place, at the
    edge of a tile of 32 keys) among a thousand, and one large sink."""
    import torch_ops
    from simply_amd.engine.context import StepContext
    from simply_amd.kernels import ops

    T, H, K, d, scale, P = 1000, 8, 2, 64, 0.3, 16
    dtype = torch.bfloat16
    q, k, v = rand((T, H, d), 50), rand((T, K, d), 51), rand((T, K, d), 52)
    sink = torch.tensor([6.0, -1.0, 0.5, 4.0, 0.0, 2.0, -3.0, 8.0], dtype=torch.float64)
    for far, asker, head in ((0, 999, 0), (15, 990, 3), (16, 999, 5), (31, 700, 7), (32, 969, 1), (511, 998, 6)):
        k[far, head // 4] = q[asker, head] * (40.0 / (q[asker, head] ** 2).sum())
    qd, kd, vd = q.to(dtype), k.to(dtype), v.to(dtype)
    want = plain.sink_softmax_attention(qd.double(), kd.double(), vd.double(), sink, scale)
    n_pages = -(-T // P)
    order = torch.randperm(n_pages + 5, generator=torch.Generator().manual_seed(2))[:n_pages]
    table = torch.full((2, n_pages), -1, dtype=torch.int32)
    table[1] = order.to(torch.int32)
    krows = torch.zeros((n_pages + 5, K, P, d), dtype=dtype)
    v_pages = torch.zeros((n_pages + 5, K, d, P), dtype=dtype)
    for t in range(T):
        krows[int(order[t // P]), :, t % P] = kd[t]
        v_pages[int(order[t // P]), :, :, t % P] = vd[t]
    k_pages = torch_ops.rows_as_stored_keys(krows).to(device)
    v_pages, table = v_pages.to(device), table.to(device)
    sinks = sink.float().to(device)
    # (these kernels have no factor on the scores: the queries carry it)
    qs = (qd.double() * scale).to(dtype).reshape(T, H * d).to(device)
    # single tokens: every row a request of its own at its position
    rows = [999, 990, 700, 969, 998, 0, 15, 16, 31, 32, 33, 512]
    meta = torch.tensor([[1, i, 1, r] for i, r in enumerate(rows)], dtype=torch.int32, device=device)
    out = torch.zeros((len(rows), H * d), dtype=dtype, device=device)
    ops.paged_attention_decode(qs[rows].contiguous(), k_pages, v_pages, table, meta, 0, len(rows), H, window=None,
                               soft_cap=None, max_kv_len=T, max_q_len=1, out=out, sinks=sinks)
    close(out, want[rows].reshape(len(rows), H * d), 3e-2, "single tokens")
    # the last 299 tokens as one portion of a prompt
    first = T - 299
    ctx = StepContext(dtype=dtype, num_tokens=299, positions=torch.arange(first, T, dtype=torch.int32, device=device),
                      token_seq=torch.ones(299, dtype=torch.int32, device=device),
                      seq_meta=torch.tensor([[1, 0, 299, first]], dtype=torch.int32, device=device), groups={},
                      request_ids=["r"], seq_slots=[1], seq_starts=[first], q_lens=[299], cu_q_lens=[0, 299])
    units, few, many, max_q = ctx.attention_units(16 // (H // K), ops.prefill_units_per_group())
    assert few == 0 and many > 0
    out = torch.zeros((299, H * d), dtype=dtype, device=device)
    ops.paged_attention_prefill(qs[first:].contiguous(), k_pages, v_pages, table, units, 0, many, H, window=None,
                                soft_cap=None, max_kv_len=T, max_q_len=max_q, out=out, sinks=sinks)
    close(out, want[first:].reshape(299, H * d), 3e-2, "a portion")
    # the sinks matter: without them the answer is another one
    without = plain.sink_softmax_attention(qd.double(), kd.double(), vd.double(), sink - 50.0, scale)
    assert float((without[first:] - want[first:]).abs().max()) > 0.3


def short_convolution(o, device, dtype):
    """Two requests in one step; the second goes on from a tail that an earlier step left; taps of very different
    size, so that a tap that is off by one shows."""
    C, n = 70, 4
    taps = torch.tensor([1.0, -10.0, 100.0, 0.1], dtype=torch.float64)[None, :] * (1.0 + rand((C, 1), 13, 0.1))
    xa, xb = rand((9, C), 14), rand((7, C), 15)
    td, xad, xbd = taps.to(dtype), xa.to(dtype), xb.to(dtype)
    want_a = plain.silu(plain.causal_conv(xad.double(), td.double()))
    want_b = plain.silu(plain.causal_conv(xbd.double(), td.double()))
    tails = torch.zeros((3, (n - 1) * C + 5), dtype=torch.float32, device=device)
    # first step: request b alone brings its first 2 tokens (fewer than the taps) into slot 2
    meta = torch.tensor([[2, 0, 2, 0]], dtype=torch.int32, device=device)
    y = o.short_conv_silu(xbd[:2].contiguous().to(device), td.to(device), tails, meta, 1, 2)
    close(y, want_b[:2], tol_of(dtype), "first portion")
    # second step: a whole (slot 0, rows 5..13) beside the rest of b (rows 0..4)
    x = torch.cat([xbd[2:], xad]).contiguous().to(device)
    meta = torch.tensor([[2, 0, 5, 2], [0, 5, 9, 0]], dtype=torch.int32, device=device)
    y = o.short_conv_silu(x, td.to(device), tails, meta, 2, 9)
    close(y[:5], want_b[2:], tol_of(dtype), "second portion from the tail")
    close(y[5:], want_a, tol_of(dtype), "a whole request beside it")
    close(tails[0, :(n - 1) * C].view(n - 1, C), xad[-(n - 1):], 0.0, "tail of a")
    close(tails[2, :(n - 1) * C].view(n - 1, C), xbd[-(n - 1):], 0.0, "tail of b")
    assert float(tails[1].abs().max()) == 0.0


def delta_inputs_of_short_steps(o, device, dtype):
    """Convolution, silu, new tails, unit q and k and the gates as one call, for steps of few tokens a request: two
    requests over three steps (2 + 1 + 9 tokens and 5 + 7 tokens), against the plain functions on the whole sequences."""
    H, G, dk, dv, n = 4, 2, 70, 9, 4
    C = 2 * G * dk + H * dv
    taps = torch.tensor([1.0, -3.0, 9.0, 0.3], dtype=torch.float64)[None, :] * (1.0 + rand((C, 1), 80, 0.1))
    a_log, dt_bias = torch.tensor([-2.0, 0.0, 0.5, 1.0], dtype=torch.float64), rand((H,), 81)
    xs = {0: rand((12, C), 82), 3: rand((12, C), 83)}
    abs_ = {0: rand((12, 2 * H), 84, 2.0), 3: rand((12, 2 * H), 85, 2.0)}
    td = taps.to(dtype)
    want = {}
    for slot in xs:
        y = plain.silu(plain.causal_conv(xs[slot].to(dtype).double(), td.double()))
        q, k = y[:, :G * dk].view(12, G, dk), y[:, G * dk:2 * G * dk].view(12, G, dk)
        y[:, :G * dk] = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5).reshape(12, -1)
        y[:, G * dk:2 * G * dk] = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).reshape(12, -1)
        ab = abs_[slot].float().double()
        want[slot] = (y, torch.sigmoid(ab[:, H:]), torch.exp(-torch.exp(a_log) * plain.softplus(ab[:, :H] + dt_bias)))
    tails = torch.zeros((4, (n - 1) * C), dtype=torch.float32, device=device)
    done = {0: 0, 3: 0}
    for step in ([(0, 2), (3, 5)], [(0, 1)], [(3, 7), (0, 9)]):
        x = torch.cat([xs[s][done[s]:done[s] + c] for s, c in step]).to(dtype).contiguous().to(device)
        ab = torch.cat([abs_[s][done[s]:done[s] + c] for s, c in step]).float().contiguous().to(device)
        meta, at = [], 0
        for s, c in step:
            meta.append([s, at, c, done[s]])
            at += c
        qkv, gates = o.delta_inputs(x, td.to(device), tails, ab, a_log.float().to(device), dt_bias.float().to(device),
                                    torch.tensor(meta, dtype=torch.int32, device=device), len(step),
                                    max(c for _, c in step), H, G, dk)
        for (s, c), (_, first, _, _) in zip(step, meta):
            y, beta, g = (w[done[s]:done[s] + c] for w in want[s])
            close(qkv[first:first + c], y, tol_of(dtype), f"slot {s} from {done[s]}")
            close(gates[first:first + c, :H], beta, 2e-6, "beta")
            close(gates[first:first + c, H:], g, 2e-5, "decay")
            done[s] += c
    for s in xs:
        close(tails[s].view(n - 1, C), xs[s].to(dtype)[-(n - 1):], 0.0, f"tail of slot {s}")
    assert float(tails[1].abs().max()) == 0.0 and float(tails[2].abs().max()) == 0.0


def delta_rule_steps(o, device, T=40, cuts=(13, 1, 2, 1, 23)):
    """The recurrence in portions against the plain one; decays close to 0 and close to 1, beta from 0 to 1."""
    H, G, dk, dv = 4, 2, 20, 70
    C = 2 * G * dk + H * dv
    x = rand((T, C), 16)
    ab = rand((T, 2 * H), 17, 3.0)
    a_log, dt_bias = torch.tensor([-3.0, 0.0, 1.0, 2.0], dtype=torch.float64), rand((H,), 18)
    q, k = x[:, :G * dk].view(T, G, dk), x[:, G * dk:2 * G * dk].view(T, G, dk)
    qn = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    kn = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(ab[:, H:])
    g = torch.exp(-torch.exp(a_log) * plain.softplus(ab[:, :H] + dt_bias))
    assert float(g.min()) < 0.01 and float(g.max()) > 0.99
    want, S = plain.delta_recurrence(qn.repeat_interleave(H // G, 1), kn.repeat_interleave(H // G, 1),
                                     x[:, 2 * G * dk:].view(T, H, dv), beta, g)
    state = torch.zeros((3, H * dk * dv + 11), dtype=torch.float32, device=device)
    got, at = [], 0
    assert sum(cuts) == T
    for c in cuts:
        part = x[at:at + c].float().contiguous().to(device)
        gates = o.delta_prepare(part, ab[at:at + c].float().contiguous().to(device), a_log.float().to(device),
                                dt_bias.float().to(device), H, G, dk)
        close(gates[:, :H], beta[at:at + c], 2e-6, "beta")
        close(gates[:, H:], g[at:at + c], 2e-5, "decay")
        meta = torch.tensor([[1, 0, c, at]], dtype=torch.int32, device=device)
        got.append(o.delta_rule(part, gates, state, meta, 1, H, G, dk, dv).cpu())
        at += c
    close(torch.cat(got), want.reshape(T, H * dv), 3e-5, "outputs")
    close(state[1, :H * dk * dv].view(H, dv, dk).transpose(1, 2), S, 3e-5, "state (stored column by column)")
    assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


def delta_rule_long_and_short_together(o, device):
    """One step with requests of 150, 64, 5 and 1 tokens, each from a state that an earlier step left in its slot:
    every request's result is what it is alone."""
    H, G, dk, dv = 3, 1, 32, 12
    C = 2 * G * dk + H * dv
    counts = {0: (7, 150), 2: (3, 64), 3: (40, 5), 1: (2, 1)}     # slot -> (tokens of the earlier step, of this one)
    a_log, dt_bias = torch.tensor([-2.0, 0.0, 1.5], dtype=torch.float64), rand((H,), 60)
    state = torch.zeros((4, H * dk * dv), dtype=torch.float32, device=device)
    want, rows, metas, xs, abs_ = {}, 0, [], [], []
    for slot, (before, now) in counts.items():
        T = before + now
        x, ab = rand((T, C), 61 + slot), rand((T, 2 * H), 71 + slot, 2.0)
        q, k = x[:, :G * dk].view(T, G, dk), x[:, G * dk:2 * G * dk].view(T, G, dk)
        qn = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
        kn = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        g = torch.exp(-torch.exp(a_log) * plain.softplus(ab[:, :H] + dt_bias))
        out, S = plain.delta_recurrence(qn.repeat_interleave(H, 1), kn.repeat_interleave(H, 1),
                                        x[:, 2 * G * dk:].view(T, H, dv), torch.sigmoid(ab[:, H:]), g)
        want[slot] = (out[before:].reshape(now, H * dv), S)
        # the earlier step, alone
        part = x[:before].float().contiguous().to(device)
        gates = o.delta_prepare(part, ab[:before].float().contiguous().to(device), a_log.float().to(device),
                                dt_bias.float().to(device), H, G, dk)
        meta = torch.tensor([[slot, 0, before, 0]], dtype=torch.int32, device=device)
        o.delta_rule(part, gates, state, meta, 1, H, G, dk, dv)
        metas.append([slot, rows, now, before])
        xs.append(x[before:])
        abs_.append(ab[before:])
        rows += now
    part = torch.cat(xs).float().contiguous().to(device)
    gates = o.delta_prepare(part, torch.cat(abs_).float().contiguous().to(device), a_log.float().to(device),
                            dt_bias.float().to(device), H, G, dk)
    meta = torch.tensor(metas, dtype=torch.int32, device=device)
    got = o.delta_rule(part, gates, state, meta, len(metas), H, G, dk, dv).cpu()
    for slot, first, now, _ in metas:
        close(got[first:first + now], want[slot][0], 3e-5, f"outputs of slot {slot}")
        close(state[slot].view(H, dv, dk).transpose(1, 2), want[slot][1], 3e-5, f"state of slot {slot}")


# --------------------------------------------------------------------------- the mixers as parts


def _load(part, dtype, device, seed, scale=0.3, fixed=None):
    tensors = {}
    for i, (name, ps) in enumerate(part.param_specs().items()):
        t = rand(ps.shape, seed + i, scale)
        if fixed and name in fixed:
            t = fixed[name]
        tensors[name] = t.to(dtype).to(device)
    part.load(tensors)
    return {k: v.double().cpu() for k, v in tensors.items()}


def attention_part(device, dtype, sizes=(40, 4, 2, 12, 20), length=50, cuts=([50], [15, 1, 1, 2, 31], [2] * 25)):
    """The attention mixer with a cache of its own, whole and in portions that cut pages, against the plain mixer.
    The sinks are large, so that one that is left out shows."""
    D, H, K, dk, dv = sizes
    eps = 1e-5
    params = dict(hidden_size=D, num_heads=H, num_kv_heads=K, key_dim=dk, value_dim=dv, scale=0.5, sinks=True,
                  qk_norm_eps=eps, output_gate=True, value_mix=None,
                  position_encoding=PartSpec("partial_rope", {"head_dim": dk, "dims": 6, "base": 50.0}))
    part = registry.MIXERS.build("sink_attention", **params)
    t = _load(part, dtype, device, 30, fixed={"sink": torch.linspace(-2.0, 4.0, H, dtype=torch.float64)})
    w = {"p.q": t["q_proj"], "p.k": t["k_proj"], "p.v": t["v_proj"], "p.g": t["gate_proj"], "p.o": t["o_proj"],
         "p.sink": t["sink"]}
    mc = {"heads": H, "kv_heads": K, "dim": dk, "vdim": dv, "scale": 0.5, "rot": {"dims": 6, "base": 50.0}}
    x = rand((length, D), 31).to(dtype)
    want = plain.attention_mixer(x.double(), torch.arange(length), w, "p.", mc, eps, {})
    without = plain.attention_mixer(x.double(), torch.arange(length), dict(w, **{"p.sink": w["p.sink"] - 30.0}), "p.", mc,
                                    eps, {})
    assert float((without - want).abs().max() / want.abs().max()) > 0.3     # the sinks matter
    tol = 3e-5 if dtype == torch.float32 else 4e-2
    for c in cuts:
        close(run_mixer(part, x.to(device), c, dtype, device), want, tol, str(c))


def delta_part(device, dtype):
    D, H, G, dk, dv, n, eps = 36, 4, 2, 12, 24, 3, 1e-5
    part = registry.MIXERS.build("gated_delta", hidden_size=D, num_heads=H, num_qk_heads=G, key_dim=dk, value_dim=dv,
                                 conv_taps=n, norm_eps=eps)
    t = _load(part, dtype, device, 40, fixed={"a_log": torch.tensor([-2.0, 0.0, 0.5, 1.0], dtype=torch.float64)})
    names = {"q_proj": "q", "k_proj": "k", "v_proj": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
             "a_proj": "a", "b_proj": "b", "a_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "gate_proj": "g",
             "o_proj": "o"}
    w = {"p." + names[k]: v for k, v in t.items()}
    mc = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": n}
    x = rand((40, D), 41).to(dtype)
    want = plain.delta_mixer(x.double(), w, "p.", mc, eps)
    tol = 5e-5 if dtype == torch.float32 else 5e-2
    for cuts in ([40], [17, 1, 1, 2, 19], [2] * 20, [1] * 40):
        close(run_mixer(part, x.to(device), cuts, dtype, device), want, tol, str(cuts))
