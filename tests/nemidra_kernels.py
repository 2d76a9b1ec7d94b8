"""Every kernel that Nemidra brought against its plain torch reference (tests/torch_ops.py) on inputs of the test's
own: requests of unequal length in one launch, states that are carried on, sizes that are no multiple of anything."""
from __future__ import annotations

import torch

import torch_ops as ref
from simply_amd.kernels import packing


def _cmp(got, want, tol, what):
    got, want = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max() / max(float(want.abs().max()), 1e-9))
    assert err < tol, (what, err)


def _meta(counts, slots, starts):
    rows, first = [], 0
    for c, s, p in zip(counts, slots, starts):
        rows.append((s, first, c, p))
        first += c
    return torch.tensor(rows, dtype=torch.int32), first


def token_tables(ops, dev, dtype):
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    g = torch.Generator().manual_seed(0)
    V, D, B = 50, 72, 13
    table, pair, pos = (torch.randn(n, D, generator=g).to(dtype) for n in (V, B + 1, 64))
    m, T = _meta([1, 5, 20], [2, 0, 3], [0, 5, 7])   # the first request is at its first token
    tokens = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    positions = torch.cat([torch.arange(p, p + c) for _, _, c, p in m.tolist()]).to(torch.int32)
    last = torch.randint(0, V, (4, 1), generator=g, dtype=torch.int32)
    last_d = last.clone().to(dev)
    got = ops.embed_sum(tokens.to(dev), positions.to(dev), m.to(dev), 3, 20, table.to(dev), pair=pair.to(dev),
                        mul_prev=1000003, mul_cur=13, last=last_d, pos=pos.to(dev))
    want = ref.embed_sum(tokens, positions, m, 3, 20, table, pair=pair, mul_prev=1000003, mul_cur=13, last=last, pos=pos)
    _cmp(got, want, 1e-6, "embed_sum")
    assert torch.equal(last_d.cpu(), last)
    z, side = torch.randn(T, 16, generator=g).to(dtype), torch.randn(V, 64, generator=g).to(dtype)
    _cmp(ops.token_gate_(z.clone().to(dev), tokens.to(dev), side.to(dev), 32, 0), ref.token_gate_(z.clone(), tokens, side, 32, 0),
         tol, "token_gate")
    x, b, y = (torch.randn(*s, generator=g).to(dtype) for s in ((T, 100), (100,), (T, 100)))
    _cmp(ops.bias_add_(x.clone().to(dev), b.to(dev)), ref.bias_add_(x.clone(), b), tol, "bias_add")
    _cmp(ops.weighted_sum(x.to(dev), 1.2, y.to(dev), 0.9), ref.weighted_sum(x, 1.2, y, 0.9), tol, "weighted_sum")


def matrix_states(ops, dev, dtype, sizes=((3, 40, 24), (2, 24, 40), (2, 128, 64), (1, 16, 20), (2, 200, 70), (1, 4, 1))):
    """Both kinds of state, requests of 1, 3, 40 and 17 tokens in one launch, from states that are not zero."""
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    g = torch.Generator().manual_seed(1)
    for H, dk, dv in sizes:
        m, T = _meta([1, 3, 40, 17], [1, 3, 0, 2], [9, 0, 4, 30])
        C = H * dk
        proj = (torch.randn(T, 2 * C + 2 * H * dv + 8, generator=g) * 0.5).to(dtype)
        z, bias = torch.randn(T, C, generator=g) * 2, torch.randn(C, generator=g).to(dtype)
        for kw, kw_d in (({}, {}), (dict(decay_bias=bias, tau=4.0), dict(decay_bias=bias.to(dev), tau=4.0))):
            gates = z if kw else torch.sigmoid(z)    # z with a bias and tau, or decays as they are
            st = torch.randn(4, C * dv + 5, generator=g) * 0.3
            st_d = st.clone().to(dev)
            got = ops.linear_state(proj.to(dev), 0, C, 2 * C, dk ** -0.5, gates.to(dev), False, H, dk, dv, False, st_d,
                                   m.to(dev), 4, **kw_d)
            want = ref.linear_state(proj, 0, C, 2 * C, dk ** -0.5, gates, False, H, dk, dv, False, st, m, 4, **kw)
            _cmp(got, want, 3e-5, ("linear_state, decays per channel", H, dk, dv, bool(kw)))
            _cmp(st_d, st, 3e-5, "its state")
        raw, gb = torch.randn(T, 2 * H, generator=g) * 3, torch.randn(2 * H, generator=g).to(dtype)
        words = C * (dv + 1)
        st = torch.randn(4, words + H, generator=g) * 0.3
        st[:, words:] = torch.rand(4, H, generator=g) * 3
        st_d = st.clone().to(dev)
        gates = ref.exp_gates(raw, gb, 12.0, H, st[:, words:], m, 4)
        gates_d = ops.exp_gates(raw.to(dev), gb.to(dev), 12.0, H, st_d[:, words:], m.to(dev), 4)
        _cmp(gates_d, gates, 3e-5, ("exp_gates", H))
        _cmp(st_d[:, words:], st[:, words:], 1e-6, "the maxima")
        got = ops.linear_state(proj.to(dev), 0, C, 2 * C, dk ** -0.5, gates_d, True, H, dk, dv, True, st_d, m.to(dev), 4)
        want = ref.linear_state(proj, 0, C, 2 * C, dk ** -0.5, gates, True, H, dk, dv, True, st, m, 4)
        _cmp(got, want, 3e-5, ("linear_state, one decay per head", H, dk, dv))
        _cmp(st_d, st, 3e-5, "its state")
        g_at = 2 * C + H * dv
        wn = torch.randn(H * dv, generator=g).to(dtype)
        _cmp(ops.normalized_readout(got, gates_d[:, 2 * H:], proj.to(dev)[:, g_at:g_at + H * dv], wn.to(dev), 1e-5, H, dv, dtype),
             ref.normalized_readout(want, gates[:, 2 * H:], proj[:, g_at:g_at + H * dv], wn, 1e-5, H, dv, dtype), max(tol, 5e-5),
             "normalized_readout")


def long_gate_scan(ops, dev):
    """The running maximum over 200 tokens of one request (several rounds of 64) equals the one over its portions."""
    g = torch.Generator().manual_seed(2)
    H = 3
    raw = torch.randn(200, 2 * H, generator=g) * 6
    whole = torch.tensor([[0, 0, 200, 0]], dtype=torch.int32)
    mx = torch.zeros(1, H)
    want = ref.exp_gates(raw, None, 12.0, H, mx, whole, 1)
    mx_d = torch.zeros(1, H).to(dev)
    got, at = [], 0
    for c in (1, 63, 64, 65, 7):
        meta = torch.tensor([[0, 0, c, at]], dtype=torch.int32, device=dev)
        got.append(ops.exp_gates(raw[at:at + c].to(dev).contiguous(), None, 12.0, H, mx_d, meta, 1))
        at += c
    _cmp(torch.cat(got), want, 2e-5, "gates in portions")
    _cmp(mx_d, mx, 1e-6, "the maxima")


def routed(ops, dev, dtype, sizes=((1, 12, 3, 192, 80), (37, 12, 3, 192, 80), (300, 8, 2, 64, 48), (50, 70, 5, 72, 40),
                                   (5, 4, 4, 32, 16), (9, 3, 1, 36, 20))):
    """Few rows and many (tiles of 16 and of 64 rows), more experts than a wave has lanes, every expert chosen, sizes
    that are no multiple of 16 or 32, rows that are not 16-byte aligned."""
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    g = torch.Generator().manual_seed(3)
    for T, E, top, D, F in sizes:
        logits = torch.randn(T, E, generator=g) * 2
        e_d, w_d = ops.route(logits.to(dev), top, 2.0)
        e_r, w_r = ref.route(logits, top, 2.0)
        assert torch.equal(e_d.cpu(), e_r), ("route", T, E)
        _cmp(w_d, w_r, 1e-5, "route: weights")
        x = torch.randn(T, D, generator=g).to(dtype)
        gs, us, ds = ([(torch.randn(*s, generator=g) * 0.1).to(dtype) for _ in range(E)] for s in ((F, D), (F, D), (D, F)))
        sh, sg = torch.randn(T, D, generator=g).to(dtype), torch.randn(T, 1, generator=g)

        def on(ws):
            return packing.stack_experts(w.to(dev) for w in ws)

        got = ops.routed_experts(x.to(dev), e_d, w_d, on(gs), on(us), on(ds), 1, shared=sh.to(dev), shared_gate=sg.to(dev))
        want = ref.routed_experts(x, e_r, w_r, packing.stack_experts(gs), packing.stack_experts(us), packing.stack_experts(ds),
                                  1, shared=sh, shared_gate=sg)
        _cmp(got, want, tol, ("routed_experts", T, E, top, D, F))
        got = ops.routed_experts(x.to(dev), e_d, w_d, on(gs), on(us), on(ds), 1)
        want = ref.routed_experts(x, e_r, w_r, packing.stack_experts(gs), packing.stack_experts(us), packing.stack_experts(ds), 1)
        _cmp(got, want, tol, ("routed_experts without a shared one", T, E))
