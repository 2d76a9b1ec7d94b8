"""Small Nemidra configurations, model folders with random weights, and the bodies of the tests that run the framework
against the plain implementation (tests/plain_nemidra.py).  A body takes the device; the CPU tests run it with the
kernels replaced by their plain torch references (the `cpu_ops` fixture), the GPU tests with the kernels themselves."""
from __future__ import annotations

import torch

import plain_nemidra as plain
from simply_amd.config import config_from_dict
from simply_amd.engine import StepEntry
from simply_amd.weights import write_random_model
from zenuzen_cases import make_executor, random_tokens, run_cut  # noqa: F401  (shared helpers)


def gla(heads, dim, vdim, tau, rank, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}, "mlp": mlp}


def parallel(left, right, left_scale, right_scale, mlp=None):
    heads, kv_heads, dim, vdim, scale, window = left
    l = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        l["mask"] = {"size": window}
    rh, rd, rv, cap = right
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": l, "right": {"heads": rh, "dim": rd, "vdim": rv, "gate_cap": cap},
                      "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def config(vocab, width, eps, layers, loop=None, bigram=(53, 7, 3), positions=256, side=4, cap=9.0):
    d = {"architecture": "Nemidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if bigram:
        d["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    if positions:
        d["max_positions"] = positions
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if side:
        d["token_side"] = {"dim": side}
    if cap:
        d["logit_softcap"] = cap
    return d


#: odd sizes everywhere; a loop over the two middle layers, three times; a window of 7 (smaller than a page of 16 and
#: larger than one of 4); every kind of feed-forward, and none
MIXED = config(83, 40, 1e-5, [
    gla(3, 12, 20, 8.0, 5, mlp=dense(56)),
    parallel((4, 2, 12, 20, 0.3, 7), (2, 8, 12, 10.0), 1.3, 0.8, mlp=moe(5, 2, 24, 1.5, shared=16)),
    gla(2, 36, 8, 3.0, 3, mlp=moe(4, 1, 20, 1.0)),
    parallel((3, 1, 20, 8, 0.25, 19), (3, 20, 70, 6.0), 0.7, 1.1),
], loop=(1, 3, 3))
#: what the others make unequal is equal or 1 here: one head, as many key heads as heads, every expert used, a loop
#: that runs once and one that starts at layer 0, a window of 1, no pair table, no side input, no cap on the logits
UNITS = config(31, 24, 1e-6, [
    parallel((1, 1, 8, 8, 0.5, 1), (1, 4, 4, 9.0), 1.0, 1.0, mlp=moe(3, 3, 8, 1.25)),
    gla(1, 4, 4, 1.0, 1),
    parallel((2, 2, 8, 4, 0.4, None), (1, 16, 8, 2.0), 1.0, 0.5, mlp=dense(16)),
], loop=(0, 2, 1), bigram=None, side=None, cap=None)
LOOP_FROM_START = config(40, 32, 1e-5, [gla(2, 8, 8, 4.0, 2, mlp=dense(24)),
                                        parallel((2, 1, 16, 16, 0.25, 5), (2, 8, 8, 8.0), 1.0, 1.0)], loop=(0, 2, 2),
                         positions=None)
#: sizes in multiples of 32 and 64 (what fast kernels may take), still small
ALIGNED = config(256, 128, 1e-5, [
    gla(2, 64, 64, 12.0, 16, mlp=moe(8, 2, 64, 1.75, shared=64)),
    parallel((4, 2, 64, 64, 0.125, 48), (2, 32, 64, 12.0), 1.25, 0.85, mlp=dense(256)),
    gla(1, 128, 128, 12.0, 8),
    parallel((8, 1, 128, 128, 0.09, 24), (1, 128, 32, 9.0), 1.0, 1.0, mlp=moe(4, 2, 128, 1.0)),
], loop=(1, 3, 2), side=16)
#: name -> (configuration, seed, standard deviation of the matrices, of the norms' weights and biases).  The wider model
#: has smaller weights: with large ones its scores are so sharp that a bfloat16 run and the plain one part ways.
CONFIGS = {"mixed": (MIXED, 21, 0.25, 0.5), "units": (UNITS, 22, 0.25, 0.5), "loop_from_start": (LOOP_FROM_START, 23, 0.25, 0.5),
           "aligned": (ALIGNED, 24, 0.05, 0.2)}


def drawn_config(seed: int) -> dict:
    """A configuration drawn at random: sizes, head counts, the order of the layers, feed-forwards, windows, the loop."""
    import random

    r = random.Random(seed)
    width = r.choice([24, 40, 56, 64, 96])

    def mlp():
        kind = r.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return dense(r.choice([16, 40, 100]))
        experts = r.choice([2, 3, 6, 9])
        return moe(experts, r.randint(1, min(experts, 3)), r.choice([8, 20, 36]), r.choice([0.5, 1.0, 1.5]),
                   shared=r.choice([None, 12, 24]))

    layers = []
    for _ in range(r.randint(2, 5)):
        if r.random() < 0.5:
            layers.append(gla(r.choice([1, 2, 3]), r.choice([4, 12, 16, 40, 72]), r.choice([4, 8, 20, 70]),
                              r.choice([1.0, 4.0, 12.0]), r.choice([1, 2, 6]), mlp=mlp()))
        else:
            kv = r.choice([1, 2, 3])
            left = (kv * r.choice([1, 2, 4]), kv, r.choice([8, 12, 32, 48]), r.choice([4, 8, 24]),
                    r.choice([0.2, 0.5]), r.choice([None, 1, 3, 4, 9, 16, 30]))
            right = (r.choice([1, 2, 3]), r.choice([4, 8, 24, 40]), r.choice([4, 12, 33]), r.choice([3.0, 12.0]))
            layers.append(parallel(left, right, r.choice([0.5, 1.0, 1.3]), r.choice([0.8, 1.0]), mlp=mlp()))
    n = len(layers)
    loop = None
    if r.random() < 0.7:
        start = r.randrange(n)
        loop = (start, r.randint(start + 1, n), r.randint(1, 3))
    return config(r.choice([50, 97, 130]), width, r.choice([1e-6, 1e-5, 1e-3]), layers, loop=loop,
                  bigram=r.choice([None, (17, 5, 11), (101, 1000003, 999983)]), positions=r.choice([None, 64]),
                  side=r.choice([None, 3, 8]), cap=r.choice([None, 5.0, 30.0]))


def write_model(name: str, out_dir: str, dtype=torch.float32, std: float | None = None, norm_std: float | None = None) -> str:
    """Writes the configuration with random weights through the framework's random-weights mode."""
    d, seed, own_std, own_norm_std = CONFIGS[name]
    return write_random_model(config_from_dict(d), out_dir, seed, dtype, std=std or own_std, norm_std=norm_std or own_norm_std)


def plain_weights(model_dir, dtype):
    """The folder's weights as the engine holds them: a bfloat16 run rounds them first."""
    w, cfg = plain.load(model_dir)
    if dtype == "bfloat16":
        w = {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()}
    return w, cfg


def rel_rows(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Every row's error (root mean square over the vocabulary) relative to the logits' root mean square."""
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def assert_engine_close(got: torch.Tensor, want: torch.Tensor, dtype: str, w, cfg, tokens, what=None) -> None:
    """32-bit: every row within 1e-4 of the logits' size, or within a few times the error that the plain implementation
    itself has in 32-bit (some of these tiny models amplify rounding: norms over four values with a tiny eps, products
    of gates).  bfloat16: a model with a few tiny experts takes another expert here and there, which moves that row and,
    through the states, some rows behind it; the typical row and the share of rows that are far off are held, which a
    fault of the logic (a window one token off, a lost state, a wrong slot) does not pass."""
    rows = rel_rows(got, want)
    assert torch.isfinite(got).all(), what
    if dtype == "float32":
        own = rel_rows(plain.forward(w, cfg, tokens, dtype=torch.float32), want)
        assert float(rows.max()) <= max(1e-4, 6.0 * float(own.max())), (what, float(rows.max()), float(own.max()))
    else:
        far = int((rows > 0.2).sum())
        assert float(rows.median()) <= 6e-2 and far <= max(1, len(rows) // 6), (what, float(rows.median()), far, len(rows))


# --------------------------------------------------------------------------- bodies


def cuts_match_plain(tmp_path, device, name, dtype="float32", length=45, page_size=4):
    """Whole prompts, a prompt and then token by token, portions of several sizes down to two tokens, all tokens one by
    one: the same logits.  The first tokens of a sequence are among the wanted places every time."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(length, cfg["vocab"], 7)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size)
    n = length
    for cuts in ([n], [n - 32] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, n - 32], [2] * (n // 2) + [1] * (n % 2), [1] * n):
        got = run_cut(ex, "r", tokens, cuts)
        assert_engine_close(got, want, dtype, w, cfg, tokens, (name, cuts))


def batches_match_alone(tmp_path, device, name, dtype="float32", page_size=4):
    """Requests of unequal length run together, portions beside single tokens, in a pool so tight that pages and state
    slots are given back and used again (freed pages are filled with NaN; a state slot keeps what its last owner
    left until the next admission): each request's logits are those of the request alone."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    V = cfg["vocab"]
    lengths = {"a": 37, "b": 9, "c": 1, "d": 22, "e": 30, "f": 2, "g": 17}
    toks = {r: random_tokens(n, V, 100 + i) for i, (r, n) in enumerate(lengths.items())}
    want = {r: plain.forward(w, cfg, t) for r, t in toks.items()}
    ex = make_executor(d, device, dtype, page_size=page_size, num_pages=26 if page_size == 4 else 8, batch=3, max_len=48,
                       poison=True)
    schedule = [
        [("a", 11), ("b", 3), ("c", 1)],          # c ends: its slot goes to d
        [("a", 2), ("b", 1), ("d", 5)],
        [("a", 1), ("b", 5), ("d", 1)],           # b ends
        [("a", 16), ("d", 2), ("e", 7)],
        [("a", 1), ("d", 1), ("e", 2)],
        [("d", 13), ("e", 1), ("a", 6)],          # a and d end
        [("e", 20), ("f", 2), ("g", 1)],          # e and f end
        [("g", 2)], [("g", 14)],
    ]
    done = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    for step in schedule:
        entries = []
        for r, n in step:
            if not ex.has_request(r):
                ex.add_request(r)
            entries.append(StepEntry(r, toks[r][done[r]:done[r] + n], list(range(n))))
        logits = ex.step(entries).cpu()
        at = 0
        for r, n in step:
            got[r].append(logits[at:at + n])
            at += n
            done[r] += n
            if done[r] == lengths[r]:
                ex.finish_request(r)
        ex.cache.check()
    assert done == lengths
    for r in toks:
        assert_engine_close(torch.cat(got[r]), want[r], dtype, w, cfg, toks[r], (name, r))


def drawn_configuration_runs(tmp_path, device, seed: int, dtype="float32"):
    """A drawn configuration, three requests of unequal length in portions beside single tokens, in a tight pool."""
    d = write_random_model(config_from_dict(drawn_config(seed)), str(tmp_path / f"m{seed}"), seed, torch.float32, std=0.3,
                           norm_std=0.4)
    w, cfg = plain_weights(d, dtype)
    toks = {r: random_tokens(n, cfg["vocab"], seed * 10 + i) for i, (r, n) in enumerate((("a", 41), ("b", 13), ("c", 26)))}
    want = {r: plain.forward(w, cfg, t) for r, t in toks.items()}
    ex = make_executor(d, device, dtype, page_size=4, num_pages=24, batch=2, max_len=44, poison=True)
    schedule = [[("a", 9), ("b", 2)], [("a", 1), ("b", 7)], [("a", 17), ("b", 1)], [("a", 2), ("b", 3)],   # b ends
                [("a", 1), ("c", 20)], [("a", 11), ("c", 1)], [("c", 2)], [("c", 3)]]
    done = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    for step in schedule:
        entries = []
        for r, n in step:
            if not ex.has_request(r):
                ex.add_request(r)
            entries.append(StepEntry(r, toks[r][done[r]:done[r] + n], list(range(n))))
        logits = ex.step(entries).cpu()
        at = 0
        for r, n in step:
            got[r].append(logits[at:at + n])
            at += n
            done[r] += n
            if done[r] == len(toks[r]):
                ex.finish_request(r)
        ex.cache.check()
    for r in toks:
        assert done[r] == len(toks[r])
        if len(toks[r]) >= 20 or dtype == "float32":   # (the typical row of a dozen is no measure)
            assert_engine_close(torch.cat(got[r]), want[r], dtype, w, cfg, toks[r], (seed, r))


def long_decoding(tmp_path, device, name, dtype="float32", prompt=5, steps=150, page_size=16):
    """A short prompt, then many tokens one by one: states and caches are carried over page borders and past every
    window."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(prompt + steps, cfg["vocab"], 21)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size, num_pages=-(-(prompt + steps) // page_size) + 1)
    got = run_cut(ex, "r", tokens, [prompt] + [1] * steps)
    assert_engine_close(got, want, dtype, w, cfg, tokens)


def layers_match_plain(tmp_path, device, name="mixed", dtype="float32"):
    """The residual stream behind every layer run (a looped layer counts each time) against the plain implementation's."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(23, cfg["vocab"], 5)
    want: list = []
    plain.forward(w, cfg, tokens, layers_out=want)
    ex = make_executor(d, device, dtype)
    ex.add_request("r")
    T, R, ctx, rows, wants, _ = ex._prepare([StepEntry("r", tokens, [len(tokens) - 1])])
    got: list = []
    ex.model.forward(ex._dev[:T], ctx, ex.cache.views, rows, after_layer=lambda i, h: got.append(h.double().cpu().clone()))
    assert len(got) == len(want) == len(ex.model.spec.schedule)
    for i, (g, x) in enumerate(zip(got, want)):
        err = float((g - x).abs().max() / x.abs().max())
        assert err < (1e-4 if dtype == "float32" else 1e-1), (i, err)


def greedy_generation(tmp_path, device, name="mixed", dtype="float32"):
    """Greedy generation through the framework's own entry point and scheduler: the plain implementation's tokens."""
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    d = write_model(name, str(tmp_path / name), std=0.4)
    w, cfg = plain.load(d)
    prompts = [random_tokens(n, cfg["vocab"], 50 + n) for n in (5, 11, 17, 3)]
    want = [plain.greedy(w, cfg, p, 6) for p in prompts]
    lm = LMInterface(d, activation_dtype=dtype, batch_size=3, max_seq_len=64, page_size=4, max_num_issue_tokens=16,
                     device=str(device))
    outs = lm.generate(prompts, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=6))
    assert [o.output_token_ids for o in outs] == want
