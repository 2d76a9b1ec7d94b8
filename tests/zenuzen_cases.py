"""Small Zenuzen configurations, model folders with random weights, and the bodies of the tests that run the
framework against the plain implementation (tests/plain_zenuzen.py).  A body takes the device; the CPU tests run
it with the kernels replaced by their plain torch references (the `cpu_ops` fixture), the GPU tests with the
kernels themselves.  Nothing here is read from outside the repository."""
from __future__ import annotations

import torch

import plain_zenuzen as plain
from simply_amd.cache import CacheManager
from simply_amd.config import EngineConfig, config_from_dict
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.context import GroupStep, StepContext
from simply_amd.engine.loading import load_model
from simply_amd.weights import write_random_model


def attention(heads, kv_heads, dim, vdim, scale, rot=None, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def delta(heads, kv_heads, dim, vdim, conv, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def config(vocab, width, mult, eps, layers):
    return {"architecture": "Zenuzen", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps},
            "layers": layers}


#: odd sizes everywhere: an attention layer first (the source of mixed values), a delta layer with a feed-forward,
#: as many q/k heads as value heads, one head, a convolution of two taps and of six, rotation of all dimensions and
#: of none, a key size above 32 and a value size above 64 (two column blocks of the state)
MIXED = config(97, 48, 0.55, 1e-6, [
    attention(4, 1, 24, 40, 0.4, rot=(8, 500.0), v_mix=True),
    delta(3, 3, 20, 24, 3, mlp=56),
    attention(2, 1, 12, 40, 0.7, v_mix=True, mlp=72),
    delta(4, 2, 36, 72, 6),
    attention(2, 2, 16, 16, 0.3, rot=(16, 10000.0)),
    delta(1, 1, 8, 8, 2),
])
#: only delta layers, and a single tap (no convolution state at all) in one of them
ONLY_DELTA = config(61, 32, 1.0, 1e-5, [delta(2, 1, 16, 16, 1, mlp=40), delta(2, 2, 12, 20, 4)])
#: only attention layers; one layer mixes values and is alone in that (it is the source and nobody reads it)
ONLY_ATTENTION = config(70, 40, 0.8, 1e-5, [
    attention(4, 4, 10, 6, 0.5, rot=(4, 100.0), mlp=30),
    attention(6, 2, 8, 12, 0.35, v_mix=True),
    attention(3, 1, 14, 4, 0.6, rot=(14, 1000.0)),
])
#: sizes in multiples of 32 and 64 (what fast kernels may take), still small
ALIGNED = config(256, 128, 0.7, 1e-5, [
    delta(4, 2, 64, 64, 4),
    attention(4, 2, 64, 64, 0.125, rot=(32, 1000000.0), v_mix=True, mlp=256),
    delta(2, 1, 128, 128, 4, mlp=128),
    attention(8, 2, 64, 64, 0.125, rot=(64, 10000.0), v_mix=True),
])
CONFIGS = {"mixed": (MIXED, 11), "only_delta": (ONLY_DELTA, 12), "only_attention": (ONLY_ATTENTION, 13),
           "aligned": (ALIGNED, 14)}


def drawn_config(seed: int) -> dict:
    """A configuration drawn at random: sizes, head counts, the order of the layers, which layers have a
    feed-forward, which mix values, how much of a head is rotated, taps, multiplier and eps."""
    import random

    r = random.Random(seed)
    width = r.choice([24, 40, 56, 64, 96])
    layers = []
    mix_shape = (r.choice([1, 2]), r.choice([8, 12, 20, 32]))      # layers that mix values agree in these
    for _ in range(r.randint(2, 6)):
        mlp = r.choice([None, None, r.choice([32, 48, 100])])
        if r.random() < 0.45:
            v_mix = r.random() < 0.6
            kv, vdim = mix_shape if v_mix else (r.choice([1, 2, 3]), r.choice([4, 8, 16, 24]))
            dim = r.choice([8, 12, 16, 32, 48])
            rot = r.choice([None, (r.choice([2, 4, dim]), r.choice([100.0, 10000.0, 1e6]))])
            layers.append(attention(kv * r.choice([1, 2, 3, 4]), kv, dim, vdim, r.choice([0.2, 0.5, dim ** -0.5]), rot=rot,
                                    v_mix=v_mix, mlp=mlp))
        else:
            g = r.choice([1, 2, 3])
            layers.append(delta(g * r.choice([1, 2, 4]), g, r.choice([4, 8, 16, 24, 40, 72]), r.choice([4, 8, 20, 70]),
                                r.choice([1, 2, 3, 4, 5, 8]), mlp=mlp))
    return config(r.choice([50, 97, 130, 300]), width, r.choice([0.3, 0.7, 1.0, 1.4]), r.choice([1e-6, 1e-5, 1e-3]), layers)


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
        assert_close_logits(torch.cat(got[r]), want[r], dtype, (seed, r))


def write_model(name: str, out_dir: str, dtype=torch.float32, std: float = 0.25, norm_std: float = 0.5) -> str:
    """Writes the configuration with random weights through the framework's random-weights mode.  Norm weights,
    sinks, decays and the mixing factor are drawn around 0 with norm_std."""
    d, seed = CONFIGS[name]
    return write_random_model(config_from_dict(d), out_dir, seed, dtype, std=std, norm_std=norm_std)


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def make_executor(model_dir, device, dtype="float32", page_size=4, num_pages=64, batch=4, max_len=256, poison=False,
                  graphs=False):
    edtype = EngineConfig(activation_dtype=dtype).dtype
    model, _ = load_model(model_dir, edtype, torch.device(device))
    cfg = EngineConfig(activation_dtype=dtype, page_size=page_size, batch_size=batch, max_seq_len=max_len,
                       max_num_issue_tokens=max_len, total_num_pages=num_pages, device=str(device), use_graphs=graphs,
                       poison_freed_pages=poison)
    return Executor(model, cfg)


def run_cut(ex, rid, tokens, cuts):
    """Feeds `tokens` in portions of the given sizes, wanting every position; returns [T, V] on the CPU."""
    out, i = [], 0
    ex.add_request(rid)
    for c in cuts:
        part = tokens[i:i + c]
        out.append(ex.step([StepEntry(rid, part, list(range(len(part))))]).cpu())
        i += len(part)
    assert i == len(tokens)
    ex.finish_request(rid)
    ex.cache.check()
    return torch.cat(out)


def rel_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest row error (root mean square over the vocabulary) relative to the logits' own root mean square."""
    got, want = got.double().cpu(), want.double().cpu()
    return float(((got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()).max())


#: bounds on rel_error: the 32-bit path is exact up to rounding.  A bfloat16 run rounds products and activations to
#: 8 bits of mantissa, layer after layer; these tiny models with their sharp softmax and norms over a handful of
#: values amplify that at single positions (the kernels' plain torch references, run on the CPU with the same
#: roundings, are 0.1 to 0.5 off at the worst position of the same sequences, the same position as the kernels, and
#: 0.01 to 0.026 on average), so a bfloat16 run is held to a bound on the average over the positions, and no more than
#: one position in twenty may be further off than BOUND.  Faults of the logic show in 32-bit, where the bound is tight.
BOUND = {"float32": 1e-4, "bfloat16": 2e-1}
MEAN_BOUND = {"float32": 1e-4, "bfloat16": 4e-2}


def assert_close_logits(got: torch.Tensor, want: torch.Tensor, dtype: str, what=None) -> None:
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    rows = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    over = int((rows > BOUND[dtype]).sum())
    allowed = 0 if dtype == "float32" else max(1, len(rows) // 20)
    assert over <= allowed and float(rows.mean()) <= MEAN_BOUND[dtype], (what, over, float(rows.max()), float(rows.mean()))


def plain_weights(model_dir, dtype):
    """The folder's weights as the engine holds them: a bfloat16 run rounds them first."""
    w, cfg = plain.load(model_dir)
    if dtype == "bfloat16":
        w = {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()}
    return w, cfg


# --------------------------------------------------------------------------- bodies


def cuts_match_plain(tmp_path, device, name, dtype="float32", length=45, page_size=4):
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(length, cfg["vocab"], 7)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size)
    n = length
    for cuts in ([n], [n - 32] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, n - 32], [2] * (n // 2) + [1] * (n % 2), [1] * n):
        got = run_cut(ex, "r", tokens, cuts)
        assert_close_logits(got, want, dtype, (name, cuts))


def batches_match_alone(tmp_path, device, name, dtype="float32", page_size=4):
    """Requests of unequal length run together, portions beside single tokens, in a pool so tight that pages and
    state slots are given back and used again (freed pages are filled with NaN): each request's logits are those of
    the request alone."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    V = cfg["vocab"]
    lengths = {"a": 37, "b": 9, "c": 1, "d": 22, "e": 30, "f": 2, "g": 17}
    toks = {r: random_tokens(n, V, 100 + i) for i, (r, n) in enumerate(lengths.items())}
    want = {r: plain.forward(w, cfg, t) for r, t in toks.items()}
    # at most three live at a time: 3 slots, and pages for 37 + 30 + 22 tokens rounded up
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
        g = torch.cat(got[r])
        assert_close_logits(g, want[r], dtype, (name, r))


def long_decoding(tmp_path, device, name, dtype="float32", prompt=5, steps=150, page_size=16):
    """A short prompt, then many tokens one by one: the state and the cache are carried over page borders."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(prompt + steps, cfg["vocab"], 21)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size, num_pages=-(-(prompt + steps) // page_size) + 1)
    got = run_cut(ex, "r", tokens, [prompt] + [1] * steps)
    assert_close_logits(got, want, dtype)


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


# --------------------------------------------------------------------------- one mixer with a cache of its own


def one_request_ctx(T, start, dtype, device, cache, rid="r"):
    """The step context of one request that brings T tokens from position `start` (its pages reserved here)."""
    cache.reserve(rid, start, T)
    tables = cache.sync_tables()
    slot = cache.slot_of(rid)
    groups = {g.group_id: GroupStep(tables[g.group_id],
                                    torch.from_numpy(cache.slot_mapping(g.group_id, rid, start, T)).to(device))
              for g in cache.groups}
    return StepContext(dtype=dtype, num_tokens=T,
                       positions=torch.arange(start, start + T, dtype=torch.int32, device=device),
                       token_seq=torch.full((T,), slot, dtype=torch.int32, device=device),
                       seq_meta=torch.tensor([[slot, 0, T, start]], dtype=torch.int32, device=device), groups=groups,
                       request_ids=[rid], seq_slots=[slot], seq_starts=[start], q_lens=[T], cu_q_lens=[0, T])


def mixer_cache(mixer, dtype, device, page_size=16, num_pages=64):
    cache = CacheManager([(mixer.cache_need(), None)], page_size=page_size, num_pages=num_pages, num_slots=2,
                         max_seq_len=num_pages * page_size, dtype=dtype, device=torch.device(device))
    cache.admit("r")
    return cache


def run_mixer(mixer, x, cuts, dtype, device, page_size=16):
    """x [T, D] through the mixer in portions; returns [T, D] float64 on the CPU."""
    cache = mixer_cache(mixer, dtype, device, page_size, num_pages=-(-x.shape[0] // page_size) + 2)
    out, at = [], 0
    for c in cuts:
        ctx = one_request_ctx(c, at, dtype, device, cache)
        out.append(mixer.forward(x[at:at + c].contiguous(), ctx, cache.views[0]).double().cpu())
        cache.mark_issued([("r", at, c)])
        at += c
    return torch.cat(out)
