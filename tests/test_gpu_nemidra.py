"""Nemidra on the GPU: every new kernel against its plain torch reference, every mechanism as a part of the framework
against the plain implementation's function (whole and in portions, keys at the edges of windows and pages), and the
engine (whole prompts, token-by-token decoding, portions down to two tokens, unequal requests together in a tight pool,
long decoding, recorded decode steps, greedy generation through the scheduler, trace replay as a child process) against
the plain implementation, in 32-bit and in bfloat16."""
import pytest
import torch

import nemidra_cases as cases
import nemidra_kernels as kern
import nemidra_mechanisms as mech
import plain_nemidra as plain
from simply_amd.engine import StepEntry
from simply_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("body", [kern.token_tables, kern.matrix_states, kern.routed])
def test_kernel(body, dtype):
    body(ops, DEV, dtype)


def test_gates_in_portions():
    kern.long_gate_scan(ops, DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("body", [mech.gla_part, mech.memory_part, mech.window_edges, mech.far_key_without_window,
                                  mech.parallel_part, mech.routed_experts_part, mech.dense_part, mech.embedding_part,
                                  mech.token_side_part])
def test_part(body, dtype):
    body(DEV, dtype)


def test_window_edges_on_the_matrix_cores():
    """Heads of 64 with values of the same size in pages of 16 keys: the bfloat16 attention kernels on the matrix cores."""
    mech.window_edges(DEV, torch.bfloat16, window=24, page_size=16, heads=4, kv_heads=2, dim=64, vdim=64, width=64, T=70)
    mech.window_edges(DEV, torch.bfloat16, window=16, page_size=16, heads=8, kv_heads=1, dim=128, vdim=128, width=64, T=70)


#: (in bfloat16 the model with top-1 routing among four tiny experts, looped three times, takes another expert now and
#: then and is left to the 32-bit runs, where the bound is tight)
RUNS = [(n, "float32") for n in ("mixed", "units", "loop_from_start", "aligned")] + \
       [(n, "bfloat16") for n in ("units", "loop_from_start", "aligned")]


@pytest.mark.parametrize("name, dtype", RUNS)
def test_cuts_match_plain(tmp_path, name, dtype):
    cases.cuts_match_plain(tmp_path, DEV, name, dtype)


@pytest.mark.parametrize("name, dtype", RUNS)
def test_batches_match_alone(tmp_path, name, dtype):
    cases.batches_match_alone(tmp_path, DEV, name, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_and_pages_of_sixteen(tmp_path, dtype):
    cases.cuts_match_plain(tmp_path, DEV, "aligned", dtype, length=171, page_size=16)


@pytest.mark.parametrize("seed", range(1, 13))
def test_drawn_configurations(tmp_path, seed):
    cases.drawn_configuration_runs(tmp_path, DEV, seed)


@pytest.mark.parametrize("seed", [1, 5, 9])
def test_drawn_configurations_bfloat16(tmp_path, seed):
    cases.drawn_configuration_runs(tmp_path, DEV, seed, "bfloat16")


@pytest.mark.parametrize("name, dtype", [("mixed", "float32"), ("aligned", "bfloat16")])
def test_long_decoding(tmp_path, name, dtype):
    cases.long_decoding(tmp_path, DEV, name, dtype, steps=150, page_size=16)


@pytest.mark.parametrize("name, dtype", [("mixed", "float32"), ("aligned", "bfloat16")])
def test_layers_match_plain(tmp_path, name, dtype):
    cases.layers_match_plain(tmp_path, DEV, name, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps(tmp_path, dtype):
    """Decode-only steps are recorded in a HIP graph and replayed: three requests decode together for 40 steps, and
    each step's logits are those of the same step run eagerly by a second engine (states, maxima and the embedding's
    last tokens advance exactly once)."""
    d = cases.write_model("mixed", str(tmp_path / "m"))
    V = plain.load(d)[1]["vocab"]
    prompts = {r: cases.random_tokens(n, V, 70 + n) for r, n in (("a", 9), ("b", 3), ("c", 14))}
    follow = {r: cases.random_tokens(40, V, 90 + len(p)) for r, p in prompts.items()}
    engines = [cases.make_executor(d, DEV, dtype, page_size=4, num_pages=64, batch=4, max_len=64, graphs=g)
               for g in (True, False)]
    for ex in engines:
        for r, p in prompts.items():
            ex.add_request(r)
        ex.step([StepEntry(r, p, []) for r, p in prompts.items()])
    for k in range(40):
        outs = [ex.step([StepEntry(r, [follow[r][k]], [0]) for r in prompts]).clone() for ex in engines]
        torch.testing.assert_close(outs[0], outs[1], rtol=0, atol=0)


def test_greedy_generation(tmp_path):
    cases.greedy_generation(tmp_path, DEV, "mixed", "float32")


def test_greedy_generation_bfloat16_runs(tmp_path):
    """The serving path as it is used: bfloat16, recorded decode steps, several steps in a row on the device."""
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    d = cases.write_model("aligned", str(tmp_path / "m"), dtype=torch.bfloat16)
    lm = LMInterface(d, activation_dtype="bfloat16", batch_size=4, max_seq_len=128, device=DEV)
    prompts = [cases.random_tokens(n, 256, n) for n in (5, 33, 17, 2, 60)]
    outs = lm.generate(prompts, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=24))
    again = lm.generate(prompts, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=24))
    assert all(len(o.output_token_ids) == 24 for o in outs)
    assert [o.output_token_ids for o in outs] == [o.output_token_ids for o in again]


def test_trace_replay_child_process(tmp_path):
    """bin/trace_run as a user starts it: a folder, steps on standard input, logits in files."""
    import json
    import os
    import subprocess

    import numpy as np

    d = cases.write_model("mixed", str(tmp_path / "m"), dtype=torch.bfloat16)
    w, cfg = plain.load(d)
    tokens = cases.random_tokens(30, cfg["vocab"], 5)
    other = cases.random_tokens(12, cfg["vocab"], 6)
    want, want_other = plain.forward(w, cfg, tokens), plain.forward(w, cfg, other)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tokens[17:19], "want": []},
                                     {"id": "y", "tokens": other[:11], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": other[11:], "want": [0]},
                                     {"id": "x", "tokens": tokens[19:], "want": [10]}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, timeout=600)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
    assert float(cases.rel_rows(got0, want[[0, 16]]).max()) <= 1e-4
    assert float(cases.rel_rows(got2[:1], want_other[[11]]).max()) <= 1e-4
    assert float(cases.rel_rows(got2[1:], want[[29]]).max()) <= 1e-4
