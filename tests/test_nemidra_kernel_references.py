"""The plain torch references of Nemidra's kernels agree with themselves where a kernel test relies on them: a state
carried through portions equals the state of the whole run (CPU)."""
import torch

import nemidra_kernels as kern
import torch_ops as ref


def test_references_run_on_the_cpu():
    kern.token_tables(ref, "cpu", torch.float32)
    kern.matrix_states(ref, "cpu", torch.float32, sizes=((2, 8, 6), (1, 4, 1)))
    kern.long_gate_scan(ref, "cpu")
    kern.routed(ref, "cpu", torch.float32, sizes=((9, 3, 1, 36, 20), (37, 6, 3, 24, 16)))
