"""The size grids of the reference's own tests, run against the oracle under this repository's tolerances.

The reference tests its native backends against ``vanilla`` on these grids with unseeded inputs and tolerances
of 0.1-0.4 (flashrnn/tests/test_lstm.py:9-46, test_gru.py, test_elman.py, test_slstm.py:9-37; ``model_test``,
flashrnn/tests/utils.py:257-340), compares the gradients of h only and leaves out those of the initial state.
Here the same shapes run seeded, both backends, all three storage types, every state and every gradient, at the
tolerances of tests/parity.py.  Every shape of the grids has a kernel on both backends."""
from itertools import product

import pytest
import torch

from parity import check_case

pytestmark = pytest.mark.gpu

# (batch sizes, head dims, sequence lengths, head counts): test_lstm.py:9-31
GRID_A = ([2, 8, 16, 64], [32, 64, 512, 1024], [1, 3], [1, 2, 4])
GRID_B = ([2, 8, 16, 64], [32, 64], [1, 3], [16, 64, 128])
EXTRA = {"lstm": [(2, 32, 1, 64)], "gru": [(2, 32, 1, 64)], "elman": [(2, 32, 1, 64)], "slstm": [(1, 32, 1, 1)]}


def combos(function):
    return list(product(*GRID_A)) + list(product(*GRID_B)) + EXTRA[function]


@pytest.mark.parametrize("backend", ["hip_fused", "hip"])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("function", ["lstm", "gru", "elman", "slstm"])
def test_reference_size_grid(gpu, function, dtype, backend):
    for i, (B, D, T, N) in enumerate(combos(function)):
        # bf16, the type the benchmark configurations use: every shape with all its gradients, as the reference's own
        # grid (flashrnn/tests/utils.py:257-340); the other two storage types: every third shape, the rest forward only
        backward = dtype == "bfloat16" or i % 3 == 0
        print(f"case grid {function} {dtype} {backend} B{B} D{D} T{T} N{N} bwd={backward}", flush=True)
        # every shape of the grid has a kernel on both backends (fp32 heads of 1024 units of the gated cells: groups of 64
        # workgroups that span the device)
        check_case(gpu, function, B, T, N, D, dtype, backend, seed=100 + i, init="zeros", backward=backward)


@pytest.mark.parametrize("dtype,B", [("bfloat16", 8), ("bfloat16", 64), ("float16", 32), ("float32", 8)])
def test_reference_long_sequence_grid(gpu, dtype, B):
    """test_lstm.py:33-39: LSTM, D = 512, T = 1024, one head, both backends."""
    for backend in ("hip_fused", "hip"):
        print(f"case long grid lstm {dtype} {backend} B{B}", flush=True)
        check_case(gpu, "lstm", B, 1024, 1, 512, dtype, backend, seed=200 + B, init="zeros")
