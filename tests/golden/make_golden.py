"""Writes tests/golden/recurrence_<function>.npz: inputs and float64 results (all states, all
gradients) of the pinned CPU oracle on one small seeded problem per function.

These vectors are produced by THIS repository's oracle (oracle/flashrnn_oracle.py) after it was
pinned against torch.nn.LSTM/GRU/RNN, the un-stabilised sLSTM recurrence and autograd
(tests/test_oracle_pins.py).  The reference ships no golden vectors for this path, and its Python
code was not imported or run to make these.  They guard the oracle and the kernels against
regressions and travel to the GPU box with the tests.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import flashrnn_oracle_backward, make_inputs  # noqa: E402

CASES = {  # function -> (B, T, N, D, seed, init)
    "lstm": (3, 6, 2, 32, 101, "randn"),
    "gru": (3, 6, 2, 32, 102, "randn"),
    "elman": (3, 6, 2, 32, 103, "randn"),
    "slstm": (3, 6, 2, 32, 104, "zeros"),
}


def main():
    for function, (B, T, N, D, seed, init) in CASES.items():
        inp = make_inputs(function, B, T, N, D, seed, init=init, round_to=torch.bfloat16,
                          grad_on="h" if function == "slstm" else "all")
        kw = {"slstm_per_element_first_step": True} if function == "slstm" else {}
        out, (dWx, dR, db, ds0) = flashrnn_oracle_backward(
            *(inp[k].double() for k in ("Wx", "R", "b", "states")), function, inp["dstates"].double(), **kw)
        np.savez_compressed(
            os.path.join(HERE, f"recurrence_{function}.npz"),
            **{k: v.numpy() for k, v in inp.items()},
            out=out.numpy(), dWx=dWx.numpy(), dR=dR.numpy(), db=db.numpy(), ds0=ds0.numpy())
        print(function, "written")


if __name__ == "__main__":
    main()
