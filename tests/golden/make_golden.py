"""Writes tests/golden/lstm_golden.npz: small seeded LSTM problems with the
expected outputs and gradients computed by torch.nn.LSTM in float64 on the CPU
(a library routine; the reference's own tests hold no golden files and compare
with nn.LSTM live, tests/test_lstm.py:160-220 of the reference).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from helpers import make_problem, nn_lstm_reference  # noqa: E402

CASES = {  # name: (T, B, I, H, h0)
    "tiny": (3, 2, 3, 4, True),
    "ragged": (10, 5, 7, 65, True),   # H = 65 as in the reference's test grid
    "nostate": (6, 3, 9, 16, False),
    "onestep": (1, 4, 5, 8, True),
}


def main():
    blob = {}
    for name, (T, B, I, H, h0) in CASES.items():
        p = make_problem(T, B, I, H, seed=100 + len(blob), h0=h0)
        r = nn_lstm_reference(p, with_state_grads=True)
        for k, v in p.items():
            if v is not None:
                blob["%s/in/%s" % (name, k)] = v.numpy().astype(np.float32)
        # inputs are stored in fp32: recompute the expectation from the rounded inputs
        p32 = {k: (v.float().double() if v is not None else None) for k, v in p.items()}
        r = nn_lstm_reference(p32, with_state_grads=True)
        for k, v in r.items():
            if v is not None:
                blob["%s/out/%s" % (name, k)] = v.numpy()
    np.savez_compressed(os.path.join(HERE, "lstm_golden.npz"), **blob)
    print("wrote", len(blob), "arrays")


if __name__ == "__main__":
    main()
