"""Writes tests/golden/config1_retained_positions.npz.

The reference ships no tests, fixtures or golden vectors, and it was not imported to make these:
they are produced by the CPU oracle (oracle/dense_ref.py), which tests/test_oracle_dense.py pins
against numpy brute force and closed forms.  The fixture freezes BASELINE config 1 -- one layer,
B=1, 8 KV heads, M=512, buffer 128, 1024-token prefill, 4096 decode steps, log beta =
logsigmoid(N(3,1)) fp32 from torch.Generator(seed=1) in the order tests/gpu_util.py draws it --
so that later changes to the oracle or to the HIP path are caught against committed data.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.dense_ref import DenseCacheRef  # noqa: E402

SEED, B, H, M, BUF, PREFILL, STEPS = 1, 1, 8, 512, 128, 1024, 4096


def log_beta_stream(gen, s):
    """The draws of tests/gpu_util.py for one append: K, V (discarded here) and log beta."""
    torch.randn(B, H, s, 128, generator=gen)
    torch.randn(B, H, s, 128, generator=gen)
    z = torch.randn(B, H, s, generator=gen) * 1.0 + 3.0
    return torch.nn.functional.logsigmoid(z)


def run():
    gen = torch.Generator().manual_seed(SEED)
    ref = DenseCacheRef()
    snaps = []
    zeros = lambda s: torch.zeros(B, H, s, 1)
    T = 0
    for step, s in enumerate([PREFILL] + [1] * STEPS):
        lb = log_beta_stream(gen, s)
        ref.update(zeros(s), zeros(s), lb, torch.arange(T, T + s), 0)
        T += s
        if s == 1 and (step - 1) % 16 == 0:
            torch.randn(B, H * 2, 1, 128, generator=gen)  # the query the parity test draws on attended steps
        before = ref.get_cache_length(0)
        ref.compress("alpha", M, BUF)
        if ref.get_cache_length(0) != before:
            snaps.append(ref.kv_positions[0][0].numpy().astype(np.uint16))
    return np.stack(snaps)


if __name__ == "__main__":
    pos = run()
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_retained_positions.npz")
    np.savez_compressed(out, positions=pos, meta=np.array([SEED, B, H, M, BUF, PREFILL, STEPS]))
    print(out, pos.shape, os.path.getsize(out), "bytes")
