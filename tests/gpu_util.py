"""Helpers shared by the GPU parity tests: seeded synthetic inputs as BASELINE.json describes them."""
import numpy as np
import torch

DEV = "cuda:0"


def draw_kv(gen, B, H, S, D=128, dtype=torch.bfloat16):
    k = torch.randn(B, H, S, D, generator=gen).to(dtype)
    v = torch.randn(B, H, S, D, generator=gen).to(dtype)
    return k, v


def draw_log_beta(gen, B, H, S, mu=3.0, sigma=1.0, dtype=torch.float32):
    z = torch.randn(B, H, S, generator=gen) * sigma + mu
    return torch.nn.functional.logsigmoid(z).to(dtype)


def boundary_ties(log_beta, positions, q_idx, keep):
    """Rows whose keep-th and (keep+1)-th scores are equal: parity on those rows is undefined."""
    sc = log_beta.to(torch.float32) * (q_idx - positions)
    top = torch.topk(sc, keep + 1, dim=-1).values
    return top[..., keep - 1] == top[..., keep]


def attn_close(got, want, atol=2e-2, rtol=1e-2):
    """The north-star tolerance: max-abs 2e-2 and relative 1e-2 against the fp32 reference."""
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    err = (got - want).abs()
    ok = bool((err <= atol + rtol * want.abs()).all())
    return ok, float(err.max())
