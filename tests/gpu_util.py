"""Helpers shared by the GPU parity tests (which call the library through its C ABI)."""
import sys

import numpy as np
import torch

import oracle as O


def say(*a):
    """Name the case before it runs, so that a fault can be traced to it."""
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def act_np(t):
    """16-bit activation tensor -> float32 numpy."""
    return t.detach().float().cpu().numpy()


def u16(t):
    return t.detach().cpu().numpy().view(np.uint16)


def u32(t):
    return t.detach().cpu().numpy().view(np.uint32)


def round_act(a, act):
    """Round float32 values through the activation type (0 = bf16, 1 = fp16)."""
    return O.round_bf16(a) if act == 0 else O.f16_to_float(O.f16_bits(a))


def act_tensor(a, ctx):
    return dev(np.asarray(a, np.float32)).to(ctx.dtype)


def gauss(rng, shape, std=1.0):
    return (rng.standard_normal(shape) * std).astype(np.float32)
