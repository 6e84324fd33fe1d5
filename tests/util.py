"""Shared helpers of the GPU parity tests: seeded host data, bit-pattern views, announce-before-launch."""
import sys

import numpy as np
import torch

import oracle

TORCH_DT = {oracle.F16: torch.float16, oracle.BF16: torch.bfloat16}


def announce(msg):
    """Name the case before the GPU step, flushed, so a fault can be attributed."""
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def to_dev(bits, dtype):
    """uint16 bit patterns (numpy) -> GPU tensor of the 16-bit float type with the same bits."""
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda()
    return t.view(TORCH_DT[dtype])


def bits_of(t):
    """GPU/CPU tensor of a 16-bit float type -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def f32_of(t):
    return t.detach().float().cpu().numpy()


def randn_bits(rng, shape, dtype, scale=1.0):
    return oracle.to_bits(rng.standard_normal(shape) * scale, dtype)
