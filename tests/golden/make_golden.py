#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run from the repo root).

The reference tree holds no fixtures for its reduction: the arithmetic lives in
ATen (fairring/device.cc:125 calls at::sum_out), and its only known-answer
checks are the all-ones and arange cases of benchmark/benchmark.cc:130-186.
The contract for this build is the sequential at::add chain in contribution
order, so the expected outputs here are produced by the installed PyTorch CPU
library itself (torch.add chain, torch.div, and for bf16 a float32 chain with
one final cast), never by this repository's oracle or kernels.

Inputs include lanes that a careless implementation gets wrong: +-0, all -0,
subnormals, +-inf, inf-inf, NaN, values that cancel, large/small mixes.
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def special_lanes(k, n, rng):
    """Overwrite the first lanes of the [k, n] float32 matrix with edge cases."""
    x = rng.standard_normal((k, n)).astype(np.float32)
    x[:, 0] = 0.0
    x[:, 1] = -0.0                      # all -0: chain keeps -0
    x[:, 2] = 0.0
    x[0, 2] = -0.0
    x[:, 3] = np.float32(1e-45)          # smallest subnormal
    x[:, 4] = np.float32(1.1754942e-38)  # largest subnormal
    x[:, 5] = np.float32(3.0e38)         # overflows to +inf part-way
    x[:, 6] = np.inf
    x[:, 7] = np.inf
    x[k - 1, 7] = -np.inf                # inf - inf = NaN at the end
    x[:, 8] = 1.0
    x[k // 2, 8] = np.nan
    x[:, 9] = np.float32(1e8)
    x[1::2, 9] = np.float32(-1e8)        # exact cancellation pairs
    x[:, 10] = np.float32(16777216.0)    # 2^24: +1 is lost, order matters
    x[1:, 10] = 1.0
    x[:, 11] = 1.0
    x[k - 1, 11] = np.float32(16777216.0)
    x[:, 12] = np.float32(1.0) + np.float32(2.0 ** -23)  # ties in rounding
    x[:, 13] = np.float32(-3.4028235e38)
    return x


def torch_chain_f32(x, scale_mode):
    t = torch.from_numpy(x)
    acc = t[0].clone()
    for k in range(1, t.shape[0]):
        acc = torch.add(acc, t[k])
    if scale_mode == "mul":
        acc = acc * (1.0 / t.shape[0])
    elif scale_mode == "div":
        acc = torch.div(acc, float(t.shape[0]))
    return acc.numpy()


def torch_chain_bf16(bits, scale_mode):
    t = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    acc = t[0].to(torch.float32)
    for k in range(1, t.shape[0]):
        acc = torch.add(acc, t[k].to(torch.float32))
    if scale_mode == "mul":
        acc = acc * (1.0 / t.shape[0])
    elif scale_mode == "div":
        acc = torch.div(acc, float(t.shape[0]))
    return acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def to_bf16_bits(x):
    t = torch.from_numpy(x).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def main():
    torch.set_num_threads(1)
    out = {}
    for name, k, n, seed, sigma in (
        ("f32_k2", 2, 1031, 11, 1.0),
        ("f32_k3", 3, 517, 12, 1.0),
        ("f32_k8", 8, 4099, 13, 0.01),
        ("f32_k17", 17, 257, 14, 1.0),
        ("f32_k64", 64, 1031, 15, 0.01),
    ):
        rng = np.random.default_rng(seed)
        x = special_lanes(k, n, rng)
        x[:, 16:] *= np.float32(sigma)
        out[name + "_in"] = x
        out[name + "_sum"] = torch_chain_f32(x, None)
        out[name + "_mul"] = torch_chain_f32(x, "mul")
        out[name + "_div"] = torch_chain_f32(x, "div")
    for name, k, n, seed, sigma in (
        ("bf16_k2", 2, 1031, 21, 1.0),
        ("bf16_k8", 8, 4099, 22, 0.01),
        ("bf16_k64", 64, 523, 23, 0.01),
    ):
        rng = np.random.default_rng(seed)
        x = special_lanes(k, n, rng)
        x[:, 16:] *= np.float32(sigma)
        bits = to_bf16_bits(x)
        out[name + "_in"] = bits
        out[name + "_sum"] = torch_chain_bf16(bits, None)
        out[name + "_mul"] = torch_chain_bf16(bits, "mul")
        out[name + "_div"] = torch_chain_bf16(bits, "div")
    np.savez_compressed(os.path.join(HERE, "ksum_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "ksum_golden.npz"),
          {k: v.shape for k, v in out.items() if k.endswith("_in")})


if __name__ == "__main__":
    main()
