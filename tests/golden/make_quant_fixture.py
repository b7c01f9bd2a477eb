"""Writes tests/golden/quant_compiled_fixture.npz: the activation quantizer
expression of the reference (gpu/model.py:69-71), typed out below, evaluated
by torch.compile (Inductor, CPU backend of the installed torch) and by torch
eager on seeded bf16 rows.  No reference file is imported.

    python tests/golden/make_quant_fixture.py
"""
import os

import numpy as np
import torch


def quant_input(input):
    s = 127 / input.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
    return (input * s).round().clamp(-128, 127).to(torch.int8), s


def bf16_bits(x32: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(np.ascontiguousarray(x32, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def main():
    rng = np.random.Generator(np.random.Philox(2024))
    rows = []
    for K in (256, 2560):
        x = rng.standard_normal((12, K), dtype=np.float32)
        x[1] *= 1e-7  # below the 1e-5 clamp
        x[2] *= 300.0
        x[3, ::7] *= 20.0  # outliers
        x[4] = 0.0
        x[5] *= 1e-3
        x[6, 0] = 3.0e38  # near the top of the bf16 range
        rows.append((K, bf16_bits(x)))
    out = {}
    compiled = torch.compile(quant_input)
    for K, xb in rows:
        xt = torch.from_numpy(xb.view(np.int16).copy()).view(torch.bfloat16)
        for tag, fn in (("compiled", compiled), ("eager", quant_input)):
            q, s = fn(xt.clone())
            assert q.dtype == torch.int8 and s.dtype == torch.bfloat16
            out[f"q_{tag}_{K}"] = q.numpy().copy()
            out[f"s_{tag}_{K}"] = s.reshape(-1).view(torch.int16).numpy().view(np.uint16).copy()
        out[f"x_{K}"] = xb
    out["torch_version"] = np.array(torch.__version__)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_compiled_fixture.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
