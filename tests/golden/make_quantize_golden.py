"""Writes tests/golden/quantize_reference.npz: input/output vectors of the reference's own
quantisers (/root/reference/quantize.py:16-67), produced by importing that module in the
container that holds the reference checkout (it needs nothing but torch).  The closed-form
invariants in tests/test_oracle_quant.py do not fix the rounding of the scale and of the
scaled values; these vectors do.

Cases, all with dtype=torch.float8_e4m3fn (FP8 max 448, the format of the gfx950 MFMA):
  rowwise_f32 / block_f32    fp32 source: every step of quantize.py is fp32 arithmetic
  rowwise_bf16 / block_bf16  bf16 source: quantize.py then computes the scale and the scaled
                             values in bf16 (quantize.py:56-63), which the kernels do not
                             mirror; kept to document that difference
Outputs are stored as quantize.py returns them (row-major fp8 bytes [rows, K], inverse scales
[rows, K/128] or [rows/128, K/128]); the test applies the layout transposes.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, "/root/reference")
import quantize as refq  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20240607)
    rows, k = 256, 256
    x = torch.randn((rows, k), generator=g) * torch.exp(torch.randn((rows, 1), generator=g) * 2.0)
    x[5, 128:256] = 0.0                      # an all-zero 1 x 128 group
    x[128:256, 128:256] = 0.0                # an all-zero 128 x 128 block
    x[17, 0:128] = 3.0                       # every element at the group maximum
    out = {"x_f32": x.numpy()}
    for tag, src in (("f32", x), ("bf16", x.to(torch.bfloat16))):
        q, s = refq.to_float8_rowwise_scale(src, dtype=torch.float8_e4m3fn)
        out[f"rowwise_{tag}_q"] = q.view(torch.uint8).numpy()
        out[f"rowwise_{tag}_s"] = s.numpy()
        q, s = refq.to_float8_block_scale(src, dtype=torch.float8_e4m3fn)
        out[f"block_{tag}_q"] = q.view(torch.uint8).numpy()
        out[f"block_{tag}_s"] = s.numpy()
    np.savez_compressed(os.path.join(HERE, "quantize_reference.npz"), **out)
    for key, v in out.items():
        print(key, v.shape, v.dtype)


if __name__ == "__main__":
    main()
