"""Writes the golden fixtures next to this file.

The reference holds no stored vectors for this path (its tests compare the
kernels with an in-process PyTorch oracle on fresh random tensors), and its
package cannot be imported in the build container, so the fixtures are produced
by this repo's oracle restatement: inputs plus the outputs of

  * ``attention_reference`` + autograd in float32   (keys o, lse, dq, dk, dv, db)
  * the float64 explicit-loop restatement            (keys *_f64; tiny case only)

They pin the oracle against drift (torch version, refactors) and give the GPU
tests fixed inputs with known answers.  Run from the repo root:

    python tests/golden/make_golden.py
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from oracle import triangle_oracle as orc  # noqa: E402


def make_case(name, b, h, n, d, seed, p_mask, full_rows=(), std=1.0, with_f64=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, n, n, d, generator=g) * std
    k = torch.randn(b, h, n, n, d, generator=g) * std
    v = torch.randn(b, h, n, n, d, generator=g) * std
    bias = torch.randn(b, h, n, n, generator=g) * std
    mask = torch.rand(b, n, n, generator=g) < p_mask
    for r in full_rows:  # rows whose keys are all masked
        mask[:, r, :] = True
    do = torch.randn(b, h, n, n, d, generator=g)
    o, dq, dk, dv, db = orc.forward_backward(q, k, v, bias, mask, do)
    lse = orc.lse_reference(q, k, bias, mask)
    out = dict(q=q, k=k, v=v, bias=bias, mask=mask, do=do, o=o, lse=lse, dq=dq, dk=dk, dv=dv, db=db)
    out = {key: val.numpy() for key, val in out.items()}
    if with_f64:
        o64, lse64, dq64, dk64, dv64, db64 = orc.brute_force_f64(q, k, v, bias, mask, do)
        out.update(o_f64=o64, lse_f64=lse64, dq_f64=dq64, dk_f64=dk64, dv_f64=dv64, db_f64=db64)
    np.savez_compressed(HERE / f"{name}.npz", **out)
    print(name, {key: val.shape for key, val in out.items() if key in ("q", "bias", "mask")})


if __name__ == "__main__":
    # tiny: also carries the float64 loop-nest answers; row 2 is fully masked
    make_case("tiny_n6_h2_d16", b=2, h=2, n=6, d=16, seed=11, p_mask=0.3, full_rows=(2,), with_f64=True)
    # the CPU-plumbing shape class of the first benchmark config, reduced to n=16
    make_case("plumb_n16_h4_d32", b=1, h=4, n=16, d=32, seed=1337, p_mask=0.1, std=32 ** -0.5)
    # ragged n (not a multiple of any tile), two batches, a fully masked row
    make_case("ragged_n19_h2_d32", b=2, h=2, n=19, d=32, seed=5, p_mask=0.5, full_rows=(7,))
