"""Writes the golden fixtures under tests/golden/ from the CPU oracle of this repository
(oracle/nvfp4_oracle.py; never from the reference's Python files).

    python tests/golden/make_golden.py

Fixtures are inputs + expected outputs as uint8/float arrays in .npz (numpy.load with
allow_pickle=False reads them).  bf16 inputs are stored as their uint16 bit patterns.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from conftest import make_input  # noqa: E402
from oracle import nvfp4_oracle as T  # noqa: E402


def bits(x):
    return x.view(torch.int16).numpy().view(np.uint16)


def main():
    # (i) 64 x 128 N(0,1) seed 0 -> nvfp4
    x = make_input((64, 128), seed=0)
    out, sf, gs = T.quantize_nvfp4(x, 0, 1)
    np.savez_compressed(os.path.join(HERE, "nvfp4_gauss_64x128.npz"), x=bits(x), out=out.numpy(), sf=sf.numpy(),
                        gs=gs.numpy())
    # (ii) the reference's value set {+-1,+-2,+-4,+-6}, ragged shape, transposed read, swizzled
    g = torch.Generator().manual_seed(1)
    vals = torch.tensor([1, 2, 4, 6, -1, -2, -4, -6], dtype=torch.bfloat16)
    x = vals[torch.randint(0, 8, (70, 45), generator=g)]
    out, sf, gs = T.quantize_nvfp4(x, 1, 0, swizzle=True)
    np.savez_compressed(os.path.join(HERE, "nvfp4_valueset_70x45_t_swz.npz"), x=bits(x), out=out.numpy(),
                        sf=sf.numpy(), gs=gs.numpy())
    # (iii) per-row fp8 / int8 with outliers, ragged
    x = make_input((37, 200), seed=2, outliers=True)
    o8, s8 = T.quantize_fp8(x, 0, 1)
    oi, si = T.quantize_int8(x, 0, 1)
    np.savez_compressed(os.path.join(HERE, "rowwise_outliers_37x200.npz"), x=bits(x), fp8=o8.numpy(), fp8_sf=s8.numpy(),
                        int8=oi.numpy(), int8_sf=si.numpy())
    # (iv) a 32 x 48 x 128 GEMM with bias
    a, b = make_input((32, 128), seed=3), make_input((48, 128), seed=4, std=0.02)
    bias = make_input((48,), seed=5)
    aq, bq = T.quantize_nvfp4(a, 0, 1), T.quantize_nvfp4(b, 0, 1)
    d = T.linear_nvfp4_contract(*aq, *bq, bias=bias, out_dtype=torch.float32)
    np.savez_compressed(os.path.join(HERE, "linear_32x48x128_bias.npz"), a=aq[0].numpy(), a_sf=aq[1].numpy(),
                        a_gs=aq[2].numpy(), b=bq[0].numpy(), b_sf=bq[1].numpy(), b_gs=bq[2].numpy(), bias=bits(bias),
                        d=d.numpy())
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
