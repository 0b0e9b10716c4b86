"""Writes tests/golden/awq_small.npz: inputs and expected outputs of one small AWQ problem.

The reference tree holds no implementation, test or vector for this path
(kuiper/include/op/matmul.h:7-9 is empty), so the expected values come from the numpy
restatement of the layout definition in tests/spec_numpy.py and from torch's own bf16 cast,
neither of which shares code with the C oracle or with the HIP kernels.

  python tests/golden/make_awq_vectors.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from mykuiperllama_amd import synth  # noqa: E402
from tests import spec_numpy as spec  # noqa: E402


def main():
    p = synth.make_awq_problem("golden_small", 2, 256, 64, group=128)
    codes = spec.unpack(p["qweight"])
    zeros = spec.unpack(p["qzeros"])
    w64 = spec.dequant_f64(p["qweight"], p["scales"], p["qzeros"], 128)
    # every product has at most 16 significant bits: float32 holds it exactly
    w_bf16 = torch.from_numpy(w64.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    y64 = spec.gemv_awq_f64(p["x"], p["qweight"], p["scales"], p["qzeros"], 128)
    np.savez_compressed(os.path.join(HERE, "awq_small.npz"),
                        x=p["x"], qweight=p["qweight"], scales=p["scales"], qzeros=p["qzeros"],
                        group=np.int64(128), codes=codes, zero_codes=zeros, w_bf16=w_bf16, y_f64=y64)
    print("wrote awq_small.npz", codes.shape, w_bf16.shape, y64.shape)


if __name__ == "__main__":
    main()
