#!/usr/bin/env python3
"""Writes tests/golden/rtn_vectors.npz: input/output vectors of the reference's round-to-nearest quantiser.

Runs in the build container only (it imports /root/reference/gptq.py, which does not travel): the
rounding of computed quotients in `Quantizer.find_params` (gptq.py:205-286) and `quantize` (gptq.py:174-178,
`scale * (clamp(round(x / scale) + zero, 0, maxq) - zero)`) is the one part of the load-time packer that
nothing else pins.  The driver loop below restates how `dumbquant` calls them per group (quantize.py:294-329:
find_params on each block of `groupsize` input columns, then quantize column by column).

Cases: mixed-sign Gaussian weights (one group and groups of 128), a matrix with exact ties on the grid, an
all-zero group, and a group of non-negative weights (where the reference's zero point is 0).
"""
import os
import sys

import numpy as np
import torch

REFERENCE = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rtn_vectors.npz")


def main():
    sys.path.insert(0, REFERENCE)
    import gptq  # the reference's gptq.py

    def reference_rtn(weight: torch.Tensor, groupsize: int):
        quantizer = gptq.Quantizer()
        quantizer.configure(4, perchannel=True, sym=False, mse=False)
        w = weight.clone().float()
        gs = w.shape[1] if groupsize == -1 else groupsize
        deq = torch.empty_like(w)
        scales, zeros = [], []
        for i in range(0, w.shape[1], gs):
            quantizer.find_params(w[:, i:i + gs], weight=True)
            scales.append(quantizer.scale.clone())
            zeros.append(quantizer.zero.clone())
            deq[:, i:i + gs] = gptq.quantize(w[:, i:i + gs], quantizer.scale, quantizer.zero, quantizer.maxq)
        return deq, torch.cat(scales, dim=1), torch.cat(zeros, dim=1)

    gen = torch.Generator().manual_seed(20240521)
    cases = {}
    cases["gauss_g-1"] = (torch.randn((16, 256), generator=gen) * 0.05, -1)
    cases["gauss_g128"] = (torch.randn((24, 384), generator=gen) * 0.02, 128)
    # exact ties: weights on half-steps of a grid whose scale is a power of two (range [-1, 0.875] -> scale 0.125)
    tie = (torch.randint(-16, 15, (8, 128), generator=gen).float()) * 0.0625
    tie[:, 0], tie[:, 1] = -1.0, 0.875
    cases["ties_g-1"] = (tie, -1)
    zg = torch.randn((8, 256), generator=gen) * 0.03
    zg[:, 128:] = 0.0            # second group all zero
    zg[3, :128] = 0.0            # and one all-zero row in the first
    cases["zero_group_g128"] = (zg, 128)
    cases["nonneg_g128"] = (torch.rand((8, 256), generator=gen) * 0.04, 128)
    out = {}
    for name, (w, g) in cases.items():
        deq, scale, zero = reference_rtn(w, g)
        out[name + "/weight"] = w.numpy().astype(np.float32)
        out[name + "/groupsize"] = np.int32(g)
        out[name + "/deq"] = deq.numpy().astype(np.float32)
        out[name + "/scale"] = scale.numpy().astype(np.float32)
        out[name + "/zero"] = zero.numpy().astype(np.float32)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, {k: v.shape for k, v in out.items() if k.endswith("/weight")})


if __name__ == "__main__":
    main()
