"""Writes the golden vectors under tests/golden/ by running the reference's own
CPU-runnable torch code (cuda_kernels/src/srrcomp/srrcomp.py) in the build
container.  Only functions that no closed form or invariant pins are recorded:

  * SRRCompUtils.randDiag(size, 'cpu', seed)      -> sign bits (the 33-bit carry of
    the SplitMix step is only provable from the reference's int64 arithmetic)
  * SRRCompUtils.EdenBinsToBits / EdenBitsToBins  -> packed words for nbits 1..8
  * SRRCompUtils.Hadamard                         -> torch butterfly output (compared
    with 1e-5 relative tolerance; its rounding differs from the kernels')

Run once:  python tests/golden/make_golden.py   (needs /root/reference; the GPU box
never runs this, it only reads the .npz fixtures).
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/cuda_kernels/src/srrcomp/srrcomp.py"


def load_reference():
    spec = importlib.util.spec_from_file_location("ref_srrcomp", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    ref = load_reference()
    utils = ref.SRRCompUtils()
    out = {}

    # randDiag
    cases = []
    for size in (8, 13, 64, 100, 1024, 4096):
        for seed in (0, 1, 42, 2 ** 31, 123456789):
            signs = utils.randDiag(size, "cpu", seed)
            cases.append((size, seed))
            out["randdiag_%d_%d" % (size, seed)] = np.packbits((signs.numpy() > 0).astype(np.uint8))
    out["randdiag_cases"] = np.array(cases, dtype=np.int64)

    # bit-plane packing
    g = torch.Generator().manual_seed(7)
    for nbits in range(1, 9):
        for nbins in (64, 256):
            bins = torch.randint(0, 1 << nbits, (nbins,), generator=g, dtype=torch.int32)
            bits = utils.EdenBinsToBits(bins.clone(), nbits)
            back = utils.EdenBitsToBins(bits.clone(), nbits)
            assert torch.equal(back.to(torch.int32), bins)
            out["pack_bins_%d_%d" % (nbits, nbins)] = bins.numpy()
            out["pack_bits_%d_%d" % (nbits, nbins)] = bits.numpy()

    # Hadamard (torch butterfly)
    for k in (3, 6, 10):
        x = torch.randn(1 << k, generator=g)
        out["had_in_%d" % k] = x.numpy().copy()
        out["had_out_%d" % k] = utils.Hadamard(x.clone()).numpy().copy()

    np.savez_compressed(os.path.join(HERE, "srrcomp_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "srrcomp_golden.npz"), len(out), "arrays")


if __name__ == "__main__":
    main()
