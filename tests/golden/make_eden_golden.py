"""Writes tests/golden/eden_golden.npz by running the reference's CPU-runnable EDEN code
(cuda_kernels/src/srrcomp/srrcomp.py, class Eden) in the build container:

  * the Lloyd-Max tables the class holds (centroids / boundaries for 1..8 bits, float32) -- the
    product computes its own tables; these numbers only check them;
  * Eden.compress / Eden.decompress on CPU tensors for a few sizes that exercise the slicing rule
    (power of two, padding below 10 %, two slices, two rotations below 1024 elements): the input,
    every slice's packed words / scale / dimensions, and the reconstruction.

Run once:  python tests/golden/make_eden_golden.py   (needs /root/reference; the GPU box only reads
the .npz).  Torch's CPU reductions and butterfly rounding differ from the kernels', so the tests compare
these vectors with stated tolerances, not bit for bit.
"""
import os

import numpy as np
import torch

from make_golden import load_reference

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = load_reference()
    eden = ref.Eden(gpuacctype="cpu")
    out = {}
    for nbits in range(1, 9):
        out["centroids_%d" % nbits] = eden.centroids[nbits].numpy().astype(np.float32)
        out["boundaries_%d" % nbits] = eden.boundaries[nbits].numpy().astype(np.float32)
    g = torch.Generator().manual_seed(11)
    cases = []
    for dim in (1024, 512, 1000, 3000, 8192):
        x = torch.randn(dim, generator=g) * 1e-3
        out["x_%d" % dim] = x.numpy().copy()
        for nbits in (1, 2, 4, 5, 8):
            for seed in (0, 42):
                data = eden.compress(x.clone(), nbits, seed)
                rec = eden.decompress(data)
                key = "%d_%d_%d" % (dim, nbits, seed)
                cases.append((dim, nbits, seed, len(data)))
                out["rec_" + key] = rec.numpy().copy()
                for k, d in enumerate(data):
                    out["packed_%s_%d" % (key, k)] = d["packed_bins"].numpy().copy()
                    out["meta_%s_%d" % (key, k)] = np.array([float(d["scale"]), d["orig_dim"], d["num_hadamard"]], np.float64)
    out["cases"] = np.array(cases, np.int64)
    np.savez_compressed(os.path.join(HERE, "eden_golden.npz"), **out)
    print("wrote eden_golden.npz", len(out), "arrays")


if __name__ == "__main__":
    main()
