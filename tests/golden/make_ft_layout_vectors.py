"""Writes golden vectors for the mixed-input GEMM weight layout.

The producer is ``quantized_weight_reorder_for_mixed_dtypes_linear_cutlass`` from the
installed PyTorch wheel (torch/quantization/_quantized_conversions.py), an independent
restatement of the same published layout.  It only accepts device tensors, so this
script has to run on a machine with a GPU:

    python tests/golden/make_ft_layout_vectors.py /tmp/ft_layout_vectors.npz

and the resulting file is committed as tests/golden/ft_layout_vectors.npz.
Inputs are seeded random bytes; for each case the file stores the input
``int8 [K, N]`` (int4: ``[K, N/2]``, low nibble = even n) and the reordered output
of the same shape.
"""
import sys

import numpy as np
import torch
from torch.quantization._quantized_conversions import (
    quantized_weight_reorder_for_mixed_dtypes_linear_cutlass as reorder,
)

CASES = [  # (name, nbit, K, N)
    ("int8_64x64", 8, 64, 64),
    ("int8_128x192", 8, 128, 192),
    ("int8_256x64", 8, 256, 64),
    ("int4_64x64", 4, 64, 64),
    ("int4_128x192", 4, 128, 192),
    ("int4_256x128", 4, 256, 128),
]


def main(path):
    out = {}
    rng = np.random.default_rng(20240607)
    for name, nbit, K, N in CASES:
        cols = N if nbit == 8 else N // 2
        a = rng.integers(-128, 128, size=(K, cols), dtype=np.int64).astype(np.int8)
        t = torch.from_numpy(a).cuda()
        r = reorder(t, torch.int8 if nbit == 8 else torch.quint4x2, transpose=False)
        r = r.cpu().numpy().view(np.int8).reshape(K, cols)
        out[name + "_in"] = a
        out[name + "_out"] = r
        print(name, a.shape, r.shape, flush=True)
    np.savez_compressed(path, **out)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/tmp/ft_layout_vectors.npz")
