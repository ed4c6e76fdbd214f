"""Writes tests/golden/kat_small.npz: a small known-answer case (inputs and the CPU oracle's outputs).

The reference ships no golden vectors for this path, and the reference itself is not imported here:
the expected values come from this repository's oracle (oracle/blockrank_oracle.py), which
tests/test_oracle_*.py pin by mathematics.  The fixture freezes those values so that a later change to
the oracle or to the kernels shows up as a difference against committed numbers.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from blockrank_amd import synthetic          # noqa: E402
from oracle import blockrank_oracle as orc   # noqa: E402


def main():
    lay = synthetic.make_layout([[6, 9, 0, 13, 5], [3, 16, 7, 1, 8]])      # prefix, three documents (one empty), query
    Nq, Nkv, D = 4, 2, 64
    scale = D ** -0.5
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.float32, "cpu", seed=1234)
    m5 = orc.additive_mask(lay.valid, torch.float32)
    out, _ = orc.sdpa_blockrank_forward(q, k, v, m5, scale)
    scores = orc.doc_scores(q.numpy(), k.numpy(), lay.valid.numpy(), lay.labels.numpy(), scale, 0.05, 16)
    rows = lay.valid.reshape(lay.B, lay.S)
    out = out.clone()
    out[~rows] = 0            # rows of padded slots are unspecified in the reference; the HIP path writes zeros
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_small.npz")
    np.savez_compressed(path, lengths=lay.lengths, H=np.int64(lay.H), q=q.numpy(), k=k.numpy(), v=v.numpy(), labels=lay.labels.numpy(),
                        scale=np.float64(scale), out=out.numpy(), scores=scores, top=orc.topk_indices(scores, 10))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
