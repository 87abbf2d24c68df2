"""Writes tests/golden/traverse_small.npz: one small, seeded search problem
with the outputs of this repository's CPU oracle.

The reference's own tests hold no golden vectors and the reference cannot be
built in this environment, so these vectors do not come from the reference:
they freeze what the pinned oracle (tests/test_oracle_*.py) computes, as a
regression fixture for the oracle itself, for the host stages and for the
device kernels.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from common import Problem  # noqa: E402


def main():
    p = Problem(n=1500, d=32, deg=16, sample_ratio=0.3, seed=77, n_query=24)
    dp, ef, k = 16, 8, 5
    init_I, init_D = p.entries(12, seed=3, dp=dp)
    B = p.query.size(0)
    cand_I = np.empty((B, 4 * ef), np.int64)
    cand_D = np.empty((B, 4 * ef), np.float32)
    oracle.traverse_cpu(cand_I, cand_D, init_I.numpy().copy(), init_D.numpy().copy(),
                        p.sub_indptr.numpy(), p.sub_indices.numpy(),
                        np.ascontiguousarray(p.x[:, :dp].numpy()),
                        np.ascontiguousarray(p.query[:, :dp].numpy()), 4 * ef)
    top_I = np.empty((B, k), np.int64)
    top_D = np.empty((B, k), np.float32)
    buf_I, buf_D = cand_I.copy(), cand_D.copy()
    oracle.traverse_refine(top_I, top_D, buf_I, buf_D, buf_I, buf_D,
                           [p.sub_indptr.numpy(), p.sub_indices.numpy()],
                           [p.indptr.numpy(), p.indices.numpy()], p.x.numpy(),
                           p.query.numpy(), ef, dp)
    np.savez_compressed(
        os.path.join(HERE, 'traverse_small.npz'),
        x=p.x.numpy(), query=p.query.numpy(), dp=dp, ef=ef, k=k, deg=p.deg,
        indptr=p.indptr.numpy().astype(np.int32),
        indices=p.indices.numpy().astype(np.int32),
        sub_indptr=p.sub_indptr.numpy().astype(np.int32),
        sub_indices=p.sub_indices.numpy().astype(np.int32),
        nodelist=p.nodelist.numpy().astype(np.int32),
        mapping=p.mapping.numpy().astype(np.int32),
        init_I=init_I.numpy().astype(np.int32), init_D=init_D.numpy(),
        cand_I=cand_I.astype(np.int32), cand_D=cand_D,
        stage2_I=buf_I.astype(np.int32), stage2_D=buf_D,
        top_I=top_I.astype(np.int32), top_D=top_D)


if __name__ == '__main__':
    main()
