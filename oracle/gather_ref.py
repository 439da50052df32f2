"""CPU restatement of the reference's stand-alone gather / scatter-add kernels.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Pinned in tests/test_oracle_gather.py by what the operations must satisfy
whatever the implementation: a permutation followed by its inverse is the
identity, gathering with an identity index is a copy, scatter-adding rows of
ones counts the index occurrences, and scatter-add equals a dense one-hot
matrix product.
"""
import numpy as np

from . import numerics


def gather_rows_ref(inp, indices):
    """output[i, :] = input[indices[i], :] (GatherKernelV2, cumm/gemm/gather.py:170-194);
    an index outside the input gives a row of zeros (this build's rule for what the reference
    leaves undefined)."""
    inp = np.asarray(inp)
    indices = np.asarray(indices, dtype=np.int64)
    out = np.zeros((indices.shape[0], inp.shape[1]), dtype=inp.dtype)
    ok = (indices >= 0) & (indices < inp.shape[0])
    out[ok] = inp[indices[ok]]
    return out


def scatter_add_rows_ref(out, inp, indices, dtype="f32"):
    """output[indices[i], :] += input[i, :] for unique indices (ScatterKernel,
    cumm/gemm/gather.py:303-331: load both fragments, add, store); each sum is formed in fp32 and
    rounded once to the storage type.  Rows with an index outside the output are dropped."""
    res = np.array(out, copy=True)
    indices = np.asarray(indices, dtype=np.int64)
    ok = (indices >= 0) & (indices < res.shape[0])
    assert np.unique(indices[ok]).shape[0] == int(ok.sum()), "indices must be unique"
    rows = indices[ok]
    total = numerics.to_f32(res[rows], dtype) + numerics.to_f32(np.asarray(inp)[: indices.shape[0]][ok], dtype)
    res[rows] = numerics.from_f32(total, dtype)
    return res
