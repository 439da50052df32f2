"""CPU oracle for the per-offset ("native") sparse convolution: one gather -> matmul -> scatter-add
per kernel offset, any kernel volume.

Test infrastructure only (see oracle/__init__.py).

This is the reference's own CPU check of its sparse-convolution kernels, restated on pair lists:
forward cumm/conv/main_real_spconv.py:309-326, backward-input :347-365, backward-weight :375-403
(``indice_pairs[0]`` = input rows, ``indice_pairs[1]`` = output rows, ``weight_ref`` [kv, K, C]).
Sums are formed in float32 over all offsets and rounded once to the storage type; bias and
activation follow LinearCombination / UnaryActivation (cumm/gemm/output_op/linear.py:108-146,
cumm/gemm/gemmmath/__init__.py:181-214).  Pinned against torch's dense conv3d and autograd with
5 x 5 x 5 and 3 x 3 x 5 kernels in tests/test_oracle_native.py.
"""
import numpy as np

from . import numerics as nm


def native_fwd_ref(inp, weight, pair_in, pair_out, counts, n_out, *, dtype, bias=None, act=nm.ACT_NONE,
                   act_alpha=0.0):
    """inp [N_in, C], weight [K, kv, C] -> output [N_out, K] in ``dtype``."""
    k_out, kv, _ = weight.shape
    acc = np.zeros((n_out, k_out), np.float32)
    xf = nm.to_f32(inp, dtype)
    for k in range(kv):
        n = int(counts[k])
        if n == 0:
            continue
        a_inds, c_inds = pair_in[k][:n], pair_out[k][:n]
        acc[c_inds] += xf[a_inds] @ nm.to_f32(weight[:, k, :], dtype).T    # output rows are unique within an offset
    if bias is not None:
        acc = nm.linear_combination_f32(acc, nm.to_f32(bias, dtype)[None, :], 1.0, 1.0)
    return nm.from_f32(nm.activation(acc, act, act_alpha), dtype)


def native_dgrad_ref(dout, weight, pair_in, pair_out, counts, n_in, *, dtype):
    """dout [N_out, K], weight [K, kv, C] -> dinp [N_in, C]."""
    _, kv, c_in = weight.shape
    acc = np.zeros((n_in, c_in), np.float32)
    gf = nm.to_f32(dout, dtype)
    for k in range(kv):
        n = int(counts[k])
        if n == 0:
            continue
        acc[pair_in[k][:n]] += gf[pair_out[k][:n]] @ nm.to_f32(weight[:, k, :], dtype)
    return nm.from_f32(acc, dtype)


def native_wgrad_ref(dout, inp, pair_in, pair_out, counts, kv, *, dtype):
    """dout [N_out, K], inp [N_in, C] -> dweight [K, kv, C]."""
    k_out, c_in = dout.shape[1], inp.shape[1]
    dw = np.zeros((k_out, kv, c_in), np.float32)
    gf, xf = nm.to_f32(dout, dtype), nm.to_f32(inp, dtype)
    for k in range(kv):
        n = int(counts[k])
        if n:
            dw[:, k, :] = gf[pair_out[k][:n]].T @ xf[pair_in[k][:n]]
    return nm.from_f32(dw, dtype)
