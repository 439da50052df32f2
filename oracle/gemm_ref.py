"""CPU oracle for ``GemmMainUnitTest.matmul2`` (dense, ShuffleAC, ShuffleAB).

Test infrastructure only (see oracle/__init__.py).

Storage dtypes are named by strings: "f32", "f16", "bf16" (uint16 bit
patterns), "s8", "s32".
"""
import numpy as np

from . import numerics as nm

NO_SHUFFLE, SHUFFLE_AC, SHUFFLE_AB = 0, 1, 2


def _is_int(dtype):
    return dtype in ("s8", "s32")


def _matmul_acc(a, b, dtype_a, dtype_b):
    """op(A) @ op(B) in the accumulator type: f32 for float inputs, exact s32
    for s8 inputs (float64 BLAS is exact while |acc| < 2**53)."""
    if _is_int(dtype_a):
        acc = a.astype(np.float64) @ b.astype(np.float64)
        assert np.all(np.abs(acc) < 2 ** 31), "s32 accumulator would overflow"
        return acc.astype(np.int64).astype(np.int32)
    return nm.to_f32(a, dtype_a) @ nm.to_f32(b, dtype_b)


def linear_combination_s32(acc, src, alpha, beta, act, act_alpha):
    """LinearCombination with dcomp = s32 (the "s8,s8,s32,s32,s32" kernels,
    cumm/gemm/main.py:350-364,500-523 of the reference): alpha, beta and act_alpha
    are members of type dcomp, i.e. the float parameters converted to int32 (C
    conversion: toward zero), cumm/gemm/output_op/linear.py:54-72; the
    combination alpha*acc + beta*src (:108-146) and the activation
    (cumm/gemm/gemmmath/__init__.py:181-214: max(x, 0); x >= 0 ? x : x*alpha)
    are int32 arithmetic, which wraps on overflow on the GPU."""
    def wrap(v):
        return ((np.asarray(v, dtype=np.int64) + 2 ** 31) % 2 ** 32 - 2 ** 31)
    ai, bi, la = int(np.float32(alpha)), int(np.float32(beta)), int(np.float32(act_alpha))
    t = wrap(ai * np.asarray(acc, dtype=np.int64))
    if bi != 0 and src is not None:
        t = wrap(t + wrap(bi * np.asarray(src, dtype=np.int64)))
    if act == nm.ACT_RELU:
        t = np.maximum(t, 0)
    elif act == nm.ACT_LEAKY_RELU:
        t = np.where(t >= 0, t, wrap(t * la))
    elif act != nm.ACT_NONE:
        raise ValueError("no integer version of activation %d" % act)
    return t.astype(np.int32)


def linear_combination(acc, src, alpha, beta, act, act_alpha, act_beta, dtype_c):
    """LinearCombination, cumm/gemm/output_op/linear.py:108-146 (with source)
    and :157-183 (beta == 0 -> the source is never read) of the reference.
    Output type s32 (of s8 operands): integer arithmetic, see linear_combination_s32."""
    if dtype_c == "s32" and np.issubdtype(np.asarray(acc).dtype, np.integer):
        return linear_combination_s32(acc, src if beta != 0.0 else None, alpha, beta, act, act_alpha)
    acc = np.asarray(acc).astype(np.float32)
    t = nm.linear_combination_f32(acc, src if beta != 0.0 else None, alpha, beta)
    t = nm.activation(t.astype(np.float32), act, act_alpha, act_beta)
    if dtype_c == "s32":
        return np.rint(t).astype(np.int32)
    if dtype_c == "s8":
        return np.clip(np.rint(t), -128, 127).astype(np.int8)
    return nm.from_f32(t, dtype_c)


def _src_f32(d, dtype_c):
    """The source operand in the arithmetic type of the combination: float32, or the integers
    themselves for an s32 output."""
    if dtype_c == "s32":
        return np.asarray(d).astype(np.int64)
    return nm.to_f32(d, dtype_c) if not _is_int(dtype_c) else d.astype(np.float32)


def split_k_ranges(k, split_k_slices, tile_k):
    """Contraction range [lo, hi) of every slice of a serial split-K GEMM: slice z owns
    ``gemm_k_size_per_split = ceil(ceil(k / tile_k) / slices) * tile_k`` consecutive elements
    (GemmUtils::get_gemm_k_size_per_split, include/tensorview/gemm/core/utils.h:30-37; use in
    cumm/gemm/kernel.py:242-243,659-667 of the reference)."""
    per = -(-(-(-k // tile_k)) // split_k_slices) * tile_k
    return [(min(z * per, k), min((z + 1) * per, k)) for z in range(split_k_slices)]


def matmul2_ref(a, b, c, *, dtype_a, dtype_b, dtype_c, trans_a=False, trans_b=False,
                trans_c=False, shuffle=NO_SHUFFLE, a_inds=None, b_inds=None, c_inds=None,
                d=None, alpha=1.0, beta=0.0, act=nm.ACT_NONE, act_alpha=0.0, act_beta=0.0,
                split_k_slices=1, tile_k=32):
    """Return the contents of ``c`` after the call (``c`` itself is not modified).

    Semantics: cumm/gemm/nvrtc_code.py:34-146 (operand roles, m/n/k) and the
    checks in cumm/gemm/main_real.py:206-229 of the reference:

    * NoShuffle : C = act(alpha * op(A) @ op(B) + beta * D)
    * ShuffleAC : C[c_inds[i]] = act(alpha * A[a_inds[i]] @ op(B) + beta * D[c_inds[i]])
                  (a_inds optional; D 1-D means a bias over n)
    * ShuffleAB : C = act(alpha * A[a_inds].T @ B[b_inds] + beta * D)
    D defaults to C.  With trans_c the result is stored transposed ([n, m]).

    ``split_k_slices`` > 1 (NoShuffle / ShuffleAB, serial split-K): slice z takes the range
    ``split_k_ranges(k, slices, tile_k)[z]`` of the contraction; slice 0 writes
    cvt(act(alpha*acc_0 + beta*D)), every later slice cvt(act(alpha*acc_z + 1*C)) in slice order
    (set_k_partition forces beta = 1, cumm/gemm/output_op/linear.py:90-99; the semaphore orders
    the slices, cumm/gemm/kernel.py:820-905 of the reference): partial results are rounded to
    the output type between slices.
    """
    out = np.array(c, copy=True)
    dd = out if d is None else d
    if shuffle == SHUFFLE_AC:
        assert not trans_a and not trans_c
        rows = a if a_inds is None else a[a_inds]
        bm = b.T if trans_b else b
        acc = _matmul_acc(rows, bm, dtype_a, dtype_b)
        if dd.ndim == 1:
            src = _src_f32(dd, dtype_c)[None, :]
        else:
            src = _src_f32(dd[c_inds], dtype_c)
        out[c_inds] = linear_combination(acc, src, alpha, beta, act, act_alpha, act_beta, dtype_c)
        return out
    if shuffle == SHUFFLE_AB:
        assert trans_a and not trans_b
        am, bm = a[a_inds].T, b[b_inds]
    else:
        am = a.T if trans_a else a
        bm = b.T if trans_b else b
    if dd.ndim == 1:
        # a 1-D D is a bias over the n dimension of the (untransposed) product
        src = _src_f32(dd, dtype_c)
        src = src[:, None] if trans_c else src[None, :]
    else:
        src = _src_f32(dd, dtype_c)
    cur_beta = beta
    for lo, hi in split_k_ranges(am.shape[1], max(1, int(split_k_slices)), tile_k):
        acc = _matmul_acc(am[:, lo:hi], bm[lo:hi], dtype_a, dtype_b)
        if trans_c:
            acc = acc.T
        out[...] = linear_combination(acc, src, alpha, cur_beta, act, act_alpha, act_beta, dtype_c)
        src, cur_beta = _src_f32(out, dtype_c), 1.0
    return out
