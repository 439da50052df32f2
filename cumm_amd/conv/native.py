"""Per-offset ("native") sparse convolution: one gather-GEMM-scatter per kernel offset.

``SparseConvAlgo.Native`` of the reference (include/tensorview/gemm/core/constants.h:34-38): what
its callers fall back to when the mask-based kernels do not apply, and the only path for kernel
volumes above 32, which 32-bit masks cannot describe (the reference's ``dynamic_mask`` loader,
cumm/gemm/blockmma/mma.py:78-269, is not built here).  The pattern is the reference's own check
of its kernels, cumm/conv/main_real_spconv.py:309-403:

    forward          out[pair_out[k]]  += inp[pair_in[k]]   @ W[:, k, :].T     (matmul2, ShuffleAC)
    backward-input   dinp[pair_in[k]]  += dout[pair_out[k]] @ W[:, k, :]       (matmul2, ShuffleAC)
    backward-weight  dW[:, k, :]        = dout[pair_out[k]].T @ inp[pair_in[k]] (matmul2, ShuffleAB)

Forward and backward-input accumulate all offsets in an fp32 image (the f16 / bf16 -> f32 kernels)
and round once at the end (``cumm_hip_finish_rows``, with bias and activation): one rounding, as
the mask-based kernels make, instead of one per offset.
"""
import ctypes
from typing import Optional

import numpy as np

from .. import _capi
from .. import tensorview as tv
from ..gemm.main import GemmMainUnitTest
from ..tensorview.gemm import Activation, GemmParams, ShuffleStrideType


_FOUND = {}


def _find(dtype: int, dtype_c: int, shuffle: ShuffleStrideType, tile_m: int, tile_n: int, trans_a: bool,
          trans_b: bool):
    key = (dtype, dtype_c, shuffle, tile_m, tile_n, trans_a, trans_b)
    if key not in _FOUND:
        for d in _descs():
            if (d.dtype_a == dtype and d.dtype_c == dtype_c and d.shuffle_type == shuffle and
                    d.tile_shape[0] == tile_m and d.tile_shape[1] == tile_n and d.trans_a == trans_a and
                    d.trans_b == trans_b and not d.trans_c):
                _FOUND[key] = d
                break
        else:
            raise RuntimeError("can't find any suitable algo for your parameters.")
    return _FOUND[key]


_DESCS = None


def _descs():
    global _DESCS
    if _DESCS is None:
        _DESCS = GemmMainUnitTest.get_all_algo_desp()
    return _DESCS


def _check(inp, weight, lists, n_rows_out):
    if inp.ndim != 2 or weight.ndim != 3:
        raise RuntimeError("error")
    if inp.dtype != weight.dtype or inp.dtype not in (tv.float16, tv.bfloat16):
        raise RuntimeError("the native path takes f16 or bf16 features and weights of one type")
    kv = weight.dim(1)
    if lists.pair_in.dim(0) != kv or lists.pair_out.dim(0) != kv or len(lists.counts) != kv:
        raise RuntimeError("pair lists and weight disagree on the kernel volume")
    if inp.dim(1) % 8 or weight.dim(0) % 8 or weight.dim(2) % 8:
        raise RuntimeError("channel counts must be multiples of 8")
    return kv


def _accumulate_steps(a, a_inds_all, c_inds_all, counts, weight, acc, trans_b, stream):
    """One validated ``GemmParams`` per offset with pairs: acc[c_inds[k]] += a[a_inds[k]] @ op(W[:, k, :])."""
    kv = weight.dim(1)
    n_ch = acc.dim(1)
    steps = []
    for k in range(kv):
        cnt = int(counts[k])
        if cnt == 0:
            continue
        p = GemmParams()
        tile_m = 128 if cnt >= 16384 else 64
        tile_n = 128 if n_ch >= 128 else 64
        p.algo_desp = _find(a.dtype, tv.float32, ShuffleStrideType.ShuffleAC, tile_m, tile_n, False, trans_b).copy()
        p.a, p.b, p.c = a, weight.select(1, k), acc
        p.a_inds = a_inds_all.select(0, k).slice_first_axis(0, cnt)
        p.c_inds = c_inds_all.select(0, k).slice_first_axis(0, cnt)
        p.alpha, p.beta = 1.0, 1.0
        p.stream = stream
        steps.append(p)
    return steps


def _finish(out, acc, bias, act_type, act_alpha, stream):
    _capi.check(_capi.lib().cumm_hip_finish_rows(
        out.byte_pointer(), out.dtype, acc.byte_pointer(), None if bias is None or bias.empty() else bias.byte_pointer(),
        out.dim(0), out.dim(1), 1.0, 1.0, act_type.value if hasattr(act_type, "value") else int(act_type),
        float(act_alpha), stream))


def _fp32_image(rows, channels, acc):
    if acc is None or acc.empty():
        acc = tv.empty([rows, channels], tv.float32, 0)
    elif acc.dtype != tv.float32 or acc.shape != [rows, channels] or acc.device < 0:
        raise RuntimeError("acc must be a device float32 tensor [%d, %d]" % (rows, channels))
    return acc


class _Plan:
    """The launches of one pass over fixed tensors and pair lists: built (and validated) once, run
    any number of times - a repeat run goes straight to the C entry points with the argument blocks
    of the first one.  The plan keeps its tensors alive."""

    def __init__(self, out, acc, steps, bias, act_type, act_alpha, stream):
        self.out, self.acc, self.steps = out, acc, steps
        self.bias, self.act_type, self.act_alpha, self.stream = bias, act_type, act_alpha, stream
        self._ctx = tv.Context()
        self._ctx.set_cuda_stream(stream)

    def __call__(self) -> None:
        self.acc.zero_(self._ctx)
        for p in self.steps:
            GemmMainUnitTest.matmul2(p)
        _finish(self.out, self.acc, self.bias, self.act_type, self.act_alpha, self.stream)

    @property
    def launches(self) -> int:
        return len(self.steps) + 2


def plan_forward(inp: tv.Tensor, weight: tv.Tensor, output: tv.Tensor, lists, *, bias: Optional[tv.Tensor] = None,
                 act_type=Activation.None_, act_alpha: float = 0.0, stream: int = 0,
                 acc: Optional[tv.Tensor] = None) -> _Plan:
    """The forward pass as a reusable plan (``plan()`` runs it): for a layer whose tensors and
    geometry stay in place from call to call."""
    _check(inp, weight, lists, output.dim(0))
    if output.ndim != 2 or output.dim(1) != weight.dim(0) or output.dtype != inp.dtype or weight.dim(2) != inp.dim(1):
        raise RuntimeError("error")
    acc = _fp32_image(output.dim(0), output.dim(1), acc)
    # W[:, k, :] is [K, C]: B stored [n, k]
    steps = _accumulate_steps(inp, lists.pair_in, lists.pair_out, lists.counts, weight, acc, True, stream)
    return _Plan(output, acc, steps, bias, act_type, act_alpha, stream)


def plan_backward_input(dout: tv.Tensor, weight: tv.Tensor, dinp: tv.Tensor, lists, *, stream: int = 0,
                        acc: Optional[tv.Tensor] = None) -> _Plan:
    _check(dout, weight, lists, dinp.dim(0))
    if dinp.ndim != 2 or dinp.dim(1) != weight.dim(2) or dout.dim(1) != weight.dim(0) or dinp.dtype != dout.dtype:
        raise RuntimeError("error")
    acc = _fp32_image(dinp.dim(0), dinp.dim(1), acc)
    # W[:, k, :] is [K, C] with K the contraction: B stored [k, n]
    steps = _accumulate_steps(dout, lists.pair_out, lists.pair_in, lists.counts, weight, acc, False, stream)
    return _Plan(dinp, acc, steps, None, Activation.None_, 0.0, stream)


def forward(inp: tv.Tensor, weight: tv.Tensor, output: tv.Tensor, lists, *, bias: Optional[tv.Tensor] = None,
            act_type=Activation.None_, act_alpha: float = 0.0, stream: int = 0, acc: Optional[tv.Tensor] = None) -> None:
    """output [N_out, K] = act(sum over offsets + bias); ``lists`` from ``pairs.pair_lists_device``
    on the forward table; ``acc``: an fp32 [N_out, K] device tensor to reuse as the image."""
    plan_forward(inp, weight, output, lists, bias=bias, act_type=act_type, act_alpha=act_alpha, stream=stream,
                 acc=acc)()


def backward_input(dout: tv.Tensor, weight: tv.Tensor, dinp: tv.Tensor, lists, *, stream: int = 0,
                   acc: Optional[tv.Tensor] = None) -> None:
    """dinp [N_in, C] = sum over offsets of dout[pair_out[k]] @ W[:, k, :] scattered to pair_in[k]."""
    plan_backward_input(dout, weight, dinp, lists, stream=stream, acc=acc)()


_NO_PAIR = {}


class _WeightPlan:
    """The per-offset launches of backward-weight, validated once (the first run goes through the
    operator's prelude, a hundred microseconds of Python per offset) and then replayed straight at
    the C entry point - on the same tensors, or on others of the same shapes and types whose
    addresses ``rebind`` writes into the argument blocks."""

    def __init__(self, steps, dout, inp, dweight):
        self.steps = steps
        self._tensors = (dout, inp, dweight)     # kept alive with the blocks that point at them
        self._blocks = None

    def __call__(self) -> None:
        for p in self.steps:
            GemmMainUnitTest.matmul2(p)
        if self._blocks is None:
            base = self._tensors[2].byte_pointer()
            self._blocks = []
            for p in self.steps:
                prep = p.__dict__.get("_prepared")
                if prep is None:
                    raise RuntimeError("the operator call left no validated argument block")
                args = prep[5]
                self._blocks.append((prep[1], prep[2], prep[3], args, int(args.ptr_C) - base, int(args.ptr_D or 0) - base))

    def rebind(self, dout_ptr: int, inp_ptr: int, dweight_ptr: int, stream: int) -> None:
        """Run on other tensors of the same shapes (device addresses), on ``stream``."""
        if self._blocks is None:
            raise RuntimeError("the plan has not run yet")
        for fn, cdesc_ref, args_ref, args, c_delta, d_delta in self._blocks:
            args.ptr_A, args.ptr_B = dout_ptr, inp_ptr
            args.ptr_C = dweight_ptr + c_delta
            if args.ptr_D:
                args.ptr_D = dweight_ptr + d_delta
            status = fn(cdesc_ref, args_ref, stream)
            if status:
                _capi.check(status)

    def release(self) -> None:
        """Forget the tensors of the first run (a caller that goes on through ``rebind`` with its
        own): the argument blocks hold addresses only, the pair lists belong to their owner."""
        if self._blocks is None:
            raise RuntimeError("the plan has not run yet")
        self.steps, self._tensors = [], None

    @property
    def launches(self) -> int:
        return len(self._blocks) if self._blocks is not None else len(self.steps)


def plan_backward_weight(dout: tv.Tensor, inp: tv.Tensor, dweight: tv.Tensor, lists, *, stream: int = 0) -> _WeightPlan:
    """Backward-weight as a reusable plan: one gathered GEMM per kernel offset into its slice of
    ``dweight`` [K, kv, C] (an offset without pairs writes zeros)."""
    kv = _check(inp, dweight, lists, dout.dim(0))
    if dout.dim(1) != dweight.dim(0) or dout.dtype != inp.dtype:
        raise RuntimeError("error")
    steps = []
    for k in range(kv):
        cnt = int(lists.counts[k])
        p = GemmParams()
        p.algo_desp = _find(inp.dtype, inp.dtype, ShuffleStrideType.ShuffleAB, 64, 64, True, False).copy()
        p.a, p.b, p.c = dout, inp, dweight.select(1, k)
        if cnt > 0:
            p.a_inds = lists.pair_out.select(0, k).slice_first_axis(0, cnt)
            p.b_inds = lists.pair_in.select(0, k).slice_first_axis(0, cnt)
        else:
            dev = inp.device
            if dev not in _NO_PAIR:
                _NO_PAIR[dev] = tv.from_numpy(np.full(32, -1, np.int32)).cuda()
            p.a_inds = p.b_inds = _NO_PAIR[dev]
        p.stream = stream
        steps.append(p)
    return _WeightPlan(steps, dout, inp, dweight)


def backward_weight(dout: tv.Tensor, inp: tv.Tensor, dweight: tv.Tensor, lists, *, split_k_slices: int = 1,
                    stream: int = 0, workspace: Optional[tv.Tensor] = None) -> None:
    """dweight[:, k, :] = dout[pair_out[k]].T @ inp[pair_in[k]] for every offset (zero without pairs)."""
    kv = _check(inp, dweight, lists, dout.dim(0))
    if dout.dim(1) != dweight.dim(0) or dout.dtype != inp.dtype:
        raise RuntimeError("error")
    for k in range(kv):
        cnt = int(lists.counts[k])
        p = GemmParams()
        p.algo_desp = _find(inp.dtype, inp.dtype, ShuffleStrideType.ShuffleAB, 64, 64, True, False).copy()
        p.a, p.b, p.c = dout, inp, dweight.select(1, k)
        if cnt > 0:
            p.a_inds = lists.pair_out.select(0, k).slice_first_axis(0, cnt)
            p.b_inds = lists.pair_in.select(0, k).slice_first_axis(0, cnt)
        else:
            # an offset without pairs: one step of absent rows (index -1) writes the zeros
            dev = inp.device
            if dev not in _NO_PAIR:
                _NO_PAIR[dev] = tv.from_numpy(np.full(32, -1, np.int32)).cuda()
            p.a_inds = p.b_inds = _NO_PAIR[dev]
        p.split_k_slices = split_k_slices if cnt >= 4096 * split_k_slices else 1
        if workspace is not None:
            p.workspace = workspace
        p.stream = stream
        GemmMainUnitTest.matmul2(p)
