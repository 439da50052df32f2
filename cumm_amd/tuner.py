"""Timing-based choice among the algorithm descriptors.

The reference leaves the choice of a descriptor to its callers: they enumerate
``get_all_algo_desp`` / ``get_all_conv_algo_desp``, keep the ones whose
``supported`` accepts the problem (``simple_select_tile_shape``,
cumm/gemm/main.py:1072-1134, is the static variant), run each once or twice and
keep the fastest per problem shape (spconv's tuner; the reference's own scripts
do the same by hand, e.g. cumm/gemm/main_real.py:789-803 for the gather
kernels).  This module is that loop for the descriptors of this build, with
the timing done by events on the caller's stream.

A candidate shares the kind of the descriptor already set in the parameter
object (operation, element types, layouts, shuffle type, int8 epilogue) and
differs in tile shape and split-k variant.  Results are cached per problem
shape; the voxel count enters the key by its power-of-two bucket, the pair density P/N
(when the caller passes the pair count) by its half-octave bucket.
"""
from typing import Callable, Dict, List, NamedTuple, Optional, Tuple

from .conv.main import ConvMainUnitTest
from .gemm.main import GemmMainUnitTest
from .tensorview import Context, CUDAEvent, Tensor
from .tensorview.gemm import (ConvAlgoDesp, ConvOpType, ConvParams, GemmAlgoDesp, GemmParams,
                              implicit_gemm_mnk)


class TuneResult(NamedTuple):
    desp: object                       # the fastest descriptor
    ms: float                          # its time per call
    tried: List[Tuple[str, float]]     # (descriptor name, ms) of every candidate that ran


def _bucket(n: int) -> int:
    return max(int(n) - 1, 0).bit_length()


def _density_bucket(num_pairs: Optional[int], n: int) -> int:
    """Half-octave bucket of P/N (pairs per position, 1 .. kernel volume); -1 when unknown."""
    if num_pairs is None or n <= 0:
        return -1
    import math
    return int(math.floor(2.0 * math.log2(max(float(num_pairs) / float(n), 1.0))))


def _light_bucket(light_prefix: int, n: int) -> int:
    """Quarter of the positions that the light_prefix hint covers (0 .. 4): with a long light end
    the 64-row descriptors run two tile shapes and rank differently against the others."""
    if n <= 0 or light_prefix <= 0:
        return 0
    return min(4, 1 + (4 * int(light_prefix)) // (n + 1))


def conv_candidates(params: ConvParams, desps: Optional[List[ConvAlgoDesp]] = None) -> List[ConvAlgoDesp]:
    """Descriptors of the same kind as ``params.conv_algo_desp`` that accept the problem."""
    cur = params.conv_algo_desp
    op = ConvOpType(cur.op_type)
    kv, C, K = params.weight.dim(1), params.input.dim(1), params.weight.dim(0)
    N = params.indices.dim(1)
    mnk = implicit_gemm_mnk(op, N, C, K, kv, -1, -1, True)
    res = []
    for d in (desps if desps is not None else ConvMainUnitTest.get_all_conv_algo_desp()):
        if (d.op_type != cur.op_type or d.ndim != cur.ndim or not d.mask_sparse or
                (d.dtype_a, d.dtype_b, d.dtype_c) != (cur.dtype_a, cur.dtype_b, cur.dtype_c) or
                d.is_int8_inference != cur.is_int8_inference or bool(d.dynamic_mask) != bool(cur.dynamic_mask) or
                (d.layout_i, d.layout_w, d.layout_o) != (cur.layout_i, cur.layout_w, cur.layout_o)):
            continue
        if params.split_k_slices > 1 and not (d.split_k_serial or d.split_k_parallel):
            continue
        if op == ConvOpType.BackwardWeight and not (params.mask_width > 0 and
                                                    params.mask_width % d.tile_shape[2] == 0):
            continue
        if not d.supported(mnk[0], mnk[1], mnk[2], C, K, params.mask_width):
            continue
        # the three-stage twin of a tile differs from it only where the contraction is walked in
        # chunks (more than 128 bytes per row): elsewhere it would be timed twice
        contraction = K if op == ConvOpType.BackwardInput else C
        if d.num_stage >= 3 and contraction * params.input.itemsize <= 128:
            continue
        res.append(d)
    return res


def gemm_candidates(params: GemmParams, desps: Optional[List[GemmAlgoDesp]] = None) -> List[GemmAlgoDesp]:
    cur = params.algo_desp
    m, n, k = GemmMainUnitTest.extract_mnk(params.a.shape, params.b.shape, cur.trans_a, cur.trans_b, cur.trans_c,
                                           cur._shuffle_int(), params.a_inds.shape, params.b_inds.shape,
                                           params.c_inds.shape)
    res = []
    for d in (desps if desps is not None else GemmMainUnitTest.get_all_algo_desp()):
        if ((d.dtype_a, d.dtype_b, d.dtype_c) != (cur.dtype_a, cur.dtype_b, cur.dtype_c) or
                (d.trans_a, d.trans_b, d.trans_c) != (cur.trans_a, cur.trans_b, cur.trans_c) or
                d._shuffle_int() != cur._shuffle_int()):
            continue
        if params.split_k_slices > 1 and not (d.split_k_serial or d.split_k_parallel):
            continue
        if not d.supported(m, n, k):
            continue
        res.append(d)
    return res


def _stream_ctx(stream: int) -> Context:
    ctx = Context()
    ctx.set_cuda_stream(stream)
    return ctx


def _save(target: Tensor, ctx: Context) -> Tensor:
    """Copy of ``target`` made on the stream the timed launches run on, so that neither the copy
    nor the restore can overtake or trail a launch on a non-blocking stream."""
    saved = Tensor(target.shape, target.dtype, target.device)
    saved.copy_(target, ctx)
    return saved


def _time_calls(run: Callable[[], None], stream: int, steps: int, warmup: int) -> float:
    for _ in range(warmup):
        run()
    start = CUDAEvent("start").record(stream)
    for _ in range(steps):
        run()
    stop = CUDAEvent("stop").record(stream)
    stop.sync()
    return CUDAEvent.duration(start, stop) / steps


class Tuner:
    """Keeps the fastest descriptor per problem shape."""

    def __init__(self, steps: int = 3, warmup: int = 1):
        self.steps, self.warmup = steps, warmup
        self.cache: Dict[tuple, TuneResult] = {}

    # ---- sparse convolution
    @staticmethod
    def conv_key(params: ConvParams, num_pairs: Optional[int] = None) -> tuple:
        """(operation, types, C, K, kernel volume, bucket of N, bucket of the pair density P/N, ...).
        ``num_pairs`` is the number of active pairs P of the geometry when the caller knows it
        (two clouds of one size and very different density want different tiles); without it
        the density does not enter the key."""
        d = params.conv_algo_desp
        n = params.indices.dim(1)
        return ("conv", ConvOpType(d.op_type).value, d.dtype_a, d.dtype_b, d.dtype_c, bool(d.is_int8_inference),
                params.input.dim(1), params.weight.dim(0), params.weight.dim(1), _bucket(n),
                _density_bucket(num_pairs, n), params.split_k_slices > 1, params.mask_width,
                bool(params.reverse_mask), _light_bucket(getattr(params, "light_prefix", 0), n))

    def tune_conv(self, params: ConvParams, desps: Optional[List[ConvAlgoDesp]] = None,
                  num_pairs: Optional[int] = None) -> TuneResult:
        """Times every candidate on ``params`` (its result tensor is saved and restored, the
        descriptor is left at the fastest) and remembers the winner."""
        key = self.conv_key(params, num_pairs)
        hit = self.cache.get(key)
        if hit is not None:
            params.conv_algo_desp = hit.desp
            return hit
        cands = conv_candidates(params, desps)
        if not cands:
            raise RuntimeError("can't find any suitable algo for your parameters.")
        op = ConvOpType(params.conv_algo_desp.op_type)
        target = {ConvOpType.Forward: params.output, ConvOpType.BackwardInput: params.input,
                  ConvOpType.BackwardWeight: params.weight}[op]
        ctx = _stream_ctx(params.stream)
        saved = _save(target, ctx)
        tried = []
        for d in cands:
            params.conv_algo_desp = d
            try:
                ms = _time_calls(lambda: ConvMainUnitTest.implicit_gemm2(params), params.stream, self.steps, self.warmup)
            except (RuntimeError, ValueError):
                continue     # e.g. a workspace this variant needs and the caller did not give
            tried.append((str(d), ms))
            target.copy_(saved, ctx)
        if not tried:
            raise RuntimeError("can't find any suitable algo for your parameters.")
        names = [n for n, _ in tried]
        best = min(tried, key=lambda t: t[1])
        res = TuneResult([d for d in cands if str(d) == best[0]][0], best[1], tried)
        assert len(set(names)) == len(names)
        params.conv_algo_desp = res.desp
        self.cache[key] = res
        return res

    # ---- GEMM
    @staticmethod
    def gemm_key(params: GemmParams) -> tuple:
        d = params.algo_desp
        m, n, k = GemmMainUnitTest.extract_mnk(params.a.shape, params.b.shape, d.trans_a, d.trans_b, d.trans_c,
                                               d._shuffle_int(), params.a_inds.shape, params.b_inds.shape,
                                               params.c_inds.shape)
        return ("gemm", d.dtype_a, d.dtype_b, d.dtype_c, d.trans_a, d.trans_b, d.trans_c, d._shuffle_int(),
                _bucket(m), n, _bucket(k), params.split_k_slices > 1)

    def tune_gemm(self, params: GemmParams, desps: Optional[List[GemmAlgoDesp]] = None) -> TuneResult:
        key = self.gemm_key(params)
        hit = self.cache.get(key)
        if hit is not None:
            params.algo_desp = hit.desp
            return hit
        cands = gemm_candidates(params, desps)
        if not cands:
            raise RuntimeError("can't find any suitable algo for your parameters.")
        ctx = _stream_ctx(params.stream)
        saved = _save(params.c, ctx)
        tried = []
        for d in cands:
            params.algo_desp = d
            try:
                ms = _time_calls(lambda: GemmMainUnitTest.matmul2(params), params.stream, self.steps, self.warmup)
            except (RuntimeError, ValueError):
                continue
            tried.append((str(d), ms))
            params.c.copy_(saved, ctx)
        if not tried:
            raise RuntimeError("can't find any suitable algo for your parameters.")
        best = min(tried, key=lambda t: t[1])
        res = TuneResult([d for d in cands if str(d) == best[0]][0], best[1], tried)
        params.algo_desp = res.desp
        self.cache[key] = res
        return res
