"""``GemmMainUnitTest``: the GEMM operator surface (matmul2 and helpers).

Host prelude of the reference's generated ``matmul2``
(cumm/gemm/main.py:1176-1335 with cumm/gemm/nvrtc_code.py:34-146): validation,
m/n/k extraction, workspace rules; the launch itself goes through the C ABI
(``cumm_hip_gemm``) to the hand-written gfx950 kernels.
"""
import bisect
import ctypes
from typing import Dict, List, Tuple

from .. import _capi
from ..tensorview import Tensor, empty, int32, uint8
from ..tensorview.gemm import (Activation, GemmAlgoDesp, GemmParams, ShuffleStrideType)

INT_MAX = 2 ** 31 - 1
ALGO_NAME = "Cdna4"   # GemmAlgoDesp.algo of every kernel in this build
_TENSOROP = {7: [16, 16, 32], 12: [16, 16, 32], 3: [16, 16, 64]}
_EPA = {7: 8, 12: 8, 3: 16}   # elements per 16-byte access


def _enum_int(v) -> int:
    return v.value if hasattr(v, "value") else int(v)


def desp_to_c(desp: GemmAlgoDesp) -> _capi.GemmDesc:
    d = _capi.GemmDesc()
    d.dtype_a, d.dtype_b, d.dtype_c = desp.dtype_a, desp.dtype_b, desp.dtype_c
    d.dacc, d.dcomp = desp.dacc, desp.dcomp
    d.trans_a, d.trans_b, d.trans_c = int(desp.trans_a), int(desp.trans_b), int(desp.trans_c)
    for i in range(3):
        d.tile_shape[i] = desp.tile_shape[i]
        d.warp_tile_shape[i] = desp.warp_tile_shape[i]
    d.num_stage = desp.num_stage
    d.shuffle_type = _enum_int(desp.shuffle_type)
    d.split_k_serial = int(desp.split_k_serial)
    d.split_k_parallel = int(desp.split_k_parallel)
    return d


def desp_from_c(d: _capi.GemmDesc, out: GemmAlgoDesp) -> GemmAlgoDesp:
    out.dtype_a, out.dtype_b, out.dtype_c = d.dtype_a, d.dtype_b, d.dtype_c
    out.dacc, out.dcomp = d.dacc, d.dcomp
    out.trans_a, out.trans_b, out.trans_c = bool(d.trans_a), bool(d.trans_b), bool(d.trans_c)
    out.tile_shape = list(d.tile_shape)
    out.warp_tile_shape = list(d.warp_tile_shape)
    out.num_stage = d.num_stage
    out.algo = ALGO_NAME
    out.tensorop = list(_TENSOROP[d.dtype_a])
    out.shuffle_type = ShuffleStrideType(d.shuffle_type)
    out.split_k_serial = bool(d.split_k_serial)
    out.split_k_parallel = bool(d.split_k_parallel)
    epa = _EPA[d.dtype_a]
    out.element_per_access_a = epa
    out.element_per_access_b = epa
    out.element_per_access_c = epa if d.dtype_c == d.dtype_a else 4   # 16-byte pieces of s32 / f32
    out.access_per_vector = 1
    out.min_arch = (9, 5)   # gfx950
    return out


def _check_shape(t: Tensor, shape, what="shape"):
    """tv::check_shape: -1 matches anything."""
    if t.ndim != len(shape) or any(e != -1 and e != s for s, e in zip(t.shape, shape)):
        raise ValueError("%s %s doesn't match expected %s" % (what, t.shape, list(shape)))


def _ptr(t: Tensor):
    return None if t.empty() else t.byte_pointer()


def _check_dtype(t: Tensor, dtype: int, what: str):
    """template_dtype_check of the reference's data_ptr<T>() (include/tensorview/tensor.h:1497)."""
    if not t.empty() and t.dtype != int(dtype):
        raise RuntimeError("%s has dtype %d, expected %d" % (what, t.dtype, int(dtype)))


def _check_device(*tens):
    devs = {t.device for t in tens if not t.empty()}
    if len(devs) > 1:
        raise ValueError("all tensors must be on the same device")
    if -1 in devs:
        raise RuntimeError("operands must be device tensors (call .cuda() first)")


class GemmMainUnitTest:
    """Static operator functions, as the reference's pybind class."""

    @staticmethod
    def get_all_algo_desp() -> List[GemmAlgoDesp]:
        """cumm/gemm/main.py:914-965 of the reference."""
        L = _capi.lib()
        n = L.cumm_hip_list_gemm_algos(None, 0)
        arr = (_capi.GemmDesc * n)()
        L.cumm_hip_list_gemm_algos(arr, n)
        return [desp_from_c(arr[i], GemmAlgoDesp()) for i in range(n)]

    @staticmethod
    def extract_mnk(a_shape, b_shape, trans_a, trans_b, trans_c, shuffle_type=0,
                    a_inds_shape=(), b_inds_shape=(), c_inds_shape=()) -> Tuple[int, int, int]:
        """cumm/gemm/main.py:967-1026 of the reference."""
        a_shape, b_shape = list(a_shape), list(b_shape)
        shuffle_type = _enum_int(shuffle_type)
        if trans_c:
            trans_a, trans_b = (not trans_b), (not trans_a)
            a_shape, b_shape = b_shape, a_shape
        if shuffle_type == ShuffleStrideType.ShuffleAC.value:
            if trans_a:
                raise RuntimeError("a of shuffle AB must be row major")
            if not len(c_inds_shape):
                raise RuntimeError("c_inds must not empty")
            m = a_inds_shape[0] if len(a_inds_shape) else a_shape[0]
            k = a_shape[int(not trans_a)]
            n = b_shape[int(not trans_b)]
        elif shuffle_type == ShuffleStrideType.ShuffleAB.value:
            if not len(a_inds_shape) or not len(b_inds_shape):
                raise RuntimeError("a_inds and c_inds must not empty")
            if not (trans_a and not trans_b):
                raise RuntimeError("shuffle AB must be nt, i.e. backward weight")
            m = a_shape[int(trans_a)]
            k = a_inds_shape[0]
            n = b_shape[int(not trans_b)]
        else:
            m = a_shape[int(trans_a)]
            k = a_shape[int(not trans_a)]
            n = b_shape[int(not trans_b)]
        return int(m), int(n), int(k)

    @staticmethod
    def align_to_power2(val: int) -> int:
        """cumm/gemm/main.py:1028-1046 of the reference."""
        r, ones = 0, val & 1
        while True:
            val >>= 1
            if not val:
                break
            r += 1
            ones += val & 1
        return (1 << r) if ones == 1 else (1 << (r + 1))

    @staticmethod
    def device_synchronize() -> None:
        _capi.check(_capi.lib().cumm_hip_device_synchronize())

    @staticmethod
    def stream_synchronize(stream: int) -> None:
        _capi.check(_capi.lib().cumm_hip_stream_synchronize(stream))

    @staticmethod
    def simple_select_tile_shape(m: int, n: int, k: int, tile_ms: List[int], tile_ns: List[int],
                                 tile_ks: List[int], tile_shape_to_algos: Dict[int, List[int]],
                                 large_k_first: bool) -> List[int]:
        """cumm/gemm/main.py:1072-1134 of the reference: the smallest listed tile
        >= each extent (the largest if none), then walk down until a key
        ``tm | tn << 20 | tk << 40`` is present."""
        def start(vals, x):
            i = bisect.bisect_left(vals, x)
            return min(i, len(vals) - 1)
        im, in_, ik = start(tile_ms, m), start(tile_ns, n), start(tile_ks, k)
        if large_k_first:
            order = ((a, b, c) for c in range(ik, -1, -1) for b in range(in_, -1, -1)
                     for a in range(im, -1, -1))
        else:
            order = ((a, b, c) for a in range(im, -1, -1) for b in range(in_, -1, -1)
                     for c in range(ik, -1, -1))
        for a, b, c in order:
            key = tile_ms[a] | (tile_ns[b] << 20) | (tile_ks[c] << 40)
            if key in tile_shape_to_algos:
                return tile_shape_to_algos[key]
        return []

    @staticmethod
    def matmul2(params: GemmParams) -> None:
        """C = act(alpha * op(A) @ op(B) + beta * D) with optional row gather /
        scatter; prelude cumm/gemm/nvrtc_code.py:34-146 of the reference."""
        desp = params.algo_desp
        prep = params.__dict__.get("_prepared")
        if prep is not None and prep[0] == (params._version, desp._version, desp.tile_shape[0],
                                            desp.tile_shape[1], desp.tile_shape[2]):
            status = prep[1](prep[2], prep[3], params.stream)
            if status:
                _capi.check(status)
            return
        params.check_valid()
        a, b, c = params.a, params.b, params.c
        d = params.d if not params.d.empty() else c
        _check_shape(a, [-1, -1])
        _check_shape(b, [-1, -1])
        _check_shape(c, [-1, -1])
        _check_device(a, b, c, d, params.a_inds, params.b_inds, params.c_inds)
        _check_dtype(a, desp.dtype_a, "a")
        _check_dtype(b, desp.dtype_b, "b")
        _check_dtype(c, desp.dtype_c, "c")
        _check_dtype(d, desp.dtype_c, "d")
        for name in ("a_inds", "b_inds", "c_inds"):
            _check_dtype(getattr(params, name), int32, name)
        a_ten, b_ten = a, b
        trans_a, trans_b, trans_c = desp.trans_a, desp.trans_b, desp.trans_c
        if trans_c:
            trans_a, trans_b = (not trans_b), (not trans_a)
            a_ten, b_ten = b_ten, a_ten
        split_k_slices = params.split_k_slices
        if not (desp.split_k_serial or desp.split_k_parallel) and split_k_slices > 1:
            raise RuntimeError("algo don't support splitk but you provide split_k_slices > 1.")
        st = desp._shuffle_int()
        a_inds, b_inds, c_inds = params.a_inds, params.b_inds, params.c_inds
        isz = lambda t: t.itemsize
        if st == ShuffleStrideType.ShuffleAC.value:
            if trans_a:
                raise RuntimeError("a of shuffle AB must be row major")
            m = a_inds.dim(0) if not a_inds.empty() else a.dim(0)
            if a.dim(0) * a.dim(1) * isz(a) >= INT_MAX:
                raise RuntimeError("your data exceed int32 range.")
            k = a_ten.dim(int(not trans_a))
            k2 = b_ten.dim(int(trans_b))
            n = b_ten.dim(int(not trans_b))
            _check_shape(c, [-1, n])
            if c_inds.dim(0) < m:
                raise RuntimeError("c_inds must hold one row number per gathered row")
        elif st == ShuffleStrideType.ShuffleAB.value:
            if not (trans_a and not trans_b):
                raise RuntimeError("shuffle AB must be nt, i.e. backward weight")
            m = a_ten.dim(int(trans_a))
            k = a_inds.dim(0)
            k2 = b_inds.dim(0)
            n = b_ten.dim(int(not trans_b))
            if a.dim(0) * a.dim(1) * isz(a) >= INT_MAX or b.dim(0) * b.dim(1) * isz(b) >= INT_MAX:
                raise RuntimeError("your data exceed int32 range.")
            # m and n are those of the swapped problem when trans_c is set, so C (stored
            # transposed, [n_orig, m_orig]) is always [m, n] here
            _check_shape(c, [m, n])
        else:
            m = a_ten.dim(int(trans_a))
            k = a_ten.dim(int(not trans_a))
            k2 = b_ten.dim(int(trans_b))
            n = b_ten.dim(int(not trans_b))
            _check_shape(c, [m, n])
        if not desp.supported(m, n, k):
            raise ValueError("this m, n, k isn't supported due to misaligned contiguous dim.")
        if k != k2:
            raise ValueError("error")
        if d.ndim == 1 and d.dim(0) != n:
            raise RuntimeError("d must be a valid bias")
        for t in (a, b, c) + ((d,) if d.ndim == 2 else ()):
            if t.stride[1] != 1:
                raise ValueError("operands must be contiguous along their last dimension")

        workspace = params.workspace
        workspace_size = desp.query_workspace_size(m, n, k, split_k_slices)
        if workspace_size > 0:
            if not workspace.empty():
                if workspace.nbytes < workspace_size:
                    raise RuntimeError("workspace at least %d bytes." % workspace_size)
            else:
                workspace = empty([workspace_size], uint8, 0)

        args = _capi.GemmArgs()
        args.m, args.n, args.k = m, n, k
        # as the reference's prelude: with trans_c the operands arrive swapped
        args.ptr_A, args.ptr_B, args.ptr_C = _ptr(a_ten), _ptr(b_ten), _ptr(c)
        args.ptr_D = _ptr(d)
        args.stride_A, args.stride_B, args.stride_C = a_ten.stride[0], b_ten.stride[0], c.stride[0]
        args.stride_D = 0 if d.ndim == 1 else d.stride[0]
        if st == ShuffleStrideType.ShuffleAC.value:
            args.indiceA = _ptr(a_inds)
            args.indiceBorC = _ptr(c_inds)
            args.indiceD = None if d.ndim == 1 else _ptr(c_inds)
        elif st == ShuffleStrideType.ShuffleAB.value:
            args.indiceA = _ptr(a_inds)
            args.indiceBorC = _ptr(b_inds)
        args.alpha, args.beta = params.alpha, params.beta
        args.act_alpha, args.act_beta = params.act_alpha, params.act_beta
        args.act_type = _enum_int(params.act_type)
        args.split_k_slices = split_k_slices
        args.workspace = _ptr(workspace)
        args.workspace_bytes = 0 if workspace.empty() else workspace.nbytes
        args.rows_A, args.rows_B, args.rows_C = a_ten.dim(0), b_ten.dim(0), c.dim(0)
        cdesc = desp_to_c(desp)
        name = repr(desp) if params.timer.enable else ""
        if name:
            params.timer.record(name, params.stream)
        fn = _capi.lib().cumm_hip_gemm
        status = fn(ctypes.byref(cdesc), ctypes.byref(args), params.stream)
        if name:
            params.timer.record(name, params.stream)
        _capi.check(status)
        if not name:
            # validated argument block for unchanged repeat calls; the workspace it may point to
            # is kept alive with it
            params.__dict__["_prepared"] = (
                (params._version, desp._version, desp.tile_shape[0], desp.tile_shape[1],
                 desp.tile_shape[2]), fn, ctypes.byref(cdesc), ctypes.byref(args), cdesc, args,
                workspace)
