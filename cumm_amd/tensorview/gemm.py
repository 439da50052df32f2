"""``tv.gemm``: descriptors and parameter bundles of the GEMM / sparse-conv operators.

Python mirror of the reference's operator ABI
(include/tensorview/gemm/core/params.h, utils.h, constants.h; Python attributes
bound in cumm/tensorview_bind.py:170-467): same attribute names, same validation
and the same exception classes (TV_ASSERT_RT_ERR -> RuntimeError,
TV_ASSERT_INVALID_ARG -> ValueError).
"""
import copy as _copy
import enum
from typing import List, Tuple


# ---- enums: include/tensorview/gemm/core/constants.h:20-55, names as bound in
# cumm/tensorview_bind.py:170-210
class ConvOpType(enum.Enum):
    Forward = 0
    BackwardInput = 1
    BackwardWeight = 2


class ConvMode(enum.Enum):
    Convolution = 0
    CrossCorrelation = 1


class ConvIterAlgo(enum.Enum):
    Analytic = 0
    Optimized = 1


class ConvLayoutType(enum.Enum):
    ChannelFirst = 0
    ChannelLast = 1
    SpatialFirst = 2


class ShuffleStrideType(enum.Enum):
    NoShuffle = 0
    ShuffleAC = 1
    ShuffleAB = 2


class SparseConvAlgo(enum.Enum):
    Native = 0
    MaskImplicitGemm = 1
    MaskSplitImplicitGemm = 2


class Activation(enum.Enum):
    None_ = 0
    ReLU = 1
    Sigmoid = 2
    LeakyReLU = 3


_UNKNOWN = -1
_SHORT = {5: "b1", 0: "f32", 3: "s8", 2: "s16", 1: "s32", 4: "f64", 8: "s64", 6: "u8", 9: "u16",
          10: "u32", 11: "u64", 7: "f16", 14: "e4m3", 15: "e5m2", 100: "x16", 101: "x32",
          102: "x48", 103: "x64", 104: "x80", 105: "x96", 106: "x128", 13: "tf32", 12: "bf16"}
_ITEMSIZE = {5: 1, 7: 2, 0: 4, 4: 8, 3: 1, 2: 2, 1: 4, 8: 8, 6: 1, 9: 2, 10: 4, 11: 8, 12: 2,
             13: 4}


def dtype_short_str(dtype: int) -> str:
    """tv::dtype_short_str, include/tensorview/dtypes.h:217-268."""
    return _SHORT.get(int(dtype), "unknown")


def div_up(a: int, b: int) -> int:
    return (a + b - 1) // b


def get_logical_tile_count(m, n, k, tile_m, tile_n, split_k_slices) -> List[int]:
    """include/tensorview/gemm/core/utils.h:21-28."""
    return [div_up(m, tile_m), div_up(n, tile_n), split_k_slices]


def get_gemm_k_size_per_split(k: int, split_k: int, tile_k: int) -> int:
    """include/tensorview/gemm/core/utils.h:30-37."""
    return div_up(div_up(k, tile_k), split_k) * tile_k


def get_spconv_logical_tile_count(m, n, k, tile_m, tile_n, split_k_slices, kv,
                                  op_type: ConvOpType) -> List[int]:
    """include/tensorview/gemm/core/utils.h:39-60: for backward weight every
    kernel offset gets its own column blocks, ceil(C / tile_n) * kv."""
    if ConvOpType(op_type) == ConvOpType.BackwardWeight:
        c = n // kv
        gy = div_up(c, tile_n) * kv
    else:
        gy = div_up(n, tile_n)
    return [div_up(m, tile_m), gy, split_k_slices]


def implicit_gemm_mnk(op_type, N, C, K, kernel_volume, in_prod, out_prod,
                      mask_sparse) -> List[int]:
    """include/tensorview/gemm/core/utils.h:62-92."""
    op_type = ConvOpType(op_type)
    if mask_sparse:
        if op_type == ConvOpType.Forward:
            return [N, K, C * kernel_volume]
        if op_type == ConvOpType.BackwardInput:
            return [N, C, K * kernel_volume]
        return [K, C * kernel_volume, N]
    if op_type == ConvOpType.Forward:
        return [N * out_prod, K, C * kernel_volume]
    if op_type == ConvOpType.BackwardInput:
        return [N * in_prod, C, K * kernel_volume]
    return [K, C * kernel_volume, N * out_prod]


def conv_iwo_012_to_abc(op_type) -> List[int]:
    """include/tensorview/gemm/core/utils.h:93-106."""
    return {ConvOpType.Forward: [0, 1, 2], ConvOpType.BackwardInput: [2, 1, 0],
            ConvOpType.BackwardWeight: [1, 2, 0]}[ConvOpType(op_type)]


def gemm_abc_012_to_iwo(op_type) -> List[int]:
    """include/tensorview/gemm/core/utils.h:107-121."""
    return {ConvOpType.Forward: [0, 1, 2], ConvOpType.BackwardInput: [2, 1, 0],
            ConvOpType.BackwardWeight: [2, 0, 1]}[ConvOpType(op_type)]


class NVRTCParams:
    """Placeholder for the reference's run-time compiled kernels
    (include/tensorview/gemm/core/nvrtc_bases.h): kernels here are built ahead of
    time, so ``cumodule`` is always None."""

    def __init__(self):
        self.cumodule = None
        self.kernel_name = ""
        self.init_kernel_name = ""
        self.constant_name = ""
        self.param_size = -1
        self.param_storage = None
        self.param_storage_cpu = None
        self.num_threads = -1
        self.smem_size = -1
        self.mode = -1


class _Versioned:
    """Counts attribute assignments so that the operators can tell cheaply whether a
    parameter object changed since they last validated it."""
    _version = 0

    def __setattr__(self, name, value):
        object.__setattr__(self, name, value)   # honours the property setters
        d = self.__dict__
        d["_version"] = d.get("_version", 0) + 1


class GemmAlgoDesp(_Versioned):
    """tv::gemm::GemmAlgoDesp, include/tensorview/gemm/core/params.h:24-164."""

    def __init__(self):
        self.dtype_a = _UNKNOWN
        self.dtype_b = _UNKNOWN
        self.dtype_c = _UNKNOWN
        self.trans_a_ = -1
        self.trans_b_ = -1
        self.trans_c_ = -1
        self.tile_shape = [-1, -1, -1]
        self.warp_tile_shape = [-1, -1, -1]
        self.num_stage = -1
        self.dacc = _UNKNOWN
        self.dcomp = _UNKNOWN
        self.algo = ""
        self.tensorop = [-1, -1, -1]
        self.split_k_serial_ = 0
        self.split_k_parallel_ = 0
        self.shuffle_type = ShuffleStrideType.NoShuffle
        self.element_per_access_a = -1
        self.element_per_access_b = -1
        self.element_per_access_c = -1
        self.access_per_vector = 1
        self.is_nvrtc = False
        self.min_arch = (0, 0)

    # bool-valued properties over the int fields (params.h:79-82, 108-113)
    trans_a = property(lambda s: s.trans_a_ == 1, lambda s, v: setattr(s, "trans_a_", 1 if v else 0))
    trans_b = property(lambda s: s.trans_b_ == 1, lambda s, v: setattr(s, "trans_b_", 1 if v else 0))
    trans_c = property(lambda s: s.trans_c_ == 1, lambda s, v: setattr(s, "trans_c_", 1 if v else 0))
    split_k_serial = property(lambda s: s.split_k_serial_ == 1,
                              lambda s, v: setattr(s, "split_k_serial_", 1 if v else 0))
    split_k_parallel = property(lambda s: s.split_k_parallel_ == 1,
                                lambda s, v: setattr(s, "split_k_parallel_", 1 if v else 0))

    def copy(self):
        # (every field is a number, a string, an enum, a tuple or a flat list of numbers: a new
        # object with new lists, without deepcopy's bookkeeping - this runs per operator call in
        # the callers that build their parameter objects afresh)
        other = object.__new__(type(self))
        d = other.__dict__
        for k, v in self.__dict__.items():
            d[k] = list(v) if isinstance(v, list) else v
        return other

    def _shuffle_int(self) -> int:
        st = self.shuffle_type
        return st.value if isinstance(st, ShuffleStrideType) else int(st)

    def check_valid(self):
        """params.h:83-107."""
        if not (self.trans_a_ != -1 and self.trans_b_ != -1 and self.trans_c_ != -1 and self.algo):
            raise RuntimeError("trans_a, trans_b, trans_c and algo must be set")
        for i in range(3):
            if not (self.tile_shape[i] > 0 and self.warp_tile_shape[i] > 0):
                raise RuntimeError("tile_shape and warp_tile_shape must be set, but they are %s %s"
                                   % (list(self.tile_shape), list(self.warp_tile_shape)))
        if self.algo not in ("Simt", "SimtDP4A", "SimtDP2A"):
            for i in range(3):
                if not self.tensorop[i] > 0:
                    raise RuntimeError("tensorop must be set, but they are %s" % list(self.tensorop))
        if _UNKNOWN in (self.dtype_a, self.dtype_b, self.dtype_c):
            raise RuntimeError("dacc and dcomp must be set to valid value")
        if _UNKNOWN in (self.dacc, self.dcomp):
            raise RuntimeError("dacc and dcomp must be set to valid value")
        if not self.num_stage > 0:
            raise RuntimeError("num_stage must larger than zero")

    def __repr__(self):
        """Kernel name string, params.h:56-78."""
        self.check_valid()
        s = self.algo + "_" + "".join(dtype_short_str(d) for d in
                                      (self.dtype_a, self.dtype_b, self.dtype_c, self.dacc, self.dcomp))
        s += ("n" if self.trans_a else "t") + ("n" if self.trans_b else "t") + \
             ("n" if self.trans_c else "t")
        s += "_m%dn%dk%d" % tuple(self.tile_shape)
        s += "m%dn%dk%d" % tuple(self.warp_tile_shape)
        s += "A%d" % self.access_per_vector
        if self.tensorop[0] != -1:
            s += "T%d%d%d" % tuple(self.tensorop)
        s += "_%d" % self.num_stage
        s += ("1" if self.split_k_serial else "0") + ("1" if self.split_k_parallel else "0")
        if self._shuffle_int() != 0:
            s += "_S%d" % self._shuffle_int()
        return s

    def query_workspace_size(self, m: int, n: int, k: int, split_k_slices: int) -> int:
        """params.h:115-132."""
        tiles = get_logical_tile_count(m, n, k, self.tile_shape[0], self.tile_shape[1],
                                       split_k_slices)
        if split_k_slices > 1:
            if self.split_k_serial:
                return 4 * tiles[0] * tiles[1]
            if self.split_k_parallel:
                return _ITEMSIZE[self.dacc] * m * n * tiles[2]
            raise ValueError("not impemented")
        return 0

    def supported(self, m: int, n: int, k: int) -> bool:
        """params.h:133-149: alignment of the contiguous dimensions."""
        lda = m if self.trans_a else k
        ldb = k if self.trans_b else n
        ldc = m if self.trans_c else n
        return self.supported_ldx(lda, ldb, ldc)

    def supported_ldx(self, lda: int, ldb: int, ldc: int) -> bool:
        """params.h:150-163."""
        res = True
        if self.element_per_access_a > 0:
            res &= lda % self.element_per_access_a == 0
        if self.element_per_access_b > 0:
            res &= ldb % self.element_per_access_b == 0
        if self.element_per_access_c > 0:
            res &= ldc % self.element_per_access_c == 0
        return res


class ConvAlgoDesp(GemmAlgoDesp):
    """tv::gemm::ConvAlgoDesp, params.h:166-327."""

    def __init__(self, ndim: int, op_type):
        super().__init__()
        self.ndim = ndim
        self.op_type = ConvOpType(op_type) if not isinstance(op_type, ConvOpType) else op_type
        self.iter_algo = ConvIterAlgo.Optimized
        self.layout_i = ConvLayoutType.ChannelLast
        self.layout_w = ConvLayoutType.ChannelLast
        self.layout_o = ConvLayoutType.ChannelLast
        self.interleave_i = 1
        self.interleave_w = 1
        self.interleave_o = 1
        self.mask_sparse = False
        self.increment_k_first = False
        self.conv2gemm_inds = conv_iwo_012_to_abc(self.op_type)
        self.gemm2conv_inds = gemm_abc_012_to_iwo(self.op_type)
        self.dynamic_mask = False
        self.is_int8_inference = False

    conv_iwo_012_to_abc = staticmethod(conv_iwo_012_to_abc)
    gemm_abc_012_to_iwo = staticmethod(gemm_abc_012_to_iwo)

    def __repr__(self):
        """params.h:197-232."""
        s = GemmAlgoDesp.__repr__(self)
        s += "_C%d%d%d" % (self.ndim, ConvOpType(self.op_type).value,
                           ConvIterAlgo(self.iter_algo).value)
        for lay, inter in ((self.layout_i, self.interleave_i), (self.layout_w, self.interleave_w),
                           (self.layout_o, self.interleave_o)):
            s += "F" if ConvLayoutType(lay) == ConvLayoutType.ChannelFirst else "L"
            if inter > 1:
                s += str(inter)
        if self.mask_sparse:
            s += "_" + ("SK" if self.increment_k_first else "SF")
        if self.dynamic_mask:
            s += "D"
        if self.is_int8_inference:
            s += "_S8"
        return s

    @property
    def dtype_input(self) -> int:
        return (self.dtype_a, self.dtype_b, self.dtype_c)[self.conv2gemm_inds[0]]

    @property
    def dtype_weight(self) -> int:
        return (self.dtype_a, self.dtype_b, self.dtype_c)[self.conv2gemm_inds[1]]

    @property
    def dtype_output(self) -> int:
        return (self.dtype_a, self.dtype_b, self.dtype_c)[self.conv2gemm_inds[2]]

    def supported(self, m: int, n: int, k: int, C: int = None, K: int = None,
                  mask_width: int = None) -> bool:
        """params.h:266-285."""
        res = GemmAlgoDesp.supported(self, m, n, k)
        if C is None:
            return res
        if self.mask_sparse:
            op = ConvOpType(self.op_type)
            if op == ConvOpType.Forward:
                res &= C % self.element_per_access_a == 0
            elif op == ConvOpType.BackwardInput:
                res &= K % self.element_per_access_a == 0
            else:
                res &= mask_width % self.tile_shape[2] == 0
                res &= K % self.element_per_access_a == 0
                res &= C % self.element_per_access_b == 0
        return bool(res)

    def query_conv_workspace_size(self, m: int, n: int, k: int, split_k_slices: int,
                                  kv: int) -> int:
        """params.h:286-307."""
        if not self.mask_sparse:
            return self.query_workspace_size(m, n, k, split_k_slices)
        tiles = get_spconv_logical_tile_count(m, n, k, self.tile_shape[0], self.tile_shape[1],
                                              split_k_slices, kv, self.op_type)
        if split_k_slices > 1:
            if self.split_k_serial:
                return 4 * tiles[0] * tiles[1]
            if self.split_k_parallel:
                return _ITEMSIZE[self.dacc] * m * n * tiles[2]
            raise ValueError("not impemented")
        return 0

    def supported_ldx_conv(self, ldi: int, ldw: int, ldo: int) -> bool:
        """params.h:308-326."""
        epas = (self.element_per_access_a, self.element_per_access_b, self.element_per_access_c)
        res = True
        for ld, idx in ((ldi, 0), (ldw, 1), (ldo, 2)):
            epa = epas[self.conv2gemm_inds[idx]]
            if epa > 0:
                res &= ld % epa == 0
        return res


def _empty_tensor():
    from . import Tensor
    return Tensor()


class GemmParams(_Versioned):
    """tv::gemm::GemmParams, params.h:329-390.  Setting ``a``/``b``/``c`` also
    records the dtype in ``algo_desp`` (params.h:366-383)."""

    def __init__(self, timer=None):
        from . import CUDAKernelTimer
        self.algo_desp = GemmAlgoDesp()
        self._a = _empty_tensor()
        self._b = _empty_tensor()
        self._c = _empty_tensor()
        self._d = _empty_tensor()
        self.split_k_slices = 1
        self.workspace = _empty_tensor()
        self.a_inds = _empty_tensor()
        self.b_inds = _empty_tensor()
        self.c_inds = _empty_tensor()
        self.alpha = 1.0
        self.beta = 0.0
        self.act_alpha = 0.0
        self.act_beta = 0.0
        self.act_type = Activation.None_
        self.stream = 0
        self.timer = timer if timer is not None else CUDAKernelTimer(False)
        self.nvrtc_params = NVRTCParams()

    def _set(self, name, val):
        setattr(self, "_" + name, val)
        setattr(self.algo_desp, "dtype_" + name, int(val.dtype))

    a = property(lambda s: s._a, lambda s, v: s._set("a", v))
    b = property(lambda s: s._b, lambda s, v: s._set("b", v))
    c = property(lambda s: s._c, lambda s, v: s._set("c", v))

    @property
    def d(self):
        return self._d

    @d.setter
    def d(self, val):
        if self._c.dtype != val.dtype:
            raise RuntimeError("d dtype must equal to c")
        self._d = val

    def check_valid(self):
        """params.h:353-364."""
        self.algo_desp.check_valid()
        if self._a.empty() or self._b.empty() or self._c.empty():
            raise RuntimeError("a,b,c must not empty")
        st = self.algo_desp._shuffle_int()
        if st == ShuffleStrideType.ShuffleAC.value:
            if self.c_inds.empty():
                raise RuntimeError("a_inds,c_inds tensor must not empty")
        elif st == ShuffleStrideType.ShuffleAB.value:
            if self.a_inds.empty() or self.b_inds.empty():
                raise RuntimeError("a_inds,b_inds tensor must not empty")


class ConvParams(_Versioned):
    """tv::gemm::ConvParams, params.h:392-428."""

    def __init__(self, ndim: int, op_type, timer=None):
        from . import CUDAKernelTimer
        self.conv_algo_desp = ConvAlgoDesp(ndim, op_type)
        self.input = _empty_tensor()
        self.weight = _empty_tensor()
        self.output = _empty_tensor()
        self.output_add = _empty_tensor()
        self.bias = _empty_tensor()
        self.scale = _empty_tensor()
        self.split_k_slices = 1
        self.padding: List[int] = []
        self.stride: List[int] = []
        self.dilation: List[int] = []
        self.alpha = 1.0
        self.beta = 0.0
        self.act_alpha = 0.0
        self.act_beta = 0.0
        self.act_type = Activation.None_
        self.mask_width = -1
        self.mask_filter = 0xFFFFFFFF
        self.reverse_mask = False
        self.verbose = False
        self.mask_int_count = 1
        self.timer = timer if timer is not None else CUDAKernelTimer(False)
        self.workspace = _empty_tensor()
        self.mask = _empty_tensor()
        self.mask_argsort = _empty_tensor()
        self.indices = _empty_tensor()
        self.mask_output = _empty_tensor()
        self.stream = 0
        # not in the reference's struct: backward-weight with a split_k_parallel descriptor adds its
        # partial sums in a fixed order (the same bits from run to run), as the reference's serial
        # split-K does, at the speed of the balanced kernels
        self.deterministic = False
        # not in the reference's struct either: a hint for forward / backward-input, the number of
        # leading positions of the sorted order in tiles of one or two kernel offsets
        # (pairs.light_prefix of the sorted mask).  0 = not given: the launch uses what the GPU sort
        # (pairs.sort_by_mask_device) or pairs.light_prefix_device left for this mask array in the
        # library's device-side table, if anything; negative = no hint.  Any value gives the same result.
        self.light_prefix = 0
        # not in the reference's struct: True = every position of a tile takes part in every kernel
        # offset of the tile's OR-ed mask (gated by its pair-table entry alone, the reference's
        # rule); False (default) = only in the offsets whose bit its own mask word has, which is
        # the same thing for masks made from the pair table and fetches less
        self.ungated_rows = False
        # not in the reference's struct: True = ``indices`` is the pair table in the order of the
        # sorted positions (pairs.pairs_by_position[_device]); forward / backward-input
        self.indices_by_position = False
        self.nvrtc_params = NVRTCParams()
