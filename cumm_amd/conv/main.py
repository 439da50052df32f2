"""``ConvMainUnitTest``: the sparse-convolution operator surface (implicit_gemm2).

Host prelude of the reference's generated ``implicit_gemm2``
(cumm/conv/main.py:483-745 with cumm/conv/nvrtc_code.py:20-197): validation,
m/n/k, operand permutation by op type, source-pointer rules and workspace; the
launch goes through the C ABI (``cumm_hip_sparse_conv``).  Only mask-based
sparse convolution (``mask_sparse``) is built; dense NHWC convolution is not.
"""
import ctypes
from typing import List, Tuple

from .. import _capi
from ..gemm.main import (INT_MAX, _check_device, _check_dtype, _check_shape, _enum_int, _ptr,
                         desp_from_c, desp_to_c)
from ..tensorview import Tensor, empty, float32, int32, uint8, uint32
from ..tensorview.gemm import (ConvAlgoDesp, ConvOpType, ConvParams, gemm_abc_012_to_iwo,
                               implicit_gemm_mnk)


def conv_desp_to_c(desp: ConvAlgoDesp) -> _capi.ConvDesc:
    c = _capi.ConvDesc()
    c.gemm = desp_to_c(desp)
    c.ndim = desp.ndim
    c.op_type = _enum_int(desp.op_type)
    c.mask_sparse = int(desp.mask_sparse)
    c.increment_k_first = int(desp.increment_k_first)
    c.dynamic_mask = int(desp.dynamic_mask)
    c.is_int8_inference = int(desp.is_int8_inference)
    return c


class ConvMainUnitTest:
    """Static operator functions, as the reference's pybind class."""

    @staticmethod
    def get_all_conv_algo_desp() -> List[ConvAlgoDesp]:
        """cumm/conv/main.py:983-1050 of the reference."""
        L = _capi.lib()
        n = L.cumm_hip_list_conv_algos(None, 0)
        arr = (_capi.ConvDesc * n)()
        L.cumm_hip_list_conv_algos(arr, n)
        out = []
        for i in range(n):
            d = ConvAlgoDesp(arr[i].ndim, ConvOpType(arr[i].op_type))
            desp_from_c(arr[i].gemm, d)
            d.mask_sparse = bool(arr[i].mask_sparse)
            d.increment_k_first = bool(arr[i].increment_k_first)
            d.dynamic_mask = bool(arr[i].dynamic_mask)
            d.is_int8_inference = bool(arr[i].is_int8_inference)
            out.append(d)
        return out

    @staticmethod
    def extract_mnk(op_type, N: int, C: int, K: int, kernel_volume: int, in_prod: int,
                    out_prod: int, mask_sparse: bool) -> Tuple[int, int, int]:
        """cumm/conv/main.py:467-481 of the reference."""
        return tuple(implicit_gemm_mnk(op_type, N, C, K, kernel_volume, in_prod, out_prod,
                                       mask_sparse))

    @staticmethod
    def implicit_gemm2_static_workspace(params: ConvParams) -> None:
        """``implicit_gemm2`` for callers that must not allocate device memory: the workspace a
        backward-weight call needs is an array of ``_capi.STATIC_WORKSPACE_BYTES`` bytes inside
        the library (``cumm_hip_sparse_conv_static_ws``); ``params.workspace`` is ignored and
        never assigned.  A problem that needs more raises ValueError.  Calls that overlap in
        time on one GPU share that array and race."""
        ConvMainUnitTest._implicit_gemm2(params, True)

    @staticmethod
    def implicit_gemm2(params: ConvParams) -> None:
        ConvMainUnitTest._implicit_gemm2(params, False)

    @staticmethod
    def _implicit_gemm2(params: ConvParams, static_ws: bool) -> None:
        desp = params.conv_algo_desp
        # A call whose parameter object has not changed since it was last validated goes
        # straight to the C ABI with the argument block prepared then.
        prep = params.__dict__.get("_prepared_static" if static_ws else "_prepared")
        if prep is not None and prep[0] == (params._version, desp._version, desp.tile_shape[0],
                                            desp.tile_shape[1], desp.tile_shape[2]):
            status = prep[1](prep[2], prep[3], params.stream)
            if status:
                _capi.check(status)
            return
        if not desp.mask_sparse:
            raise RuntimeError("can't find any suitable algo for your parameters. "
                               "(dense convolution is not built)")
        op_type = ConvOpType(desp.op_type)
        inp, weight, output = params.input, params.weight, params.output
        bias, scale, output_add = params.bias, params.scale, params.output_add
        indices, mask, mask_argsort = params.indices, params.mask, params.mask_argsort
        mask_output, mask_width = params.mask_output, params.mask_width
        split_k_slices = params.split_k_slices
        if inp.ndim != 2:
            raise RuntimeError("error")
        if weight.ndim != 3:
            raise RuntimeError("error")
        if output.ndim != 2:
            raise RuntimeError("error")
        if not (desp.split_k_serial or desp.split_k_parallel) and split_k_slices > 1:
            raise RuntimeError("algo don't support splitk but you provide split_k_slices > 1.")
        # tv::gemm::ConvParams::mask_int_count (params.h:413): 32-bit mask words per position.  As in
        # the reference's kernels the count follows from the descriptor and the kernel volume -
        # ceil(kernel volume / 32) with dynamic_mask, else 1 (cumm/conv/kernel.py:827-838) - and the
        # field may say the same thing or stay at its default of 1.
        mask_words = (weight.dim(1) + 31) // 32 if desp.dynamic_mask else 1
        if int(getattr(params, "mask_int_count", 1)) not in (1, mask_words):
            raise RuntimeError("mask_int_count must be %d for this descriptor and kernel volume" % mask_words)
        K = weight.dim(0)
        C = inp.dim(1)
        if output.dim(1) != K:
            raise RuntimeError("error")
        _check_device(inp, weight, output, bias, scale, output_add, indices, mask, mask_argsort,
                      mask_output)
        # The reference takes every operand through data_ptr<T>(), which throws on another
        # element type (include/tensorview/tensor.h:1497, 2027): the kernels derive all extents
        # from the descriptor's element sizes.
        _check_dtype(inp, desp.dtype_input, "input")
        _check_dtype(weight, desp.dtype_weight, "weight")
        _check_dtype(output, desp.dtype_output, "output")
        _check_dtype(indices, int32, "indices")
        _check_dtype(mask_argsort, int32, "mask_argsort")
        _check_dtype(mask, uint32, "mask")
        _check_dtype(mask_output, uint32, "mask_output")
        if desp.is_int8_inference:
            _check_dtype(bias, float32, "bias")
            _check_dtype(scale, float32, "scale")
        else:
            _check_dtype(bias, desp.dtype_output, "bias")
        inv = gemm_abc_012_to_iwo(op_type)
        iwo = [inp, weight, output]
        a_ten, b_ten, c_ten = iwo[inv[0]], iwo[inv[1]], iwo[inv[2]]
        if not desp.is_int8_inference:
            if not output_add.empty():
                raise ValueError("only int8 inference support output_add not empty ")
        else:
            if bias.empty() or scale.empty():
                raise RuntimeError("int8 inference must have both scale and bias")
        if output_add.empty():
            if desp.is_int8_inference or bias.empty():
                d_ten = c_ten
            else:
                d_ten = bias
        else:
            if output_add.dtype != output.dtype or output_add.shape != output.shape:
                raise RuntimeError("output and output_add must have same dtype and shape")
            d_ten = output_add
        if op_type == ConvOpType.BackwardWeight:
            if not (mask_width > 0 and mask_width % desp.tile_shape[2] == 0):
                raise RuntimeError("error")
        if indices.empty() or mask.empty() or mask_argsort.empty():
            raise RuntimeError("error")
        kernel_volume = weight.dim(1)
        _check_shape(indices, [kernel_volume, -1])
        N = indices.dim(1)
        if weight.dim(2) != C:
            raise RuntimeError("error")
        if op_type == ConvOpType.BackwardWeight:
            if N != output.dim(0):
                raise RuntimeError("error")
            if N * C * b_ten.itemsize >= INT_MAX or N * K * a_ten.itemsize >= INT_MAX:
                raise RuntimeError("your data exceed int32 range.")
        elif op_type == ConvOpType.Forward:
            if N != output.dim(0):
                raise RuntimeError("error")
            if N * C * a_ten.itemsize >= INT_MAX:
                raise RuntimeError("your data exceed int32 range.")
        else:
            if N * K * a_ten.itemsize >= INT_MAX:
                raise RuntimeError("your data exceed int32 range.")
            if N != inp.dim(0):
                raise RuntimeError("error")
        mnk = implicit_gemm_mnk(op_type, N, C, K, kernel_volume, -1, -1, True)
        if not desp.supported(mnk[0], mnk[1], mnk[2], C, K, mask_width):
            raise RuntimeError("error")
        if mask_argsort.dim(0) < N:
            raise RuntimeError("error")
        if op_type == ConvOpType.BackwardWeight:
            if mask.dim(0) < (N + mask_width - 1) // mask_width:
                raise RuntimeError("error")
        elif mask.size < N * mask_words or (mask.ndim == 2 and mask.dim(1) != mask_words):
            raise RuntimeError("error")
        for t in (inp, weight, output):
            if not t.is_contiguous():
                raise ValueError("input, weight and output must be contiguous")
        if (not bias.empty() and bias.dim(0) != K) or (not scale.empty() and scale.dim(0) != K):
            raise RuntimeError("bias and scale must have one entry per output channel")

        workspace_size = desp.query_conv_workspace_size(mnk[0], mnk[1], mnk[2], split_k_slices,
                                                        kernel_volume)
        ordered = bool(getattr(params, "deterministic", False)) and op_type == ConvOpType.BackwardWeight \
            and desp.split_k_parallel and split_k_slices > 1
        if ordered and params.workspace.empty():
            # the fixed-order variant keeps one partial block per workgroup: sized by the library
            workspace_size = int(_capi.lib().cumm_hip_query_wgrad_ordered_workspace(N, C, K, kernel_volume, mask_width))
            if workspace_size < 0:
                raise ValueError("the fixed-order backward-weight does not take these sizes")
        if static_ws:
            workspace = Tensor()
        else:
            if workspace_size > 0:
                if not params.workspace.empty():
                    if params.workspace.nbytes < workspace_size:
                        raise RuntimeError("workspace at least %d bytes." % workspace_size)
                else:
                    # as in the reference the allocation stays in the caller's params object
                    params.workspace = empty([workspace_size], uint8, 0)
            workspace = params.workspace

        args = _capi.SparseConvArgs()
        args.ptr_A, args.ptr_B, args.ptr_C = _ptr(a_ten), _ptr(b_ten), _ptr(c_ten)
        args.ptr_D = _ptr(d_ten)
        args.alpha, args.beta = params.alpha, params.beta
        args.act_alpha, args.act_beta = params.act_alpha, params.act_beta
        args.act_type = _enum_int(params.act_type)
        args.split_k_slices = split_k_slices
        args.workspace = _ptr(workspace)
        args.workspace_bytes = 0 if workspace.empty() else workspace.nbytes
        args.mask_ptr = _ptr(mask)
        if op_type == ConvOpType.Forward and not mask_output.empty():
            tiles = (N + desp.tile_shape[0] - 1) // desp.tile_shape[0]
            if mask_output.size < tiles * mask_words:
                raise RuntimeError("mask_output needs one word (mask_int_count words) per tile of tile_shape[0] positions")
            args.mask_out_ptr = _ptr(mask_output)
        args.indice_ptr = _ptr(indices)
        args.mask_argsort_ptr = _ptr(mask_argsort)
        args.mask_filter = params.mask_filter & 0xFFFFFFFF
        args.reverse_mask = int(bool(params.reverse_mask))
        args.mask_width = mask_width
        args.ndim, args.N, args.C, args.K = desp.ndim, N, C, K
        args.kernel_volume = kernel_volume
        args.mode, args.groups = 1, 1      # ConvMode.CrossCorrelation, ungrouped: all the reference's mask kernels do
        args.d_is_bias = int(not bias.empty())
        args.deterministic = int(ordered)
        args.bias_pointer = _ptr(bias)
        args.scale_pointer = _ptr(scale)
        args.rows_in, args.rows_out = inp.dim(0), output.dim(0)
        # (0 = not given: the launch looks for the count input preparation left on the device;
        # negative = no hint at all)
        args.light_prefix = max(-1, min(int(getattr(params, "light_prefix", 0)), N)) \
            if op_type != ConvOpType.BackwardWeight else 0
        args.ungated_rows = int(bool(getattr(params, "ungated_rows", False)))
        args.indices_by_position = int(bool(getattr(params, "indices_by_position", False))) \
            if op_type != ConvOpType.BackwardWeight else 0
        cdesc = conv_desp_to_c(desp)
        name = repr(desp) if params.timer.enable else ""
        if name:
            params.timer.record(name, params.stream)
        fn = _capi.lib().cumm_hip_sparse_conv_static_ws if static_ws else _capi.lib().cumm_hip_sparse_conv
        status = fn(ctypes.byref(cdesc), ctypes.byref(args), params.stream)
        if name:
            params.timer.record(name, params.stream)
        _capi.check(status)
        if not name:
            # remember the validated argument block (the tensors it points into stay referenced
            # by params; any later assignment to params or the descriptor invalidates it)
            params.__dict__["_prepared_static" if static_ws else "_prepared"] = (
                (params._version, desp._version, desp.tile_shape[0], desp.tile_shape[1],
                 desp.tile_shape[2]), fn, ctypes.byref(cdesc), ctypes.byref(args), cdesc, args)
