"""torch.Tensor <-> tv.Tensor without copies, and autograd functions around the mask-based sparse
convolution (forward = implicit_gemm2 Forward, backward = BackwardInput + BackwardWeight).

``torch2tensor`` / ``tensor2torch`` stand where the reference's ``PyTorchTools.torch2tensor`` /
``tensor2torch`` do (cumm/bindings.py:53-86 over include/tensorview/torch_utils.h).  torch is
plumbing here: it owns activations, parameters and the stream (allocation, zero fill, making a
tensor contiguous); every computing kernel that runs is this library's, including the ReLU gate
and the bias gradient of the backward pass.  Imported on demand: nothing else in the package
needs torch.
"""
import ctypes
from typing import Optional, Sequence, Tuple

import torch

from . import _capi, pairs, tuner
from . import tensorview as tv
from .conv.main import ConvMainUnitTest
from .tensorview.gemm import Activation, ConvOpType, ConvParams

_TORCH_TO_TV = {torch.float32: tv.float32, torch.float16: tv.float16, torch.bfloat16: tv.bfloat16,
                torch.int32: tv.int32, torch.int8: tv.int8, torch.uint8: tv.uint8, torch.int64: tv.int64,
                torch.int16: tv.int16, torch.float64: tv.float64, torch.bool: tv.bool_}
_TV_TO_TORCH = {v: k for k, v in _TORCH_TO_TV.items()}
# torch has no full unsigned support: tensor2torch(cast_uint_to_int=True) views them as signed
_UINT_AS_INT = {tv.uint32: torch.int32, tv.uint16: torch.int16, tv.uint64: torch.int64}
_TYPESTR = {torch.float32: "<f4", torch.float16: "<f2", torch.int32: "<i4", torch.int8: "|i1", torch.uint8: "|u1",
            torch.int64: "<i8", torch.int16: "<i2", torch.float64: "<f8", torch.bool: "|b1"}


def torch2tensor(t: torch.Tensor) -> tv.Tensor:
    """A tv.Tensor over the storage of ``t`` (any strides); ``t`` is kept alive by the view."""
    if t.dtype not in _TORCH_TO_TV:
        raise ValueError("unsupported torch dtype %s" % t.dtype)
    device = t.device.index if t.is_cuda else -1
    if t.is_cuda and device is None:
        device = torch.cuda.current_device()
    return tv.from_blob_strided(t.data_ptr(), list(t.shape), list(t.stride()), _TORCH_TO_TV[t.dtype], device,
                                keepalive=t)


class _DeviceArray:
    """What torch.as_tensor needs to wrap device memory in place."""

    def __init__(self, ten: tv.Tensor, typestr: str, itemsize: int):
        self._keep = ten
        self.__cuda_array_interface__ = {
            "shape": tuple(ten.shape), "typestr": typestr, "data": (ten.byte_pointer(), False), "version": 2,
            "strides": tuple(s * itemsize for s in ten.stride)}


def tensor2torch(ten: tv.Tensor, clone: bool = True, cast_uint_to_int: bool = False) -> torch.Tensor:
    """The reference's signature (clone=True copies; clone=False shares the memory and keeps ``ten``
    alive)."""
    dt = ten.dtype
    if dt in _UINT_AS_INT:
        if not cast_uint_to_int:
            raise ValueError("torch has no such unsigned type: pass cast_uint_to_int=True")
        tdt = _UINT_AS_INT[dt]
    elif dt in _TV_TO_TORCH:
        tdt = _TV_TO_TORCH[dt]
    else:
        raise ValueError("unsupported tv dtype %d" % dt)
    if ten.empty():
        return torch.empty(list(ten.shape), dtype=tdt, device="cuda" if ten.device >= 0 else "cpu")
    if ten.device < 0:
        arr = ten.numpy_view()
        res = torch.from_numpy(arr).view(tdt) if tdt != torch.bfloat16 else torch.from_numpy(arr).view(torch.bfloat16)
    else:
        carrier = torch.int16 if tdt == torch.bfloat16 else tdt
        res = torch.as_tensor(_DeviceArray(ten, _TYPESTR[carrier], ten.itemsize), device="cuda:%d" % ten.device)
        if tdt == torch.bfloat16:
            res = res.view(torch.bfloat16)
    return res.clone() if clone else res


def current_stream() -> int:
    return int(torch.cuda.current_stream().cuda_stream)


_TUNER = tuner.Tuner(steps=3, warmup=1)


_DESP_LIKE = {}


def _desp_like(dtype, op, parallel=False, dynamic=False):
    """A descriptor of the wanted kind (the tuner then picks the tile); looked up once per kind:
    building the table of all descriptors costs more than a forward launch.  ``dynamic``: several
    mask words per position (kernel volumes above 32)."""
    key = (dtype, op, parallel, dynamic)
    if key not in _DESP_LIKE:
        for d in ConvMainUnitTest.get_all_conv_algo_desp():
            if (d.dtype_a == dtype and d.dtype_c == dtype and ConvOpType(d.op_type) == op and not d.is_int8_inference and
                    bool(d.split_k_parallel) == parallel and d.mask_sparse and bool(d.dynamic_mask) == dynamic):
                _DESP_LIKE[key] = d
                break
        else:
            raise RuntimeError("can't find any suitable algo for your parameters.")
    return _DESP_LIKE[key].copy()


class _Launch:
    """The validated argument block of one operator call, replayed with other tensors of the same
    shapes: the first call goes through the operator's prelude (and the tuner), a repeat patches the
    pointers of the tensors that change from call to call into the block and calls the C entry
    point - a layer of a network makes the same call every iteration, and the prelude costs several
    times what the kernel does."""

    _FIELDS = ("ptr_A", "ptr_B", "ptr_C", "ptr_D", "bias_pointer", "workspace")

    def __init__(self, params: ConvParams, roles):
        prep = params.__dict__.get("_prepared")
        if prep is None:
            raise RuntimeError("the operator call left no validated argument block")
        self.fn, self.cdesc, self.args = prep[1], prep[4], prep[5]
        self.params = params       # keeps the geometry's tensors alive
        self.fields = {}
        for role, t in roles.items():
            ptr = t.data_ptr()
            if t.numel() == 0:     # an empty tensor has no address to find in the block: nothing to patch
                self.fields[role] = []
                continue
            self.fields[role] = [f for f in self._FIELDS if ptr and getattr(self.args, f) == ptr]
            if not self.fields[role]:
                raise RuntimeError("the argument block does not point at the %s tensor" % role)
        # the tensors of the first call are replaced by the caller's on every replay: only the
        # geometry's stay referenced here (a backward-weight workspace can be tens of megabytes)
        from .tensorview import Tensor as _T
        for name in ("input", "weight", "output", "bias", "workspace"):
            if name in roles:
                params.__dict__[name] = _T()

    def __call__(self, stream: int, **tensors) -> None:
        for role, t in tensors.items():
            ptr = t.data_ptr()
            for f in self.fields[role]:
                setattr(self.args, f, ptr)
        status = self.fn(ctypes.byref(self.cdesc), ctypes.byref(self.args), stream)
        if status:
            _capi.check(status)


class SparseConvGeometry:
    """Pair tables, masks and sorts of one convolution geometry, built on the GPU once and shared by
    every layer (and every pass) that uses it.  Kernel volumes up to 32 have one mask word per
    position; above that (up to 128, e.g. 5 x 5 x 5) the masks have ``ceil(kv / 32)`` words, forward
    and backward-input run on the ``dynamic_mask`` descriptors, and backward-weight - which has no
    such kernel, in the reference neither - goes offset by offset over the pair lists."""

    def __init__(self, coords: torch.Tensor, spatial_shape: Sequence[int], ksize=(3, 3, 3), stride=None,
                 padding=(1, 1, 1), dilation=(1, 1, 1), batch_size: int = 1):
        if coords.dtype != torch.int32 or not coords.is_cuda or coords.dim() != 2 or coords.shape[1] != 4:
            raise ValueError("coords must be a cuda int32 tensor [N, 4] of (batch, z, y, x)")
        coords = coords.contiguous()
        stream = current_stream()
        c_tv = torch2tensor(coords)
        self.subm = stride is None
        self.n_in = int(coords.shape[0])
        self.kv = int(ksize[0]) * int(ksize[1]) * int(ksize[2])
        if self.subm:
            t = pairs.subm_pairs_device(c_tv, spatial_shape, ksize, dilation, stream=stream)
            self.out_coords, self.out_shape = coords, tuple(int(s) for s in spatial_shape)
        else:
            t = pairs.sparse_conv_pairs_device(c_tv, spatial_shape, ksize, stride, padding, dilation,
                                               batch_size=batch_size, stream=stream)
            self.out_coords, self.out_shape = tensor2torch(t.out_coords, clone=False), t.out_shape
        self.indices_fwd, self.indices_bwd = t.indices_fwd, t.indices_bwd
        self.n_out = int(t.indices_fwd.dim(1))
        self.words = (self.kv + 31) // 32
        self.lists = None
        if self.kv > 32:
            # the builders give no masks for these volumes: made from the tables, sorted by offset
            # count and word pattern; the per-offset lists serve backward-weight
            mf = pairs.masks_from_pairs_device(t.indices_fwd, stream=stream)
            self.mask_fwd, self.order_fwd = pairs.sort_by_mask_words_device(mf, stream=stream)
            if self.subm:
                self.mask_bwd, self.order_bwd = self.mask_fwd, self.order_fwd
            else:
                mb = pairs.masks_from_pairs_device(t.indices_bwd, stream=stream)
                self.mask_bwd, self.order_bwd = pairs.sort_by_mask_words_device(mb, stream=stream)
            self.lists = pairs.pair_lists_device(t.indices_fwd, stream=stream)
            self.light_fwd = self.light_bwd = 0
            self.indices_fwd_pos = pairs.pairs_by_position_device(self.indices_fwd, self.order_fwd, stream=stream)
            self.indices_bwd_pos = pairs.pairs_by_position_device(self.indices_bwd, self.order_bwd, stream=stream)
            self._reduced = {}
            self._launches = {}
            return
        # (a mask has one bit per kernel offset: a filter of that width spares the sort the passes over
        # the bits above it)
        bits = (1 << self.kv) - 1 if self.kv < 32 else 0xFFFFFFFF
        # (the library's order by offset count where the masks leave room for the count: same rows,
        # lighter tiles, and the few many-offset tiles in a short run at the end)
        by_count = self.kv <= 27
        self.mask_fwd, self.order_fwd = pairs.sort_by_mask_device(t.mask_fwd, mask_filter=bits, stream=stream,
                                                                  by_offset_count=by_count)
        if self.subm:      # the forward masks serve the backward-input pass, bit-reversed in the kernel
            self.mask_bwd, self.order_bwd = self.mask_fwd, self.order_fwd
        else:
            self.mask_bwd, self.order_bwd = pairs.sort_by_mask_device(t.mask_bwd, mask_filter=bits, stream=stream,
                                                                      by_offset_count=by_count)
        # (how far the light end of each sorted order reaches - the hint of the forward and
        # backward-input launches - stays on the device: the sort leaves it in the library's table
        # under the sorted array's address and the launches look it up there; 0 = not given here)
        self.light_fwd = self.light_bwd = 0
        # the pair tables once more in the order of the sorted positions: what forward and
        # backward-input read (a tile's entries for one offset are then consecutive in memory);
        # backward-weight keeps the table by row
        self.indices_fwd_pos = pairs.pairs_by_position_device(self.indices_fwd, self.order_fwd, stream=stream)
        self.indices_bwd_pos = pairs.pairs_by_position_device(self.indices_bwd, self.order_bwd, stream=stream)
        self._reduced = {}
        self._launches = {}      # validated calls of the layers on this geometry, see _Launch

    def reduced_mask_buffer(self, width: int) -> tv.Tensor:
        """One word per run of ``width`` sorted output positions: the forward launch writes the
        OR of the run's masks here (its ``mask_output``), and backward-weight reads it."""
        if width not in self._reduced:
            tiles = (self.n_out + width - 1) // width
            buf = torch.zeros(max(tiles, 1), dtype=torch.int32, device=self.out_coords.device)
            self._reduced[width] = (torch2tensor(buf).type_view(tv.uint32), buf)
        return self._reduced[width][0]


class _SparseConvFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, features, weight, bias, geometry: SparseConvGeometry, relu: bool):
        features, weight = features.contiguous(), weight.contiguous()
        if features.dim() != 2 or features.shape[0] != geometry.n_in:
            raise ValueError("features must be [%d, C]: one row per input site of the geometry" % geometry.n_in)
        if weight.dim() != 3 or weight.shape[1] != geometry.kv or weight.shape[2] != features.shape[1]:
            raise ValueError("weight must be [K, %d, %d]" % (geometry.kv, features.shape[1]))
        dtype = _TORCH_TO_TV[features.dtype]
        out = torch.empty((geometry.n_out, weight.shape[0]), dtype=features.dtype, device=features.device)
        if bias is not None:
            bias = bias.contiguous()
        key = ("fwd", dtype, weight.dtype, tuple(features.shape), tuple(weight.shape),
               None if bias is None else (bias.dtype, tuple(bias.shape)), relu)
        hit = geometry._launches.get(key)
        if hit is not None:
            launch, tile_m = hit
            if bias is not None:
                launch(current_stream(), input=features, weight=weight, output=out, bias=bias)
            else:
                launch(current_stream(), input=features, weight=weight, output=out)
            ctx.geometry, ctx.relu, ctx.has_bias, ctx.tile_m = geometry, relu, bias is not None, tile_m
            ctx.save_for_backward(features, weight, out if relu else None)
            return out
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = _desp_like(dtype, ConvOpType.Forward, dynamic=geometry.words > 1)
        p.input, p.weight, p.output = torch2tensor(features), torch2tensor(weight), torch2tensor(out)
        p.indices, p.mask, p.mask_argsort = geometry.indices_fwd_pos, geometry.mask_fwd, geometry.order_fwd
        p.indices_by_position = True
        p.mask_int_count = geometry.words
        p.light_prefix = geometry.light_fwd
        if bias is not None:
            p.bias, p.beta = torch2tensor(bias), 1.0
        if relu:
            p.act_type = Activation.ReLU
        p.stream = current_stream()
        _TUNER.tune_conv(p)
        # the tile masks the forward launch computes anyway are what backward-weight needs
        # (not for several mask words: that backward-weight walks the pair lists)
        tile_m = int(p.conv_algo_desp.tile_shape[0])
        if geometry.words == 1:
            p.mask_output = geometry.reduced_mask_buffer(tile_m)
        ConvMainUnitTest.implicit_gemm2(p)
        roles = {"input": features, "weight": weight, "output": out}
        if bias is not None:
            roles["bias"] = bias
        geometry._launches[key] = (_Launch(p, roles), tile_m)
        ctx.geometry, ctx.relu, ctx.has_bias, ctx.tile_m = geometry, relu, bias is not None, tile_m
        ctx.save_for_backward(features, weight, out if relu else None)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        features, weight, out = ctx.saved_tensors
        g: SparseConvGeometry = ctx.geometry
        grad_out = grad_out.contiguous()
        dtype = _TORCH_TO_TV[features.dtype]
        stream = current_stream()
        lib = _capi.lib()
        if ctx.relu:       # the gradient passes where the fused ReLU let the output through
            gated = torch.empty_like(grad_out)
            _capi.check(lib.cumm_hip_relu_backward(gated.data_ptr(), grad_out.data_ptr(), out.data_ptr(),
                                                   grad_out.numel(), dtype, stream))
            grad_out = gated
        grad_in = grad_w = grad_b = None
        if ctx.needs_input_grad[0]:
            # inputs that feed no output site sit in tiles the kernel skips (mask 0): zero them
            grad_in = torch.empty_like(features) if g.subm else torch.zeros_like(features)
            key = ("dgrad", dtype, tuple(weight.shape))
            launch = g._launches.get(key)
            if launch is not None:
                launch(stream, input=grad_in, weight=weight, output=grad_out)
            else:
                p = ConvParams(3, ConvOpType.BackwardInput)
                p.conv_algo_desp = _desp_like(dtype, ConvOpType.BackwardInput, dynamic=g.words > 1)
                p.input, p.weight, p.output = torch2tensor(grad_in), torch2tensor(weight), torch2tensor(grad_out)
                p.indices, p.mask, p.mask_argsort = g.indices_bwd_pos, g.mask_bwd, g.order_bwd
                p.indices_by_position = True
                p.mask_int_count = g.words
                p.reverse_mask = g.subm
                p.light_prefix = g.light_bwd
                p.stream = stream
                _TUNER.tune_conv(p)
                ConvMainUnitTest.implicit_gemm2(p)
                g._launches[key] = _Launch(p, {"input": grad_in, "weight": weight, "output": grad_out})
        if ctx.needs_input_grad[1] and g.words > 1:
            # no mask kernel for this pass: one gathered GEMM per kernel offset, straight into its
            # slice of the gradient (an offset without pairs writes zeros)
            from .conv import native
            grad_w = torch.empty_like(weight)
            key = ("wgrad_per_offset", dtype, tuple(weight.shape), tuple(features.shape), tuple(grad_out.shape))
            plan = g._launches.get(key)
            if plan is None:      # validated once (the prelude costs 0.1 ms of Python per offset), replayed after
                plan = native.plan_backward_weight(torch2tensor(grad_out), torch2tensor(features), torch2tensor(grad_w),
                                                   g.lists, stream=stream)
                plan()
                plan.release()      # (later calls bring their own tensors)
                g._launches[key] = plan
            else:
                plan.rebind(grad_out.data_ptr(), features.data_ptr(), grad_w.data_ptr(), stream)
        elif ctx.needs_input_grad[1]:
            grad_w = torch.empty_like(weight)
            # torch's switch for reproducible results selects the fixed-order sum of the partial blocks
            deterministic = bool(torch.are_deterministic_algorithms_enabled())
            key = ("wgrad", dtype, tuple(weight.shape), ctx.tile_m, deterministic)
            hit = g._launches.get(key)
            if hit is not None:
                launch, need = hit
                # the workspace comes from torch's caching allocator (the prelude's own would be a
                # device allocation per call)
                ws = torch.empty(need, dtype=torch.uint8, device=grad_out.device)
                launch(stream, input=features, weight=grad_w, output=grad_out, workspace=ws)
            else:
                p = ConvParams(3, ConvOpType.BackwardWeight)
                p.conv_algo_desp = _desp_like(dtype, ConvOpType.BackwardWeight, parallel=True)
                p.input, p.weight, p.output = torch2tensor(features), torch2tensor(grad_w), torch2tensor(grad_out)
                p.indices, p.mask, p.mask_argsort = g.indices_fwd, g.reduced_mask_buffer(ctx.tile_m), g.order_fwd
                p.mask_width, p.split_k_slices = ctx.tile_m, 32
                p.deterministic = deterministic
                n_pos, k_out, kv, c_in = int(grad_out.shape[0]), int(weight.shape[0]), int(weight.shape[1]), int(weight.shape[2])
                need = p.conv_algo_desp.query_conv_workspace_size(k_out, kv * c_in, n_pos, p.split_k_slices, kv)
                if deterministic:
                    need = max(need, int(lib.cumm_hip_query_wgrad_ordered_workspace(n_pos, c_in, k_out, kv, ctx.tile_m)))
                need = max(int(need), 256)
                ws = torch.empty(need, dtype=torch.uint8, device=grad_out.device)
                p.workspace = torch2tensor(ws)
                p.stream = stream
                ConvMainUnitTest.implicit_gemm2(p)
                g._launches[key] = (_Launch(p, {"input": features, "weight": grad_w, "output": grad_out, "workspace": ws}), need)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            rows, k_out = int(grad_out.shape[0]), int(grad_out.shape[1])
            grad_b = torch.empty(k_out, dtype=grad_out.dtype, device=grad_out.device)
            need = int(lib.cumm_hip_column_sum_workspace(rows, k_out))
            ws = torch.empty(max(need, 4), dtype=torch.uint8, device=grad_out.device)
            _capi.check(lib.cumm_hip_column_sum(grad_b.data_ptr(), grad_out.data_ptr(), rows, k_out, dtype,
                                                ws.data_ptr(), need, stream))
        return grad_in, grad_w, grad_b, None, None


def sparse_conv(features: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                geometry: SparseConvGeometry, relu: bool = False) -> torch.Tensor:
    """features [N_in, C], weight [K, kv, C] (f16 / bf16, cuda) -> [N_out, K]; differentiable in
    features, weight and bias."""
    return _SparseConvFunction.apply(features, weight, bias, geometry, relu)


class SparseConv3d(torch.nn.Module):
    """A layer over :func:`sparse_conv`: submanifold when its geometry was built without a stride."""

    def __init__(self, in_channels: int, out_channels: int, ksize=(3, 3, 3), bias: bool = True, relu: bool = False,
                 dtype=torch.float16, device="cuda"):
        super().__init__()
        kv = int(ksize[0]) * int(ksize[1]) * int(ksize[2])
        w = torch.randn(out_channels, kv, in_channels, device=device) * (2.0 / (kv * in_channels)) ** 0.5
        self.weight = torch.nn.Parameter(w.to(dtype))
        self.bias = torch.nn.Parameter(torch.zeros(out_channels, dtype=dtype, device=device)) if bias else None
        self.relu = relu

    def forward(self, features: torch.Tensor, geometry: SparseConvGeometry) -> torch.Tensor:
        return sparse_conv(features, self.weight, self.bias, geometry, self.relu)
