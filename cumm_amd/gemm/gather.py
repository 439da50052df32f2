"""Stand-alone row gather and row scatter-add: host mirror of the reference's
``GatherAll`` / ``ScatterAll`` (cumm/gemm/gather.py:391-497 and :499-617).

    gather:   output[i, :]           = input[indices[i], :]
    scatter:  output[indices[i], :] += input[i, :]        (indices unique)

The reference compiles one kernel per (tile_m, tile_k_bytes, bytes_per_access,
num_threads) and lets the caller time them; the same parameter lists and the
same ``supported`` checks are kept so that such callers run unchanged, but
every combination maps to the one HIP kernel behind ``cumm_hip_gather_rows`` /
``cumm_hip_scatter_add_rows`` (one lane per 16 bytes, whole rows per wave),
which needs no tuning: the copy is bound by HBM bandwidth.
"""
from typing import List, Tuple

from .. import _capi
from ..tensorview import Tensor, bfloat16, float16, float32, tvdtype_itemsize


def _gather_params() -> List[Tuple[int, int, int, int]]:
    """Enumeration order of GatherAll.__init__ (cumm/gemm/gather.py:398-415)."""
    res, seen = [], set()
    for tile_k_bytes in [4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048]:
        for tile_m in [1, 2, 4, 8]:
            for bytes_per_access in [4, 8, 16]:
                for num_threads in [64, 128, 256]:
                    if num_threads * bytes_per_access > tile_k_bytes * tile_m:
                        continue
                    key = (tile_m, tile_k_bytes, bytes_per_access, num_threads)
                    if key not in seen:
                        seen.add(key)
                        res.append(key)
    return res


def _scatter_params() -> List[Tuple[int, int, int, int]]:
    """Enumeration order of ScatterAll.__init__ (cumm/gemm/gather.py:506-525)."""
    res, seen = [], set()
    for tile_k_bytes in [64, 128, 256, 512, 1024, 2048]:
        for tile_m in [1, 2, 4, 8]:
            for bytes_per_access in [4, 8, 16]:
                for num_threads in [128, 256]:
                    if num_threads * bytes_per_access > tile_k_bytes * tile_m:
                        continue
                    key = (tile_m, tile_k_bytes, bytes_per_access, num_threads)
                    if key not in seen:
                        seen.add(key)
                        res.append(key)
    return res


def _check_rows(output: Tensor, input: Tensor, indices: Tensor):
    # TV_ASSERT_RT_ERR in Gather.gather / Scatter.scatter (cumm/gemm/gather.py:237-238, 369-370)
    if not (input.ndim == 2 and output.ndim == 2 and input.dim(1) == output.dim(1)):
        raise RuntimeError("error: output and input must be matrices with the same number of columns")
    if input.dtype != output.dtype:
        raise RuntimeError("error: output and input must have the same dtype")
    if indices.ndim != 1 or tvdtype_itemsize(indices.dtype) != 4:
        raise RuntimeError("error: indices must be a vector of 32-bit integers")
    if -1 in (output.device, input.device, indices.device):
        raise RuntimeError("operands must be device tensors (call .cuda() first)")


class GatherAll:
    """``lib.cumm.gemm.gather.GatherAll()`` of the reference."""

    def __init__(self):
        self._params = set(_gather_params())

    @staticmethod
    def get_all_gather_params() -> List[Tuple[int, int, int, int]]:
        return _gather_params()

    @staticmethod
    def supported(bytes_per_access: int, channel_size: int, dtype: int) -> bool:
        """cumm/gemm/gather.py:459-468."""
        return (channel_size * tvdtype_itemsize(dtype)) % bytes_per_access == 0

    @staticmethod
    def stream_synchronize(stream: int = 0) -> None:
        _capi.check(_capi.lib().cumm_hip_stream_synchronize(stream))

    def gather(self, output: Tensor, input: Tensor, indices: Tensor, tile_m: int = 8, tile_k_bytes: int = 512,
               bytes_per_access: int = 4, num_threads: int = 128, stream: int = 0) -> None:
        """cumm/gemm/gather.py:482-497 (dispatch) and :224-256 (checks, launch)."""
        if (tile_m, tile_k_bytes, bytes_per_access, num_threads) not in self._params:
            raise RuntimeError("can't find a suitable gather")
        _check_rows(output, input, indices)
        if not self.supported(bytes_per_access, input.dim(1), input.dtype):
            raise RuntimeError("not supported. use supported() to check first")
        m = indices.dim(0)
        if output.dim(0) < m:
            raise RuntimeError("output has fewer rows than indices")
        _capi.check(_capi.lib().cumm_hip_gather_rows(
            output.byte_pointer() if not output.empty() else None,
            input.byte_pointer() if not input.empty() else None,
            indices.byte_pointer() if not indices.empty() else None,
            m, input.dim(0), input.dim(1) * tvdtype_itemsize(input.dtype), stream))


class ScatterAll:
    """``lib.cumm.gemm.gather.ScatterAll()`` of the reference (float32 there; float16 and bfloat16
    are accepted as well: the sum is formed in fp32 and rounded once)."""

    _DTYPES = (float32, float16, bfloat16)

    def __init__(self):
        self._params = set(_scatter_params())

    @staticmethod
    def get_all_scatter_params() -> List[Tuple[int, int, int, int]]:
        return _scatter_params()

    def supported_scatter(self, tile_m: int, tile_k_bytes: int, bytes_per_access: int, num_threads: int,
                          channel_size: int, dtype: int) -> bool:
        """cumm/gemm/gather.py:574-589."""
        if (tile_m, tile_k_bytes, bytes_per_access, num_threads) not in self._params or dtype not in self._DTYPES:
            return False
        return (channel_size * tvdtype_itemsize(dtype)) % bytes_per_access == 0

    @staticmethod
    def stream_synchronize(stream: int = 0) -> None:
        _capi.check(_capi.lib().cumm_hip_stream_synchronize(stream))

    def scatter(self, output: Tensor, input: Tensor, indices: Tensor, tile_m: int = 8, tile_k_bytes: int = 256,
                bytes_per_access: int = 16, num_threads: int = 128, stream: int = 0) -> None:
        """cumm/gemm/gather.py:603-617 (dispatch) and :356-389 (checks, launch)."""
        _check_rows(output, input, indices)
        if (tile_m, tile_k_bytes, bytes_per_access, num_threads) not in self._params or \
                input.dtype not in self._DTYPES:
            raise RuntimeError("can't find a suitable scatter")
        if (input.dim(1) * tvdtype_itemsize(input.dtype)) % bytes_per_access != 0:
            raise RuntimeError("not supported. use supported() to check first")
        m = indices.dim(0)
        if input.dim(0) < m:
            raise RuntimeError("input has fewer rows than indices")
        _capi.check(_capi.lib().cumm_hip_scatter_add_rows(
            output.byte_pointer() if not output.empty() else None,
            input.byte_pointer() if not input.empty() else None,
            indices.byte_pointer() if not indices.empty() else None,
            m, output.dim(0), input.dim(1), int(input.dtype), stream))
