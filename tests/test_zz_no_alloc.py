"""GPU parity of the entry point that allocates nothing: ``cumm_hip_sparse_conv_static_ws`` (the
library's own static workspace) against ``cumm_hip_sparse_conv`` with a caller-provided workspace,
backward-weight, two calls in a row, the second on a smaller input.

Serial split-K is deterministic: compared bit for bit.  The balanced (split_k_parallel) kernels
add fp32 partial sums with atomics in no fixed order: compared within the f16/bf16 tolerance of
1e-2 (fp32 accumulate), against the existing entry point and against the oracle; their fixed-order
variant splits the sum by the number of workgroups its workspace has slots for, so it is compared
with the oracle within the tolerance and with itself bit for bit.
"""
import numpy as np
import pytest

from oracle import conv_ref

from cumm_amd import _capi, pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import ConvOpType, ConvParams

import helpers as H

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _wgrad_params(seed, n, c_in, k_out, dtype, desp, split_k, mask_width=64):
    rng = np.random.default_rng(seed)
    grid = (12, 40, 36)
    coords = synth.clustered_voxels(rng, n, grid, 6, sigma=3.0)
    pt = pairs.subm_pairs(coords, grid)
    n_out = pt.indices_fwd.shape[1]
    feat = H.to_storage(rng.normal(0, 1, size=(n_out, c_in)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, mask_width)

    def make():
        p = ConvParams(3, ConvOpType.BackwardWeight)
        p.conv_algo_desp = desp
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
        p.mask_width = mask_width
        p.split_k_slices = split_k
        p.alpha, p.beta = 0.5, 1.0
        return p

    def oracle(serial):
        return conv_ref.implicit_gemm_wgrad_ref(
            dout, feat, dw0, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
            dtype_in=dtype, dtype_w=dtype, alpha=0.5, beta=1.0,
            split_k_slices=split_k if serial else 1, tile_k=32)
    return make, oracle


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_static_workspace_serial_split_k_bit_exact(dtype):
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64)
    # the second call is smaller: it must not see what the first left in the shared array
    for seed, n, c_in, k_out in ((31, 3000, 64, 96), (32, 1100, 32, 64)):
        print("case static_ws serial", dtype, n, c_in, k_out, flush=True)
        make, oracle = _wgrad_params(seed, n, c_in, k_out, dtype, desp, split_k=4)
        p_ref = make()
        ConvMainUnitTest.implicit_gemm2(p_ref)
        assert not p_ref.workspace.empty()          # the existing entry point got a workspace
        p_new = make()
        ConvMainUnitTest.implicit_gemm2_static_workspace(p_new)
        assert p_new.workspace.empty()              # nothing was allocated for the new one
        got, want = H.host(p_new.weight), H.host(p_ref.weight)
        np.testing.assert_array_equal(got, want)
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(oracle(True), dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_static_workspace_balanced(dtype):
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    for seed, n, c_in, k_out in ((33, 3000, 128, 128), (34, 900, 64, 72)):
        print("case static_ws balanced", dtype, n, c_in, k_out, flush=True)
        make, oracle = _wgrad_params(seed, n, c_in, k_out, dtype, desp, split_k=8)
        p_ref = make()
        ConvMainUnitTest.implicit_gemm2(p_ref)
        p_new = make()
        ConvMainUnitTest.implicit_gemm2_static_workspace(p_new)
        assert p_new.workspace.empty()
        got = H.as_f32(H.host(p_new.weight), dtype)
        assert H.rel_err(got, H.as_f32(H.host(p_ref.weight), dtype)) < TOL
        assert H.rel_err(got, H.as_f32(oracle(False), dtype)) < TOL
        # an unchanged repeat call (the validated-arguments path) gives the same again
        ConvMainUnitTest.implicit_gemm2_static_workspace(p_new)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_static_workspace_fixed_order(dtype):
    """The fixed-order backward-weight on the static workspace: as many workgroups as its 8 MiB hold
    slots for; the same bits twice in a row, also after a call on another problem in between."""
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    results = []
    for seed, n, c_in, k_out in ((36, 3000, 128, 128), (37, 900, 64, 72), (36, 3000, 128, 128)):
        print("case static_ws fixed order", dtype, n, c_in, k_out, flush=True)
        make, oracle = _wgrad_params(seed, n, c_in, k_out, dtype, desp, split_k=8)
        p_new = make()
        p_new.deterministic = True
        ConvMainUnitTest.implicit_gemm2_static_workspace(p_new)
        assert p_new.workspace.empty()
        got = H.host(p_new.weight)
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(oracle(False), dtype)) < TOL
        results.append(got)
    np.testing.assert_array_equal(results[0], results[2])


def test_static_workspace_rejects_what_does_not_fit():
    dtype = "f16"
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    c_in = k_out = 288          # 288 * 27 * 288 * 4 bytes > 8 MiB
    assert 4 * k_out * 27 * c_in > _capi.STATIC_WORKSPACE_BYTES
    make, _ = _wgrad_params(35, 300, c_in, k_out, dtype, desp, split_k=2)
    with pytest.raises(ValueError, match="static"):
        ConvMainUnitTest.implicit_gemm2_static_workspace(make())
