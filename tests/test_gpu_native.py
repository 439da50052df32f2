"""Kernel volumes above 32 end to end on the GPU: pair tables and per-offset pair lists bit-exact
against the host builders, and the per-offset ("native") convolution - forward, backward-input,
backward-weight - against the oracle (the reference's own gather -> matmul -> scatter-add check,
cumm/conv/main_real_spconv.py:309-403) and, on a small grid, against torch's dense conv3d.
Tolerance for f16 / bf16: max relative error 1e-2 (fp32 accumulate)."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv import native
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import Activation, ConvOpType, ConvParams
from oracle import native_ref

pytestmark = pytest.mark.gpu
TOL = 1e-2

CASES = {"subm555": dict(ksize=(5, 5, 5), stride=None, padding=(2, 2, 2)),
         "strided335": dict(ksize=(3, 3, 5), stride=(2, 2, 2), padding=(1, 1, 2)),
         "subm333": dict(ksize=(3, 3, 3), stride=None, padding=(1, 1, 1))}


def _tables(case, coords, grid):
    g = CASES[case]
    dc = H.dev(coords, "i32")
    if g["stride"] is None:
        host = pairs.subm_pairs(coords, grid, ksize=g["ksize"])
        devt = pairs.subm_pairs_device(dc, grid, ksize=g["ksize"])
    else:
        host = pairs.sparse_conv_pairs(coords, grid, ksize=g["ksize"], stride=g["stride"], padding=g["padding"])
        devt = pairs.sparse_conv_pairs_device(dc, grid, ksize=g["ksize"], stride=g["stride"], padding=g["padding"])
    return host, devt


@pytest.mark.parametrize("case", ["subm555", "strided335", "subm333"])
def test_pair_tables_and_lists_bit_exact(case):
    print("case native tables", case, flush=True)
    coords, grid = H.small_cloud(61, 5000, grid=(14, 40, 36))
    host, devt = _tables(case, coords, grid)
    np.testing.assert_array_equal(H.host(devt.indices_fwd), host.indices_fwd)
    np.testing.assert_array_equal(H.host(devt.indices_bwd), host.indices_bwd)
    kv = host.indices_fwd.shape[0]
    if kv > 32:
        assert devt.mask_fwd is None and host.mask_fwd is None
    else:
        np.testing.assert_array_equal(H.host(devt.mask_fwd), host.mask_fwd)
    want = pairs.pair_lists(host.indices_fwd)
    got = pairs.pair_lists_device(devt.indices_fwd)
    np.testing.assert_array_equal(got.counts, want.counts)
    gin, gout = H.host(got.pair_in), H.host(got.pair_out)
    for k in range(kv):
        n = int(want.counts[k])
        np.testing.assert_array_equal(gin[k][:n], want.pair_in[k][:n])
        np.testing.assert_array_equal(gout[k][:n], want.pair_out[k][:n])


def test_mask_kernels_still_reject_large_kernel_volumes():
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 64, 64)
    n = 100
    p.input, p.weight = tv.zeros([n, 64], tv.float16, 0), tv.zeros([64, 125, 64], tv.float16, 0)
    p.output = tv.zeros([n, 64], tv.float16, 0)
    p.indices = tv.zeros([125, n], tv.int32, 0)
    p.mask, p.mask_argsort = tv.zeros([n], tv.uint32, 0), tv.zeros([n], tv.int32, 0)
    with pytest.raises(ValueError, match="kernel volume"):
        ConvMainUnitTest.implicit_gemm2(p)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", ["subm555", "strided335"])
def test_native_forward_backward(dtype, case):
    print("case native conv", dtype, case, flush=True)
    coords, grid = H.small_cloud(62, 4000, grid=(14, 40, 36))
    rng = np.random.default_rng(63)
    c_in, k_out = 64, 128
    host, devt = _tables(case, coords, grid)
    kv = host.indices_fwd.shape[0]
    n_in, n_out = coords.shape[0], host.indices_fwd.shape[1]
    lists_h = pairs.pair_lists(host.indices_fwd)
    lists_d = pairs.pair_lists_device(devt.indices_fwd)
    feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.03, size=(k_out, kv, c_in)).astype(np.float32), dtype)
    bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    d_feat, d_w, d_dout = H.dev(feat, dtype), H.dev(w, dtype), H.dev(dout, dtype)
    # forward with bias + ReLU
    out = tv.zeros([n_out, k_out], H.TV_DTYPE[dtype], 0)
    native.forward(d_feat, d_w, out, lists_d, bias=H.dev(bias, dtype), act_type=Activation.ReLU)
    ref = native_ref.native_fwd_ref(feat, w, lists_h.pair_in, lists_h.pair_out, lists_h.counts, n_out, dtype=dtype,
                                    bias=bias, act=1)
    got = H.as_f32(H.host(out), dtype)
    assert got.min() >= 0.0
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL
    assert H.rel_err_rows(got, H.as_f32(ref, dtype)) < TOL
    # backward-input
    dinp = tv.zeros([n_in, c_in], H.TV_DTYPE[dtype], 0)
    native.backward_input(d_dout, d_w, dinp, lists_d)
    ref_d = native_ref.native_dgrad_ref(dout, w, lists_h.pair_in, lists_h.pair_out, lists_h.counts, n_in, dtype=dtype)
    assert H.rel_err(H.as_f32(H.host(dinp), dtype), H.as_f32(ref_d, dtype)) < TOL
    # backward-weight (offsets without pairs must come out zero: start from garbage)
    dw = H.dev(H.to_storage(rng.normal(0, 1, size=(k_out, kv, c_in)).astype(np.float32), dtype), dtype)
    native.backward_weight(d_dout, d_feat, dw, lists_d)
    ref_w = native_ref.native_wgrad_ref(dout, feat, lists_h.pair_in, lists_h.pair_out, lists_h.counts, kv, dtype=dtype)
    assert H.rel_err(H.as_f32(H.host(dw), dtype), H.as_f32(ref_w, dtype)) < TOL


def test_native_forward_against_dense_conv3d():
    """5 x 5 x 5 submanifold forward on a small grid against torch's dense cross-correlation of
    the densified cloud (f16 inputs, float64 reference)."""
    torch = pytest.importorskip("torch")
    import torch.nn.functional as F
    rng = np.random.default_rng(64)
    grid = (10, 12, 12)
    coords = synth.clustered_voxels(rng, 400, grid, 3, sigma=2.5)
    c_in, k_out, ksize = 16, 32, (5, 5, 5)
    devt = pairs.subm_pairs_device(H.dev(coords, "i32"), grid, ksize=ksize)
    lists = pairs.pair_lists_device(devt.indices_fwd)
    n = coords.shape[0]
    feat = rng.normal(0, 1, size=(n, c_in)).astype(np.float16)
    w_ref = rng.normal(0, 0.1, size=(125, k_out, c_in)).astype(np.float16)
    weight = np.ascontiguousarray(w_ref.transpose(1, 0, 2))
    out = tv.zeros([n, k_out], tv.float16, 0)
    native.forward(H.dev(feat, "f16"), H.dev(weight, "f16"), out, lists)
    dense = torch.zeros(1, c_in, *grid, dtype=torch.float64)
    dense[0, :, coords[:, 1], coords[:, 2], coords[:, 3]] = torch.from_numpy(feat.T.astype(np.float64))
    wt = torch.from_numpy(w_ref.astype(np.float64)).reshape(5, 5, 5, k_out, c_in).permute(3, 4, 0, 1, 2).contiguous()
    want = F.conv3d(dense, wt, padding=2)[0, :, coords[:, 1], coords[:, 2], coords[:, 3]].T.numpy()
    assert H.rel_err(H.host(out).astype(np.float32), want.astype(np.float32)) < TOL


def test_plan_runs_again_on_new_contents():
    """A forward plan is validated once; a second run reads the tensors' current contents."""
    rng = np.random.default_rng(65)
    grid = (8, 10, 10)
    coords = synth.clustered_voxels(rng, 300, grid, 3, sigma=2.5)
    c_in, k_out = 16, 16
    host = pairs.subm_pairs(coords, grid, ksize=(5, 5, 5))
    devt = pairs.subm_pairs_device(H.dev(coords, "i32"), grid, ksize=(5, 5, 5))
    lists_h, lists_d = pairs.pair_lists(host.indices_fwd), pairs.pair_lists_device(devt.indices_fwd)
    n = coords.shape[0]
    weight = rng.normal(0, 0.1, size=(k_out, 125, c_in)).astype(np.float16)
    d_feat = tv.zeros([n, c_in], tv.float16, 0)
    out = tv.zeros([n, k_out], tv.float16, 0)
    plan = native.plan_forward(d_feat, H.dev(weight, "f16"), out, lists_d)
    assert plan.launches == int((lists_h.counts > 0).sum()) + 2
    for seed in (1, 2):
        feat = np.random.default_rng(seed).normal(0, 1, size=(n, c_in)).astype(np.float16)
        d_feat.copy_(tv.from_numpy(feat))
        plan()
        ref = native_ref.native_fwd_ref(feat, weight, lists_h.pair_in, lists_h.pair_out, lists_h.counts, n, dtype="f16")
        assert H.rel_err(H.host(out).astype(np.float32), ref.astype(np.float32)) < TOL
