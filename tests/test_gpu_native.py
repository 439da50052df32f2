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


def test_static_mask_descriptors_reject_large_kernel_volumes():
    """One mask word per position describes 32 offsets: a descriptor without dynamic_mask refuses more."""
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 64, 64)
    n = 100
    p.input, p.weight = tv.zeros([n, 64], tv.float16, 0), tv.zeros([64, 125, 64], tv.float16, 0)
    p.output = tv.zeros([n, 64], tv.float16, 0)
    p.indices = tv.zeros([125, n], tv.int32, 0)
    p.mask, p.mask_argsort = tv.zeros([n], tv.uint32, 0), tv.zeros([n], tv.int32, 0)
    with pytest.raises(ValueError, match="kernel volume"):
        ConvMainUnitTest.implicit_gemm2(p)
    p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 64, 64, dynamic_mask=True)
    p.mask_int_count = 2                      # four words for 125 offsets, nothing else
    with pytest.raises(RuntimeError, match="mask_int_count"):
        ConvMainUnitTest.implicit_gemm2(p)
    with pytest.raises(RuntimeError):         # masks of one word per position: too short
        p.mask_int_count = 4
        ConvMainUnitTest.implicit_gemm2(p)


@pytest.mark.parametrize("case", ["subm555", "strided335", "subm333"])
def test_masks_and_sort_for_several_words_bit_exact(case):
    """cumm_hip_masks_from_pairs and cumm_hip_sort_by_mask_words against their host mirrors."""
    print("case dynamic masks", case, flush=True)
    coords, grid = H.small_cloud(66, 6000, grid=(14, 40, 36))
    host, devt = _tables(case, coords, grid)
    for table_h, table_d in ((host.indices_fwd, devt.indices_fwd), (host.indices_bwd, devt.indices_bwd)):
        want = pairs.masks_from_pairs(table_h)
        got = pairs.masks_from_pairs_device(table_d)
        np.testing.assert_array_equal(H.host(got), want)
        ms_ref, order_ref = pairs.sort_by_mask_words(want)
        ms, order = pairs.sort_by_mask_words_device(got)
        np.testing.assert_array_equal(H.host(order), order_ref)
        np.testing.assert_array_equal(H.host(ms), ms_ref)


@pytest.mark.parametrize("dtype,tile,c_in,k_out", [("f16", (64, 64), 64, 64), ("bf16", (128, 128), 64, 128),
                                                    ("f16", (128, 128), 128, 128), ("bf16", (64, 64), 160, 72)])
@pytest.mark.parametrize("case", ["subm555", "strided335"])
def test_dynamic_mask_forward_backward_input(dtype, tile, c_in, k_out, case):
    """Kernel volumes above 32 through implicit_gemm2 in ONE launch: a dynamic_mask descriptor,
    ceil(kv / 32) mask words per position (masks and order from the GPU preparation, bit-exact
    above), against the oracle - forward with bias + ReLU and the tile masks it writes,
    backward-input on the backward masks, and for the submanifold case backward-input on the
    forward masks reversed in the kernel; the pair table by row and by position."""
    print("case dynamic mask conv", dtype, tile, c_in, k_out, case, flush=True)
    from oracle import conv_ref, numerics as onm
    coords, grid = H.small_cloud(67, 4000, grid=(14, 40, 36))
    rng = np.random.default_rng(68)
    host, devt = _tables(case, coords, grid)
    kv, n_out = host.indices_fwd.shape
    n_in = coords.shape[0]
    words = (kv + 31) // 32
    mf_d = pairs.masks_from_pairs_device(devt.indices_fwd)
    ms_d, order_d = pairs.sort_by_mask_words_device(mf_d)
    ms, order = H.host(ms_d), H.host(order_d)
    feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.03, size=(k_out, kv, c_in)).astype(np.float32), dtype)
    bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    out0 = H.to_storage(np.zeros((n_out, k_out), np.float32), dtype)
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, host.indices_fwd, ms, order, tile_m=tile[0], dtype_in=dtype,
                                                 dtype_w=dtype, dtype_out=dtype, beta=1.0, bias=bias, act=onm.ACT_RELU)
    tiles = (n_out + tile[0] - 1) // tile[0]
    outs = []
    for by_pos in (False, True):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile, dynamic_mask=True)
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        p.bias, p.beta, p.act_type = H.dev(bias, dtype), 1.0, Activation.ReLU
        p.indices = pairs.pairs_by_position_device(devt.indices_fwd, order_d) if by_pos else devt.indices_fwd
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        p.mask_output = tv.zeros([tiles, words], tv.uint32, 0)
        p.mask_int_count = words
        ConvMainUnitTest.implicit_gemm2(p)
        got = H.as_f32(H.host(p.output), dtype)
        assert got.min() >= 0.0
        assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL
        np.testing.assert_array_equal(H.host(p.mask_output), ref_mo)
        outs.append(H.host(p.output))
    np.testing.assert_array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))

    # backward-input on the masks of the backward table
    mb_d = pairs.masks_from_pairs_device(devt.indices_bwd)
    msb_d, orderb_d = pairs.sort_by_mask_words_device(mb_d)
    din0 = H.to_storage(np.zeros((n_in, c_in), np.float32), dtype)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, host.indices_bwd, H.host(msb_d), H.host(orderb_d), tile_m=tile[0],
                                             dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    runs = [(msb_d, orderb_d, False)]
    if case == "subm555":
        runs.append((ms_d, order_d, True))      # the forward masks, reversed end for end in the kernel
    for mask_d, ord_d, reverse in runs:
        pd = ConvParams(3, ConvOpType.BackwardInput)
        pd.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, *tile, dynamic_mask=True)
        pd.input, pd.weight, pd.output = H.dev(din0, dtype), H.dev(w, dtype), H.dev(dout, dtype)
        pd.indices, pd.mask, pd.mask_argsort = devt.indices_bwd, mask_d, ord_d
        pd.reverse_mask = reverse
        ConvMainUnitTest.implicit_gemm2(pd)
        if reverse:
            ref_r = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, host.indices_bwd, ms, order, tile_m=tile[0], dtype_in=dtype,
                                                     dtype_w=dtype, dtype_out=dtype, reverse_mask=True)
            assert H.rel_err(H.as_f32(H.host(pd.input), dtype), H.as_f32(ref_r, dtype)) < TOL
        assert H.rel_err(H.as_f32(H.host(pd.input), dtype), H.as_f32(ref_d, dtype)) < TOL


def test_dynamic_mask_descriptor_with_a_small_kernel_volume():
    """A dynamic_mask descriptor on a 3 x 3 x 3 kernel has one word per position and gives what
    the static descriptor gives, bit for bit."""
    coords, grid = H.small_cloud(69, 3000)
    rng = np.random.default_rng(70)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    feat = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), "f16")
    w = H.to_storage(rng.normal(0, 0.05, size=(64, 27, 64)).astype(np.float32), "f16")
    outs = []
    for dyn in (False, True):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 64, 64, dynamic_mask=dyn)
        p.input, p.weight, p.output = H.dev(feat, "f16"), H.dev(w, "f16"), tv.zeros([n, 64], tv.float16, 0)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
        ConvMainUnitTest.implicit_gemm2(p)
        outs.append(H.host(p.output))
    np.testing.assert_array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))


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


def test_backward_weight_plan_replays_on_other_tensors():
    """The backward-weight plan validates its per-offset launches once; ``rebind`` then runs them
    on other tensors of the same shapes by address (what the torch bridge does every iteration),
    also after the plan has let go of the first run's tensors."""
    rng = np.random.default_rng(66)
    grid = (8, 10, 10)
    coords = synth.clustered_voxels(rng, 300, grid, 3, sigma=2.5)
    c_in, k_out = 16, 24
    host = pairs.subm_pairs(coords, grid, ksize=(5, 5, 5))
    devt = pairs.subm_pairs_device(H.dev(coords, "i32"), grid, ksize=(5, 5, 5))
    lists_h, lists_d = pairs.pair_lists(host.indices_fwd), pairs.pair_lists_device(devt.indices_fwd)
    n = coords.shape[0]

    def data(seed):
        r = np.random.default_rng(seed)
        return (r.normal(0, 1, size=(n, k_out)).astype(np.float16), r.normal(0, 1, size=(n, c_in)).astype(np.float16))

    dout, feat = data(1)
    d_dout, d_feat, d_dw = H.dev(dout, "f16"), H.dev(feat, "f16"), tv.zeros([k_out, 125, c_in], tv.float16, 0)
    plan = native.plan_backward_weight(d_dout, d_feat, d_dw, lists_d)
    plan()
    assert plan.launches == 125
    ref = native_ref.native_wgrad_ref(dout, feat, lists_h.pair_in, lists_h.pair_out, lists_h.counts, 125, dtype="f16")
    assert H.rel_err(H.host(d_dw).astype(np.float32), ref.astype(np.float32)) < TOL
    plan.release()
    dout2, feat2 = data(2)
    e_dout, e_feat = H.dev(dout2, "f16"), H.dev(feat2, "f16")
    e_dw = H.dev(np.full((k_out, 125, c_in), 7.0, np.float16), "f16")     # every slice is written, also those without pairs
    plan.rebind(e_dout.byte_pointer(), e_feat.byte_pointer(), e_dw.byte_pointer(), 0)
    ref2 = native_ref.native_wgrad_ref(dout2, feat2, lists_h.pair_in, lists_h.pair_out, lists_h.counts, 125, dtype="f16")
    assert H.rel_err(H.host(e_dw).astype(np.float32), ref2.astype(np.float32)) < TOL
