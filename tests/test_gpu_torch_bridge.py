"""torch <-> tv.Tensor views and the autograd functions over the sparse convolution, against the
same convolution written with torch indexing in fp32 (autograd gives the reference gradients)."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs
from cumm_amd import tensorview as tv

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _reference(feat32, w32, bias32, ind_f, relu):
    """out[o] = sum_k W[:, k, :] @ x[ind[k][o]] over the valid pairs, in fp32 on the CPU."""
    n_out = ind_f.shape[1]
    out = torch.zeros(n_out, w32.shape[0])
    for k in range(ind_f.shape[0]):
        o = np.nonzero(ind_f[k] >= 0)[0]
        if o.size:
            out = out.index_add(0, torch.as_tensor(o), feat32[torch.as_tensor(ind_f[k][o].astype(np.int64))] @ w32[:, k, :].T)
    if bias32 is not None:
        out = out + bias32
    return torch.relu(out) if relu else out


def test_views_share_memory_both_ways():
    from cumm_amd import torch_bridge as tb
    t = torch.arange(24, dtype=torch.float16, device="cuda").reshape(4, 6)
    v = tb.torch2tensor(t)
    assert v.shape == [4, 6] and v.dtype == tv.float16 and v.byte_pointer() == t.data_ptr()
    np.testing.assert_array_equal(H.host(v), t.cpu().numpy())
    back = tb.tensor2torch(v, clone=False)
    assert back.data_ptr() == t.data_ptr() and torch.equal(back, t)
    back[1, 2] = 100.0
    assert float(t[1, 2]) == 100.0
    assert tb.tensor2torch(v, clone=True).data_ptr() != t.data_ptr()
    # a strided view, bf16, and an unsigned tensor
    s = tb.torch2tensor(t[:, ::2])
    np.testing.assert_array_equal(H.host(s), t[:, ::2].cpu().numpy())
    b = torch.randn(5, 3, device="cuda").to(torch.bfloat16)
    assert torch.equal(tb.tensor2torch(tb.torch2tensor(b), clone=False), b)
    u = tv.zeros([7], tv.uint32, 0)
    with pytest.raises(ValueError):
        tb.tensor2torch(u)
    assert tb.tensor2torch(u, cast_uint_to_int=True).dtype == torch.int32


@pytest.mark.parametrize("strided", [False, True, "pad0"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_autograd_matches_torch_indexing(dtype, strided):
    from cumm_amd import torch_bridge as tb
    print("case torch bridge", dtype, strided, flush=True)
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    coords, grid = H.small_cloud(21, 2500)
    padding = (1, 1, 1)
    if strided == "pad0":
        # stride 2 without padding on even axes: the inputs on the last plane of an axis feed no
        # output site.  A whole plane of them fills several 128-row tiles whose mask is zero, which
        # the backward-input kernel skips: their gradient must still come back as zero.
        padding = (0, 0, 0)
        zz, yy = np.meshgrid(np.arange(grid[0]), np.arange(grid[1]), indexing="ij")
        plane = np.stack([np.zeros(zz.size, np.int64), zz.ravel(), yy.ravel(),
                          np.full(zz.size, grid[2] - 1)], axis=1).astype(np.int32)
        coords = np.unique(np.concatenate([coords, plane]), axis=0).astype(np.int32)
    c_in, k_out = 64, 96
    torch.manual_seed(3)
    geo = tb.SparseConvGeometry(torch.as_tensor(coords, device="cuda"), grid, stride=(2, 2, 2) if strided else None,
                                padding=padding)
    host = pairs.sparse_conv_pairs(coords, grid, padding=padding) if strided else pairs.subm_pairs(coords, grid)
    if strided == "pad0":
        assert int((host.mask_bwd == 0).sum()) >= 3 * 128
    np.testing.assert_array_equal(H.host(geo.indices_fwd), host.indices_fwd)
    def rel(a, b):
        return float((a.float().cpu() - b).abs().max() / b.abs().max().clamp_min(1e-6))

    # the second pass runs on other tensors (the first pass's stay alive, so the addresses differ):
    # the bridge replays the argument blocks it validated in the first pass with the new pointers
    held = []
    for trip in range(2):
        feat = (torch.randn(coords.shape[0], c_in)).to(tdt)
        weight = (torch.randn(k_out, 27, c_in) * 0.05).to(tdt)
        bias = (torch.randn(k_out) * 0.1).to(tdt)
        gout = torch.randn(geo.n_out, k_out).to(tdt)

        f_d = feat.cuda().requires_grad_(True)
        w_d = weight.cuda().requires_grad_(True)
        b_d = bias.cuda().requires_grad_(True)
        out = tb.sparse_conv(f_d, w_d, b_d, geo, relu=True)
        g_d = gout.cuda()
        out.backward(g_d)
        held += [f_d, w_d, b_d, out, g_d]

        f_r = feat.float().requires_grad_(True)
        w_r = weight.float().requires_grad_(True)
        b_r = bias.float().requires_grad_(True)
        ref = _reference(f_r, w_r, b_r, host.indices_fwd, relu=True)
        # the ReLU gate of the reference must be the GPU's own (outputs within rounding of zero differ)
        gate = (out.detach().float().cpu() > 0).float()
        pre = _reference(f_r, w_r, b_r, host.indices_fwd, relu=False)
        (pre * gate * gout.float()).sum().backward()

        assert rel(out.detach(), ref.detach()) < 1e-2, trip
        assert rel(f_d.grad, f_r.grad) < 1e-2, trip
        assert rel(w_d.grad, w_r.grad) < 1e-2, trip
        assert rel(b_d.grad, b_r.grad) < 1e-2, trip
    assert len(geo._launches) == 3

    # other shapes on the same geometry do not meet the remembered calls
    with pytest.raises(ValueError):
        tb.sparse_conv(f_d[:-1], w_d, b_d, geo, relu=True)
    with pytest.raises(ValueError):
        tb.sparse_conv(f_d, w_d[:, :26], b_d, geo, relu=True)


@pytest.mark.parametrize("case", ["subm555", "strided335"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_autograd_with_kernel_volumes_above_32(dtype, case):
    """5 x 5 x 5 submanifold and strided 3 x 3 x 5 layers through the bridge: masks of several words
    made and sorted on the GPU, forward and backward-input on the dynamic_mask descriptors (one
    launch each), backward-weight offset by offset over the pair lists; outputs and all three
    gradients against the convolution written with torch indexing in fp32."""
    from cumm_amd import torch_bridge as tb
    print("case torch bridge large kernel", dtype, case, flush=True)
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    coords, grid = H.small_cloud(31, 1500, grid=(12, 30, 28))
    if case == "subm555":
        ksize, stride, padding = (5, 5, 5), None, (2, 2, 2)
        host = pairs.subm_pairs(coords, grid, ksize)
    else:
        ksize, stride, padding = (3, 3, 5), (2, 2, 2), (1, 1, 2)
        host = pairs.sparse_conv_pairs(coords, grid, ksize, stride, padding)
    kv = ksize[0] * ksize[1] * ksize[2]
    geo = tb.SparseConvGeometry(torch.as_tensor(coords, device="cuda"), grid, ksize=ksize, stride=stride, padding=padding)
    assert geo.words == (kv + 31) // 32 and geo.kv == kv
    np.testing.assert_array_equal(H.host(geo.indices_fwd), host.indices_fwd)
    c_in, k_out = 64, 64
    torch.manual_seed(5)

    def rel(a, b):
        return float((a.float().cpu() - b).abs().max() / b.abs().max().clamp_min(1e-6))

    for trip in range(2):
        feat = torch.randn(coords.shape[0], c_in).to(tdt)
        weight = (torch.randn(k_out, kv, c_in) * 0.03).to(tdt)
        bias = (torch.randn(k_out) * 0.1).to(tdt)
        gout = torch.randn(geo.n_out, k_out).to(tdt)
        f_d, w_d, b_d = (t.cuda().requires_grad_(True) for t in (feat, weight, bias))
        out = tb.sparse_conv(f_d, w_d, b_d, geo, relu=True)
        out.backward(gout.cuda())
        f_r, w_r, b_r = (t.float().requires_grad_(True) for t in (feat, weight, bias))
        ref = _reference(f_r, w_r, b_r, host.indices_fwd, relu=True)
        gate = (out.detach().float().cpu() > 0).float()
        pre = _reference(f_r, w_r, b_r, host.indices_fwd, relu=False)
        (pre * gate * gout.float()).sum().backward()
        assert rel(out.detach(), ref.detach()) < 1e-2, trip
        assert rel(f_d.grad, f_r.grad) < 1e-2, trip
        assert rel(w_d.grad, w_r.grad) < 1e-2, trip
        assert rel(b_d.grad, b_r.grad) < 1e-2, trip


def test_module_stack_runs_and_trains_a_step():
    from cumm_amd import torch_bridge as tb
    coords, grid = H.small_cloud(22, 3000)
    c = torch.as_tensor(coords, device="cuda")
    geo = tb.SparseConvGeometry(c, grid)
    down = tb.SparseConvGeometry(c, grid, stride=(2, 2, 2))
    torch.manual_seed(1)
    l1 = tb.SparseConv3d(32, 64, relu=True)
    l2 = tb.SparseConv3d(64, 64, relu=True)
    l3 = tb.SparseConv3d(64, 128)
    x = torch.randn(coords.shape[0], 32, device="cuda").half()
    params = list(l1.parameters()) + list(l2.parameters()) + list(l3.parameters())
    y = l3(l2(l1(x, geo), geo) + l1(x, geo), down)          # a residual connection by torch
    assert y.shape == (down.n_out, 128) and torch.isfinite(y.float()).all()
    loss = y.float().pow(2).mean()
    loss.backward()
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() for p in params)
    assert float(l1.weight.grad.float().abs().max()) > 0


def test_deterministic_switch_gives_the_same_weight_gradient_twice():
    """torch.use_deterministic_algorithms(True) selects the fixed-order backward-weight: two
    backward passes over the same tensors give the same bits (and the value stays within
    tolerance of the default variant's)."""
    from cumm_amd import torch_bridge as tb
    coords, grid = H.small_cloud(23, 3000)
    geo = tb.SparseConvGeometry(torch.as_tensor(coords, device="cuda"), grid)
    torch.manual_seed(2)
    layer = tb.SparseConv3d(64, 64, relu=True)
    x = torch.randn(coords.shape[0], 64, device="cuda").half()

    def weight_grad():
        layer.zero_grad(set_to_none=True)
        layer(x, geo).float().pow(2).mean().backward()
        return layer.weight.grad.clone()

    default = weight_grad()
    was = torch.are_deterministic_algorithms_enabled()
    torch.use_deterministic_algorithms(True)
    try:
        first, second = weight_grad(), weight_grad()
    finally:
        torch.use_deterministic_algorithms(was)
    assert torch.equal(first, second)
    scale = float(default.float().abs().max())
    assert float((first.float() - default.float()).abs().max()) < 1e-2 * scale
