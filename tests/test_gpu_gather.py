"""GatherAll.gather / ScatterAll.scatter through the C ABI against the oracle (copies and single
fp32 additions: bit-exact)."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import tensorview as tv
from cumm_amd.gemm.gather import GatherAll, ScatterAll
from oracle import gather_ref

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,channels", [("f32", 128), ("f32", 3), ("f16", 64), ("f16", 6), ("s8", 64),
                                            ("bf16", 40), ("f32", 1)])
def test_gather_rows(dtype, channels):
    print("case gather", dtype, channels, flush=True)
    rng = np.random.default_rng(10 + channels)
    rows, m = 5000, 3777
    a = H.to_storage(rng.integers(-100, 100, size=(rows, channels)).astype(np.float32), dtype)
    idx = rng.integers(0, rows, size=m).astype(np.int32)      # repeats allowed
    idx[7], idx[100] = -1, rows                               # outside: rows of zeros
    out = tv.zeros([m, channels], H.TV_DTYPE[dtype], 0)
    lib = GatherAll()
    for params in [(8, 512, 4, 128), (1, 256, 4, 64)]:
        if not lib.supported(params[2], channels, H.TV_DTYPE[dtype]):
            continue
        lib.gather(out, H.dev(a, dtype), H.dev(idx, "i32"), *params)
        np.testing.assert_array_equal(H.host(out), gather_ref.gather_rows_ref(a, idx))


def test_gather_reference_test_shape_and_parameter_list():
    """The reference's own check (cumm/gemm/main_real.py:775-810): 64000 x 128 f32, a shuffled
    identity, every parameter set that supports the shape."""
    rng = np.random.default_rng(12315)
    m, k = 64000, 128
    a = rng.uniform(-2, 2, size=(m, k)).astype(np.float32)
    inds = rng.permutation(m).astype(np.int32)
    lib = GatherAll()
    params = lib.get_all_gather_params()
    assert len(params) == len(set(params)) and (8, 512, 4, 128) in params and (1, 4, 4, 64) not in params
    a_tv, inds_tv = H.dev(a, "f32"), H.dev(inds, "i32")
    for p in params[::17]:
        c_tv = tv.zeros([m, k], tv.float32, 0)
        assert lib.supported(p[2], k, tv.float32)
        lib.gather(c_tv, a_tv, inds_tv, *p)
        lib.stream_synchronize()
        np.testing.assert_array_equal(H.host(c_tv), a[inds])


@pytest.mark.parametrize("dtype,channels", [("f32", 128), ("f32", 3), ("f16", 64), ("f16", 6), ("bf16", 40)])
def test_scatter_add_rows(dtype, channels):
    print("case scatter", dtype, channels, flush=True)
    rng = np.random.default_rng(20 + channels)
    rows, m = 6000, 4100
    inp = H.to_storage(rng.normal(0, 1, size=(m, channels)).astype(np.float32), dtype)
    out = H.to_storage(rng.normal(0, 1, size=(rows, channels)).astype(np.float32), dtype)
    idx = rng.permutation(rows + 2)[:m].astype(np.int32) - 1   # unique, one -1 and one == rows possible
    lib = ScatterAll()
    out_tv = H.dev(out, dtype)
    assert lib.supported_scatter(8, 256, 4, 128, channels, H.TV_DTYPE[dtype])
    lib.scatter(out_tv, H.dev(inp, dtype), H.dev(idx, "i32"), 8, 256, 4, 128)
    np.testing.assert_array_equal(H.host(out_tv), gather_ref.scatter_add_rows_ref(out, inp, idx, dtype))


def test_gather_then_scatter_round_trip_full_size():
    """1 M rows of 128 bytes: gather with a permutation, scatter-add into zeros with the same
    permutation gives the input back (size-independent property)."""
    rng = np.random.default_rng(3)
    n, c = 1_000_000, 64
    a = rng.integers(-1000, 1000, size=(n, c)).astype(np.float16)
    perm = rng.permutation(n).astype(np.int32)
    a_tv, p_tv = H.dev(a, "f16"), H.dev(perm, "i32")
    g = tv.zeros([n, c], tv.float16, 0)
    GatherAll().gather(g, a_tv, p_tv)
    back = tv.zeros([n, c], tv.float16, 0)
    ScatterAll().scatter(back, g, p_tv)
    np.testing.assert_array_equal(H.host(back), a)


def test_gather_scatter_errors():
    a = tv.zeros([16, 6], tv.float16, 0)
    idx = tv.zeros([4], tv.int32, 0)
    with pytest.raises(RuntimeError):
        GatherAll().gather(tv.zeros([4, 8], tv.float16, 0), a, idx)            # column mismatch
    with pytest.raises(RuntimeError):
        GatherAll().gather(tv.zeros([4, 6], tv.float16, 0), a, idx, 8, 512, 16, 128)   # 12 bytes % 16
    with pytest.raises(RuntimeError):
        GatherAll().gather(tv.zeros([4, 6], tv.float16, 0), a, idx, 3, 512, 4, 128)    # no such kernel
    with pytest.raises(RuntimeError):
        ScatterAll().scatter(tv.zeros([16, 6], tv.int8, 0), tv.zeros([4, 6], tv.int8, 0), idx)   # dtype
    assert not ScatterAll().supported_scatter(8, 256, 16, 128, 6, tv.float16)
    GatherAll().gather(tv.zeros([0, 6], tv.float16, 0), a, tv.zeros([0], tv.int32, 0))   # empty: no-op
