"""Random shapes through matmul2, against the oracle.

Dense GEMM (all transposes, outputs in the operands' or the accumulator's type, serial split-K),
gather-GEMM-scatter (ShuffleAC) and the gathered weight-gradient GEMM (ShuffleAB, with split-K)
for f16, bf16 and s8, with sizes, tiles and index sets drawn from a seeded generator - down to
one row and up to a few thousand, most of them no multiple of any tile.  Each case prints its
parameters before it runs.  s8 / s32 results bit-exact, f16 / bf16 within 1e-2.
"""
import json

import numpy as np
import pytest

import helpers as H
from oracle import gemm_ref
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import GemmParams, ShuffleStrideType

pytestmark = pytest.mark.gpu
TOL = 1e-2
TILE_K = {"s8": 64, "f16": 32, "bf16": 32}
WIDE = {"s8": "s32", "f16": "f32", "bf16": "f32"}


def rand(rng, shape, dtype, scale=1.0):
    if dtype == "s8":
        return rng.integers(-127, 128, size=shape).astype(np.int8)
    return H.to_storage((rng.uniform(-1, 1, size=shape) * scale).astype(np.float32), dtype)


def compare(got, ref, dtype):
    if dtype in ("s8", "s32"):
        return float((np.asarray(got) != np.asarray(ref)).sum())
    return H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype))


def one_case(seed):
    rng = np.random.default_rng(seed)
    dtype = str(rng.choice(["f16", "bf16", "s8"]))
    kind = str(rng.choice(["dense", "ac", "ab"]))
    align = 16 if dtype == "s8" else 8
    desc = dict(seed=seed, dtype=dtype, kind=kind)
    if kind == "dense":
        tile = tuple(int(x) for x in rng.choice([64, 128], size=1)) * 2
        ta, tb, tc = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        m = int(rng.integers(1, 60)) * align
        n = int(rng.integers(1, 60)) * align
        k = int(rng.integers(1, 90)) * align
        wide = bool(rng.integers(0, 2)) and not tc
        split = int(rng.choice([1, 1, 2, 4])) if not wide or dtype == "s8" else 1
        beta = float(rng.choice([0.0, 1.0]))
        alpha = 1.0 if dtype != "s8" or wide else 2e-5
        out_t = WIDE[dtype] if wide else dtype
        desc.update(tile=tile, ta=ta, tb=tb, tc=tc, m=m, n=n, k=k, wide=wide, split=split, beta=beta)
        print("case", json.dumps(desc), flush=True)
        a = rand(rng, (k, m) if ta else (m, k), dtype)
        b = rand(rng, (n, k) if tb else (k, n), dtype, 0.1)
        if out_t == "s32":
            c0 = rng.integers(-1000, 1000, size=(n, m) if tc else (m, n)).astype(np.int32)
        elif out_t == "f32":
            c0 = rng.uniform(-1, 1, size=(m, n)).astype(np.float32)
        else:
            c0 = rand(rng, (n, m) if tc else (m, n), dtype)
        try:
            desp = H.find_gemm_desp(dtype, ShuffleStrideType.NoShuffle, *tile, ta, tb, tc, dtype_c=out_t)
        except KeyError:
            return True, 0.0, desc
        p = GemmParams()
        p.algo_desp = desp
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, out_t)
        p.alpha, p.beta, p.split_k_slices = alpha, beta, split
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=out_t, trans_a=ta, trans_b=tb, trans_c=tc,
                                   alpha=alpha, beta=beta, split_k_slices=split, tile_k=TILE_K[dtype])
        err = compare(H.host(p.c), ref, out_t)
    elif kind == "ac":
        tile = tuple(int(x) for x in rng.choice([64, 128], size=2))
        tb = bool(rng.integers(0, 2))
        rows = int(rng.integers(1, 6000))
        m = int(rng.integers(1, rows + 1))
        n = int(rng.integers(1, 33)) * align
        k = int(rng.integers(1, 33)) * align
        beta = float(rng.choice([0.0, 1.0]))
        alpha = 1.0 if dtype != "s8" else 1e-4
        desc.update(tile=tile, tb=tb, rows=rows, m=m, n=n, k=k, beta=beta)
        print("case", json.dumps(desc), flush=True)
        a = rand(rng, (rows, k), dtype)
        b = rand(rng, (n, k) if tb else (k, n), dtype, 0.1)
        a_inds = rng.permutation(rows)[:m].astype(np.int32)
        c_inds = rng.permutation(rows)[:m].astype(np.int32)
        c0 = rand(rng, (rows, n), dtype)
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, *tile, False, tb)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
        p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
        p.alpha, p.beta = alpha, beta
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_b=tb, shuffle=gemm_ref.SHUFFLE_AC,
                                   a_inds=a_inds, c_inds=c_inds, alpha=alpha, beta=beta)
        err = compare(H.host(p.c), ref, dtype)
    else:
        tile = tuple(int(x) for x in rng.choice([64, 128], size=1)) * 2
        rows = int(rng.integers(1, 6000))
        kk = int(rng.integers(1, rows + 1))          # contraction = gathered rows
        m = int(rng.integers(1, 25)) * align
        n = int(rng.integers(1, 25)) * align
        split = int(rng.choice([1, 1, 2, 4]))
        beta = float(rng.choice([0.0, 1.0]))
        alpha = 1.0 if dtype != "s8" else 2e-5
        desc.update(tile=tile, rows=rows, k=kk, m=m, n=n, split=split, beta=beta)
        print("case", json.dumps(desc), flush=True)
        a = rand(rng, (rows, m), dtype)              # trans_a: A stored [k, m]
        b = rand(rng, (rows, n), dtype, 0.1)         # B stored [k, n]
        a_inds = rng.permutation(rows)[:kk].astype(np.int32)
        b_inds = rng.permutation(rows)[:kk].astype(np.int32)
        c0 = rand(rng, (m, n), dtype)
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAB, *tile, True, False)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
        p.a_inds, p.b_inds = H.dev(a_inds, "i32"), H.dev(b_inds, "i32")
        p.alpha, p.beta, p.split_k_slices = alpha, beta, split
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_a=True, trans_b=False,
                                   shuffle=gemm_ref.SHUFFLE_AB, a_inds=a_inds, b_inds=b_inds, alpha=alpha, beta=beta,
                                   split_k_slices=split, tile_k=TILE_K[dtype])
        err = compare(H.host(p.c), ref, dtype)
    ok = err == 0 if dtype == "s8" else err < TOL
    return ok, err, desc


@pytest.mark.parametrize("block", range(6))
def test_random_gemm_shapes_against_the_oracle(block):
    bad = []
    for it in range(80):
        ok, err, desc = one_case(9000000 + block * 1000 + it)
        if not ok:
            bad.append((desc, err))
    assert not bad, bad
