"""Mint tests/golden/desp_golden.json from the reference's own descriptor logic.

Runs in the build container only: it loads oracle/_ref/libcummref_host.so, which
oracle/Makefile compiles from the reference's header-only host structs
(include/tensorview/gemm/core/params.h, utils.h) where they lie under
/root/reference.  The JSON holds inputs and the reference's answers (kernel name
strings, validity errors, alignment checks, workspace sizes, m/n/k, tile counts);
tests/test_desp.py replays them against the Python mirror in cumm_amd.tensorview.gemm.

    make -C oracle ref && python tests/golden/make_desp_golden.py
"""
import ctypes
import itertools
import json
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(ROOT, "oracle", "_ref", "libcummref_host.so")

FIELDS = ["dtype_a", "dtype_b", "dtype_c", "trans_a", "trans_b", "trans_c", "ts0", "ts1", "ts2",
          "wts0", "wts1", "wts2", "num_stage", "dacc", "dcomp", "top0", "top1", "top2",
          "split_k_serial", "split_k_parallel", "shuffle", "epa_a", "epa_b", "epa_c", "apv",
          "ndim", "op_type", "mask_sparse", "inc_k_first", "dyn_mask", "int8_infer"]


def load():
    lib = ctypes.CDLL(LIB)
    assert lib.ref_field_count() == len(FIELDS)
    return lib


def arr(d):
    return (ctypes.c_int * len(FIELDS))(*[d[f] for f in FIELDS])


def base_desc(**kw):
    d = dict(dtype_a=7, dtype_b=7, dtype_c=7, trans_a=0, trans_b=1, trans_c=0, ts0=64, ts1=64,
             ts2=32, wts0=32, wts1=32, wts2=32, num_stage=2, dacc=0, dcomp=0, top0=16, top1=8,
             top2=8, split_k_serial=0, split_k_parallel=0, shuffle=0, epa_a=8, epa_b=8, epa_c=8,
             apv=1, ndim=3, op_type=0, mask_sparse=1, inc_k_first=1, dyn_mask=0, int8_infer=0)
    d.update(kw)
    return d


def main():
    lib = load()
    rng = random.Random(20240607)
    buf = ctypes.create_string_buffer(2048)
    out3 = (ctypes.c_int * 3)()
    cases = []
    descs = []
    dtypes = [(7, 7, 7, 0, 0), (12, 12, 12, 0, 0), (3, 3, 3, 1, 0), (0, 0, 0, 0, 0), (3, 3, 1, 1, 1),
              (7, 7, 0, 0, 0)]
    for (da, db, dc, dacc, dcomp), algo, shuffle, splits, op in itertools.product(
            dtypes, ["Turing", "Ampere", "Simt", "Cdna4"], [0, 1, 2], [(0, 0), (1, 0), (0, 1)],
            [0, 1, 2]):
        ts = rng.choice([(64, 64, 32), (128, 64, 32), (128, 128, 32), (32, 64, 64), (64, 128, 64)])
        wts = rng.choice([(32, 32, 32), (16, 64, 32), (64, 64, 64)])
        tr = {0: (0, 1, 0), 1: (0, 0, 0), 2: (1, 0, 0)}[op]
        top = (-1, -1, -1) if algo == "Simt" else rng.choice([(16, 8, 8), (16, 16, 32), (16, 16, 64)])
        d = base_desc(dtype_a=da, dtype_b=db, dtype_c=dc, dacc=dacc, dcomp=dcomp, trans_a=tr[0],
                      trans_b=tr[1], trans_c=tr[2], ts0=ts[0], ts1=ts[1], ts2=ts[2], wts0=wts[0],
                      wts1=wts[1], wts2=wts[2], top0=top[0], top1=top[1], top2=top[2],
                      split_k_serial=splits[0], split_k_parallel=splits[1], shuffle=shuffle,
                      epa_a=rng.choice([-1, 4, 8, 16]), epa_b=rng.choice([-1, 4, 8, 16]),
                      epa_c=rng.choice([-1, 4, 8, 16]), apv=rng.choice([1, 2]),
                      num_stage=rng.choice([2, 3]), op_type=op,
                      mask_sparse=rng.choice([0, 1]), inc_k_first=rng.choice([0, 1]),
                      dyn_mask=rng.choice([0, 1]), int8_infer=rng.choice([0, 1]))
        descs.append((d, algo))
    rng.shuffle(descs)
    descs = descs[:90]
    # invalid descriptors: the reference's check_valid messages
    descs.append((base_desc(trans_a=-1), "Turing"))
    descs.append((base_desc(ts0=-1), "Turing"))
    descs.append((base_desc(top0=-1), "Turing"))
    descs.append((base_desc(dtype_a=-1), "Turing"))
    descs.append((base_desc(dacc=-1), "Turing"))
    descs.append((base_desc(num_stage=0), "Turing"))
    descs.append((base_desc(), ""))
    for d, algo in descs:
        a = arr(d)
        algo_b = algo.encode()
        rec = {"desc": d, "algo": algo}
        rc = lib.ref_gemm_repr(a, algo_b, buf, len(buf))
        rec["gemm_repr"] = [rc, buf.value.decode()]
        rc = lib.ref_conv_repr(a, algo_b, buf, len(buf))
        rec["conv_repr"] = [rc, buf.value.decode()]
        lib.ref_conv_dtypes_iwo(a, algo_b, out3)
        rec["dtypes_iwo"] = list(out3)
        probes = []
        for _ in range(4):
            m, n, k = rng.choice([64, 72, 100, 1000, 4096]), rng.choice([64, 96, 1728, 3456]), \
                rng.choice([64, 60, 1728, 120000])
            split = rng.choice([1, 2, 8, 32])
            kv = 27
            C, K, mw = rng.choice([64, 60, 128]), rng.choice([64, 72, 128]), rng.choice([32, 64, 48, 128])
            probes.append({
                "m": m, "n": n, "k": k, "split": split, "kv": kv, "C": C, "K": K, "mask_width": mw,
                "gemm_ws": lib.ref_gemm_workspace(a, algo_b, m, n, k, split),
                "conv_ws": lib.ref_conv_workspace(a, algo_b, m, n, k, split, kv),
                "gemm_supported": lib.ref_gemm_supported(a, algo_b, m, n, k),
                "gemm_supported_ldx": lib.ref_gemm_supported_ldx(a, algo_b, m, n, k),
                "conv_supported": lib.ref_conv_supported(a, algo_b, m, n, k, C, K, mw),
            })
        rec["probes"] = probes
        cases.append(rec)
    funcs = {"mnk": [], "tile_count": [], "spconv_tile_count": [], "iwo_abc": [], "k_per_split": []}
    for op in range(3):
        a3, b3 = (ctypes.c_int * 3)(), (ctypes.c_int * 3)()
        lib.ref_iwo_abc(op, a3, b3)
        funcs["iwo_abc"].append({"op": op, "iwo2abc": list(a3), "abc2iwo": list(b3)})
        for N, C, K, kv, ip, op_, ms in [(1000, 64, 64, 27, -1, -1, 1), (119989, 64, 64, 27, -1, -1, 1),
                                         (2, 16, 32, 9, 100, 81, 0), (300000, 64, 128, 27, -1, -1, 1)]:
            lib.ref_implicit_gemm_mnk(op, N, C, K, kv, ip, op_, ms, out3)
            funcs["mnk"].append({"op": op, "N": N, "C": C, "K": K, "kv": kv, "in_prod": ip,
                                 "out_prod": op_, "mask_sparse": ms, "mnk": list(out3)})
        for m, n, k, tm, tn, split, kv in [(64, 1728, 120000, 64, 64, 32, 27), (128, 3456, 1000, 64, 64, 4, 27),
                                           (120000, 64, 1728, 128, 64, 1, 27), (130, 27 * 130, 999, 64, 64, 2, 27)]:
            lib.ref_tile_count(m, n, k, tm, tn, split, out3)
            funcs["tile_count"].append({"m": m, "n": n, "k": k, "tm": tm, "tn": tn, "split": split,
                                        "out": list(out3)})
            lib.ref_spconv_tile_count(m, n, k, tm, tn, split, kv, op, out3)
            funcs["spconv_tile_count"].append({"m": m, "n": n, "k": k, "tm": tm, "tn": tn,
                                               "split": split, "kv": kv, "op": op, "out": list(out3)})
    for k, split, tk in [(1000, 4, 32), (120000, 32, 32), (64, 1, 32), (33, 2, 32)]:
        funcs["k_per_split"].append({"k": k, "split": split, "tile_k": tk,
                                     "out": lib.ref_gemm_k_size_per_split(k, split, tk)})
    with open(os.path.join(HERE, "desp_golden.json"), "w") as f:
        json.dump({"fields": FIELDS, "cases": cases, "funcs": funcs}, f, separators=(",", ":"), sort_keys=True)
    print("wrote", len(cases), "descriptor cases")


if __name__ == "__main__":
    main()
