"""The Python mirror of GemmAlgoDesp / ConvAlgoDesp and the m/n/k helpers against the
reference's own descriptor logic: golden answers minted from the reference headers
(tests/golden/desp_golden.json), and the live oracle/_ref library where it is built."""
import ctypes
import json
import os

import pytest

from cumm_amd.tensorview import gemm as G

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, "golden", "desp_golden.json")))


def make_desps(rec):
    d, algo = rec["desc"], rec["algo"]

    def fill(x):
        x.dtype_a, x.dtype_b, x.dtype_c = d["dtype_a"], d["dtype_b"], d["dtype_c"]
        x.trans_a_, x.trans_b_, x.trans_c_ = d["trans_a"], d["trans_b"], d["trans_c"]
        x.tile_shape = [d["ts0"], d["ts1"], d["ts2"]]
        x.warp_tile_shape = [d["wts0"], d["wts1"], d["wts2"]]
        x.num_stage, x.dacc, x.dcomp, x.algo = d["num_stage"], d["dacc"], d["dcomp"], algo
        x.tensorop = [d["top0"], d["top1"], d["top2"]]
        x.split_k_serial_, x.split_k_parallel_ = d["split_k_serial"], d["split_k_parallel"]
        x.shuffle_type = G.ShuffleStrideType(d["shuffle"])
        x.element_per_access_a, x.element_per_access_b = d["epa_a"], d["epa_b"]
        x.element_per_access_c, x.access_per_vector = d["epa_c"], d["apv"]
        return x
    g = fill(G.GemmAlgoDesp())
    c = fill(G.ConvAlgoDesp(d["ndim"], G.ConvOpType(d["op_type"])))
    c.mask_sparse, c.increment_k_first = bool(d["mask_sparse"]), bool(d["inc_k_first"])
    c.dynamic_mask, c.is_int8_inference = bool(d["dyn_mask"]), bool(d["int8_infer"])
    return g, c


def _name_or_error(desp):
    try:
        return 0, repr(desp)
    except RuntimeError as e:
        return 1, str(e)


@pytest.mark.parametrize("rec", GOLDEN["cases"], ids=lambda r: r["gemm_repr"][1][:60].replace("\n", " "))
def test_descriptor_against_reference(rec):
    g, c = make_desps(rec)
    for desp, key in ((g, "gemm_repr"), (c, "conv_repr")):
        rc, text = _name_or_error(desp)
        ref_rc, ref_text = rec[key]
        assert rc == ref_rc
        if rc == 0:
            assert text == ref_text
        else:
            # the reference prefixes file(line) and the failed expression; the message must match
            assert text.split(" [")[0] in ref_text
    assert [c.dtype_input, c.dtype_weight, c.dtype_output] == rec["dtypes_iwo"]
    for pr in rec["probes"]:
        m, n, k = pr["m"], pr["n"], pr["k"]
        for desp, fn, key in ((g, lambda: g.query_workspace_size(m, n, k, pr["split"]), "gemm_ws"),
                              (c, lambda: c.query_conv_workspace_size(m, n, k, pr["split"], pr["kv"]),
                               "conv_ws")):
            try:
                got = fn()
            except ValueError:
                got = -1   # "not impemented": split-K asked of a descriptor without split-K
            assert got == pr[key]
        assert int(g.supported(m, n, k)) == pr["gemm_supported"]
        assert int(g.supported_ldx(m, n, k)) == pr["gemm_supported_ldx"]
        assert int(c.supported(m, n, k, pr["C"], pr["K"], pr["mask_width"])) == pr["conv_supported"]


def test_helper_functions_against_reference():
    f = GOLDEN["funcs"]
    for r in f["iwo_abc"]:
        assert G.conv_iwo_012_to_abc(r["op"]) == r["iwo2abc"]
        assert G.gemm_abc_012_to_iwo(r["op"]) == r["abc2iwo"]
    for r in f["mnk"]:
        assert G.implicit_gemm_mnk(r["op"], r["N"], r["C"], r["K"], r["kv"], r["in_prod"],
                                   r["out_prod"], bool(r["mask_sparse"])) == r["mnk"]
    for r in f["tile_count"]:
        assert G.get_logical_tile_count(r["m"], r["n"], r["k"], r["tm"], r["tn"], r["split"]) == r["out"]
    for r in f["spconv_tile_count"]:
        assert G.get_spconv_logical_tile_count(r["m"], r["n"], r["k"], r["tm"], r["tn"], r["split"],
                                               r["kv"], r["op"]) == r["out"]
    for r in f["k_per_split"]:
        assert G.get_gemm_k_size_per_split(r["k"], r["split"], r["tile_k"]) == r["out"]


def test_live_reference_library_if_built():
    """Where oracle/_ref has been built (needs the reference tree), query it directly."""
    lib_path = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libcummref_host.so")
    if not os.path.exists(lib_path):
        pytest.skip("oracle/_ref not built (the reference tree is not on this machine)")
    lib = ctypes.CDLL(lib_path)
    out3 = (ctypes.c_int * 3)()
    for op in range(3):
        for N, C, K, kv in [(7, 8, 16, 27), (123457, 64, 64, 27), (5, 128, 256, 8)]:
            lib.ref_implicit_gemm_mnk(op, N, C, K, kv, -1, -1, 1, out3)
            assert G.implicit_gemm_mnk(op, N, C, K, kv, -1, -1, True) == list(out3)
            m, n, k = G.implicit_gemm_mnk(op, N, C, K, kv, -1, -1, True)
            lib.ref_spconv_tile_count(m, n, k, 64, 64, 3, kv, op, out3)
            assert G.get_spconv_logical_tile_count(m, n, k, 64, 64, 3, kv, op) == list(out3)


def test_params_setters_record_dtypes():
    """GemmParams.a/b/c setters also write algo_desp.dtype_* (params.h:366-383 of the reference)."""
    from cumm_amd import tensorview as tv
    import numpy as np
    p = G.GemmParams()
    p.a = tv.from_numpy(np.zeros((2, 8), np.float16))
    p.b = tv.from_numpy(np.zeros((2, 8), np.int8))
    p.c = tv.from_numpy(np.zeros((2, 2), np.float32))
    assert (p.algo_desp.dtype_a, p.algo_desp.dtype_b, p.algo_desp.dtype_c) == (7, 3, 0)
    with pytest.raises(RuntimeError):
        p.d = tv.from_numpy(np.zeros((2, 2), np.float16))   # d dtype must equal to c
    with pytest.raises(RuntimeError):
        p.check_valid()
