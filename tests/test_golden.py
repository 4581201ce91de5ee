"""The CPU oracle against the committed known-answer fixtures of tests/golden/ (computed by
tests/golden/make_fixtures.py with numpy / torch only, independently of the oracle), and the
fixtures against their generator."""
import importlib.util
import os

import numpy as np
import pytest

import helpers as H
import oracle
from oracle import layouts as L
from oracle import routing as R

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _generator():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_fixture_files_are_what_the_generator_writes():
    for name, d in _generator().all_fixtures().items():
        on_disk = load(name)
        assert sorted(on_disk) == sorted(k for k, v in d.items() if v is not None), name
        for k, v in on_disk.items():
            assert np.array_equal(v, np.asarray(d[k])), f"{name}.{k}"


@pytest.mark.parametrize("fmt", H.FORMATS)
def test_oracle_grouped_ops_match_the_fixtures(fmt):
    d = load("grouped_" + fmt)
    for gemv in (False, True):
        got = oracle.grouped_gemm(oracle.FMT_BY_NAME[fmt], d["x"], d["weight"], d.get("scale"), d.get("offset"),
                                  d["group_list"], round_bf16=not gemv)
        H.assert_close(got, d["y_gemv" if gemv else "y_gemm"], what=f"oracle {fmt} gemv={gemv}")


@pytest.mark.parametrize("block", [32, 16])
def test_oracle_dequant_matches_the_fixture_bit_for_bit(block):
    d = load("dequant_fp4")
    assert np.array_equal(oracle.dequant_fp4_bf16(d["codes"], d[f"scale_b{block}"], block), d[f"out_b{block}"])


def test_oracle_layouts_match_the_prepack_fixture():
    d = load("prepack_fp4")
    assert np.array_equal(L.fp4ref_from_checkpoint(d["ckpt"]), d["weight_out"])
    assert np.array_equal(L.fp4ref_scale_from_checkpoint(d["scale"], d["scale2"]), d["scale_out"])


def test_oracle_routing_matches_the_fixture():
    d = load("route")
    ids, w = R.route_topk(d["logits"], int(d["topk"]))
    assert np.array_equal(ids, d["ids"])
    assert np.allclose(w, d["weight"], rtol=1e-6, atol=1e-9)
    gl, rt, roc = R.route_sort(ids, d["logits"].shape[1])
    assert np.array_equal(gl, d["group_list"]) and np.array_equal(rt, d["row_token"])
    assert np.array_equal(roc, d["row_of_choice"])
