"""Replays the committed golden vectors (written by the reference's compiled C path, see
tests/golden/make_golden.py): bit for bit against the CPU oracle, and through the HIP
path at the parity bar of the device kernels."""
from pathlib import Path

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from hc_cases import call_add, call_read
from helpers import assert_parity, call_decode, call_group, call_route, forward_with

GOLDEN = Path(__file__).resolve().parent / "golden"
FORWARD = sorted(p.stem for p in GOLDEN.glob("forward_*.npz"))


def load_forward(name):
    data = np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
    h, e, k, i, s, dp, norm = (int(v) for v in data["config"])
    cfg = abi.moe_config(h, e, k, i, s, dp, bool(norm))
    weights = pf.LayerWeights(cfg, [data[f"tensor{j}"].copy() for j in range(8)], [int(t) for t in data["types"]])
    return cfg, weights, data["x"].copy(), data["y_bits"].view(np.float32), data["ids"], data["w_bits"].view(np.float32)


def test_fixtures_exist():
    assert len(FORWARD) == 4 and (GOLDEN / "route_512_top10.npz").exists()


@pytest.mark.parametrize("name", FORWARD)
def test_oracle_reproduces_forward_fixture(oracle, name):
    cfg, weights, x, y, ids, w = load_forward(name)
    got = forward_with(oracle, cfg, weights, x)
    np.testing.assert_array_equal(got[0].view(np.uint32), y.view(np.uint32))
    np.testing.assert_array_equal(got[1], ids)
    np.testing.assert_array_equal(got[2].view(np.uint32), w.view(np.uint32))


def test_oracle_reproduces_route_group_and_decode_fixtures(oracle):
    data = np.load(GOLDEN / "route_512_top10.npz", allow_pickle=False)
    cfg = abi.moe_config(8, 512, 10, 5, 3)
    st, p, ids, w, _ = call_route(oracle, cfg, data["logits"])
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(p.view(np.uint32), data["p_bits"])
    np.testing.assert_array_equal(ids, data["ids"])
    np.testing.assert_array_equal(w.view(np.uint32), data["w_bits"])
    st, off, cur, p2r, r2p = call_group(oracle, cfg, data["ids"])
    np.testing.assert_array_equal(off[:513], data["offsets"])
    np.testing.assert_array_equal(p2r[:160], data["pair_to_row"])
    np.testing.assert_array_equal(r2p[:160], data["row_to_pair"])
    for gtype, name in ((abi.GGUF_Q4_K, "decode_q4k"), (abi.GGUF_IQ2_XXS, "decode_iq2xxs")):
        data = np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
        for row in range(4):
            st, out = call_decode(oracle, data["raw"].copy(), gtype, 768, 4, row)
            np.testing.assert_array_equal(out.view(np.uint32), data["rows_bits"][row])


def replay_hc_fixture(api):
    data = np.load(GOLDEN / "hc_read_add.npz", allow_pickle=False)
    cases = sorted(int(k[6:]) for k in data.files if k.startswith("normed"))
    assert len(cases) == 3
    for n in cases:
        normed, logits = data[f"normed{n}"].copy(), data[f"logits{n}"].copy()
        st, mixed, _ = call_read(api, normed, logits)
        assert st == abi.QW4_OK
        np.testing.assert_array_equal(mixed.view(np.uint32), data[f"mixed_bits{n}"], err_msg=f"read, case {n}")
        residual = normed.copy()
        assert call_add(api, residual, data[f"block{n}"].copy(), data[f"inject{n}"].copy())[0] == abi.QW4_OK
        np.testing.assert_array_equal(residual.view(np.uint32), data[f"residual_bits{n}"], err_msg=f"add, case {n}")


def test_oracle_reproduces_hc_fixture(oracle):
    replay_hc_fixture(oracle)


@pytest.mark.gpu
def test_hip_path_reproduces_hc_fixture_bit_for_bit(product):
    replay_hc_fixture(product)


@pytest.mark.gpu
@pytest.mark.parametrize("name", FORWARD)
def test_hip_path_reproduces_forward_fixture(product, name):
    cfg, weights, x, y, ids, w = load_forward(name)
    got = forward_with(product, cfg, weights, x)
    assert_parity(*got, y, ids, w, label=name)


@pytest.mark.gpu
def test_hip_path_reproduces_route_group_and_decode_fixtures(product):
    data = np.load(GOLDEN / "route_512_top10.npz", allow_pickle=False)
    cfg = abi.moe_config(8, 512, 10, 5, 3)
    st, p, ids, w, _ = call_route(product, cfg, data["logits"])
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(ids, data["ids"])
    np.testing.assert_array_equal(p.view(np.uint32), data["p_bits"])
    np.testing.assert_array_equal(w.view(np.uint32), data["w_bits"])
    st, off, cur, p2r, r2p = call_group(product, cfg, data["ids"])
    np.testing.assert_array_equal(off[:513], data["offsets"])
    np.testing.assert_array_equal(p2r[:160], data["pair_to_row"])
    np.testing.assert_array_equal(r2p[:160], data["row_to_pair"])
    for gtype, name in ((abi.GGUF_Q4_K, "decode_q4k"), (abi.GGUF_IQ2_XXS, "decode_iq2xxs")):
        data = np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
        for row in range(4):
            st, out = call_decode(product, data["raw"].copy(), gtype, 768, 4, row)
            np.testing.assert_array_equal(out.view(np.uint32), data["rows_bits"][row])
