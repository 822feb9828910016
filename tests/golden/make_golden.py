#!/usr/bin/env python3
"""Writes tests/golden/*.npz by running the reference's own compiled C path.

Runs only in the container where /root/reference is mounted: `make -C oracle`
compiles the reference's sources where they lie into oracle/_ref/libqwen4_ref.so,
and this script feeds it seeded inputs and stores inputs and outputs.  The
fixtures are data only (packed weight bytes, activations, expected outputs as
raw bit patterns); tests/test_golden.py replays them against the CPU oracle
(no GPU) and against the HIP path (GPU).
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import picoforge_amd as pf  # noqa: E402
from picoforge_amd import abi  # noqa: E402
from helpers import call_decode, call_group, call_route, forward_with, make_layer_inputs  # noqa: E402
from hc_cases import call_add, call_read, random_case  # noqa: E402

OUT = Path(__file__).resolve().parent

FORWARD_CASES = {
    # name: hidden, experts, top_k, inter, shared_inter, type, tokens, seed
    "forward_f32_tiny": (8, 4, 2, 5, 3, abi.GGUF_F32, 33, 21),
    "forward_f32_wide": (64, 16, 4, 24, 12, abi.GGUF_F32, 9, 22),
    "forward_q4k": (256, 4, 2, 256, 256, abi.GGUF_Q4_K, 6, 23),
    "forward_iq2xxs": (256, 6, 3, 256, 256, abi.GGUF_IQ2_XXS, 6, 24),
}


HC_CASES = [(5, 3, 7, 1.0), (3, 4, 256, 4.0), (2, 4, 64, 30.0)]   # tokens, streams, hidden, logit scale


def write_hc(ref):
    """qwen4_hc_read and qwen4_hc_add of the reference on seeded inputs, the exp branches included."""
    arrays = {}
    for n, (t, h, w, scale) in enumerate(HC_CASES):
        normed, logits, block, inject = random_case(t, h, w, 26 + n, scale=scale)
        logits.ravel()[:4] = (0.0, -0.0, 89.0, -104.0)
        st, mixed, _ = call_read(ref, normed, logits)
        assert st == 0
        residual = normed.copy()
        assert call_add(ref, residual, block, inject)[0] == 0
        arrays.update({f"normed{n}": normed, f"logits{n}": logits, f"block{n}": block, f"inject{n}": inject,
                       f"mixed_bits{n}": mixed.view(np.uint32), f"residual_bits{n}": residual.view(np.uint32)})
    np.savez_compressed(OUT / "hc_read_add.npz", **arrays)


def main():
    from oracle.load import load_reference
    ref = load_reference()
    if ref is None:
        sys.exit("oracle/_ref/libqwen4_ref.so missing: run make -C oracle where the reference is mounted")
    write_hc(ref)
    if "--only-hc" in sys.argv:
        return
    for name, (h, e, k, i, s, gtype, tokens, seed) in FORWARD_CASES.items():
        cfg = abi.moe_config(h, e, k, i, s)
        weights, x = make_layer_inputs(cfg, gtype, tokens, seed=seed, std=0.02 if gtype else 0.2)
        y, ids, w = forward_with(ref, cfg, weights, x)
        np.savez_compressed(OUT / f"{name}.npz", config=np.array([h, e, k, i, s, i, 1], dtype=np.uint32),
                            types=np.array(weights.types, dtype=np.uint32), x=x, y_bits=y.view(np.uint32), ids=ids,
                            w_bits=w.view(np.uint32), **{f"tensor{j}": weights.raw[j] for j in range(8)})
    rng = np.random.default_rng(25)
    cfg = abi.moe_config(8, 512, 10, 5, 3)
    z = rng.normal(0, 1.2, (16, 512)).astype(np.float32)
    z[1] = 0
    z[2] = np.round(z[2] * 2) / 2
    z[3, :20] = z[3, 0]
    st, p, ids, w, _ = call_route(ref, cfg, z)
    assert st == 0
    st, off, cur, p2r, r2p = call_group(ref, cfg, ids)
    assert st == 0
    np.savez_compressed(OUT / "route_512_top10.npz", logits=z, p_bits=p.view(np.uint32), ids=ids,
                        w_bits=w.view(np.uint32), offsets=off[:513], pair_to_row=p2r[:160], row_to_pair=r2p[:160])
    for gtype, size, name in ((abi.GGUF_Q4_K, 144, "decode_q4k"), (abi.GGUF_IQ2_XXS, 66, "decode_iq2xxs")):
        blocks = rng.integers(0, 256, (4 * 3, size), dtype=np.uint8)
        blocks[:, 0:2] = rng.uniform(-1, 1, (12, 1)).astype(np.float16).view(np.uint8)
        if gtype == abi.GGUF_Q4_K:
            blocks[:, 2:4] = rng.uniform(-1, 1, (12, 1)).astype(np.float16).view(np.uint8)
        raw = blocks.reshape(-1)
        rows = np.stack([call_decode(ref, raw, gtype, 768, 4, r)[1] for r in range(4)])
        np.savez_compressed(OUT / f"{name}.npz", raw=raw, rows_bits=rows.view(np.uint32))
    print("wrote", sorted(p.name for p in OUT.glob("*.npz")))


if __name__ == "__main__":
    main()
