"""Writes tests/golden/*.npz from the reference's own modules.cpp, compiled in place by `make -C oracle ref`.

Run in the authoring container only (it needs /root/reference to build oracle/_ref/libsd3_ref.so):
    make -C oracle ref && python tests/golden/make_golden.py
Inputs are regenerated from seeds by tests/cases.py; the fixtures hold the reference's outputs only."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import cases  # noqa: E402
import oracle_lib as ol  # noqa: E402


def main():
    if ol.reference() is None:
        raise SystemExit("oracle/_ref/libsd3_ref.so is missing: run `make -C oracle ref` first")
    out = {}
    for name in cases.BLOCK_CASES:
        k = cases.block_case(name)
        c, x = ol.ref_dit_block(k["y"], k["c"], k["x"], k["params"], k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
        out[name + ".c"] = c
        out[name + ".x"] = x
    for name in cases.DIT_CASES:
        k = cases.dit_case(name)
        out[name + ".out"] = ol.ref_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
    np.savez_compressed(os.path.join(HERE, "reference_outputs.npz"), **out)
    if "--with-reference-test-config" in sys.argv:  # about a minute of single-core CPU
        k = cases.dit_reference_test_case()
        big = ol.ref_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
        np.savez_compressed(os.path.join(HERE, "reference_dit_test_config.npz"), out=big.astype(np.float32))
        out["dit_reference_test.out"] = big
    for k, v in out.items():
        print(f"{k:28s} {str(v.shape):18s} absmax {np.abs(v).max():.4f}")


if __name__ == "__main__":
    main()
