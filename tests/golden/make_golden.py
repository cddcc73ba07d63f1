"""Writes tests/golden/layer_c1_*.npz: inputs and float64 expected outputs of the tiny default-variant
configuration (E=4, d=64, h=256, [2,16,64]) and of its cpm_2 / base_layer / reference-as-coded
siblings, computed by oracle/moe_oracle.py after its pins pass (tests/test_oracle_pins.py).

The reference ships no golden vectors and cannot be run; these fixtures freeze the pinned oracle's
answers so that a later change to the oracle, the C restatement or the kernels shows up as a diff
against committed data.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402

CASES = {
    "default_rms_relu": ("default", "rms", "relu"),
    "cpm2_rms_relu": ("cpm_2", "rms", "relu"),
    "base_rms_relu": ("base_layer", "rms", "relu"),
    "cpm2_centered_gated": ("cpm_2", "centered", "gated_gelu"),
}


def main():
    E, d, h, T, seed = 4, 64, 256, 32, 0
    out_dir = os.path.dirname(os.path.abspath(__file__))
    for name, (variant, norm, ffn) in CASES.items():
        x, c, g = O.draw_inputs(seed, T, d, E)
        ws = [O.draw_expert(seed, e, d, h, ffn) for e in range(E)]
        r = O.moe_layer(x, c, variant, ws, layernorm_weight=g, norm_kind=norm, ffn_kind=ffn)
        arrays = dict(x=x, centroids=c, layernorm_weight=g, out=r["out"], sel=r["sel"], coeff=r["coeff"],
                      count=r["count"], offset=r["offset"], pos=r["pos"])
        for e, w in enumerate(ws):
            for k, v in w.items():
                arrays[f"{e}/{k}"] = v
        np.savez_compressed(os.path.join(out_dir, f"layer_c1_{name}.npz"), **arrays)
        print(name, "min top-2 gap", O.top2_relative_gap(r["aff"]).min())


if __name__ == "__main__":
    main()
