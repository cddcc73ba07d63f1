"""The C/OpenMP restatement (benchmark CPU baseline) against the pinned float64 numpy oracle."""
import numpy as np
import pytest

from oracle import moe_cpu
from oracle import moe_oracle as O


@pytest.mark.parametrize("variant,norm,ffn", [
    ("default", "rms", "relu"), ("cpm_2", "rms", "relu"), ("base_layer", "rms", "relu"),
    ("cpm_2", "centered", "gated_gelu"),
])
def test_c_layer_matches_numpy_oracle(variant, norm, ffn):
    T, d, h, E = 150, 72, 136, 5
    x, c, g = O.draw_inputs(3, T, d, E)
    ws = [O.draw_expert(3, e, d, h, ffn) for e in range(E)]
    slots = [moe_cpu.pack_slot(w, ffn) for w in ws]
    y, sel, count = moe_cpu.layer(x, c, variant, slots, gamma=g if variant == "cpm_2" else None, h=h,
                                  norm_kind=norm, ffn_kind=ffn)
    ref = O.moe_layer(x, c, variant, ws, layernorm_weight=g, norm_kind=norm, ffn_kind=ffn)
    assert (O.top2_relative_gap(ref["aff"]) > 1e-4).all()
    np.testing.assert_array_equal(sel, ref["sel"])
    np.testing.assert_array_equal(count, ref["count"])
    scale = np.abs(ref["out"]).max()
    assert np.abs(y - ref["out"]).max() <= 1e-4 * scale


def test_c_layer_identity_and_nan():
    x, c, g = O.draw_inputs(4, 64, 32, 4)
    y, sel, count = moe_cpu.layer(x, c, "cpm_2", None, gamma=g)
    np.testing.assert_array_equal(y, x)
    x[3, :] = np.nan
    with pytest.raises(FloatingPointError):
        moe_cpu.layer(x, c, "default", None)
    assert moe_cpu.load().moe_cpu_threads() >= 1
