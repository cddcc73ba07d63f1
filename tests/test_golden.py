"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py) against
the oracle, the C restatement and - on the GPU - the library."""
import glob
import os

import numpy as np
import pytest

from oracle import moe_cpu
from oracle import moe_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "layer_c1_*.npz")))
KINDS = {"default_rms_relu": ("default", "rms", "relu"), "cpm2_rms_relu": ("cpm_2", "rms", "relu"),
         "base_rms_relu": ("base_layer", "rms", "relu"), "cpm2_centered_gated": ("cpm_2", "centered", "gated_gelu")}


def load(path):
    z = np.load(path)  # allow_pickle stays False
    name = os.path.basename(path)[len("layer_c1_"):-4]
    variant, norm, ffn = KINDS[name]
    E = z["centroids"].shape[0]
    keys = ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight") if ffn == "gated_gelu" else \
        ("layer_norm_weight", "wi_weight", "wo_weight")
    ws = [{k: z[f"{e}/{k}"] for k in keys} for e in range(E)]
    return z, variant, norm, ffn, ws


def test_fixtures_exist():
    assert len(FILES) == 4


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_oracle_reproduces_golden(path):
    z, variant, norm, ffn, ws = load(path)
    r = O.moe_layer(z["x"], z["centroids"], variant, ws, layernorm_weight=z["layernorm_weight"], norm_kind=norm, ffn_kind=ffn)
    np.testing.assert_array_equal(r["sel"], z["sel"])
    np.testing.assert_array_equal(r["pos"], z["pos"])
    np.testing.assert_array_equal(r["count"], z["count"])
    np.testing.assert_allclose(r["out"], z["out"], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_c_restatement_matches_golden(path):
    z, variant, norm, ffn, ws = load(path)
    slots = [moe_cpu.pack_slot(w, ffn) for w in ws]
    y, sel, count = moe_cpu.layer(z["x"], z["centroids"], variant, slots,
                                  gamma=z["layernorm_weight"] if variant == "cpm_2" else None,
                                  h=ws[0]["wo_weight"].shape[1], norm_kind=norm, ffn_kind=ffn)
    np.testing.assert_array_equal(sel, z["sel"])
    np.testing.assert_array_equal(count, z["count"])
    assert np.abs(y - z["out"]).max() <= 1e-4 * np.abs(z["out"]).max()


@pytest.mark.gpu
@pytest.mark.parametrize("mc", [2, 4])
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_library_matches_golden(torch_cuda, path, mc):
    from infmoe_amd import MoELayerConfig, MoELayerPlugin
    from tests.gpu_util import assert_close
    torch = torch_cuda
    z, variant, norm, ffn, ws = load(path)
    E, d = z["centroids"].shape
    h = ws[0]["wo_weight"].shape[1]
    cfg = MoELayerConfig(seq_len=16, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=mc,
                         moe_variant=variant, sublayer_type="T5_FF", max_batch_size=2, expert_centroids=z["centroids"],
                         layernorm_weight=z["layernorm_weight"] if variant == "cpm_2" else None, norm_kind=norm, ffn_kind=ffn)
    plugin = MoELayerPlugin(cfg).create_plugin()
    for e, w in enumerate(ws):
        for k, v in w.items():
            plugin.set_expert_weights(e, k, v)
    plugin.configure([2, 16, d])
    plugin.initialize()
    y = plugin.forward(torch.from_numpy(z["x"].reshape(2, 16, d)).cuda()).cpu().numpy().reshape(-1, d)
    count, stats = plugin.last_routing()
    np.testing.assert_array_equal(count, z["count"])  # no near ties in these fixtures
    assert stats["near_ties"] == 0 and stats["nan_rows"] == 0
    assert_close(y, z["out"], what=os.path.basename(path))
    plugin.terminate()
