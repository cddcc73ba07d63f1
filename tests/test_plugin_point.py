"""The expert plug-in point (include/infmoe_sublayer.h; the reference's MoESubLayer,
plugin/sublayers/SubLayer.h:18-48, README.md:100-107): an expert type built outside the library
(tests/plugin_point/toy_sublayer.hip -> libtoy_sublayer.so) registers itself and is then created, streamed
and run through the ordinary C ABI."""
import ctypes as C
import os

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin, capi
from oracle import moe_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
TOY = os.path.join(HERE, "plugin_point", "libtoy_sublayer.so")


@pytest.fixture(scope="module")
def toy():
    capi.load()  # libinfmoe.so first, with RTLD_GLOBAL: the toy links against it
    if not os.path.isfile(TOY):
        pytest.fail(f"{TOY} not built: run `make -C tests/plugin_point` (the build entry point does)")
    lib = C.CDLL(TOY)
    assert lib.toy_register() == capi.OK
    return lib


def toy_config(E, d, mc, variant, B, S, seed=5, kind="ToyAffine"):
    x, c, g = O.draw_inputs(seed, B * S, d, E)
    cfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=16, max_concurrency=mc,
                         moe_variant=variant, sublayer_type=kind, max_batch_size=B, expert_centroids=c,
                         layernorm_weight=g if variant == "cpm_2" else None)
    return cfg, x, c, g


def test_registered_type_is_accepted_and_unknown_ones_still_are_not(toy):
    cfg, *_ = toy_config(4, 32, 2, "default", 2, 8)
    plugin = MoELayerPlugin(cfg).create_plugin()
    small = plugin.workspace_size([2, 8, 32])
    assert plugin.workspace_size([2, 80, 32]) > small > 0
    plugin.destroy()
    cfg.sublayer_type = "ToyAffineX"
    with pytest.raises(capi.InfMoEError) as ei:
        MoELayerPlugin(cfg).create_plugin()
    assert ei.value.status == capi.ERR_UNSUPPORTED
    assert toy.toy_register() == capi.OK  # registering again replaces the factory


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["default", "cpm_2", "base_layer"])
@pytest.mark.parametrize("mc", [1, 2, 6])  # streamed through one or two slots; resident (the library's default grouped run)
def test_out_of_tree_expert_runs_on_both_schedules(toy, torch_cuda, variant, mc):
    torch = torch_cuda
    E, d, B, S = 6, 48, 3, 40
    cfg, x, c, g = toy_config(E, d, mc, variant, B, S)
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([B, S, d])
    plugin.initialize()
    y = plugin.forward(torch.from_numpy(x.reshape(B, S, d)).cuda())
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(B * S, d)
    sel, coeff, aff = O.gate(x, c, variant, g)
    assert (O.top2_relative_gap(aff) >= 1e-6).all()
    count, stats = plugin.last_routing()
    np.testing.assert_array_equal(count, np.bincount(sel, minlength=E))
    post = x.astype(np.float64) * (sel[:, None] + 2.0) + 0.5 * sel[:, None]
    if variant == "base_layer":
        a = O.sigmoid(coeff)[:, None]
        post = a * post + (1 - a) * x
    np.testing.assert_allclose(y, post, rtol=2e-6, atol=1e-6)
    plugin.terminate()


@pytest.mark.gpu
@pytest.mark.parametrize("d", [48, 1024, 130])  # rows in registers, 16 bytes at a time; the same, longer; scalar path
def test_expert_type_that_asks_for_row_statistics(toy, torch_cuda, d):
    """A sub-layer whose rowStatsKind() is the centered norm gets (mean, 1/sqrt(biased variance + 1e-6)) of each of
    its rows from the layer's scatter, here with means far from zero."""
    torch = torch_cuda
    E, B, S = 5, 2, 33
    cfg, x, c, g = toy_config(E, d, E, "default", B, S, seed=9, kind="ToyStandardize")
    x = (x + np.random.default_rng(1).uniform(-5, 5, size=(B * S, 1))).astype(np.float32)
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([B, S, d])
    plugin.initialize()
    y = plugin.forward(torch.from_numpy(x.reshape(B, S, d)).cuda())
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(B * S, d)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=2e-6)
    plugin.terminate()
