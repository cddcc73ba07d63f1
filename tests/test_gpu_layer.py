"""Whole-layer parity through infmoe_create .. infmoe_enqueue against the float64 oracle."""
import os

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin, Plugin, capi
from oracle import moe_oracle as O
from tests.gpu_util import assert_close, check_assignment, dev

pytestmark = pytest.mark.gpu


def make_layer(T_shape, E, d, h, mc, variant, sublayer="T5_FF", norm="rms", ffn="relu", seed=0, bias=None,
               weight_file="", tweak=None):
    B, S = T_shape
    x, c, g = O.draw_inputs(seed, B * S, d, E)
    cfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=mc,
                         moe_variant=variant, sublayer_type=sublayer, max_batch_size=B, expert_centroids=c,
                         layernorm_weight=g if variant == "cpm_2" else None, weight_file_path=weight_file,
                         norm_kind=norm, ffn_kind=ffn)
    plugin = MoELayerPlugin(cfg).create_plugin()
    ws = None
    if sublayer == "T5_FF":
        ws = [O.draw_expert(seed, e, d, h, ffn) for e in range(E)]
        if tweak is not None:
            tweak(x, ws)
        if not weight_file:
            for e, w in enumerate(ws):
                for k, v in w.items():
                    plugin.set_expert_weights(e, k, v)
    if bias is not None:
        plugin.set_score_bias(bias)
    plugin.configure([B, S, d])
    plugin.initialize()
    return plugin, x, c, g, ws


def run_and_check(torch, plugin, x, c, g, ws, T_shape, variant, sublayer="T5_FF", norm="rms", ffn="relu", bias=None):
    B, S = T_shape
    d = x.shape[1]
    y = plugin.forward(dev(torch, x.reshape(B, S, d)))
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(B * S, d)
    count, stats = plugin.last_routing()
    ref = O.moe_layer(x, c, variant, ws, layernorm_weight=g, sublayer_type=sublayer, norm_kind=norm, ffn_kind=ffn,
                      score_bias=bias)
    # assignment: bit-exact outside the 1e-6 relative top-2 gap
    exempt = check_assignment_from_counts(count, ref, stats)
    if exempt:
        # A token whose two best float64 scores are closer than 1e-6 relative may go to either of the
        # two experts.  Rows are independent, so its output row must equal the oracle's row under one of
        # the two choices; the choice that matches is the device's, and with it the counts must agree.
        gap = O.top2_relative_gap(ref["aff"])
        toks = np.flatnonzero(gap < 1e-6)
        second = np.argsort(-ref["aff"][toks], axis=1, kind="stable")[:, 1]
        alt_sel = ref["sel"].copy()
        alt_sel[toks] = second
        alt = O.moe_layer(x, c, variant, ws, layernorm_weight=g, sublayer_type=sublayer, norm_kind=norm, ffn_kind=ffn,
                          score_bias=bias, sel_override=alt_sel)
        dev_sel = ref["sel"].copy()
        want = ref["out"].copy()
        scale = np.abs(ref["out"]).max()
        for t in toks:
            if np.abs(y[t] - ref["out"][t]).max() > np.abs(y[t] - alt["out"][t]).max():
                dev_sel[t] = alt_sel[t]
                want[t] = alt["out"][t]
            assert np.abs(y[t] - want[t]).max() <= 1e-4 * scale, f"near-tie token {t} matches neither of its two experts"
        np.testing.assert_array_equal(count, np.bincount(dev_sel, minlength=len(count)))
        assert_close(y, want, what=f"layer {variant}/{sublayer} ({exempt} near-tie tokens)")
        ref = dict(ref, out=want, sel=dev_sel)
    else:
        assert_close(y, ref["out"], what=f"layer {variant}/{sublayer}")
    return y, ref, count, stats


def check_assignment_from_counts(count, ref, stats):
    gap = O.top2_relative_gap(ref["aff"])
    exempt = int((gap < 1e-6).sum())
    if exempt == 0:
        np.testing.assert_array_equal(count, ref["count"])
    assert stats["nan_rows"] == 0
    assert stats["near_ties"] == exempt
    return exempt


@pytest.mark.parametrize("mc", [2, 4])  # streamed through 2 slots / all 4 experts resident
def test_config1_tiny_default(torch_cuda, mc):
    shape, E, d, h = (2, 16), 4, 64, 256
    plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "default")
    run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "default")
    plugin.terminate()


@pytest.mark.parametrize("variant", ["default", "cpm_2", "base_layer"])
@pytest.mark.parametrize("mc", [2, 8])
def test_identity_sublayer_reproduces_input(torch_cuda, variant, mc):
    shape, E, d = (3, 50), 8, 96
    plugin, x, c, g, _ = make_layer(shape, E, d, 128, mc, variant, sublayer="Identity", seed=3)
    y = plugin.forward(dev(torch_cuda, x.reshape(3, 50, d)))
    y = y.cpu().numpy().reshape(-1, d)
    if variant == "base_layer":
        np.testing.assert_allclose(y, x, rtol=1e-6, atol=1e-7)  # a*x + (1-a)*x
    else:
        np.testing.assert_array_equal(y, x)  # plugin/sublayers/IdentityLayer.hh:34-40
    plugin.terminate()


@pytest.mark.parametrize("variant,norm,ffn", [
    ("cpm_2", "rms", "relu"), ("base_layer", "rms", "relu"), ("default", "rms", "relu"),
    ("cpm_2", "centered", "gated_gelu"),  # the reference's code as written
    ("base_layer", "centered", "gated_gelu"),
])
@pytest.mark.parametrize("mc", [2, 6])
def test_variants_streamed_and_resident(torch_cuda, variant, norm, ffn, mc):
    shape, E, d, h = (4, 100), 6, 128, 384
    plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, variant, norm=norm, ffn=ffn, seed=5)
    run_and_check(torch_cuda, plugin, x, c, g, ws, shape, variant, norm=norm, ffn=ffn)
    plugin.terminate()


@pytest.mark.parametrize("shape", [(4, 128), (1, 24), (1, 8)])  # matrix-core tiles, tall and short; few-row kernel
@pytest.mark.parametrize("norm", ["centered", "rms"])
def test_rows_with_a_large_mean_and_weights_with_a_common_sign(torch_cuda, shape, norm):
    """Rows with a mean of several standard deviations against weights that all have one sign: x W'^T and
    mean * colsum(W') are then both hundreds of times larger than their difference, the case in which applying
    a CENTERED norm after the first product, as rstd * (x W'^T - mean * colsum(W')), loses most (it missed the
    oracle by eight times the bound, so the centered norm runs first, as a launch of its own; only the rms
    norm, which subtracts nothing, rides on the product as rstd * (x W'^T)).  Either way the layer has to meet
    the float64 oracle, which norms first, to the usual bound."""
    E, d, h = 4, 2048, 512

    def tweak(x, ws):
        rng = np.random.default_rng(77)
        x += rng.uniform(-4, 4, size=(x.shape[0], 1)).astype(np.float32)  # per-row mean of up to 4 sigma
        for w in ws:
            for k in w:
                if k.startswith("wi"):
                    w[k] += np.float32(2.0 / np.sqrt(d))  # two standard deviations of the entries: nearly all positive

    plugin, x, c, g, ws = make_layer(shape, E, d, h, E, "default", norm=norm, seed=23, tweak=tweak)
    run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "default", norm=norm)
    plugin.terminate()


# 300 tokens over 5 experts: the few-rows-per-expert kernels (tokens <= 64 * experts); 320 tokens with a score
# bias that sends most of them to expert 0: the same kernels with an expert cut into several 96-row tiles next to
# experts of a few rows; 600 tokens: the tall-tile kernels
@pytest.mark.parametrize("shape,skew", [((2, 150), 0.0), ((2, 160), 0.6), ((4, 150), 0.0)])
@pytest.mark.parametrize("variant", ["cpm_2", "base_layer"])
def test_output_is_bit_identical_for_every_max_concurrency(torch_cuda, variant, shape, skew):
    """Streamed experts run one set of launches per expert, resident ones one grouped set: same
    arithmetic, same bits."""
    torch = torch_cuda
    E, d, h = 5, 64, 192
    bias = np.array([skew, 0, 0, 0, 0], np.float32) if skew else None
    outs = []
    for mc in (1, 2, 3, 5, 9):
        plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, variant, seed=8, bias=bias)
        if mc == 5:
            y, ref, count, _ = run_and_check(torch, plugin, x, c, g, ws, shape, variant, bias=bias)
            assert not skew or (count.max() > 96 and count.min() < 40), count
        outs.append(plugin.forward(dev(torch, x.reshape(*shape, d))).cpu().numpy())
        plugin.terminate()
    for o in outs[1:]:
        np.testing.assert_array_equal(o, outs[0])


@pytest.mark.parametrize("mc", [1, 2, 3, 4, 6])
def test_slots_keep_experts_between_calls(torch_cuda, mc):
    """Streamed experts stay in their slots: an expert needed again is not copied again, whatever mix of
    experts the calls need, and the output is that of the resident layer bit for bit on every call."""
    torch = torch_cuda
    shape, E, d, h = (2, 80), 8, 64, 192
    B, S = shape
    resident, x, c, g, ws = make_layer(shape, E, d, h, E, "cpm_2", seed=83)
    streamed, *_ = make_layer(shape, E, d, h, mc, "cpm_2", seed=83)
    rng = np.random.default_rng(1)
    # inputs that need different subsets of the experts: all of them, then tokens of three experts only, ...
    sel = O.gate(x, c, "cpm_2", g)[0]
    inputs = [x, x[np.isin(sel, [0, 1, 2])][:B * S // 4], x[np.isin(sel, [1, 2, 5, 6])][:B * S // 4], x, x]
    history = []
    for i, xi in enumerate(inputs):
        xi = np.ascontiguousarray(xi)
        dx = dev(torch, xi.reshape(1, -1, d))
        want = resident.forward(dx)
        got = streamed.forward(dx)
        assert torch.equal(got, want), f"call {i} differs from the resident layer"
        count, _ = streamed.last_routing()
        needed = set(np.flatnonzero(count > 0).tolist())
        copies, hits = streamed.last_streaming()
        assert copies + hits == len(needed) and 0 <= hits <= mc
        history.append((needed, copies, hits))
    assert len(history[0][0]) == E and history[0][1:] == (E, 0)      # first call: every expert copied
    assert history[1][0] == {0, 1, 2} and history[2][0] == {1, 2, 5, 6}
    if mc >= 3:
        assert history[2][2] >= 2          # experts 1 and 2 ran in call 1 and were still there
    if mc >= 6:
        assert history[2][1] <= 2          # ... and with room to spare nothing else was displaced for them
    # calls 3 and 4 need all eight experts: after call 3 every slot holds one of them, so call 4 copies the rest only
    assert history[4][2] == mc and history[4][1] == E - mc
    assert_close(got.cpu().numpy().reshape(-1, d), O.moe_layer(x, c, "cpm_2", ws, layernorm_weight=g)["out"], what="last call")
    assert resident.last_streaming() == (0, 0)
    resident.terminate()
    streamed.terminate()


def test_new_weights_empty_the_slots(torch_cuda):
    torch = torch_cuda
    shape, E, d, h = (2, 40), 4, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, 4 - 1, "default", seed=89)
    dx = dev(torch, x.reshape(2, 40, d))
    plugin.forward(dx)
    plugin.forward(dx)
    copies, hits = plugin.last_streaming()
    assert hits > 0
    ws[1] = O.draw_expert(90, 1, d, h)
    for k, v in ws[1].items():
        plugin.set_expert_weights(1, k, v)
    y = plugin.forward(dx).cpu().numpy().reshape(-1, d)
    copies, hits = plugin.last_streaming()
    assert hits == 0 and copies > 0
    assert_close(y, O.moe_layer(x, c, "default", ws)["out"], what="after new weights")
    plugin.terminate()


@pytest.mark.parametrize("d,h", [(40, 72), (30, 50)])  # multiples of 4 but not of 32; not even of 4
@pytest.mark.parametrize("variant,ffn", [("cpm_2", "relu"), ("base_layer", "gated_gelu")])
@pytest.mark.parametrize("mc", [2, 4])
def test_sizes_the_matrix_core_kernels_do_not_take(torch_cuda, d, h, variant, ffn, mc):
    shape, E = (3, 50), 4
    plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, variant, ffn=ffn, seed=47)
    run_and_check(torch_cuda, plugin, x, c, g, ws, shape, variant, ffn=ffn)
    plugin.terminate()


def test_output_may_alias_input(torch_cuda):
    """The input is copied into the routed buffer before anything writes the output, so a caller
    may pass one buffer for both."""
    torch = torch_cuda
    shape, E, d, h = (2, 90), 4, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, E, "base_layer", seed=53)
    y, ref, _, _ = run_and_check(torch, plugin, x, c, g, ws, shape, "base_layer")
    buf = dev(torch, x.reshape(2, 90, d))
    ws_bytes = plugin.workspace_size([2, 90, d])
    work = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    plugin.enqueue([2, 90, d], buf.data_ptr(), buf.data_ptr(), work.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(buf.cpu().numpy().reshape(-1, d), y)
    plugin.terminate()


@pytest.mark.parametrize("skew", [0.0, 1.5])
def test_decode_shape_uses_few_row_kernels_and_matches(torch_cuda, skew):
    """Up to two tokens per expert: experts of up to 8 rows go to the few-row kernel.  32 tokens over 16 experts:
    some experts get no rows, most 1..5; with a score bias one gets more than 8 and goes to the matrix-core
    kernel in the same call.  Both schedules, same bits."""
    shape, E, d, h = (32, 1), 16, 256, 640
    bias = np.array([0, 0, 0, skew] + [0] * 12, np.float32) if skew else None
    outs = []
    for mc in (16, 2):
        plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "cpm_2", seed=13, bias=bias)
        y, ref, count, _ = run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "cpm_2", bias=bias)
        assert count.sum() == 32 and ((count > 0) & (count <= 8)).any()
        assert not skew or count.max() > 8, count
        outs.append(y)
        plugin.terminate()
    np.testing.assert_array_equal(outs[0], outs[1])


@pytest.mark.parametrize("ffn", ["relu", "gated_gelu"])
def test_skewed_routing_with_score_bias(torch_cuda, ffn):
    """Experts of very different sizes, some cut into several row tiles (of equal height): the grouped
    and the per-expert launches cut alike, so both schedules give the same bits."""
    shape, E, d, h = (8, 256), 16, 128, 256
    x, c, _ = O.draw_inputs(17, 8 * 256, d, E)
    bias = O.zipf_score_bias(x, c, s=1.2)
    outs = []
    for mc in (E, 3):  # resident; streamed, where the experts run largest first
        plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "base_layer", ffn=ffn, seed=17, bias=bias)
        y, ref, count, _ = run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "base_layer", ffn=ffn, bias=bias)
        assert count.max() > 4 * max(count.min(), 1)  # the histogram really is skewed
        assert count.max() > 256                      # and some expert needs more than one row tile
        assert ((count > 128) & (count <= 256)).any()  # and one lies between the tile heights of the two forms
        outs.append(y)
        plugin.terminate()
    np.testing.assert_array_equal(outs[0], outs[1])


def test_all_tokens_to_one_expert_and_empty_experts(torch_cuda):
    shape, E, d, h = (1, 300), 4, 64, 128
    bias = np.array([0, 0, 100, 0], np.float32)
    for mc in (2, 4):
        plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "default", seed=19, bias=bias)
        y, ref, count, _ = run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "default", bias=bias)
        np.testing.assert_array_equal(count, [0, 0, 300, 0])
        plugin.terminate()


@pytest.mark.parametrize("variant", ["cpm_2", "base_layer"])
def test_near_tie_tokens_are_compared_under_either_expert(torch_cuda, variant):
    """Two centroids that differ by one unit in the last place of one element: every token they win is a
    near tie (float64 gap far below 1e-6 relative), counted by the device and exempt from bit-exact
    assignment; its output row must still be the oracle's row under one of the two experts."""
    shape, E, d, h = (2, 60), 4, 64, 128
    B, S = shape
    x, c, g = O.draw_inputs(71, B * S, d, E)
    c[1] = c[0]
    c[1, 5] = np.nextafter(c[0, 5], np.float32(1.0))
    cfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=E,
                         moe_variant=variant, sublayer_type="T5_FF", max_batch_size=B, expert_centroids=c,
                         layernorm_weight=g if variant == "cpm_2" else None)
    plugin = MoELayerPlugin(cfg).create_plugin()
    ws = [O.draw_expert(71, e, d, h) for e in range(E)]
    for e, w in enumerate(ws):
        for k, v in w.items():
            plugin.set_expert_weights(e, k, v)
    plugin.configure([B, S, d])
    plugin.initialize()
    y, ref, count, stats = run_and_check(torch_cuda, plugin, x, c, g, ws, shape, variant)
    assert stats["near_ties"] >= 10  # about half the tokens pick one of the twins
    plugin.terminate()


@pytest.mark.parametrize("mc", [2, 6])  # experts streamed / resident
@pytest.mark.parametrize("variant", ["cpm_2", "base_layer"])
def test_batch_size_may_change_from_call_to_call(torch_cuda, variant, mc):
    """The batch dimension is dynamic (the reference takes it from the input descriptor of every enqueue,
    plugin/MoELayerPlugin.cc:284-289): one handle, one workspace sized for the largest batch, calls of 4, 1, 0, 3
    and 4 sequences, each against the oracle on its own tokens."""
    torch = torch_cuda
    S, E, d, h = 40, 6, 128, 256
    plugin, x, c, g, ws = make_layer((4, S), E, d, h, mc, variant, seed=31)
    x3 = x.reshape(4, S, d)
    for B in (4, 1, 0, 3, 4):
        y = plugin.forward(dev(torch, x3[:B]))
        torch.cuda.synchronize()
        assert tuple(y.shape) == (B, S, d)
        if B == 0:
            continue
        xb = x3[:B].reshape(B * S, d)
        ref = O.moe_layer(xb, c, variant, ws, layernorm_weight=g)
        assert (O.top2_relative_gap(ref["aff"]) >= 1e-6).all()
        count, stats = plugin.last_routing()
        np.testing.assert_array_equal(count, ref["count"])
        assert_close(y.cpu().numpy().reshape(B * S, d), ref["out"], what=f"batch of {B}")
    plugin.terminate()


def test_single_token(torch_cuda):
    shape, E, d, h = (1, 1), 4, 64, 128
    for mc in (2, 4):
        plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "cpm_2", seed=23)
        run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "cpm_2")
        plugin.terminate()


def test_token_permutation_equivariance(torch_cuda):
    torch = torch_cuda
    shape, E, d, h = (1, 200), 6, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, E, "cpm_2", seed=29)
    y = plugin.forward(dev(torch, x.reshape(1, 200, d))).cpu().numpy().reshape(-1, d)
    perm = np.random.default_rng(0).permutation(200)
    yp = plugin.forward(dev(torch, x[perm].reshape(1, 200, d))).cpu().numpy().reshape(-1, d)
    # same expert, same row content; only the row's place inside the expert's tile changes
    assert_close(yp, y[perm], rtol=1e-6, what="permutation")
    plugin.terminate()


def test_clone_shares_weights_and_serialization_round_trip(torch_cuda):
    torch = torch_cuda
    shape, E, d, h = (2, 40), 4, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, 4, "cpm_2", seed=31)
    dx = dev(torch, x.reshape(2, 40, d))
    y = plugin.forward(dx).cpu().numpy()
    twin = plugin.clone()
    twin.configure([2, 40, d])
    twin.initialize()
    np.testing.assert_array_equal(twin.forward(dx).cpu().numpy(), y)
    blob = plugin.serialize()
    back = Plugin.deserialize(blob)
    assert back.serialize() == blob
    twin.terminate()
    plugin.terminate()


@pytest.mark.parametrize("mc", [2, 4])  # experts streamed (each clone its own slots and copy stream) / resident
def test_clones_driven_from_two_threads_at_once(torch_cuda, mc):
    """Stacked layers share one sub-layer (plugin/MoELayerPlugin.cc:114-127).  Two clones, each called from a thread
    of its own on a stream of its own with a batch of its own, while the other runs: every output has to be the one the
    layer gives when nothing else is going on."""
    import threading
    torch = torch_cuda
    E, d, h = 4, 128, 256
    shapes = [(2, 60), (3, 33)]
    plugin, x0, c, g, ws = make_layer(shapes[0], E, d, h, mc, "cpm_2", seed=57)
    twin = plugin.clone()
    twin.configure([shapes[1][0], shapes[1][1], d])
    twin.initialize()
    x1 = O.draw_inputs(58, shapes[1][0] * shapes[1][1], d, E)[0]
    layers = [plugin, twin]
    xs = [dev(torch, x0.reshape(*shapes[0], d)), dev(torch, x1.reshape(*shapes[1], d))]
    want = [layers[i].forward(xs[i]).clone() for i in range(2)]
    torch.cuda.synchronize()
    for i, x in enumerate((x0, x1)):
        ref = O.moe_layer(x, c, "cpm_2", ws, layernorm_weight=g)
        assert_close(want[i].cpu().numpy().reshape(-1, d), ref["out"], what=f"clone {i} alone")
    errors = []

    def drive(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(25):
                    y = layers[i].forward(xs[i])
                    stream.synchronize()
                    if not torch.equal(y, want[i]):
                        errors.append(f"clone {i}: output differs")
                        return
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append(f"clone {i}: {exc!r}")

    threads = [threading.Thread(target=drive, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors
    twin.terminate()
    plugin.terminate()


def save_experts(path, ws, compressed=False):
    arrays = {f"{e}/{k}": v for e, w in enumerate(ws) for k, v in w.items()}
    (np.savez_compressed if compressed else np.savez)(path, **arrays)


@pytest.mark.parametrize("variant,norm,ffn,from_file", [
    ("cpm_2", "rms", "relu", True), ("base_layer", "centered", "gated_gelu", False), ("cpm_2", "centered", "gated_gelu", True)])
def test_deserialized_layer_and_clone_match_the_oracle(torch_cuda, tmp_path, variant, norm, ffn, from_file):
    """serialize -> deserialize gives a layer that, initialised and run, computes what the oracle computes
    (plugin/MoELayerPlugin.cc:104-143,418-458: the engine file holds the parameters and the weight file's
    path, not the weights); so does a clone, which shares its parent's sub-layer (:83-102)."""
    torch = torch_cuda
    shape, E, d, h = (3, 70), 5, 96, 160
    B, S = shape
    ws = [O.draw_expert(67, e, d, h, ffn) for e in range(E)]
    path = ""
    if from_file:
        path = os.path.join(tmp_path, "experts.npz")
        save_experts(path, ws, compressed=True)  # deflated members
    plugin, x, c, g, _ = make_layer(shape, E, d, h, 2, variant, norm=norm, ffn=ffn, seed=67, weight_file=path)
    blob = plugin.serialize()
    plugin.terminate()
    plugin.destroy()

    back = Plugin.deserialize(blob)
    if not from_file:  # no path in the blob: the weights come by pointer again
        for e, w in enumerate(ws):
            for k, v in w.items():
                back.set_expert_weights(e, k, v)
    back.configure([B, S, d])
    back.initialize()
    y, ref, count, _ = run_and_check(torch, back, x, c, g, ws, shape, variant, norm=norm, ffn=ffn)
    if variant == "base_layer":  # the mix really is active: the plain gather of the expert output differs
        plain = O.moe_layer(x, c, "default", ws, norm_kind=norm, ffn_kind=ffn)["out"]
        assert np.abs(y - plain).max() > 1e-3 * np.abs(plain).max()

    twin = back.clone()
    twin.configure([B, S, d])
    twin.initialize()
    run_and_check(torch, twin, x, c, g, ws, shape, variant, norm=norm, ffn=ffn)
    back.terminate()  # the clone keeps the shared sub-layer (and its weights) alive
    y2, *_ = run_and_check(torch, twin, x, c, g, ws, shape, variant, norm=norm, ffn=ffn)
    np.testing.assert_array_equal(y2, y)
    twin.terminate()


def test_npz_with_a_transposed_matrix_is_rejected(torch_cuda, tmp_path):
    """wo saved as [h][d] has the element count of [d][h]; the reference checks the count only
    (plugin/sublayers/T5FFLayer.cc:83) and would read it as if it were [d][h]."""
    E, d, h = 2, 32, 64
    ws = [O.draw_expert(73, e, d, h) for e in range(E)]
    ws[1]["wo_weight"] = np.ascontiguousarray(ws[1]["wo_weight"].T)
    path = os.path.join(tmp_path, "bad.npz")
    save_experts(path, ws)
    x, c, g = O.draw_inputs(73, 8, d, E)
    cfg = MoELayerConfig(seq_len=8, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=2,
                         moe_variant="default", sublayer_type="T5_FF", max_batch_size=1, expert_centroids=c,
                         weight_file_path=path)
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([1, 8, d])
    with pytest.raises(capi.InfMoEError) as ei:
        plugin.initialize()
    assert ei.value.status == capi.ERR_INVALID_ARGUMENT and "1/wo_weight" in ei.value.message
    # a file of the other FFN kind names the cause
    cfg.ffn_kind = "gated_gelu"
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([1, 8, d])
    with pytest.raises(capi.InfMoEError) as ei:
        plugin.initialize()
    assert ei.value.status == capi.ERR_MISSING_FIELD and "ffn_kind" in ei.value.message


@pytest.mark.parametrize("variant", ["cpm_2", "base_layer"])
@pytest.mark.parametrize("mc", [2, 4])  # experts streamed / resident
def test_nan_input_one_contract_for_both_schedules(torch_cuda, variant, mc):
    """A token with a NaN in its row (the reference asserts, plugin/cuda/moe.cu:70,184): the call completes,
    that token's output row is NaN in full, every other row is the oracle's, the count is in the routing
    report, and INFMOE_ERR_NAN is returned once - by the same call when experts are streamed (it waits for
    the routing anyway), by the next call when they are resident: a deferred notice that names the call, while
    that next call is itself queued in full and gives the right output."""
    torch = torch_cuda
    shape, E, d, h = (1, 20), 4, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, variant, seed=37)
    clean = x.copy()
    x[7, 3] = np.nan
    dims = [1, 20, d]
    xin = dev(torch, x.reshape(1, 20, d))
    y = torch.zeros_like(xin)
    work = torch.empty(plugin.workspace_size(dims), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    if mc < E:
        with pytest.raises(capi.InfMoEError) as ei:
            plugin.enqueue(dims, xin.data_ptr(), y.data_ptr(), work.data_ptr(), stream)
        assert ei.value.status == capi.ERR_NAN
    else:
        plugin.enqueue(dims, xin.data_ptr(), y.data_ptr(), work.data_ptr(), stream)
    torch.cuda.synchronize()
    out = y.cpu().numpy().reshape(20, d)
    assert np.isnan(out[7]).all()
    ref = O.moe_layer(clean, c, variant, ws, layernorm_weight=g)
    others = np.arange(20) != 7
    assert_close(out[others], ref["out"][others], what="rows next to a NaN row")
    if mc >= E:
        # resident: the report comes with the next call, once, and names the call that met the NaN (the first on
        # this handle); the call that carries the notice is queued in full: a valid batch is not lost
        y2 = torch.zeros_like(xin)
        cin = dev(torch, clean.reshape(1, 20, d))
        with pytest.raises(capi.InfMoEError) as ei:
            plugin.enqueue(dims, cin.data_ptr(), y2.data_ptr(), work.data_ptr(), stream)
        assert ei.value.status == capi.ERR_NAN and "call number 1 " in ei.value.message and "(number 2)" in ei.value.message
        torch.cuda.synchronize()
        assert_close(y2.cpu().numpy().reshape(20, d), ref["out"], what="the call that carries the deferred notice")
    assert_close(plugin.forward(dev(torch, clean.reshape(1, 20, d))).cpu().numpy().reshape(20, d), ref["out"], what="after the report")
    # the routing report tells of the NaN rows too, and then the next call does not repeat it
    if mc >= E:
        plugin.enqueue(dims, xin.data_ptr(), y.data_ptr(), work.data_ptr(), stream)
        count, stats = plugin.last_routing()
        assert stats["nan_rows"] == 1 and count.sum() == 20
        plugin.forward(dev(torch, clean.reshape(1, 20, d)))
        with pytest.raises(capi.InfMoEError) as ei:
            plugin.forward(xin, check_nan=True)
        assert ei.value.status == capi.ERR_NAN
    plugin.terminate()


def test_weights_from_npz_file(torch_cuda, tmp_path):
    shape, E, d, h = (2, 30), 3, 64, 128
    ws = [O.draw_expert(41, e, d, h, "gated_gelu") for e in range(E)]
    arrays = {}
    for e, w in enumerate(ws):
        for k, v in w.items():
            # wo saved as a transposed view, as python/infmoe/config.py:52 does: numpy stores it Fortran-ordered
            arrays[f"{e}/{k}"] = np.ascontiguousarray(v.T).T if k == "wo_weight" else v
    path = os.path.join(tmp_path, "experts.npz")
    np.savez(path, **arrays)
    plugin, x, c, g, _ = make_layer(shape, E, d, h, 2, "cpm_2", norm="centered", ffn="gated_gelu", seed=41,
                                    weight_file=path)
    run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "cpm_2", norm="centered", ffn="gated_gelu")
    plugin.terminate()


def test_enqueue_before_initialize_is_an_error(torch_cuda):
    x, c, g = O.draw_inputs(0, 8, 16, 2)
    cfg = MoELayerConfig(seq_len=8, expert_count=2, embedding_size=16, hidden_size=32, max_concurrency=2,
                         moe_variant="default", sublayer_type="Identity", max_batch_size=1, expert_centroids=c)
    plugin = MoELayerPlugin(cfg).create_plugin()
    with pytest.raises(capi.InfMoEError) as ei:
        plugin.forward(dev(torch_cuda, x.reshape(1, 8, 16)))
    assert ei.value.status == capi.ERR_STATE


def test_layer_can_be_captured_in_a_graph_and_replayed(torch_cuda):
    """The resident schedule makes no host wait and no allocation, so after one eager call it can be
    captured; every replay, with eager work in between, must reproduce the eager result bit for bit."""
    torch = torch_cuda
    shape, E, d, h = (4, 64), 8, 128, 256
    plugin, x, c, g, ws = make_layer(shape, E, d, h, E, "cpm_2", seed=43)
    xs = [dev(torch, np.roll(x, k, axis=0).reshape(4, 64, d)) for k in range(3)]
    eager = [plugin.forward(v).clone() for v in xs]
    dims = [4, 64, d]
    wsb = torch.empty(plugin.workspace_size(dims), dtype=torch.uint8, device="cuda")
    xin = xs[0].clone()
    yout = torch.empty_like(xin)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plugin.enqueue(dims, xin.data_ptr(), yout.data_ptr(), wsb.data_ptr(), side.cuda_stream)  # warm
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plugin.enqueue(dims, xin.data_ptr(), yout.data_ptr(), wsb.data_ptr(), side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(2):
        for k, v in enumerate(xs):
            xin.copy_(v)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(yout, eager[k]), f"replay {rep}/{k} differs from the eager result"
            assert torch.equal(plugin.forward(v), eager[k])  # eager work between replays
    plugin.terminate()


def test_phase_timing_keeps_the_last_calls(torch_cuda):
    torch = torch_cuda
    shape, E, d, h = (2, 64), 4, 64, 128
    plugin, x, c, g, ws = make_layer(shape, E, d, h, E, "cpm_2", seed=59)
    xd = dev(torch, x.reshape(2, 64, d))
    with pytest.raises(RuntimeError):
        plugin.last_timing()  # nothing timed yet
    plugin.set_timing(3)
    for _ in range(5):
        plugin.forward(xd)
    hist = plugin.timing_history(10)
    assert len(hist) == 3  # the last three of five calls
    for phases in hist:
        assert set(phases) == set(plugin.PHASES)
        assert all(v >= 0.0 for v in phases.values())
        assert phases["expert_gemm1"] > 0.0 and phases["gating"] > 0.0
    # the same events read twice: the runtime converts ticks to milliseconds anew on every query
    assert plugin.last_timing() == pytest.approx(hist[-1], rel=1e-3, abs=1e-5)
    assert len(plugin.timing_history(2)) == 2
    plugin.set_timing(False)
    plugin.forward(xd)
    with pytest.raises(RuntimeError):
        plugin.last_timing()
    plugin.terminate()


@pytest.mark.parametrize("E,mc", [(130, 130), (130, 3), (64, 64)])
def test_many_experts(torch_cuda, E, mc):
    """More experts than one gating pass scores (128), most of them with a handful of rows."""
    shape, d, h = (7, 100), 64, 96
    plugin, x, c, g, ws = make_layer(shape, E, d, h, mc, "cpm_2", seed=61)
    y, ref, count, _ = run_and_check(torch_cuda, plugin, x, c, g, ws, shape, "cpm_2")
    assert count.sum() == 700 and (count > 0).sum() > E // 2
    plugin.terminate()


def test_streamed_layer_called_from_alternating_streams(torch_cuda):
    """The weight slots of a streamed layer outlive a call; a call on another stream than the last one's waits for
    that call's end on the device.  Calls alternate between two streams without any host synchronisation in
    between, each with its own buffers, and every output is the resident layer's, bit for bit."""
    torch = torch_cuda
    shape, E, d, h = (2, 96), 8, 64, 192
    B, S = shape
    resident, x, c, g, ws = make_layer(shape, E, d, h, E, "cpm_2", seed=97)
    streamed, *_ = make_layer(shape, E, d, h, 3, "cpm_2", seed=97)
    rng = np.random.default_rng(2)
    inputs = [dev(torch, (x * s).reshape(B, S, d)) for s in (1.0, 0.5, 2.0, 1.5, 0.25, 3.0)]
    want = [resident.forward(v).clone() for v in inputs]
    torch.cuda.synchronize()
    dims = [B, S, d]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.zeros_like(v) for v in inputs]
    works = [torch.empty(streamed.workspace_size(dims), dtype=torch.uint8, device="cuda") for _ in streams]
    for i, v in enumerate(inputs):
        s = streams[i % 2]
        streamed.enqueue(dims, v.data_ptr(), outs[i].data_ptr(), works[i % 2].data_ptr(), s.cuda_stream)
    torch.cuda.synchronize()
    for i in range(len(inputs)):
        assert torch.equal(outs[i], want[i]), f"call {i} (stream {i % 2}) differs from the resident layer"
    resident.terminate()
    streamed.terminate()
