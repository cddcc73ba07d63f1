"""Pins for oracle/moe_oracle.py: each oracle function is checked against something
that does not share its formula (a library routine, a closed form, an invariant or a
brute-force loop), chosen so that a dropped term, wrong sign, wrong axis or transposed
operand fails.  The reference ships no tests or golden vectors, so these are the pins.
"""
import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

RNG = np.random.default_rng(1234)


# ---------------------------------------------------------------- norms
def test_centered_norm_matches_torch_layer_norm():
    x = RNG.standard_normal((7, 33)) * 3 + 1.5
    g = 1 + 0.1 * RNG.standard_normal(33)
    want = F.layer_norm(torch.tensor(x), (33,), weight=torch.tensor(g), bias=None, eps=1e-6).numpy()
    np.testing.assert_allclose(O.layernorm(x, g, "centered"), want, rtol=1e-12, atol=1e-12)


def test_centered_norm_invariants():
    x = RNG.standard_normal((5, 64)) * 2
    ones = np.ones(64)
    y = O.layernorm(x, ones, "centered")
    np.testing.assert_allclose(y.mean(axis=1), 0, atol=1e-12)
    var = x.var(axis=1)
    np.testing.assert_allclose(y.var(axis=1), var / (var + 1e-6), rtol=1e-10)
    np.testing.assert_allclose(O.layernorm(x + 7.25, ones, "centered"), y, atol=1e-9)
    assert np.all(O.layernorm(np.full((2, 64), 3.0), ones, "centered") == 0)


def test_rms_norm_matches_hf_t5_layernorm():
    from transformers.models.t5.modeling_t5 import T5LayerNorm
    x = RNG.standard_normal((6, 48)) + 0.3
    g = 1 + 0.1 * RNG.standard_normal(48)
    m = T5LayerNorm(48, eps=1e-6).double()
    with torch.no_grad():
        m.weight.copy_(torch.tensor(g))
        want = m(torch.tensor(x)).numpy()
    # HF evaluates the mean square in float32 whatever the module dtype, hence 1e-6
    np.testing.assert_allclose(O.layernorm(x, g, "rms"), want, rtol=2e-6, atol=1e-7)
    ms = (x * x).mean(axis=1, keepdims=True)  # and the closed form itself, to double precision
    np.testing.assert_allclose(O.layernorm(x, g, "rms") * np.sqrt(ms + 1e-6), g * x, rtol=1e-13)


def test_rms_norm_is_not_centered_and_scale_equivariant():
    x = RNG.standard_normal((4, 32)) + 5.0
    ones = np.ones(32)
    y = O.layernorm(x, ones, "rms")
    assert np.all(np.abs(y.mean(axis=1)) > 0.5)  # a centred norm would give ~0
    np.testing.assert_allclose(O.layernorm(1000 * x, ones, "rms"), y, rtol=1e-6)
    np.testing.assert_allclose((y * y).mean(axis=1), 1.0, rtol=1e-6)


# ---------------------------------------------------------------- scoring / argmax
def test_score_one_hot_selects_centroid_entries():
    E, d = 5, 9
    c = RNG.standard_normal((E, d))  # [E][d]
    x = np.eye(d)
    aff = O.score(x, c)
    assert aff.shape == (d, E)
    np.testing.assert_array_equal(aff, c.T)  # token k picks c[e][k]; a transposed layout would not even shape-match
    np.testing.assert_allclose(O.score(x, c, score_bias=np.arange(E)), c.T + np.arange(E))


def test_select_top1_brute_force_and_ties():
    aff = RNG.integers(-3, 4, size=(200, 7)).astype(np.float64)  # many exact ties
    sel, coeff = O.select_top1(aff)
    np.testing.assert_array_equal(sel, np.argmax(aff, axis=1))  # numpy: first occurrence
    np.testing.assert_array_equal(coeff, aff.max(axis=1))
    for t in range(aff.shape[0]):
        best, pos = None, -1
        for e in range(aff.shape[1]):
            if best is None or aff[t, e] > best:
                best, pos = aff[t, e], e
        assert pos == sel[t]


def test_select_top1_nan_row_raises_and_partial_nan_does_not():
    with pytest.raises(FloatingPointError):
        O.select_top1(np.array([[np.nan, np.nan]]))
    sel, _ = O.select_top1(np.array([[np.nan, 1.0, 0.5]]))
    assert sel[0] == 1


def test_top2_gap():
    aff = np.array([[1.0, 3.0, 2.0], [-4.0, -4.0, -9.0], [0.5, 0.5000001, 0.1]])
    gap = O.top2_relative_gap(aff)
    np.testing.assert_allclose(gap, [1 / 3, 0.0, 1e-7 / 0.5000001], rtol=1e-6)


# ---------------------------------------------------------------- count / sort
@pytest.mark.parametrize("T,E", [(1, 1), (1, 4), (17, 3), (256, 64), (1000, 7)])
def test_expert_count_matches_numpy_stable_sort(T, E):
    sel = RNG.integers(0, E, size=T).astype(np.int32)
    count, offset, pos = O.expert_count(sel, E)
    np.testing.assert_array_equal(count, np.bincount(sel, minlength=E))
    np.testing.assert_array_equal(offset, np.concatenate([[0], np.cumsum(count)]))
    np.testing.assert_array_equal(pos, np.argsort(sel, kind="stable"))
    assert sorted(pos.tolist()) == list(range(T))
    assert np.all(np.diff(sel[pos]) >= 0)


def test_expert_count_all_to_one_and_empty_experts():
    sel = np.full(9, 2, np.int32)
    count, offset, pos = O.expert_count(sel, 4)
    np.testing.assert_array_equal(count, [0, 0, 9, 0])
    np.testing.assert_array_equal(offset, [0, 0, 0, 9, 9])
    np.testing.assert_array_equal(pos, np.arange(9))


# ---------------------------------------------------------------- scatter / gather / mix
def test_scatter_gather_roundtrip_and_direction():
    x = RNG.standard_normal((11, 6))
    coeff = RNG.standard_normal(11)
    pos = RNG.permutation(11).astype(np.int32)
    routed, rc = O.scatter(x, coeff, pos)
    for r in range(11):  # brute force: routed row r is token pos[r]
        np.testing.assert_array_equal(routed[r], x[pos[r]])
        assert rc[r] == coeff[pos[r]]
    np.testing.assert_array_equal(O.gather(routed, pos), x)  # inverse, exactly


def test_mix_and_gather_closed_form_and_limits():
    post = RNG.standard_normal((8, 5))
    routed = RNG.standard_normal((8, 5))
    pos = RNG.permutation(8).astype(np.int32)
    c = RNG.standard_normal(8)
    out = O.mix_and_gather(post, routed, c, pos)
    a = scipy.special.expit(c)
    for r in range(8):
        np.testing.assert_allclose(out[pos[r]], a[r] * post[r] + (1 - a[r]) * routed[r], rtol=1e-12)
    np.testing.assert_allclose(O.mix_and_gather(post, routed, np.full(8, 50.0), pos), O.gather(post, pos), atol=1e-12)
    np.testing.assert_allclose(O.mix_and_gather(post, routed, np.full(8, -50.0), pos), O.gather(routed, pos), atol=1e-12)
    np.testing.assert_allclose(O.sigmoid([0.0, 1.0]), [0.5, 1 / (1 + np.exp(-1))])


# ---------------------------------------------------------------- FFN
def test_gelu_dot_matches_torch_tanh_gelu():
    a = RNG.standard_normal(1000) * 3
    b = RNG.standard_normal(1000)
    want = (F.gelu(torch.tensor(a), approximate="tanh") * torch.tensor(b)).numpy()
    np.testing.assert_allclose(O.gelu_dot(a, b), want, rtol=1e-9, atol=1e-12)


def _hf_t5_ff(d, h, gated):
    from transformers import T5Config
    from transformers.models.t5.modeling_t5 import T5LayerFF
    cfg = T5Config(d_model=d, d_ff=h, dropout_rate=0.0, layer_norm_epsilon=1e-6,
                   feed_forward_proj="gated-gelu" if gated else "relu")
    return T5LayerFF(cfg).double().eval()


def test_t5ff_relu_matches_hf_t5_v1_0_layer():
    d, h = 24, 40
    m = _hf_t5_ff(d, h, gated=False)
    w = O.draw_expert(3, 0, d, h, "relu")
    with torch.no_grad():
        m.layer_norm.weight.copy_(torch.tensor(w["layer_norm_weight"], dtype=torch.float64))
        m.DenseReluDense.wi.weight.copy_(torch.tensor(w["wi_weight"], dtype=torch.float64))  # [h,d]
        m.DenseReluDense.wo.weight.copy_(torch.tensor(w["wo_weight"], dtype=torch.float64))  # [d,h]
        x = RNG.standard_normal((9, d))
        want = m(torch.tensor(x)).numpy()
    np.testing.assert_allclose(O.t5ff_run(x, w, "rms", "relu"), want, rtol=1e-5, atol=1e-6)


def test_t5ff_gated_gelu_matches_hf_t5_v1_1_layer():
    d, h = 16, 56
    m = _hf_t5_ff(d, h, gated=True)
    w = O.draw_expert(4, 1, d, h, "gated_gelu")
    with torch.no_grad():
        m.layer_norm.weight.copy_(torch.tensor(w["layer_norm_weight"], dtype=torch.float64))
        m.DenseReluDense.wi_0.weight.copy_(torch.tensor(w["wi_0_weight"], dtype=torch.float64))
        m.DenseReluDense.wi_1.weight.copy_(torch.tensor(w["wi_1_weight"], dtype=torch.float64))
        m.DenseReluDense.wo.weight.copy_(torch.tensor(w["wo_weight"], dtype=torch.float64))
        x = RNG.standard_normal((5, d))
        want = m(torch.tensor(x)).numpy()
    # HF's "gelu_new" is the same tanh form the reference codes (plugin/cuda/ops/gelu.cu:7-16)
    np.testing.assert_allclose(O.t5ff_run(x, w, "rms", "gated_gelu"), want, rtol=1e-5, atol=1e-6)


def test_t5ff_centered_norm_path_and_zero_wo():
    d, h = 12, 20
    w = O.draw_expert(5, 0, d, h, "gated_gelu")
    x = RNG.standard_normal((4, d))
    ln = F.layer_norm(torch.tensor(x), (d,), weight=torch.tensor(w["layer_norm_weight"], dtype=torch.float64), eps=1e-6)
    h0 = ln @ torch.tensor(w["wi_0_weight"], dtype=torch.float64).T
    h1 = ln @ torch.tensor(w["wi_1_weight"], dtype=torch.float64).T
    want = torch.tensor(x) + (F.gelu(h0, approximate="tanh") * h1) @ torch.tensor(w["wo_weight"], dtype=torch.float64).T
    np.testing.assert_allclose(O.t5ff_run(x, w, "centered", "gated_gelu"), want.numpy(), rtol=1e-9)
    w0 = dict(w, wo_weight=np.zeros_like(w["wo_weight"]))
    np.testing.assert_array_equal(O.t5ff_run(x, w0, "centered", "gated_gelu"), x)


# ---------------------------------------------------------------- whole layer
def test_parse_flags():
    assert O.parse_flags("cpm_2") == (True, False)
    assert O.parse_flags("base_layer") == (False, True)
    assert O.parse_flags("default") == (False, False)
    with pytest.raises(ValueError):
        O.parse_flags("switch")


@pytest.mark.parametrize("variant", ["default", "cpm_2"])
def test_layer_identity_sublayer_is_identity(variant):
    x, c, g = O.draw_inputs(0, 40, 16, 5)
    r = O.moe_layer(x, c, variant, None, layernorm_weight=g, sublayer_type="Identity")
    np.testing.assert_array_equal(r["out"], x.astype(np.float64))


def test_layer_base_layer_identity_is_identity_to_rounding():
    x, c, g = O.draw_inputs(0, 40, 16, 5)
    r = O.moe_layer(x, c, "base_layer", None, sublayer_type="Identity")
    np.testing.assert_allclose(r["out"], x, rtol=1e-12)


def test_layer_equals_per_token_brute_force_and_is_permutation_equivariant():
    T, d, h, E = 24, 8, 12, 3
    x, c, g = O.draw_inputs(7, T, d, E)
    ws = [O.draw_expert(7, e, d, h) for e in range(E)]
    r = O.moe_layer(x, c, "cpm_2", ws, layernorm_weight=g)
    for t in range(T):  # independent per-token evaluation, no sort involved
        xn = g * x[t].astype(np.float64) / np.sqrt(np.mean(x[t].astype(np.float64) ** 2) + 1e-6)
        e = int(np.argmax(c.astype(np.float64) @ xn))
        assert e == r["sel"][t]
        np.testing.assert_allclose(r["out"][t], O.t5ff_run(x[t:t + 1], ws[e], "rms", "relu")[0], rtol=1e-12)
    perm = RNG.permutation(T)
    rp = O.moe_layer(x[perm], c, "cpm_2", ws, layernorm_weight=g)
    np.testing.assert_allclose(rp["out"], r["out"][perm], rtol=1e-12)


def test_cpm2_norm_is_used_for_scoring_only():
    T, d, h, E = 16, 8, 12, 4
    x, c, g = O.draw_inputs(9, T, d, E)
    ws = [O.draw_expert(9, e, d, h) for e in range(E)]
    a = O.moe_layer(x, c, "cpm_2", ws, layernorm_weight=g)
    b = O.moe_layer(x, c, "default", ws, sel_override=a["sel"])
    np.testing.assert_array_equal(a["out"], b["out"])  # experts saw the raw input in both


def test_zipf_bias_skews_counts():
    x, c, _ = O.draw_inputs(2, 4096, 32, 16)
    b = O.zipf_score_bias(x, c, s=1.2)
    sel, _ = O.select_top1(O.score(x, c, b))
    cnt = np.bincount(sel, minlength=16)
    assert cnt[0] > 4 * cnt[-1] and cnt.min() > 0
