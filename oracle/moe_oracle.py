"""CPU restatement (numpy, float64) of InfMoE's MoELayerPlugin hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests, the smoke check and
the benchmark's CPU-baseline leg may import it; the shipped library never does.

Every function cites the reference file:line it restates (paths are relative to
the Harry-Chen/InfMoE tree).  Two defects of the public reference are *not*
reproduced, the intended math is used instead:
  * plugin/MoELayerPlugin.cc:373,391-392 offsets expert rows by a token count
    without multiplying by the row length -> here row stride `d` is applied;
  * plugin/MoELayerPlugin.cc:411 gathers the pre-expert buffer for the
    default / cpm_2 variants -> here the post-expert buffer is gathered.

The reference code and its README disagree about the norm and the FFN form, so
both are explicit parameters:
  norm_kind: "centered" = plugin/cuda/ops/layernorm.cu:136-174 as coded
             "rms"      = README.md:115 / comment at plugin/sublayers/T5FFLayer.cc:98
  ffn_kind:  "gated_gelu" = plugin/sublayers/T5FFLayer.cc:105-138 as coded (wi_0, wi_1, wo)
             "relu"       = the two-matrix dense_relu_dense the benchmark configs name (wi, wo)

Pin status (tests/test_oracle_pins.py): every function below is checked against
an independent library routine, closed form, invariant or brute force; none is
"parity unpinned".  The third-party arithmetic the reference delegates to
(cuBLAS SGEMM, thrust::transform, CUDA rsqrt/tanh/exp) is pinned by its
mathematical definition only.
"""
from __future__ import annotations

import numpy as np

EPS = 1e-6  # plugin/MoELayerPlugin.cc:324 and plugin/sublayers/T5FFLayer.cc:102 pass (double)1e-6

VARIANTS = ("default", "cpm_2", "base_layer")
NORM_KINDS = ("rms", "centered")
FFN_KINDS = ("relu", "gated_gelu")


def parse_flags(moe_variant: str):
    """plugin/MoELayerPlugin.cc:44-58 -> (layernormOnInputBeforeScore, baseLayerOutputMix)."""
    if moe_variant == "base_layer":
        return False, True
    if moe_variant == "cpm_2":
        return True, False
    if moe_variant == "default":
        return False, False
    raise ValueError(f"unsupported moe variant: {moe_variant}")


def layernorm(x, gamma, norm_kind: str, eps: float = EPS):
    """Row-wise norm with gamma only (beta is nullptr at both call sites).

    centered: plugin/cuda/ops/layernorm.cu:149,157-161 -> gamma*(x-mu)*rsqrt(var+eps), biased var.
    rms:      README.md:115 -> gamma * x / sqrt(mean(x^2) + eps).
    """
    x = np.asarray(x, dtype=np.float64)
    gamma = np.asarray(gamma, dtype=np.float64)
    if norm_kind == "centered":
        mu = x.mean(axis=-1, keepdims=True)
        var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
        return gamma * ((x - mu) / np.sqrt(var + eps))
    if norm_kind == "rms":
        ms = (x * x).mean(axis=-1, keepdims=True)
        return gamma * (x / np.sqrt(ms + eps))
    raise ValueError(f"unknown norm kind: {norm_kind}")


def score(x_aff, centroids, score_bias=None):
    """plugin/MoELayerPlugin.cc:332-337: aff[t,e] = sum_k x_aff[t,k] * centroids[e,k].

    `centroids` is in the reference's in-memory layout [E][d]
    (lda = token_len with OP_T; python/infmoe/config.py:27-28).
    `score_bias[E]` is a test-harness extension (skewed routing); None on the plugin path.
    """
    aff = np.asarray(x_aff, np.float64) @ np.asarray(centroids, np.float64).T
    if score_bias is not None:
        aff = aff + np.asarray(score_bias, np.float64)[None, :]
    return aff


def select_top1(aff):
    """plugin/cuda/moe.cu:60-75: first maximum wins (strict '>' scanning ascending index).

    A row the scan cannot order (NaN) leaves the position at -1 and trips the
    assert at plugin/cuda/moe.cu:70; that is raised here.
    Returns (sel int32[T], coeff float64[T]).
    """
    aff = np.asarray(aff, np.float64)
    T, E = aff.shape
    sel = np.full(T, -1, np.int32)
    best = np.full(T, -np.finfo(np.float32).max)
    for e in range(E):  # literal restatement of the scan; vectorised over rows
        better = aff[:, e] > best
        best = np.where(better, aff[:, e], best)
        sel = np.where(better, e, sel).astype(np.int32)
    if (sel < 0).any():
        raise FloatingPointError("row with no orderable score (NaN)")
    return sel, best


def top2_relative_gap(aff):
    """(s1 - s2) / max(|s1|, tiny) per row; rows under 1e-6 are exempt from bit-exact assignment."""
    aff = np.asarray(aff, np.float64)
    if aff.shape[1] < 2:
        return np.full(aff.shape[0], np.inf)
    part = np.partition(aff, -2, axis=1)
    s1, s2 = part[:, -1], part[:, -2]
    return (s1 - s2) / np.maximum(np.abs(s1), np.finfo(np.float64).tiny)


def expert_count(sel, n_expert: int):
    """plugin/cuda/moe.cu:181-199 (+ offset[E] = T preset at plugin/MoELayerPlugin.cc:350-351).

    Histogram, exclusive prefix, stable counting sort.  Routed row r holds
    original token pos[r].  Returns (count[E], offset[E+1], pos[T]) int32.
    """
    sel = np.asarray(sel)
    T = sel.shape[0]
    count = np.zeros(n_expert, np.int32)
    for t in range(T):
        count[sel[t]] += 1
    offset = np.zeros(n_expert + 1, np.int32)
    for e in range(1, n_expert):
        offset[e] = offset[e - 1] + count[e - 1]
    offset[n_expert] = T
    cursor = offset[:n_expert].copy()
    pos = np.empty(T, np.int32)
    for t in range(T):
        pos[cursor[sel[t]]] = t
        cursor[sel[t]] += 1
    return count, offset, pos


def scatter(x, coeff, pos):
    """plugin/cuda/moe.cu:98-113: routed[r,:] = x[pos[r],:], routed_coeff[r] = coeff[pos[r]]."""
    return np.asarray(x)[pos], np.asarray(coeff)[pos]


def gather(buf, pos):
    """plugin/cuda/moe.cu:89-96: out[pos[r],:] = buf[r,:]."""
    out = np.empty_like(buf)
    out[pos] = buf
    return out


def sigmoid(v):
    """plugin/cuda/common.cuh:24-27."""
    return 1.0 / (1.0 + np.exp(-np.asarray(v, np.float64)))


def mix_and_gather(post, routed, routed_coeff, pos):
    """plugin/cuda/moe.cu:115-127: a = sigmoid(coeff[r]); out[pos[r],:] = a*post[r,:] + (1-a)*routed[r,:]."""
    a = sigmoid(routed_coeff)[:, None]
    mixed = a * np.asarray(post, np.float64) + (1.0 - a) * np.asarray(routed, np.float64)
    out = np.empty_like(mixed)
    out[pos] = mixed
    return out


def gelu_dot(a, b):
    """plugin/cuda/ops/gelu.cu:7-16: a * 0.5*(1+tanh(a*(C*a*a+B))) * b."""
    a = np.asarray(a, np.float64)
    B = 0.7978845608028654
    C = 0.035677408136300125
    cdf = 0.5 * (1.0 + np.tanh(a * (C * a * a + B)))
    return a * cdf * np.asarray(b, np.float64)


def t5ff_run(x, w: dict, norm_kind: str, ffn_kind: str):
    """plugin/sublayers/T5FFLayer.cc:90-141: out = x + FFN(norm(x)).

    Weights use the reference's in-memory (torch Linear) layouts
    (plugin/sublayers/T5FFLayer.cc:112-138; python/infmoe/config.py:46-52):
      layer_norm_weight [d]
      gated_gelu: wi_0_weight [h,d], wi_1_weight [h,d], wo_weight [d,h]
      relu:       wi_weight   [h,d],                    wo_weight [d,h]
    """
    x = np.asarray(x, np.float64)
    ln = layernorm(x, w["layer_norm_weight"], norm_kind)
    wo = np.asarray(w["wo_weight"], np.float64)
    if ffn_kind == "gated_gelu":
        h0 = ln @ np.asarray(w["wi_0_weight"], np.float64).T
        h1 = ln @ np.asarray(w["wi_1_weight"], np.float64).T
        hid = gelu_dot(h0, h1)
    elif ffn_kind == "relu":
        hid = np.maximum(ln @ np.asarray(w["wi_weight"], np.float64).T, 0.0)
    else:
        raise ValueError(f"unknown ffn kind: {ffn_kind}")
    return x + hid @ wo.T


def identity_run(x, w=None, *_):
    """plugin/sublayers/IdentityLayer.hh:34-40: out = in."""
    return np.array(x, copy=True)


def gate(x, centroids, moe_variant, layernorm_weight=None, norm_kind="rms", score_bias=None):
    """plugin/MoELayerPlugin.cc:312-345: optional norm (scoring only), score, top-1.

    Returns (sel, coeff, aff)."""
    ln_before, _ = parse_flags(moe_variant)
    x = np.asarray(x, np.float64)
    x_aff = x
    if ln_before:
        if layernorm_weight is None:
            raise ValueError("cpm_2 requires layernorm_weight")  # plugin/MoELayerPlugin.cc:76-79
        x_aff = layernorm(x, layernorm_weight, norm_kind)
    aff = score(x_aff, centroids, score_bias)
    sel, coeff = select_top1(aff)
    return sel, coeff, aff


def moe_layer(x, centroids, moe_variant, expert_weights, *, layernorm_weight=None,
              sublayer_type="T5_FF", norm_kind="rms", ffn_kind="relu", score_bias=None,
              sel_override=None):
    """plugin/MoELayerPlugin.cc:279-416, intended math.

    x: [T,d] (tokens already flattened, :288-289).  expert_weights: list of dicts
    (ignored for Identity).  `sel_override` lets a parity test feed the device's
    assignment so the output comparison is not polluted by exempt near-tie tokens.
    Returns dict(out, sel, coeff, aff, count, offset, pos).
    """
    x = np.asarray(x, np.float64)
    E = np.asarray(centroids).shape[0]
    _, mix = parse_flags(moe_variant)
    sel, coeff, aff = gate(x, centroids, moe_variant, layernorm_weight, norm_kind, score_bias)
    if sel_override is not None:
        sel = np.asarray(sel_override, np.int32)
        coeff = aff[np.arange(x.shape[0]), sel]
    count, offset, pos = expert_count(sel, E)
    routed, routed_coeff = scatter(x, coeff, pos)  # experts get the RAW input (:354)
    post = np.empty_like(routed)
    for e in range(E):  # ascending, empties skipped (:361-363,383-384)
        if count[e] == 0:
            continue
        rows = slice(offset[e], offset[e] + count[e])
        if sublayer_type == "T5_FF":
            post[rows] = t5ff_run(routed[rows], expert_weights[e], norm_kind, ffn_kind)
        elif sublayer_type == "Identity":
            post[rows] = identity_run(routed[rows])
        else:
            raise ValueError(f"unsupported sublayer type: {sublayer_type}")
    out = mix_and_gather(post, routed, routed_coeff, pos) if mix else gather(post, pos)
    return dict(out=out, sel=sel, coeff=coeff, aff=aff, count=count, offset=offset, pos=pos)


# ----------------------------------------------------------------------------
# Synthetic inputs shared by tests, smoke and bench (not part of the reference).
# One SeedSequence child per tensor so tensors can be drawn independently.
# ----------------------------------------------------------------------------
_TENSOR_IDS = {"x": 0, "centroids": 1, "layernorm_weight": 2, "score_bias": 3}


def _rng(seed: int, *key: int):
    return np.random.default_rng(np.random.SeedSequence(entropy=seed, spawn_key=tuple(key)))


def draw_inputs(seed, T, d, E):
    """x ~ N(0,1) [T,d]; centroids ~ N(0,1/d) drawn logical [d,E], handed over as [E][d];
    gating gamma = 1 + 0.1 N(0,1)."""
    x = _rng(seed, 0).standard_normal((T, d)).astype(np.float32)
    cent_logical = (_rng(seed, 1).standard_normal((d, E)) / np.sqrt(d)).astype(np.float32)
    gamma = (1.0 + 0.1 * _rng(seed, 2).standard_normal(d)).astype(np.float32)
    return x, np.ascontiguousarray(cent_logical.T), gamma


def draw_expert(seed, e, d, h, ffn_kind="relu"):
    """Per-expert weights: gamma = 1+0.1N, wi ~ N(0,1/d) logical [d,h] -> stored [h][d],
    wo ~ N(0,1/h) logical [h,d] -> stored [d][h]."""
    w = {"layer_norm_weight": (1.0 + 0.1 * _rng(seed, 100 + e, 0).standard_normal(d)).astype(np.float32)}
    if ffn_kind == "relu":
        wi = (_rng(seed, 100 + e, 1).standard_normal((d, h)) / np.sqrt(d)).astype(np.float32)
        w["wi_weight"] = np.ascontiguousarray(wi.T)
    else:
        for j, name in enumerate(("wi_0_weight", "wi_1_weight")):
            wi = (_rng(seed, 100 + e, 1 + j).standard_normal((d, h)) / np.sqrt(d)).astype(np.float32)
            w[name] = np.ascontiguousarray(wi.T)
    wo = (_rng(seed, 100 + e, 3).standard_normal((h, d)) / np.sqrt(h)).astype(np.float32)
    w["wo_weight"] = np.ascontiguousarray(wo.T)
    return w


def zipf_score_bias(x, centroids, s=1.2, iters=30):
    """Per-expert additive score bias so that argmax counts follow p_e ~ (e+1)^-s.

    Simple fixed-point calibration on the host (harness only, not a reference attribute)."""
    aff = np.asarray(x, np.float64) @ np.asarray(centroids, np.float64).T
    T, E = aff.shape
    target = (np.arange(1, E + 1) ** (-s))
    target = target / target.sum()
    bias = np.zeros(E)
    for _ in range(iters):
        sel = np.argmax(aff + bias, axis=1)
        p = np.bincount(sel, minlength=E) / T
        bias += 0.5 * (np.log(target) - np.log(np.maximum(p, 0.5 / T)))
    return bias.astype(np.float32)
