"""Helpers of the GPU parity tests: device buffers come from torch (plumbing only), every
computation under test goes through the C ABI, every expectation comes from the oracle."""
import ctypes as C

import numpy as np

from infmoe_amd import capi

RTOL = 1e-4  # tolerance of the layer output against the float64 oracle (FP32 arithmetic)


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def stream_ptr(torch):
    return torch.cuda.current_stream().cuda_stream


def assert_close(got, want, rtol=RTOL, what=""):
    """max |got - want| <= rtol * max |want| and elementwise |diff| <= rtol * (|want| + rms(want))."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    diff = np.abs(got - want)
    scale = max(np.abs(want).max(), 1e-30)
    assert diff.max() <= rtol * scale, f"{what}: max rel err {diff.max() / scale:.3e} > {rtol}"
    rms = np.sqrt((want ** 2).mean())
    bad = diff > rtol * (np.abs(want) + rms)
    assert not bad.any(), f"{what}: {bad.sum()} elements off, worst {diff.max():.3e}"


def pack_slot(w, ffn_kind):
    """One expert's device slot [gamma | wi(_0) | (wi_1) | wo] (plugin/sublayers/T5FFLayer.cc:100-131)."""
    keys = ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight") if ffn_kind == "gated_gelu" \
        else ("layer_norm_weight", "wi_weight", "wo_weight")
    return np.concatenate([np.asarray(w[k], np.float32).ravel() for k in keys])


def check_assignment(sel_dev, oracle_aff, stats=None):
    """Bit-exact assignment except tokens whose float64 top-2 gap is below 1e-6 relative."""
    from oracle import moe_oracle as O
    want, _ = O.select_top1(oracle_aff)
    gap = O.top2_relative_gap(oracle_aff)
    exempt = gap < 1e-6
    mism = (np.asarray(sel_dev) != want) & ~exempt
    assert not mism.any(), f"{mism.sum()} non-exempt tokens assigned differently (first: {np.flatnonzero(mism)[:5]})"
    return int(exempt.sum())
