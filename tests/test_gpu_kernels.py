"""Parity of every kernel-level C entry point against the float64 oracle, on the GPU."""
import numpy as np
import pytest

from infmoe_amd import capi
from oracle import moe_oracle as O
from tests.gpu_util import assert_close, check_assignment, dev, pack_slot, stream_ptr

pytestmark = pytest.mark.gpu
NORM = capi.NORM_KINDS
FFN = capi.FFN_KINDS


# ------------------------------------------------------------------ gating
def run_gate(lib, torch, x, c, gamma, norm, bias=None, scratch=True):
    """scratch=True hands over the optional scratch memory (filled with 0xFF bytes: any contents are
    allowed), which lets the kernel split the embedding dimension; False runs the one-pass form."""
    T, d = x.shape
    E = c.shape[0]
    dx, dc = dev(torch, x), dev(torch, c)
    dg = dev(torch, gamma) if gamma is not None else None
    db = dev(torch, bias) if bias is not None else None
    sel = torch.full((T,), -7, dtype=torch.int32, device="cuda")
    coeff = torch.zeros(T, dtype=torch.float32, device="cuda")
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    ws = torch.full((max(lib.infmoe_gate_top1_scratch_bytes(T, d, E), 16),), 255, dtype=torch.uint8, device="cuda") if scratch else None
    capi.check(lib.infmoe_gate_top1(T, d, E, dx.data_ptr(), dc.data_ptr(), dg.data_ptr() if dg is not None else None,
                                    NORM[norm], db.data_ptr() if db is not None else None, sel.data_ptr(),
                                    coeff.data_ptr(), stats.data_ptr(), ws.data_ptr() if scratch else None,
                                    stream_ptr(torch)))
    torch.cuda.synchronize()
    return sel.cpu().numpy(), coeff.cpu().numpy(), stats.cpu().numpy()


@pytest.mark.parametrize("T,d,E,norm,use_bias", [
    (32, 64, 4, "none", False),      # tiny default-variant config
    (80, 4, 2, "rms", False),        # reference example shape (d smaller than one chunk)
    (100, 4096, 32, "rms", False),   # cpm_2 shape
    (77, 130, 5, "centered", False), # row length not a multiple of 4: scalar path
    (1, 256, 16, "rms", False),
    (300, 2048, 64, "none", True),   # base_layer shape with score bias
    (50, 512, 200, "centered", True),  # more than 128 experts: several passes
    (64, 4096, 32, "centered", False),
    (2048, 2048, 16, "centered", False),  # 2 slices of the embedding dimension
    (16389, 256, 8, "rms", True),         # 64-token workgroups, ragged last group
    (40, 4096, 200, "rms", False),        # several passes over experts and several slices
    (1024, 1024, 32, "rms", False),       # 16-token workgroups, 4 slices
    (40, 1030, 8, "rms", False),          # scalar path (row length not a multiple of 4) with slices
    (7, 4098, 130, "none", False),        # scalar path, two passes over experts, slices
])
@pytest.mark.parametrize("scratch", [True, False])
def test_gate_top1_matches_oracle(lib, torch_cuda, T, d, E, norm, use_bias, scratch):
    torch = torch_cuda
    x, c, g = O.draw_inputs(11, T, d, E)
    x = x + (0.3 if norm == "centered" else 0.0)  # a mean for the centred norm to remove
    bias = (0.2 * np.random.default_rng(5).standard_normal(E)).astype(np.float32) if use_bias else None
    sel, coeff, stats = run_gate(lib, torch, x, c, g if norm != "none" else None, norm, bias, scratch=scratch)
    xa = O.layernorm(x, g, norm) if norm != "none" else x.astype(np.float64)
    aff = O.score(xa, c, bias)
    exempt = check_assignment(sel, aff)
    assert stats[0] == exempt
    assert stats[1] == 0
    want = aff[np.arange(T), sel]
    assert_close(coeff, want, what="coeff")


@pytest.mark.parametrize("d", [32, 1024])  # one chunk; several slices
def test_gate_top1_exact_ties_pick_lowest_index(lib, torch_cuda, d):
    torch = torch_cuda
    rng = np.random.default_rng(3)
    T, E = 64, 24
    x = rng.integers(-2, 3, size=(T, d)).astype(np.float32)  # small integers: scores are exact
    c = rng.integers(-1, 2, size=(E, d)).astype(np.float32)
    c[7] = c[3]
    c[19] = c[3]  # identical centroids -> exact ties
    sel, coeff, stats = run_gate(lib, torch, x, c, None, "none")
    aff = O.score(x, c)
    want, best = O.select_top1(aff)
    np.testing.assert_array_equal(sel, want)  # lowest index among equal maxima, also after re-scoring
    np.testing.assert_array_equal(coeff, best.astype(np.float32))
    assert stats[0] == int((O.top2_relative_gap(aff) < 1e-6).sum())


@pytest.mark.parametrize("d", [64, 2048])  # one chunk; several slices
def test_gate_top1_counts_nan_rows(lib, torch_cuda, d):
    torch = torch_cuda
    x, c, g = O.draw_inputs(2, 40, d, 8)
    x[5, 3] = np.nan
    x[33, :] = np.nan
    sel, coeff, stats = run_gate(lib, torch, x, c, g, "rms")
    assert stats[1] == 2
    ok = np.ones(40, bool)
    ok[[5, 33]] = False
    aff = O.score(O.layernorm(x[ok], g, "rms"), c)
    np.testing.assert_array_equal(sel[ok], O.select_top1(aff)[0])


def test_gate_near_tie_is_rescored_in_float64(lib, torch_cuda):
    """Two centroids 3e-6 relative apart: above the 1e-6 exemption, at the edge of what FP32
    accumulation over 1024 terms can order, so the float64 re-scoring has to decide."""
    torch = torch_cuda
    T, d, E = 48, 1024, 8
    x, c, g = O.draw_inputs(4, T, d, E)
    c = c.astype(np.float64)
    c[:] *= 0.1
    c[5] = 1.0 * np.sign(np.arange(d) % 2 - 0.5) / np.sqrt(d)
    c = c.astype(np.float32)
    c[2] = (c[5].astype(np.float64) * (1 + 3e-6)).astype(np.float32)  # 3e-6 relative apart: must be ordered
    sel, coeff, stats = run_gate(lib, torch, x, c, None, "none")
    aff = O.score(x, c)
    exempt = check_assignment(sel, aff)
    assert stats[2] >= 1  # the float64 path ran
    assert stats[0] == exempt


@pytest.mark.parametrize("T,d", [(300, 8192), (1536, 8192), (2048, 16384)])  # one-kernel / sliced form; slab form
@pytest.mark.parametrize("norm", ["none", "rms"])
def test_gate_adversarial_same_sign_near_ties(lib, torch_cuda, T, d, norm):
    """The case in which FP32 accumulation is worst: every term of every dot product has the same sign, the
    rows are long, and the experts' scores lie a few 1e-6 relative apart (above the 1e-6 exemption, so the
    assignment has to be the float64 one).  The re-scoring threshold (8 eps times the Cauchy-Schwarz bound of a
    score, at least 4e-6 of the best score) is an empirical choice, not a worst-case bound of a length-d FP32
    sum; this pins it where it is most at risk."""
    torch = torch_cuda
    E = 16
    rng = np.random.default_rng(d + T)
    x = (np.abs(rng.standard_normal((T, d))) + 0.5).astype(np.float32)
    c0 = (np.abs(rng.standard_normal(d)) + 0.1) / np.sqrt(d)
    order = rng.permutation(E)  # the best expert is not the last index
    c = np.stack([c0 * (1.0 + 2.5e-6 * order[e]) for e in range(E)]).astype(np.float32)
    g = (1.0 + 0.1 * np.abs(rng.standard_normal(d))).astype(np.float32)
    sel, coeff, stats = run_gate(lib, torch, x, c, g if norm != "none" else None, norm)
    xa = O.layernorm(x, g, norm) if norm != "none" else x.astype(np.float64)
    aff = O.score(xa, c)
    gap = O.top2_relative_gap(aff)
    assert (gap < 1e-5).all() and (gap > 1e-6).mean() > 0.9  # near ties everywhere, nearly none of them exempt
    exempt = check_assignment(sel, aff)
    assert stats[0] == exempt
    assert stats[2] >= T // 2  # FP32 could not be trusted with most of them: the float64 path decided
    assert_close(coeff, aff[np.arange(T), sel], what="coeff")


# ------------------------------------------------------------------ count / sort
@pytest.mark.parametrize("T,E,mode", [
    (1, 1, "rand"), (1, 4, "rand"), (32, 4, "rand"), (1023, 7, "rand"), (1024, 32, "rand"), (1025, 32, "rand"),
    (4096, 32, "rand"), (16384, 64, "zipf"), (5000, 300, "rand"), (3000, 5, "one"),
])
def test_expert_count_is_bit_exact(lib, torch_cuda, T, E, mode):
    torch = torch_cuda
    rng = np.random.default_rng(T * 31 + E)
    if mode == "rand":
        sel = rng.integers(0, E, size=T).astype(np.int32)
    elif mode == "one":
        sel = np.full(T, E - 2, np.int32)
    else:
        p = np.arange(1, E + 1) ** -1.2
        sel = rng.choice(E, size=T, p=p / p.sum()).astype(np.int32)
    dsel = dev(torch, sel)
    pos = torch.full((T,), -1, dtype=torch.int32, device="cuda")
    count = torch.full((E,), -1, dtype=torch.int32, device="cuda")
    offset = torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")
    scratch = torch.empty(max(lib.infmoe_expert_count_scratch_bytes(T, E), 1), dtype=torch.uint8, device="cuda")
    capi.check(lib.infmoe_expert_count(T, E, dsel.data_ptr(), pos.data_ptr(), count.data_ptr(), offset.data_ptr(),
                                       scratch.data_ptr(), stream_ptr(torch)))
    torch.cuda.synchronize()
    wc, wo, wp = O.expert_count(sel, E)
    np.testing.assert_array_equal(count.cpu().numpy(), wc)
    np.testing.assert_array_equal(offset.cpu().numpy(), wo)
    np.testing.assert_array_equal(pos.cpu().numpy(), wp)


# ------------------------------------------------------------------ scatter / gather / mix
@pytest.mark.parametrize("T,d", [(1, 4), (33, 64), (257, 130), (512, 4096), (100, 2048)])
def test_scatter_gather_mix(lib, torch_cuda, T, d):
    torch = torch_cuda
    rng = np.random.default_rng(T + d)
    x = rng.standard_normal((T, d)).astype(np.float32)
    coeff = rng.standard_normal(T).astype(np.float32)
    pos = rng.permutation(T).astype(np.int32)
    dx, dc, dp = dev(torch, x), dev(torch, coeff), dev(torch, pos)
    routed = torch.zeros_like(dx)
    rc = torch.zeros_like(dc)
    s = stream_ptr(torch)
    capi.check(lib.infmoe_expert_scatter(T, d, dx.data_ptr(), dc.data_ptr(), dp.data_ptr(), routed.data_ptr(), rc.data_ptr(), s))
    wr, wrc = O.scatter(x, coeff, pos)
    np.testing.assert_array_equal(routed.cpu().numpy(), wr)
    np.testing.assert_array_equal(rc.cpu().numpy(), wrc)
    back = torch.zeros_like(dx)
    capi.check(lib.infmoe_expert_gather(T, d, routed.data_ptr(), dp.data_ptr(), back.data_ptr(), s))
    np.testing.assert_array_equal(back.cpu().numpy(), x)  # gather(scatter(x)) == x exactly
    post = rng.standard_normal((T, d)).astype(np.float32)
    dpost = dev(torch, post)
    out = torch.zeros_like(dx)
    capi.check(lib.infmoe_expert_mix_gather(T, d, dp.data_ptr(), routed.data_ptr(), dpost.data_ptr(), rc.data_ptr(), out.data_ptr(), s))
    want = O.mix_and_gather(post, wr, wrc, pos)
    assert_close(out.cpu().numpy(), want, rtol=1e-6, what="mix")


# ------------------------------------------------------------------ norm
@pytest.mark.parametrize("rows,d", [(1, 4), (5, 64), (37, 130), (64, 4096), (3, 10240), (2, 8200)])
@pytest.mark.parametrize("kind", ["rms", "centered"])
def test_layernorm(lib, torch_cuda, rows, d, kind):
    torch = torch_cuda
    rng = np.random.default_rng(rows * 7 + d)
    x = (rng.standard_normal((rows, d)) * 2 + 0.7).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    dx, dg = dev(torch, x), dev(torch, g)
    out = torch.zeros_like(dx)
    capi.check(lib.infmoe_layernorm(out.data_ptr(), dx.data_ptr(), rows, d, dg.data_ptr(), NORM[kind], stream_ptr(torch)))
    assert_close(out.cpu().numpy(), O.layernorm(x, g, kind), rtol=1e-5, what="norm")


# ------------------------------------------------------------------ expert
def run_t5ff(lib, torch, x, w, norm, ffn):
    rows, d = x.shape
    h = w["wo_weight"].shape[1]
    slot = dev(torch, pack_slot(w, ffn))
    assert slot.numel() * 4 == lib.infmoe_t5ff_weight_bytes(d, h, FFN[ffn])
    dx = dev(torch, x)
    out = torch.zeros_like(dx)
    ws = torch.empty(max(lib.infmoe_t5ff_workspace_bytes(rows, d, h, FFN[ffn]), 16), dtype=torch.uint8, device="cuda")
    capi.check(lib.infmoe_t5ff_run(rows, d, h, NORM[norm], FFN[ffn], slot.data_ptr(), dx.data_ptr(), out.data_ptr(),
                                   ws.data_ptr(), stream_ptr(torch)))
    torch.cuda.synchronize()
    return out.cpu().numpy()


# tile shapes (16-row units + 4-row groups): 33 -> 2+1, 40 -> 2+2, 44 -> 2+3, 45 -> 3+0, 49 -> 3+1 (an odd
# unit and a group), 97 -> 6+1, 130 -> 8+1, 147 -> 9+1, 161 / 172 -> 10+1 / 10+3 (32-float steps), 250 -> 15+3
@pytest.mark.parametrize("rows", [1, 2, 3, 5, 8, 9, 16, 17, 33, 40, 44, 45, 49, 97, 100, 128, 130, 140, 147, 161, 172,
                                  250, 255, 256, 257, 300, 600])
@pytest.mark.parametrize("d,h", [(64, 256), (256, 96)])  # 64-float and (h = 96) 32-float K steps
def test_t5ff_row_counts(lib, torch_cuda, rows, d, h):
    w = O.draw_expert(21, 0, d, h, "relu")
    x = O.draw_inputs(rows, rows, d, 2)[0]
    got = run_t5ff(lib, torch_cuda, x, w, "rms", "relu")
    assert_close(got, O.t5ff_run(x, w, "rms", "relu"), what=f"t5ff rows={rows}")


# the benchmark's K (4096 into the first product, 10240 into the second) at the row counts of decode batches of
# a few hundred tokens: few-row kernel (5), one 16-row unit (12), one unit + two 4-row groups... (24 -> 2 units),
# three units (48), a 32-row block + a 16-row block + a group (52); every row count from 9 to 64 takes the
# few-rows-per-expert form of the matrix-core kernel (a call of at most 64 rows per expert): all of its tile
# shapes - one to four 16-row units, and from 32 rows on whole units plus one or two 4-row groups - are met
@pytest.mark.parametrize("rows", [5, 9, 12, 16, 17, 24, 31, 33, 36, 40, 41, 48, 52, 57, 64])
def test_t5ff_row_counts_at_full_width(lib, torch_cuda, rows):
    d, h = 4096, 10240
    w = O.draw_expert(26, 0, d, h, "relu")
    x = O.draw_inputs(rows, rows, d, 2)[0]
    got = run_t5ff(lib, torch_cuda, x, w, "rms", "relu")
    assert_close(got, O.t5ff_run(x, w, "rms", "relu"), what=f"t5ff rows={rows} at {d}x{h}")


# the two-matrix form keeps two accumulator sets: tiles of up to 192 rows, taller experts in equal tiles
@pytest.mark.parametrize("rows", [9, 130, 192, 193, 400])
def test_t5ff_gated_row_counts(lib, torch_cuda, rows):
    d, h = 64, 256
    w = O.draw_expert(24, 0, d, h, "gated_gelu")
    x = O.draw_inputs(rows, rows, d, 2)[0]
    got = run_t5ff(lib, torch_cuda, x, w, "centered", "gated_gelu")
    assert_close(got, O.t5ff_run(x, w, "centered", "gated_gelu"), what=f"gated t5ff rows={rows}")


@pytest.mark.parametrize("d,h", [(64, 256), (128, 320), (20, 36), (6, 10), (512, 1280), (4096, 256)])
@pytest.mark.parametrize("norm,ffn", [("rms", "relu"), ("centered", "gated_gelu"), ("rms", "gated_gelu"), ("centered", "relu")])
@pytest.mark.parametrize("rows", [4, 70])
def test_t5ff_shapes_and_kinds(lib, torch_cuda, d, h, norm, ffn, rows):
    w = O.draw_expert(22, 1, d, h, ffn)
    x = O.draw_inputs(5, rows, d, 2)[0] + 0.25
    got = run_t5ff(lib, torch_cuda, x, w, norm, ffn)
    assert_close(got, O.t5ff_run(x, w, norm, ffn), what=f"t5ff {d}x{h} {norm} {ffn}")


def test_t5ff_zero_wo_returns_input(lib, torch_cuda):
    d, h = 64, 128
    w = O.draw_expert(23, 0, d, h, "relu")
    w["wo_weight"][:] = 0
    x = O.draw_inputs(6, 40, d, 2)[0]
    np.testing.assert_array_equal(run_t5ff(lib, torch_cuda, x, w, "rms", "relu"), x)
