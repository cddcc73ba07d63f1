"""Parity at the benchmark's full sizes.  The float64 oracle cannot run whole 687-GFLOP layers in
seconds, so at these sizes the checks are (1) the gating of every token against the oracle (cheap:
T x d x E), (2) every output row of a sample of tokens against a per-token oracle evaluation with the
expert the device chose - rows are independent, so this is exact parity for the sampled rows - and
(3) size-independent properties: counts sum to T, an Identity sub-layer returns its input bit for bit."""
import ctypes as C

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin, capi
from oracle import moe_oracle as O
from tests.gpu_util import assert_close, check_assignment, stream_ptr

pytestmark = pytest.mark.gpu


def slot_weights(slot, d, h, ffn):
    if ffn == "gated_gelu":
        return {"layer_norm_weight": slot[:d], "wi_0_weight": slot[d:d + d * h].reshape(h, d),
                "wi_1_weight": slot[d + d * h:d + 2 * d * h].reshape(h, d), "wo_weight": slot[d + 2 * d * h:].reshape(d, h)}
    return {"layer_norm_weight": slot[:d], "wi_weight": slot[d:d + d * h].reshape(h, d),
            "wo_weight": slot[d + d * h:].reshape(d, h)}


def device_gate(lib, torch, x2d, cent, gamma, norm, bias):
    T, d = x2d.shape
    E = cent.shape[0]
    sel = torch.empty(T, dtype=torch.int32, device="cuda")
    coeff = torch.empty(T, dtype=torch.float32, device="cuda")
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    db = torch.from_numpy(bias).cuda() if bias is not None else None
    ws = torch.empty(max(lib.infmoe_gate_top1_scratch_bytes(T, d, E), 16), dtype=torch.uint8, device="cuda")
    capi.check(lib.infmoe_gate_top1(T, d, E, x2d.data_ptr(), cent.data_ptr(), gamma.data_ptr() if norm != "none" else None,
                                    capi.NORM_KINDS[norm], db.data_ptr() if db is not None else None, sel.data_ptr(),
                                    coeff.data_ptr(), stats.data_ptr(), ws.data_ptr(), stream_ptr(torch)))
    torch.cuda.synchronize()
    return sel.cpu().numpy(), coeff.cpu().numpy(), stats.cpu().numpy()


# the last case is the three-matrix form the reference's code computes, at c2's sizes
@pytest.mark.parametrize("name,experts_to_check,rows_per_expert,ffn",
                         [("c2", 2, 24, "relu"), ("c5", 5, 8, "relu"), ("c4", 3, 16, "relu"), ("c2", 2, 16, "gated_gelu")])
def test_full_size_layer_sampled_rows(lib, torch_cuda, name, experts_to_check, rows_per_expert, ffn):
    torch = torch_cuda
    import bench
    cfg = dict(bench.CONFIGS[name], ffn=ffn)
    E, d, h = cfg["E"], cfg["d"], cfg["h"]
    B, S = cfg["shape"]
    T = B * S
    variant = cfg["variant"]
    plugin, x, cent, gamma, slots, bias = bench.build_layer(torch, cfg, keep_host=True)
    y = plugin.forward(x.contiguous())
    torch.cuda.synchronize()
    count, stats = plugin.last_routing()
    assert count.sum() == T and stats["nan_rows"] == 0

    # (1) gating of every token
    xh = x.reshape(T, d).cpu().numpy()
    ch, gh = cent.cpu().numpy(), gamma.cpu().numpy()
    xa = O.layernorm(xh, gh, "rms") if variant == "cpm_2" else xh.astype(np.float64)
    aff = O.score(xa, ch, bias)
    sel, coeff, gstats = device_gate(lib, torch, x.reshape(T, d), cent, gamma, "rms" if variant == "cpm_2" else "none", bias)
    exempt = check_assignment(sel, aff)
    assert gstats[0] == exempt == stats["near_ties"]
    np.testing.assert_array_equal(np.bincount(sel, minlength=E), count)
    assert_close(coeff, aff[np.arange(T), sel], what="coeff")

    # (2) sampled rows, per-token oracle with the device's expert
    yh = y.reshape(T, d).cpu().numpy()
    active = np.flatnonzero(count > 0)
    order = active[np.argsort(count[active])]
    chosen = list(dict.fromkeys([order[0], order[-1], *order[:: max(1, len(order) // experts_to_check)]]))[:experts_to_check]
    checked = 0
    for e in chosen:
        w = slot_weights(slots[e], d, h, ffn)
        toks = np.flatnonzero(sel == e)[:rows_per_expert]
        post = O.t5ff_run(xh[toks], w, "rms", ffn)
        if variant == "base_layer":
            a = O.sigmoid(aff[toks, e])[:, None]
            post = a * post + (1 - a) * xh[toks].astype(np.float64)
        assert_close(yh[toks], post, what=f"{name} expert {e} ({count[e]} rows)")
        checked += len(toks)
    assert checked >= min(rows_per_expert, T)
    plugin.terminate()


def test_full_size_streamed_equals_resident(torch_cuda):
    """The same layer with its experts streamed through two slots (10.7 GB over the host link per call)
    and with all of them resident: the same bits."""
    torch = torch_cuda
    import bench
    outs = []
    for name in ("c2", "c3"):  # equal but for max_concurrency: 32 (resident) and 2
        plugin, x, *_ = bench.build_layer(torch, bench.CONFIGS[name], keep_host=False)
        outs.append(plugin.forward(x.contiguous()).clone())
        torch.cuda.synchronize()
        plugin.terminate()
    assert torch.equal(outs[0], outs[1])


def test_full_size_identity_returns_input(torch_cuda):
    torch = torch_cuda
    T, d, E = 4096, 4096, 32
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    x = torch.randn(8, 512, d, generator=gen, device="cuda")
    cent = (torch.randn(E, d, generator=gen, device="cuda") / 64).cpu().numpy()
    cfg = MoELayerConfig(seq_len=512, expert_count=E, embedding_size=d, hidden_size=10240, max_concurrency=2,
                         moe_variant="cpm_2", sublayer_type="Identity", max_batch_size=8, expert_centroids=cent,
                         layernorm_weight=np.ones(d, np.float32))
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([8, 512, d])
    plugin.initialize()
    y = plugin.forward(x)
    assert torch.equal(y, x)
    count, _ = plugin.last_routing()
    assert count.sum() == T and (count > 0).all()
    plugin.terminate()
