"""A layer initialised from an expert_weight_file of real size: 14 experts of the headline layer's dimensions
(4096 x 10240, 335 MB each), 4.7 GB in all, so that the archive has zip64 structures and the last expert lies
beyond 4 GiB - the only way the reference obtains weights is to load such a file whole
(plugin/sublayers/T5FFLayer.cc:143-147, plugin/thirdparty/cnpy/cnpy.cpp:229-276).  Two experts hold drawn
weights (one of them the last); the others hold zeros, written as holes (tests/npz_large.py), and with zero
weights an expert returns its input."""
import shutil
import zipfile

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin
from oracle import moe_oracle as O
from tests.gpu_util import assert_close, dev
from tests.npz_large import write_npz

pytestmark = pytest.mark.gpu


def test_layer_from_a_weight_file_of_more_than_four_gib(torch_cuda, tmp_path):
    torch = torch_cuda
    if shutil.disk_usage(tmp_path).free < (2 << 30):
        pytest.skip("less than 2 GiB free under the temporary directory (the archive stores 0.7 GB of drawn weights)")
    E, d, h, B, S = 14, 4096, 10240, 4, 56
    real = {2: O.draw_expert(31, 2, d, h), 13: O.draw_expert(31, 13, d, h)}
    members = []
    for e in range(E):
        for key, shape in (("layer_norm_weight", (d,)), ("wi_weight", (h, d)), ("wo_weight", (d, h))):
            members.append((f"{e}/{key}", real[e][key] if e in real else shape))
    path = tmp_path / "experts.npz"
    write_npz(path, members)
    with zipfile.ZipFile(path) as z:  # the last expert's members start beyond 4 GiB
        assert min(i.header_offset for i in z.infolist() if i.filename.startswith("13/")) > (1 << 32)

    x, c, g = O.draw_inputs(31, B * S, d, E)
    cfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=E,
                         moe_variant="cpm_2", sublayer_type="T5_FF", max_batch_size=B, expert_centroids=c,
                         layernorm_weight=g, weight_file_path=str(path))
    plugin = MoELayerPlugin(cfg).create_plugin()
    plugin.configure([B, S, d])
    plugin.initialize()
    y = plugin.forward(dev(torch, x.reshape(B, S, d)))
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(B * S, d)
    count, stats = plugin.last_routing()
    plugin.terminate()

    sel = O.gate(x, c, "cpm_2", g)[0]
    np.testing.assert_array_equal(count, np.bincount(sel, minlength=E))
    assert stats["nan_rows"] == 0 and count[2] > 0 and count[13] > 0
    for e, w in real.items():  # every row of the two experts that hold weights, against the float64 oracle
        rows = np.flatnonzero(sel == e)
        assert_close(y[rows], O.t5ff_run(x[rows], w, "rms", "relu"), what=f"expert {e} read from beyond {'4 GiB' if e == 13 else 'the start'}")
    others = ~np.isin(sel, list(real))
    np.testing.assert_array_equal(y[others], x[others])  # zero weights: the expert adds nothing to its input
