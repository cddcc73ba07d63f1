"""The layer against the float64 oracle at token counts one below, at and one above every point where the
host picks another kernel or another launch sequence, with routing that is even and routing that a score bias
sends mostly to the first experts:

  tokens <= 2 * experts      every expert through the row-streaming kernel, tall ones in runs of eight rows
  tokens <= 64 * experts     row tiles of at most 96 rows, two workgroups per compute unit
  tokens >= 1024             gating by slices with the centroid slice in the LDS (row length a multiple of 128)
  tokens >  1024             the counting sort ranks blocks of 1024 tokens; the gating's second launch has
                             already counted each block's tokens per expert
"""
import numpy as np
import pytest

from tests.test_gpu_layer import make_layer, run_and_check

pytestmark = pytest.mark.gpu


def skewed(E, skew):
    """A score bias that falls linearly from `skew` at expert 0 to nothing at the last one."""
    if not skew or E < 2:
        return None
    return (skew * (1.0 - np.arange(E) / (E - 1))).astype(np.float32)


CASES = [
    # (experts, embedding, hidden, token counts, skews)
    (16, 256, 384, (31, 32, 33), (0.0, 5.0)),            # 2 * experts = 32
    (5, 128, 160, (10, 11, 40), (0.0, 3.0)),             # 2 * experts = 10; 40 tokens mostly on one expert
    (4, 128, 256, (255, 256, 257), (0.0, 3.0)),          # 64 * experts = 256
    (8, 256, 128, (511, 512, 513), (0.0, 3.0)),          # 64 * experts = 512
    (8, 256, 128, (1023, 1024, 1025, 2047, 2048, 2049, 3001), (0.0, 3.0)),   # blocks of 1024 tokens
    (64, 1024, 64, (1024, 1025, 2050), (0.0, 3.0)),      # the same with 64 experts: four score blocks a token
    (128, 2048, 32, (1500,), (0.0, 3.0)),                # the widest layer the sliced gating takes
    (130, 2048, 32, (1500,), (0.0,)),                    # and one too wide for it
]


@pytest.mark.parametrize("E,d,h,tokens,skews", CASES, ids=[f"E{c[0]}-d{c[1]}-T{c[3][0]}" for c in CASES])
@pytest.mark.parametrize("variant,ffn", [("cpm_2", "relu"), ("base_layer", "gated_gelu")])
def test_layer_at_kernel_choice_boundaries(torch_cuda, E, d, h, tokens, skews, variant, ffn):
    for T in tokens:
        for skew in skews:
            bias = skewed(E, skew)
            print(f"case E={E} d={d} h={h} T={T} skew={skew} {variant}/{ffn}", flush=True)
            plugin, x, c, g, ws = make_layer((1, T), E, d, h, E, variant, ffn=ffn, seed=300 + T % 97, bias=bias)
            _, _, count, _ = run_and_check(torch_cuda, plugin, x, c, g, ws, (1, T), variant, ffn=ffn, bias=bias)
            assert int(count.sum()) == T
            if skew and T >= 4 * E:
                assert count.max() >= 2 * T // E, f"the bias did not skew the routing: {count}"
            plugin.terminate()
