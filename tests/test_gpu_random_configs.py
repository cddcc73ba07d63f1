"""Seeded random layer configurations against the float64 oracle: sizes, variants, norms, feed-forward
kinds and slot counts in combinations nobody wrote down by hand (one expert, more experts than tokens, row
lengths that leave the fast paths, token counts on either side of every kernel choice)."""
import numpy as np
import pytest

from tests.test_gpu_layer import make_layer, run_and_check

pytestmark = pytest.mark.gpu


def draw(seed):
    rng = np.random.default_rng(1000 + seed)
    E = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 17, 33, 64, 130]))
    d = int(rng.choice([4, 8, 20, 30, 32, 48, 64, 96, 128, 256, 320, 384, 512, 1024]))
    h = int(rng.choice([8, 12, 32, 50, 64, 96, 160, 256, 512]))
    B = int(rng.choice([1, 2, 3, 5]))
    S = int(rng.choice([1, 2, 7, 16, 33, 100, 257, 411]))
    mc = int(rng.choice([1, 2, 3, E, E + 1]))
    variant = str(rng.choice(["default", "cpm_2", "base_layer"]))
    norm = str(rng.choice(["rms", "centered"]))
    ffn = str(rng.choice(["relu", "gated_gelu"]))
    return dict(E=E, d=d, h=h, shape=(B, S), mc=mc, variant=variant, norm=norm, ffn=ffn, seed=int(rng.integers(1, 10000)))


@pytest.mark.parametrize("seed", range(64))
def test_random_configuration_matches_the_oracle(torch_cuda, seed):
    k = draw(seed)
    print(f"case {seed}: {k}", flush=True)
    plugin, x, c, g, ws = make_layer(k["shape"], k["E"], k["d"], k["h"], k["mc"], k["variant"], norm=k["norm"],
                                     ffn=k["ffn"], seed=k["seed"])
    run_and_check(torch_cuda, plugin, x, c, g, ws, k["shape"], k["variant"], norm=k["norm"], ffn=k["ffn"])
    # the same call again: with streamed experts the slots now hold some of them
    run_and_check(torch_cuda, plugin, x, c, g, ws, k["shape"], k["variant"], norm=k["norm"], ffn=k["ffn"])
    plugin.terminate()
