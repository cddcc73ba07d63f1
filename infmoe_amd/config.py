"""Layer configuration of the Python binding.

The field names and their order are the reference's (python/infmoe/config.py:9-25), because scripts
written against it construct the dataclass by keyword or position; `norm_kind` and `ffn_kind` are the
two explicit switches of this build.  The helpers that fill a configuration with synthetic tensors
keep the reference's method names and array layouts (centroids [E][d], input-side matrices [h][d],
wo [d][h], npz members "<expert>/<key>", README.md:121) but draw from a seeded generator, give every
expert its own values, and scale by 1/fan_in so that a layer built from them computes finite numbers.
"""
from __future__ import annotations

import pathlib
import warnings
from dataclasses import dataclass, field
from typing import Dict, Iterator, Optional, Tuple

import numpy as np

_KEYS = {
    "relu": ("layer_norm_weight", "wi_weight", "wo_weight"),
    "gated_gelu": ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight"),
}


@dataclass
class MoELayerConfig:
    seq_len: int
    expert_count: int
    embedding_size: int
    hidden_size: int
    max_concurrency: int
    moe_variant: str
    sublayer_type: str
    max_batch_size: int
    expert_centroids: Optional[np.ndarray] = None   # [expert_count, embedding_size]
    layernorm_weight: Optional[np.ndarray] = None   # [embedding_size], required for cpm_2
    weight_file_path: str = ""
    norm_kind: str = "rms"          # "rms" | "centered"
    ffn_kind: str = "relu"          # "relu" (wi, wo) | "gated_gelu" (wi_0, wi_1, wo)
    seed: int = field(default=0, repr=False)  # of the generators below

    def _rng(self, stream: int) -> np.random.Generator:
        return np.random.default_rng(np.random.SeedSequence(entropy=self.seed, spawn_key=(stream,)))

    def generate_random_centroids(self) -> None:
        shape = (self.expert_count, self.embedding_size)
        self.expert_centroids = self._rng(1).random(shape, dtype=np.float32)

    def generate_random_layernorm_weight(self) -> None:
        self.layernorm_weight = self._rng(2).random(self.embedding_size, dtype=np.float32)

    def weight_keys(self) -> Tuple[str, ...]:
        return _KEYS[self.ffn_kind]

    def expert_arrays(self, expert: int) -> Iterator[Tuple[str, np.ndarray]]:
        """(npz member name, array) of one expert, in slot order."""
        d, h = self.embedding_size, self.hidden_size
        rng = self._rng(100 + expert)
        for key in self.weight_keys():
            if key == "layer_norm_weight":
                value = rng.random(d, dtype=np.float32)
            elif key == "wo_weight":
                value = rng.random((d, h), dtype=np.float32) / np.float32(h)
            else:
                value = rng.random((h, d), dtype=np.float32) / np.float32(d)
            yield f"{expert}/{key}", value

    def generate_random_weight_file(self, weight_path: str, overwrite: bool) -> None:
        """Writes the experts' arrays to `weight_path` (.npz) and points the configuration at it.
        An existing file is kept, with a warning, unless `overwrite`."""
        target = pathlib.Path(weight_path)
        if target.is_file() and not overwrite:
            warnings.warn(f"{target} is already there and is used as it is (pass overwrite=True to replace it)")
        else:
            members: Dict[str, np.ndarray] = {}
            for expert in range(self.expert_count):
                members.update(self.expert_arrays(expert))
            with open(target, "wb") as out:  # np.savez would append ".npz" to a name without it
                np.savez(out, **members)
        self.weight_file_path = str(target)
