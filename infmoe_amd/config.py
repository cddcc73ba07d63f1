"""Layer configuration: same fields as the reference's dataclass
(python/infmoe/config.py:9-25) plus the explicit norm / FFN kinds of this build."""
from __future__ import annotations

import os
import sys
from dataclasses import dataclass
from typing import Optional

import numpy as np


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

    def generate_random_centroids(self) -> None:
        # python/infmoe/config.py:27-28
        self.expert_centroids = np.random.rand(self.expert_count, self.embedding_size).astype("f")

    def generate_random_layernorm_weight(self) -> None:
        # python/infmoe/config.py:30-31
        self.layernorm_weight = np.random.rand(self.embedding_size).astype("f")

    def weight_keys(self):
        if self.ffn_kind == "gated_gelu":
            return ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight")
        return ("layer_norm_weight", "wi_weight", "wo_weight")

    def generate_random_weight_file(self, weight_path: str, overwrite: bool) -> None:
        """npz with members '<n>/<key>' (python/infmoe/config.py:33-54, README.md:121).
        Input-side matrices are [hidden, embedding], wo is [embedding, hidden]."""
        if os.path.isfile(weight_path):
            if overwrite:
                os.remove(weight_path)
            else:
                print(f"WARNING: weight file to generate exists: {weight_path}", file=sys.stderr)
                self.weight_file_path = weight_path
                return
        weights = {}
        d, h = self.embedding_size, self.hidden_size
        for i in range(self.expert_count):
            for key in self.weight_keys():
                if key == "layer_norm_weight":
                    w = np.random.rand(d)
                elif key == "wo_weight":
                    w = np.random.rand(d, h) / h
                else:
                    w = np.random.rand(h, d) / d
                weights[f"{i}/{key}"] = w.astype("f")
        np.savez(weight_path, **weights)
        self.weight_file_path = weight_path
