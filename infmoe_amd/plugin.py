"""Python binding of the layer: the counterpart of python/infmoe/plugin.py:43-119.

`MoELayerPlugin(config).create_plugin()` marshals the configuration into the same named fields
the reference hands to TensorRT's plugin creator and returns a `Plugin` that wraps the C ABI
handle (configure / workspace_size / initialize / enqueue / terminate / destroy).  Tensors are
torch ROCm tensors used for device memory and streams only; every computation happens in
libinfmoe.so.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import numpy as np

from . import capi
from .config import MoELayerConfig

PLUGIN_INFO = {"name": "MoELayerPlugin", "version": "1"}  # python/infmoe/plugin.py:11-14


def _i32_array(values: Sequence[int]):
    return (C.c_int32 * len(values))(*values)


class Plugin:
    """Owns one infmoe_plugin handle."""

    def __init__(self, handle: int, expert_count: int, embedding_size: int):
        self._h = C.c_void_p(handle)
        self._lib = capi.load()
        self.expert_count = expert_count
        self.embedding_size = embedding_size
        self._workspace = None

    # -- lifecycle -------------------------------------------------------------------------
    def set_expert_weights(self, expert: int, key: str, array: np.ndarray) -> None:
        a = np.ascontiguousarray(array, dtype=np.float32)
        capi.check(self._lib.infmoe_set_expert_weights(self._h, expert, key.encode(), a.ctypes.data, a.size))

    def set_expert_weights_ptr(self, expert: int, key: str, host_ptr: int, count: int) -> None:
        capi.check(self._lib.infmoe_set_expert_weights(self._h, expert, key.encode(), host_ptr, count))

    def set_score_bias(self, bias: Optional[np.ndarray]) -> None:
        if bias is None:
            capi.check(self._lib.infmoe_set_score_bias(self._h, None))
        else:
            b = np.ascontiguousarray(bias, dtype=np.float32)
            assert b.size == self.expert_count
            capi.check(self._lib.infmoe_set_score_bias(self._h, b.ctypes.data))

    def configure(self, dims: Sequence[int]) -> None:
        capi.check(self._lib.infmoe_configure(self._h, _i32_array(dims), len(dims)))

    def workspace_size(self, dims: Sequence[int]) -> int:
        out = C.c_size_t(0)
        capi.check(self._lib.infmoe_workspace_size(self._h, _i32_array(dims), len(dims), C.byref(out)))
        return out.value

    def initialize(self) -> None:
        capi.check(self._lib.infmoe_initialize(self._h))

    def enqueue(self, dims: Sequence[int], input_ptr: int, output_ptr: int, workspace_ptr: int, stream: int) -> None:
        ins = (C.c_void_p * 1)(input_ptr)
        outs = (C.c_void_p * 1)(output_ptr)
        capi.check(self._lib.infmoe_enqueue(self._h, _i32_array(dims), len(dims), ins, outs, workspace_ptr, stream))

    def last_routing(self):
        count = (C.c_int32 * self.expert_count)()
        stats = (C.c_int32 * 3)()
        capi.check(self._lib.infmoe_last_routing(self._h, count, stats))
        return np.array(count[:], np.int32), dict(near_ties=stats[0], nan_rows=stats[1], rescored=stats[2])

    def last_streaming(self):
        """(experts copied host-to-device, experts served from a slot kept from an earlier call) of the last call."""
        copies, hits = C.c_int32(0), C.c_int32(0)
        capi.check(self._lib.infmoe_last_streaming(self._h, C.byref(copies), C.byref(hits)))
        return copies.value, hits.value

    PHASES = ("gating", "count_sort", "scatter", "expert_norm", "expert_gemm1", "expert_gemm2", "gather")

    def set_timing(self, enable) -> None:
        """False / 0: off.  True / 1: keep the phase marks of the last call.  n: of the last n calls."""
        capi.check(self._lib.infmoe_set_timing(self._h, int(enable)))

    def timing_history(self, max_calls: int) -> list:
        """Phase times (ms) of the last min(max_calls, kept) calls, oldest first."""
        n = len(self.PHASES)
        ms = (C.c_float * (n * max_calls))()
        got = C.c_int32(0)
        capi.check(self._lib.infmoe_timing_history(self._h, ms, max_calls, C.byref(got)))
        return [dict(zip(self.PHASES, ms[i * n:(i + 1) * n])) for i in range(got.value)]

    def last_timing(self) -> dict:
        ms = (C.c_float * len(self.PHASES))()
        capi.check(self._lib.infmoe_last_timing(self._h, ms))
        return dict(zip(self.PHASES, ms[:]))

    def clone(self) -> "Plugin":
        out = C.c_void_p()
        capi.check(self._lib.infmoe_clone(self._h, C.byref(out)))
        return Plugin(out.value, self.expert_count, self.embedding_size)

    def serialize(self) -> bytes:
        n = C.c_size_t(0)
        capi.check(self._lib.infmoe_serialization_size(self._h, C.byref(n)))
        buf = C.create_string_buffer(n.value)
        capi.check(self._lib.infmoe_serialize(self._h, buf, n.value))
        return buf.raw

    @staticmethod
    def deserialize(data: bytes, name: str = "moe_layer_plugin") -> "Plugin":
        lib = capi.load()
        out = C.c_void_p()
        capi.check(lib.infmoe_deserialize(name.encode(), data, len(data), C.byref(out)))
        E, d = np.frombuffer(data, np.int32, 2, 8)
        return Plugin(out.value, int(E), int(d))

    def terminate(self) -> None:
        capi.check(self._lib.infmoe_terminate(self._h))

    def destroy(self) -> None:
        if self._h:
            self._lib.infmoe_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass

    # -- torch convenience -----------------------------------------------------------------
    def forward(self, x, check_nan: bool = False):
        """x: torch float32 ROCm tensor [B, S, d] -> new tensor of the same shape.

        check_nan: wait for the call's routing and raise InfMoEError(ERR_NAN) if a token had no orderable
        score (a NaN in its row), as the reference asserts (plugin/cuda/moe.cu:70); costs a host wait.
        Without it such a token's output row is NaN and a later call reports the error once."""
        import torch
        assert x.is_cuda and x.dtype == torch.float32 and x.dim() == 3 and x.is_contiguous()
        dims = list(x.shape)
        need = self.workspace_size(dims)
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
        y = torch.empty_like(x)
        stream = torch.cuda.current_stream(x.device).cuda_stream
        self.enqueue(dims, x.data_ptr(), y.data_ptr(), self._workspace.data_ptr(), stream)
        if check_nan:
            _, stats = self.last_routing()
            if stats["nan_rows"] > 0:
                raise capi.InfMoEError(capi.ERR_NAN, f"{stats['nan_rows']} token(s) have no orderable score (NaN input?)")
        return y


class MoELayerPlugin:
    """Builds the field collection and creates the plugin (python/infmoe/plugin.py:43-119)."""

    def __init__(self, config: MoELayerConfig, namespace: str = "") -> None:
        self._lib = capi.load()
        if self._lib.infmoe_plugin_name().decode() != PLUGIN_INFO["name"]:
            raise RuntimeError("libinfmoe.so does not provide MoELayerPlugin")
        self.__check_config(config)
        self.__config = config

    @property
    def config(self) -> MoELayerConfig:
        return self.__config

    @staticmethod
    def __check_config(config: MoELayerConfig) -> None:
        # python/infmoe/plugin.py:77-90; the library does the remaining checks
        assert config.expert_count > 0
        assert config.seq_len > 0
        assert config.embedding_size > 0
        assert config.hidden_size > 0
        assert config.max_concurrency > 0
        assert config.max_batch_size > 0
        assert config.sublayer_type != ""
        assert config.expert_centroids is not None and config.expert_centroids.size > 0
        assert config.moe_variant != ""

    def get_layer_attributes(self):
        """List of (name, buffer, type, length) in the reference's order (python/infmoe/plugin.py:101-117)."""
        c = self.config
        keep = []

        def ints(v):
            a = np.array([v], np.int32)
            keep.append(a)
            return a.ctypes.data, capi.FIELD_INT32, 1

        def floats(v):
            a = np.ascontiguousarray(v, np.float32)
            keep.append(a)
            return a.ctypes.data, capi.FIELD_FLOAT32, a.size

        def chars(v):
            b = C.create_string_buffer(v.encode("utf-8"))
            keep.append(b)
            return C.cast(b, C.c_void_p).value, capi.FIELD_UNKNOWN, len(b.raw)

        attrs = [
            ("expert_count", *ints(c.expert_count)),
            ("embedding_size", *ints(c.embedding_size)),
            ("hidden_size", *ints(c.hidden_size)),
            ("max_concurrency", *ints(c.max_concurrency)),
            ("expert_centroids", *floats(c.expert_centroids)),
        ]
        if c.weight_file_path:
            attrs.append(("expert_weight_file", *chars(c.weight_file_path)))
        attrs += [
            ("expert_sublayer_type", *chars(c.sublayer_type)),
            ("moe_variant", *chars(c.moe_variant)),
        ]
        if c.layernorm_weight is not None:
            attrs.append(("layernorm_weight", *floats(c.layernorm_weight)))
        attrs += [("norm_kind", *chars(c.norm_kind)), ("ffn_kind", *chars(c.ffn_kind))]
        return attrs, keep

    def create_plugin(self, plugin_name: str = "moe_layer_plugin") -> Plugin:
        attrs, keep = self.get_layer_attributes()
        fields = (capi.Field * len(attrs))()
        for f, (name, ptr, typ, length) in zip(fields, attrs):
            f.name, f.data, f.type, f.length = name.encode(), ptr, typ, length
        out = C.c_void_p()
        capi.check(self._lib.infmoe_create(plugin_name.encode(), fields, len(attrs), C.byref(out)))
        del keep
        return Plugin(out.value, self.config.expert_count, self.config.embedding_size)
