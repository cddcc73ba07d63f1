"""Host logic of the C ABI that needs no GPU: exported symbols, attribute parsing and its error
codes (the reference asserts or exits in each of these cases), shapes, workspace sizing,
serialisation.  No compute entry point is called here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin, Plugin, capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "infmoe.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(infmoe_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    lib = capi.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/infmoe.h but not exported"
    assert declared == set(capi.PROTOTYPES), declared ^ set(capi.PROTOTYPES)
    assert lib.infmoe_plugin_name() == b"MoELayerPlugin" and lib.infmoe_plugin_version() == b"1"


def fields(**kw):
    """Build an infmoe_field array from python values; returns (array, n, keepalive)."""
    keep, items = [], []
    for name, v in kw.items():
        if isinstance(v, int):
            a = np.array([v], np.int32)
            items.append((name, a.ctypes.data, capi.FIELD_INT32, 1))
        elif isinstance(v, str):
            a = C.create_string_buffer(v.encode())
            items.append((name, C.cast(a, C.c_void_p).value, capi.FIELD_UNKNOWN, len(a.raw)))
        else:
            a = np.ascontiguousarray(v, np.float32)
            items.append((name, a.ctypes.data, capi.FIELD_FLOAT32, a.size))
        keep.append(a)
    arr = (capi.Field * len(items))()
    for f, (name, ptr, typ, n) in zip(arr, items):
        f.name, f.data, f.type, f.length = name.encode(), ptr, typ, n
    return arr, len(items), keep


GOOD = dict(expert_count=4, embedding_size=8, hidden_size=16, max_concurrency=2,
            expert_centroids=np.zeros(32, np.float32), expert_sublayer_type="T5_FF", moe_variant="default")


def create(**kw):
    lib = capi.load()
    arr, n, keep = fields(**kw)
    out = C.c_void_p()
    status = lib.infmoe_create(b"layer", arr, n, C.byref(out))
    return status, out, lib.infmoe_last_error().decode()


def test_create_ok_and_destroy():
    status, h, _ = create(**GOOD)
    assert status == capi.OK and h.value
    capi.load().infmoe_destroy(h)


@pytest.mark.parametrize("change,expected", [
    (dict(bogus_field=1), capi.ERR_UNKNOWN_FIELD),                      # MoELayerPluginCreator.cc:111-114
    (dict(expert_centroids=np.zeros(31, np.float32)), capi.ERR_INVALID_ARGUMENT),  # :122
    (dict(moe_variant="cpm_2"), capi.ERR_MISSING_FIELD),                # MoELayerPlugin.cc:76-79
    (dict(moe_variant="switch"), capi.ERR_UNSUPPORTED),                 # MoELayerPlugin.cc:53-56
    (dict(expert_sublayer_type="Conv"), capi.ERR_UNSUPPORTED),          # MoELayerPlugin.cc:37-40
    (dict(expert_weight_file="/nonexistent/w.npz"), capi.ERR_IO),       # MoELayerPluginCreator.cc:132-136
    (dict(expert_weight_file="/tmp"), capi.ERR_IO),                     # :137-140 not a regular file
    (dict(layernorm_weight=np.ones(7, np.float32)), capi.ERR_INVALID_ARGUMENT),  # :126-128
    (dict(max_concurrency=0), capi.ERR_INVALID_ARGUMENT),               # :121
    (dict(norm_kind="batch"), capi.ERR_UNSUPPORTED),
    (dict(ffn_kind="swiglu"), capi.ERR_UNSUPPORTED),
])
def test_create_rejects_bad_attributes(change, expected):
    status, h, msg = create(**{**GOOD, **change})
    assert status == expected, msg
    assert not h.value and msg


@pytest.mark.parametrize("missing", ["expert_count", "embedding_size", "hidden_size", "expert_centroids",
                                     "expert_sublayer_type", "moe_variant"])
def test_create_requires_fields(missing):
    kw = {k: v for k, v in GOOD.items() if k != missing}
    status, h, msg = create(**kw)
    assert status == capi.ERR_MISSING_FIELD, msg  # MoELayerPluginCreator.cc:118-125


def test_max_concurrency_defaults_to_two():
    lib = capi.load()
    dims = (C.c_int32 * 3)(2, 5, 8)
    sizes = []
    for kw in (GOOD, {k: v for k, v in GOOD.items() if k != "max_concurrency"}):
        status, h, msg = create(**kw)
        assert status == capi.OK, msg
        out = C.c_size_t()
        assert lib.infmoe_workspace_size(h, dims, 3, C.byref(out)) == capi.OK
        sizes.append(out.value)
        lib.infmoe_destroy(h)
    assert sizes[0] == sizes[1]  # MoELayerPluginCreator.cc:65


def test_configure_and_workspace_shape_checks():
    lib = capi.load()
    status, h, _ = create(**GOOD)
    assert lib.infmoe_configure(h, (C.c_int32 * 2)(3, 8), 2) == capi.ERR_INVALID_ARGUMENT  # MoELayerPlugin.cc:176
    assert lib.infmoe_configure(h, (C.c_int32 * 3)(3, 5, 9), 3) == capi.ERR_INVALID_ARGUMENT  # :177
    assert lib.infmoe_configure(h, (C.c_int32 * 3)(3, 5, 8), 3) == capi.OK
    out = C.c_size_t()
    assert lib.infmoe_workspace_size(h, (C.c_int32 * 3)(3, 5, 9), 3, C.byref(out)) == capi.ERR_INVALID_ARGUMENT
    lib.infmoe_destroy(h)


def workspace(kw, dims):
    lib = capi.load()
    status, h, msg = create(**kw)
    assert status == capi.OK, msg
    out = C.c_size_t()
    assert lib.infmoe_workspace_size(h, (C.c_int32 * 3)(*dims), 3, C.byref(out)) == capi.OK
    lib.infmoe_destroy(h)
    return out.value


def test_workspace_size_accounting():
    E, d, h = 4, 8, 16
    slot = 4 * (d + 2 * d * h)
    streamed = workspace(GOOD, (2, 50, d))
    resident = workspace({**GOOD, "max_concurrency": E}, (2, 50, d))
    # the weight slots of streamed experts and the resident experts are both memory of the layer (the reference
    # carves the slots from the workspace, MoELayerPlugin.cc:243-264; slots that keep experts between calls
    # cannot live in memory the caller may hand to others between calls)
    assert streamed == resident and slot > 0
    T = 100
    floor = 4 * (T * (d + h) + 3 * T + 2 * T + 2 * T * d)  # sub-layer scratch, sel/pos/rowExpert, coeffs, routed+post
    assert floor <= resident <= floor + 64 * 256
    assert workspace({**GOOD, "max_concurrency": E}, (2, 100, d)) > resident
    gated = workspace({**GOOD, "ffn_kind": "gated_gelu"}, (2, 50, d))
    assert gated == streamed  # one hidden buffer in either form: the gelu*mul product is formed in the GEMM epilogue
    ident = workspace({**GOOD, "expert_sublayer_type": "Identity"}, (2, 50, d))
    assert ident < resident


def test_set_expert_weights_validates_before_touching_the_device():
    lib = capi.load()
    status, h, _ = create(**GOOD)
    w = np.zeros(8 * 16, np.float32)
    p = w.ctypes.data
    assert lib.infmoe_set_expert_weights(h, 9, b"wi_weight", p, w.size) == capi.ERR_INVALID_ARGUMENT
    assert lib.infmoe_set_expert_weights(h, 0, b"wi_0_weight", p, w.size) == capi.ERR_UNKNOWN_FIELD  # relu layer
    assert lib.infmoe_set_expert_weights(h, 0, b"wi_weight", p, w.size - 1) == capi.ERR_INVALID_ARGUMENT  # T5FFLayer.cc:69
    assert lib.infmoe_set_expert_weights(h, 0, b"wi_weight", None, w.size) == capi.ERR_INVALID_ARGUMENT
    lib.infmoe_destroy(h)
    status, h, _ = create(**{**GOOD, "expert_sublayer_type": "Identity"})
    assert lib.infmoe_set_expert_weights(h, 0, b"wi_weight", p, w.size) == capi.ERR_UNSUPPORTED
    lib.infmoe_destroy(h)


def test_enqueue_before_initialize_and_null_handle():
    lib = capi.load()
    status, h, _ = create(**GOOD)
    dims = (C.c_int32 * 3)(1, 2, 8)
    ins, outs = (C.c_void_p * 1)(256), (C.c_void_p * 1)(512)
    assert lib.infmoe_enqueue(h, dims, 3, ins, outs, 1024, None) == capi.ERR_STATE
    assert lib.infmoe_enqueue(None, dims, 3, ins, outs, 1024, None) == capi.ERR_INVALID_ARGUMENT
    assert lib.infmoe_last_routing(h, None, None) == capi.ERR_STATE
    lib.infmoe_destroy(h)


def test_serialization_round_trip_and_rejects_garbage():
    rng = np.random.default_rng(0)
    cfg = MoELayerConfig(seq_len=5, expert_count=3, embedding_size=8, hidden_size=12, max_concurrency=2,
                         moe_variant="cpm_2", sublayer_type="T5_FF", max_batch_size=2,
                         expert_centroids=rng.standard_normal((3, 8)).astype("f"),
                         layernorm_weight=rng.standard_normal(8).astype("f"), norm_kind="centered", ffn_kind="gated_gelu")
    p = MoELayerPlugin(cfg).create_plugin()
    blob = p.serialize()
    q = Plugin.deserialize(blob)
    assert q.serialize() == blob
    assert q.workspace_size([2, 5, 8]) == p.workspace_size([2, 5, 8])
    head = np.frombuffer(blob, np.int32, 9)
    assert list(head[2:8]) == [3, 8, 12, 2, capi.NORM_CENTERED, capi.FFN_GATED_GELU] and head[8] == 1
    assert np.array_equal(np.frombuffer(blob, np.float32)[-8:], cfg.layernorm_weight)
    lib = capi.load()
    out = C.c_void_p()
    assert lib.infmoe_deserialize(b"x", blob[:40], 40, C.byref(out)) == capi.ERR_INVALID_ARGUMENT
    assert lib.infmoe_deserialize(b"x", b"\0" * len(blob), len(blob), C.byref(out)) == capi.ERR_INVALID_ARGUMENT
    assert lib.infmoe_deserialize(b"x", blob[:-4], len(blob) - 4, C.byref(out)) == capi.ERR_INVALID_ARGUMENT
    for word, value in ((6, 7), (7, -1), (12, 5)):  # norm kind, ffn kind, number of centroid floats
        bad = np.frombuffer(blob, np.int32).copy()
        bad[word] = value
        assert lib.infmoe_deserialize(b"x", bad.tobytes(), bad.nbytes, C.byref(out)) != capi.OK


def test_binding_marshals_reference_field_names():
    cfg = MoELayerConfig(seq_len=4, expert_count=2, embedding_size=4, hidden_size=8, max_concurrency=2,
                         moe_variant="cpm_2", sublayer_type="T5_FF", max_batch_size=1)
    cfg.generate_random_centroids()
    cfg.generate_random_layernorm_weight()
    assert cfg.expert_centroids.shape == (2, 4)  # [E][d], python/infmoe/config.py:27-28
    attrs, keep = MoELayerPlugin(cfg).get_layer_attributes()
    names = [a[0] for a in attrs]
    assert names[:5] == ["expert_count", "embedding_size", "hidden_size", "max_concurrency", "expert_centroids"]
    assert {"expert_sublayer_type", "moe_variant", "layernorm_weight"} <= set(names)


def test_generated_weight_file_has_reference_key_names(tmp_path):
    cfg = MoELayerConfig(seq_len=4, expert_count=2, embedding_size=4, hidden_size=8, max_concurrency=2,
                         moe_variant="default", sublayer_type="T5_FF", max_batch_size=1, ffn_kind="gated_gelu")
    path = os.path.join(tmp_path, "w.npz")
    cfg.generate_random_weight_file(path, overwrite=True)
    with np.load(path) as z:
        assert set(z.files) == {f"{e}/{k}" for e in range(2)
                                for k in ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight")}  # README.md:121
        assert z["0/wi_0_weight"].shape == (8, 4) and z["1/wo_weight"].shape == (4, 8)


def test_header_is_plain_c_and_usable_without_hip_headers(tmp_path):
    """include/infmoe.h compiles as C99 (-pedantic, no HIP or C++ headers on the include path) and a C program
    linked against libinfmoe.so drives the host side of the life cycle: tests/c_abi/use_from_c.c."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    assert gcc is not None, "gcc is needed for this test"
    capi.load()  # fails loudly when the library has not been built
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib_dir = os.path.join(root, "infmoe_amd", "lib")
    exe = str(tmp_path / "use_from_c")
    r = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I" + os.path.join(root, "include"),
                        os.path.join(root, "tests", "c_abi", "use_from_c.c"), "-L" + lib_dir, "-linfmoe",
                        "-Wl,-rpath," + lib_dir, "-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    first, second = r.stdout.strip().splitlines()
    assert first.startswith("name=MoELayerPlugin version=1 workspace=")
    assert f"bad_dims_status={capi.ERR_INVALID_ARGUMENT} " in first and "expected embedding_size = 64" in first
    assert second == f"bad_variant_status={capi.ERR_UNSUPPORTED}"


@pytest.mark.parametrize("E,d,h,variant,tmax", [
    (32, 4096, 10240, "cpm_2", 9000),     # the headline layer: the gating cuts d into more slices for fewer tokens
    (64, 2048, 8192, "base_layer", 18000),
    (4, 64, 256, "default", 3000),
    (128, 1024, 512, "default", 5000),
    (7, 384, 96, "cpm_2", 3000),
])
def test_workspace_size_never_shrinks_as_tokens_grow(E, d, h, variant, tmax):
    """A caller sizes ONE workspace for its largest batch (getWorkspaceSize, plugin/MoELayerPlugin.cc:253-273) and
    then calls with any smaller batch; enqueue lays the blocks out from the call's own token count, so the size has
    to be non-decreasing in the token count or a smaller batch would be laid out past the end of the buffer."""
    lib = capi.load()
    kw = dict(expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=E,
              expert_centroids=np.zeros(E * d, np.float32), expert_sublayer_type="T5_FF", moe_variant=variant)
    if variant == "cpm_2":
        kw["layernorm_weight"] = np.ones(d, np.float32)
    for ffn in ("relu", "gated_gelu"):
        status, hnd, msg = create(**kw, ffn_kind=ffn)
        assert status == capi.OK, msg
        out = C.c_size_t()
        prev, worst = 0, 0
        for t in range(0, tmax + 1):
            assert lib.infmoe_workspace_size(hnd, (C.c_int32 * 3)(1, t, d), 3, C.byref(out)) == capi.OK
            worst = max(worst, prev - out.value)
            prev = max(prev, out.value)
        lib.infmoe_destroy(hnd)
        assert worst == 0, f"a smaller batch needs up to {worst} bytes more than a larger one"
