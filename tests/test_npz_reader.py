"""The npz reader behind expert_weight_file (the counterpart of cnpy::npz_load,
plugin/thirdparty/cnpy/cnpy.cpp:229-276) against numpy's own writer: stored, deflated and
Fortran-ordered members, wrong shapes and dtypes, and files that are truncated or not archives.
Host memory only."""
import ctypes as C
import os
import zipfile

import numpy as np
import pytest

from infmoe_amd import capi


def read(path, name, rows, cols):
    lib = capi.load()
    out = np.full(rows * max(cols, 1), np.nan, np.float32)
    status = lib.infmoe_npz_read_f32(str(path).encode(), name.encode(), out.ctypes.data, rows, cols)
    return status, out, lib.infmoe_last_error().decode()


@pytest.fixture
def arrays():
    rng = np.random.default_rng(3)
    return {"0/layer_norm_weight": rng.standard_normal(12).astype("f"),
            "0/wi_weight": rng.standard_normal((20, 12)).astype("f"),
            "0/wo_weight": rng.standard_normal((12, 20)).astype("f")}


@pytest.mark.parametrize("compressed", [False, True])
def test_reads_what_numpy_wrote(tmp_path, arrays, compressed):
    path = tmp_path / "w.npz"
    (np.savez_compressed if compressed else np.savez)(path, **arrays)
    with zipfile.ZipFile(path) as z:  # the writer really used the method under test
        assert {i.compress_type for i in z.infolist()} == {zipfile.ZIP_DEFLATED if compressed else zipfile.ZIP_STORED}
    for name, a in arrays.items():
        rows, cols = (a.shape[0], 0) if a.ndim == 1 else a.shape
        status, got, msg = read(path, name, rows, cols)
        assert status == capi.OK, msg
        np.testing.assert_array_equal(got.reshape(a.shape), a)
        status, got, _ = read(path, name + ".npy", rows, cols)  # member names carry the suffix inside the zip
        assert status == capi.OK


@pytest.mark.parametrize("compressed", [False, True])
def test_fortran_ordered_member_is_transposed_into_c_order(tmp_path, arrays, compressed):
    # python/infmoe/config.py:52 saves w.transpose(): numpy then writes fortran_order True
    a = arrays["0/wo_weight"]
    view = np.ascontiguousarray(a.T).T
    assert view.flags.f_contiguous and not view.flags.c_contiguous
    path = tmp_path / "f.npz"
    (np.savez_compressed if compressed else np.savez)(path, **{"0/wo_weight": view})
    status, got, msg = read(path, "0/wo_weight", *a.shape)
    assert status == capi.OK, msg
    np.testing.assert_array_equal(got.reshape(a.shape), a)


def test_shape_must_match_not_only_the_count(tmp_path, arrays):
    path = tmp_path / "w.npz"
    np.savez(path, **arrays)
    status, _, msg = read(path, "0/wo_weight", 20, 12)  # same 240 floats, transposed meaning
    assert status == capi.ERR_INVALID_ARGUMENT and "(12,20,)" in msg
    status, _, _ = read(path, "0/wo_weight", 240, 0)
    assert status == capi.ERR_INVALID_ARGUMENT
    status, _, _ = read(path, "0/layer_norm_weight", 12, 1)
    assert status == capi.ERR_INVALID_ARGUMENT
    status, _, msg = read(path, "0/absent", 12, 0)
    assert status == capi.ERR_MISSING_FIELD and "0/absent" in msg


def test_other_dtypes_are_rejected(tmp_path):
    path = tmp_path / "d.npz"
    np.savez(path, a=np.zeros(4, np.float64), b=np.zeros(4, ">f4"), c=np.zeros(4, np.int32))
    for name in "abc":
        status, _, msg = read(path, name, 4, 0)
        assert status == capi.ERR_IO and "dtype" in msg


def test_files_that_are_not_archives(tmp_path, arrays):
    good = tmp_path / "w.npz"
    np.savez_compressed(good, **arrays)
    blob = good.read_bytes()
    cases = {
        "empty.npz": b"",
        "noise.npz": np.random.default_rng(0).bytes(4096),
        "head_only.npz": blob[: len(blob) // 2],           # end record cut off
        "tail_only.npz": blob[len(blob) // 2:],            # directory points before the start of the file
        "zeros_inside.npz": blob[:40] + b"\0" * 200 + blob[240:],  # member data and headers damaged
    }
    for fname, data in cases.items():
        path = tmp_path / fname
        path.write_bytes(data)
        for name, a in arrays.items():
            rows, cols = (a.shape[0], 0) if a.ndim == 1 else a.shape
            status, got, msg = read(path, name, rows, cols)
            if status == capi.OK:  # a member the damage did not reach
                assert fname == "zeros_inside.npz" and name != "0/layer_norm_weight"
                np.testing.assert_array_equal(got.reshape(a.shape), a)
            else:
                assert status in (capi.ERR_IO, capi.ERR_INVALID_ARGUMENT, capi.ERR_MISSING_FIELD), (fname, name, status, msg)
    status, _, _ = read(tmp_path / "missing.npz", "a", 1, 0)
    assert status == capi.ERR_IO
    status, _, _ = read(tmp_path, "a", 1, 0)  # a directory
    assert status == capi.ERR_IO


def test_garbage_npy_headers(tmp_path):
    """Members whose npy header lacks a key, a colon or a closing quote are refused, not crashed on."""
    def member(header_text):
        h = header_text.encode()
        h += b" " * (-(10 + len(h) + 1) % 64) + b"\n"
        return b"\x93NUMPY\x01\x00" + len(h).to_bytes(2, "little") + h + np.zeros(4, "<f4").tobytes()

    headers = [
        "{'descr': '<f4', 'fortran_order' False, 'shape': (4,), }",   # no colon
        "{'descr': '<f4', 'fortran_order':", "{'descr': '<f4",         # cut short
        "{'fortran_order': False, 'shape': (4,), }",                   # no descr
        "{'descr': '<f4', 'fortran_order': Maybe, 'shape': (4,), }",
        "{'descr': '<f4', 'fortran_order': False, 'shape': 4, }",      # no tuple
        "{'descr': '<f4', 'fortran_order': False, 'shape': (4, }",
        "",
    ]
    for i, text in enumerate(headers):
        path = tmp_path / f"h{i}.npz"
        with zipfile.ZipFile(path, "w") as z:
            z.writestr("a.npy", member(text))
        status, _, msg = read(path, "a", 4, 0)
        assert status == capi.ERR_IO, (text, status, msg)
    path = tmp_path / "ok.npz"
    with zipfile.ZipFile(path, "w") as z:
        z.writestr("a.npy", member("{'descr': '<f4', 'fortran_order': False, 'shape': (4,), }"))
    assert read(path, "a", 4, 0)[0] == capi.OK
    with zipfile.ZipFile(tmp_path / "bomb.npz", "w") as z:  # header promises more data than the member holds
        z.writestr("a.npy", member("{'descr': '<f4', 'fortran_order': False, 'shape': (400,), }"))
    assert read(tmp_path / "bomb.npz", "a", 400, 0)[0] == capi.ERR_IO
