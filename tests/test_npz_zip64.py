"""The npz reader on archives of the size real expert files have (plugin/thirdparty/cnpy/cnpy.cpp:179-189,229-276
read such files whole): more members than the 16-bit count of the plain end record holds, and members that
start beyond 4 GiB - the zip64 end record, its locator, and 64-bit offsets in the central directory.  The large
members are zeros written as holes (tests/npz_large.py); host memory only."""
import os
import shutil
import zipfile

import numpy as np
import pytest

from infmoe_amd import capi
from tests.npz_large import write_npz
from tests.test_npz_reader import read


def test_more_members_than_the_short_end_record_counts(tmp_path):
    """70 000 small members: zipfile has to write the zip64 end record and its locator (the 16-bit member count
    of the plain record reads 0xFFFF); the first, the last and one in the middle are read back."""
    path = tmp_path / "many.npz"
    rng = np.random.default_rng(5)
    picks = {0: rng.standard_normal(7).astype("f"), 34567: rng.standard_normal((3, 5)).astype("f"),
             69999: rng.standard_normal(11).astype("f")}
    tiny = np.zeros(1, np.float32)
    write_npz(path, ((f"{i}/layer_norm_weight", picks.get(i, tiny)) for i in range(70000)))
    with zipfile.ZipFile(path) as z:
        assert len(z.infolist()) == 70000
    with open(path, "rb") as f:  # the archive really ends in a zip64 end record + locator + plain end record
        f.seek(-(22 + 20), os.SEEK_END)
        assert f.read(4) == b"PK\x06\x07"
    for i, a in picks.items():
        rows, cols = (a.shape[0], 0) if a.ndim == 1 else a.shape
        status, got, msg = read(path, f"{i}/layer_norm_weight", rows, cols)
        assert status == capi.OK, msg
        np.testing.assert_array_equal(got.reshape(a.shape), a)
    status, _, msg = read(path, "70000/layer_norm_weight", 1, 0)
    assert status == capi.ERR_MISSING_FIELD


def test_members_beyond_four_gib(tmp_path):
    """An archive of 4.4 GB: one member of zeros that alone exceeds 4 GiB (its sizes live in the zip64 extra field),
    then members whose local headers start beyond 4 GiB (64-bit offsets in the central directory, which itself lies
    beyond 4 GiB, so the end record is the zip64 one)."""
    if shutil.disk_usage(tmp_path).free < (1 << 30):
        pytest.skip("less than 1 GiB free under the temporary directory")
    path = tmp_path / "big.npz"
    rng = np.random.default_rng(6)
    wi = rng.standard_normal((24, 40)).astype("f")
    wo = rng.standard_normal((40, 24)).astype("f")
    head = rng.standard_normal(9).astype("f")
    big = (1100, 1 << 20)  # 4.4e9 bytes of float32 zeros
    write_npz(path, [("0/layer_norm_weight", head), ("0/wi_weight", big), ("1/wi_weight", wi), ("1/wo_weight", wo)])
    assert os.path.getsize(path) > (1 << 32) + (1 << 27)
    assert os.stat(path).st_blocks * 512 < (1 << 28), "the zeros were meant to be holes"
    with zipfile.ZipFile(path) as z:
        info = {i.filename: i for i in z.infolist()}
        assert info["1/wi_weight.npy"].header_offset > (1 << 32) and info["0/wi_weight.npy"].file_size > (1 << 32)
    for name, a in (("0/layer_norm_weight", head), ("1/wi_weight", wi), ("1/wo_weight", wo)):
        rows, cols = (a.shape[0], 0) if a.ndim == 1 else a.shape
        status, got, msg = read(path, name, rows, cols)
        assert status == capi.OK, msg
        np.testing.assert_array_equal(got.reshape(a.shape), a)
    # the member of more than 4 GiB itself: its shape is checked against the caller's before anything is read
    status, _, msg = read(path, "0/wi_weight", 8, 8)
    assert status == capi.ERR_INVALID_ARGUMENT, msg
