"""The npz reader under AddressSanitizer + UndefinedBehaviorSanitizer on damaged archives (host code only, no
GPU): tests/npz_sanitize/harness.cpp is compiled with g++ together with infmoe_amd/csrc/npz_reader.cpp and fed a
corpus made here - sound archives (stored, deflated, Fortran order), then each with bytes flipped, zeroed,
truncated or with its length fields overwritten.  Every file has to be answered with a status."""
import io
import os
import shutil
import subprocess
import zipfile

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
ROWS, COLS = 6, 10


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.fail("g++ is needed to build the sanitizer harness")
    exe = str(tmp_path_factory.mktemp("npz_sanitize") / "harness")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-static-libasan", "-static-libubsan",  # the runtimes inside the program, whatever else the process loads first
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", f"-I{ROOT}/include", f"-I{ROOT}/infmoe_amd/csrc",
           os.path.join(HERE, "npz_sanitize", "harness.cpp"), os.path.join(ROOT, "infmoe_amd", "csrc", "npz_reader.cpp"),
           "-lz", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def archives():
    rng = np.random.default_rng(12)
    members = {"0/wi_weight": rng.standard_normal((ROWS, COLS)).astype(np.float32),
               "0/wo_weight": np.asfortranarray(rng.standard_normal((COLS, ROWS)).astype(np.float32)),
               "0/layer_norm_weight": rng.standard_normal(ROWS).astype(np.float32),
               "0/other_type": np.arange(ROWS * COLS, dtype=np.float64).reshape(ROWS, COLS)}
    out = []
    for save in (np.savez, np.savez_compressed):
        buf = io.BytesIO()
        save(buf, **members)
        out.append(buf.getvalue())
    # an archive whose members carry no sizes in their local headers (a zip written as a stream)
    buf = io.BytesIO()
    with zipfile.ZipFile(buf, "w", zipfile.ZIP_DEFLATED) as z:
        for k, v in members.items():
            with z.open(k + ".npy", "w", force_zip64=True) as f:
                np.lib.format.write_array(f, v)
    out.append(buf.getvalue())
    return out


def mutants(blob, rng, n):
    size = len(blob)
    for _ in range(n):
        b = bytearray(blob)
        kind = rng.integers(0, 6)
        if kind == 0:    # a few flipped bytes anywhere
            for p in rng.integers(0, size, rng.integers(1, 8)):
                b[p] ^= int(rng.integers(1, 256))
        elif kind == 1:  # truncated
            b = b[:rng.integers(0, size)]
        elif kind == 2:  # a zeroed stretch
            p = int(rng.integers(0, size))
            b[p:p + int(rng.integers(1, 64))] = bytes(min(int(rng.integers(1, 64)), size - p))
        elif kind == 3:  # damage near the end: end-of-central-directory and central directory
            for p in rng.integers(max(0, size - 400), size, rng.integers(1, 6)):
                b[p] = int(rng.integers(0, 256))
        elif kind == 4:  # a 32-bit field set to an extreme value, anywhere 4-aligned or not
            p = int(rng.integers(0, max(1, size - 4)))
            b[p:p + 4] = [(0xff, 0xff, 0xff, 0xff), (0xff, 0xff, 0xff, 0x7f), (0, 0, 0, 0x80), (1, 0, 0, 0)][int(rng.integers(0, 4))]
        else:            # damage inside an npy header (shape, descr, fortran_order text)
            at = blob.find(b"'shape'")
            if at > 0:
                for p in rng.integers(at - 40, at + 40, rng.integers(1, 4)):
                    b[p] = int(rng.integers(32, 127))
        yield bytes(b)


def test_reader_answers_damaged_archives_with_a_status(harness, tmp_path):
    rng = np.random.default_rng(99)
    paths = []
    sound = archives()
    for i, blob in enumerate(sound):
        p = tmp_path / f"sound{i}.npz"
        p.write_bytes(blob)
        paths.append(str(p))
    for i, blob in enumerate(sound):
        for j, m in enumerate(mutants(blob, rng, 250)):
            p = tmp_path / f"m{i}_{j}.npz"
            p.write_bytes(m)
            paths.append(str(p))
    (tmp_path / "empty.npz").write_bytes(b"")
    paths.append(str(tmp_path / "empty.npz"))
    paths.append(str(tmp_path / "missing.npz"))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([harness, str(ROWS), str(COLS), *paths], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-4000:]
    lines = r.stdout.strip().splitlines()
    assert len(lines) == len(paths)
    # the sound archives: four members each; wi reads as (ROWS, COLS), wo (Fortran order) as (COLS, ROWS), gamma as (ROWS,)
    for line in lines[:len(sound)]:
        assert line.split() == ["0", "4", "3"], line
    assert lines[-1].split()[0] != "0" and lines[-2].split()[0] != "0"
    rejected = sum(1 for line in lines[len(sound):] if line.split()[0] != "0")
    assert 0 < rejected < len(lines)  # some damage is fatal to the archive, some only to a member
