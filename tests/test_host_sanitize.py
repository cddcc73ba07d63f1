"""The library's host code under AddressSanitizer + UndefinedBehaviorSanitizer, fed damaged serialised layers
(no GPU needed).  tests/host_sanitize/harness.cpp is compiled with g++ together with the library's own .cpp
files and linked with the device objects of the normal build; infmoe_deserialize then parses 1200 blobs - sound
ones of four layer kinds, and each with bytes flipped, truncated, zeroed or its length fields overwritten."""
import glob
import os
import shutil
import subprocess

import numpy as np
import pytest

from infmoe_amd import MoELayerConfig, MoELayerPlugin, capi

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "infmoe_amd", "csrc")


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    gxx = shutil.which("g++")
    assert gxx is not None, "g++ is needed to build the sanitizer harness"
    device_objects = sorted(glob.glob(os.path.join(CSRC, "build", "kernels_*.hip.o")))
    if not device_objects:
        pytest.fail("no device objects under infmoe_amd/csrc/build: build the library first (python -m infmoe_amd.build)")
    exe = str(tmp_path_factory.mktemp("host_sanitize") / "harness")
    host = [os.path.join(CSRC, f) for f in ("c_api.cpp", "moe_layer.cpp", "npz_reader.cpp", "sublayers/sublayer.cpp",
                                            "sublayers/t5ff_layer.cpp")]
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-static-libasan", "-static-libubsan", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", f"-I{ROOT}/include",
           f"-I{CSRC}", os.path.join(HERE, "host_sanitize", "harness.cpp"), *host, *device_objects,
           "-L/opt/rocm/lib", "-lamdhip64", "-lz", "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def sound_blobs():
    rng = np.random.default_rng(3)
    out = []
    for variant, sub, norm, ffn, E, d in (("cpm_2", "T5_FF", "rms", "relu", 4, 64), ("base_layer", "T5_FF", "centered", "gated_gelu", 3, 32),
                                          ("default", "Identity", "rms", "relu", 130, 8), ("cpm_2", "T5_FF", "centered", "relu", 1, 4)):
        cfg = MoELayerConfig(seq_len=8, expert_count=E, embedding_size=d, hidden_size=2 * d, max_concurrency=2,
                             moe_variant=variant, sublayer_type=sub, max_batch_size=2,
                             expert_centroids=rng.standard_normal((E, d)).astype(np.float32),
                             layernorm_weight=np.ones(d, np.float32) if variant == "cpm_2" else None,
                             norm_kind=norm, ffn_kind=ffn)
        plugin = MoELayerPlugin(cfg).create_plugin()
        out.append(plugin.serialize())
        plugin.destroy()
    return out


def mutants(blob, rng, n):
    size = len(blob)
    for _ in range(n):
        b = bytearray(blob)
        kind = rng.integers(0, 5)
        if kind == 0:    # a few flipped bytes anywhere
            for p in rng.integers(0, size, rng.integers(1, 6)):
                b[p] ^= int(rng.integers(1, 256))
        elif kind == 1:  # truncated, or with a tail added
            b = b[:rng.integers(0, size)] if rng.integers(0, 4) else b + bytes(rng.integers(1, 64))
        elif kind == 2:  # damage in the header words (sizes, counts, string lengths)
            for p in rng.integers(0, min(size, 64), rng.integers(1, 4)):
                b[p] = int(rng.integers(0, 256))
        elif kind == 3:  # a 32-bit field set to an extreme value
            p = int(rng.integers(0, max(1, min(size, 96) - 4)))
            b[p:p + 4] = [(0xff, 0xff, 0xff, 0xff), (0xff, 0xff, 0xff, 0x7f), (0, 0, 0, 0x80), (0, 0, 0, 0)][int(rng.integers(0, 4))]
        else:            # a zeroed stretch
            p = int(rng.integers(0, size))
            b[p:p + 32] = bytes(min(32, size - p))
        yield bytes(b)


def test_deserialize_answers_damaged_blobs_with_a_status(harness, tmp_path):
    rng = np.random.default_rng(17)
    sound = sound_blobs()
    paths = []
    for i, blob in enumerate(sound):
        p = tmp_path / f"sound{i}.bin"
        p.write_bytes(blob)
        paths.append(str(p))
    for i, blob in enumerate(sound):
        for j, m in enumerate(mutants(blob, rng, 300)):
            p = tmp_path / f"m{i}_{j}.bin"
            p.write_bytes(m)
            paths.append(str(p))
    (tmp_path / "empty.bin").write_bytes(b"")
    paths.append(str(tmp_path / "empty.bin"))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([harness, *paths], capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0 and "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-4000:]
    lines = r.stdout.strip().splitlines()
    assert len(lines) == len(paths)
    for blob, line in zip(sound, lines):  # a sound blob comes back and re-serialises to the same number of bytes
        assert line.split() == [str(capi.OK), str(len(blob))], line
    assert lines[-1].split()[0] != str(capi.OK)
    rejected = sum(1 for line in lines[len(sound):] if line.split()[0] != str(capi.OK))
    assert rejected > len(lines) // 3  # most damage is noticed (a flipped bit inside a centroid is not damage)


def test_create_answers_odd_field_collections_with_a_status(harness):
    """4000 field collections (fields missing, doubled, unknown, empty, null, of the wrong type, sizes that do not fit
    each other) through infmoe_create and, where a layer comes back, through the host side of its life cycle."""
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([harness, "--create", "7", "4000"], capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0 and "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, (r.stdout[-500:], r.stderr[-4000:])
    accepted = int(r.stdout.strip().split()[-1])
    assert 200 < accepted < 3800  # both outcomes are exercised
