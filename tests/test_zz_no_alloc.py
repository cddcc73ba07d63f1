"""infmoe_expert_count_noalloc (scratch in a device array of the library, nothing allocated) against
infmoe_expert_count (caller-supplied scratch) and the oracle: bit-exact, on calls in a row that share
the array, a later one smaller than an earlier one."""
import numpy as np
import pytest

from infmoe_amd import capi
from oracle import moe_oracle as O
from tests.gpu_util import dev, stream_ptr

pytestmark = pytest.mark.gpu

MAX_INTS = 65536  # INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS


def draw_sel(T, E, seed):
    rng = np.random.default_rng(seed)
    p = np.arange(1, E + 1) ** -0.7
    return rng.choice(E, size=T, p=p / p.sum()).astype(np.int32)


def run_both(lib, torch, sel, E):
    T = len(sel)
    dsel = dev(torch, sel)
    outs = []
    for noalloc in (False, True):
        pos = torch.full((T,), -1, dtype=torch.int32, device="cuda")
        count = torch.full((E,), -1, dtype=torch.int32, device="cuda")
        offset = torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")
        if noalloc:
            capi.check(lib.infmoe_expert_count_noalloc(T, E, dsel.data_ptr(), pos.data_ptr(), count.data_ptr(),
                                                       offset.data_ptr(), stream_ptr(torch)))
        else:
            scratch = torch.empty(max(lib.infmoe_expert_count_scratch_bytes(T, E), 1), dtype=torch.uint8, device="cuda")
            capi.check(lib.infmoe_expert_count(T, E, dsel.data_ptr(), pos.data_ptr(), count.data_ptr(),
                                               offset.data_ptr(), scratch.data_ptr(), stream_ptr(torch)))
        torch.cuda.synchronize()
        outs.append((count.cpu().numpy(), offset.cpu().numpy(), pos.cpu().numpy()))
    return outs


def test_noalloc_matches_scratch_entry_point_on_calls_in_a_row(lib, torch_cuda):
    torch = torch_cuda
    # large first (many blocks leave their histograms in the array), then smaller ones, then large again
    for T, E, seed in [(40000, 64, 1), (3000, 32, 2), (700, 32, 3), (1, 5, 4), (16384, 64, 5)]:
        sel = draw_sel(T, E, seed)
        print(f"noalloc case T={T} E={E} seed={seed}", flush=True)
        with_scratch, static = run_both(lib, torch, sel, E)
        want = O.expert_count(sel, E)
        for got_a, got_b, w, name in zip(with_scratch, static, want, ("count", "offset", "pos")):
            np.testing.assert_array_equal(got_b, got_a, err_msg=f"{name} T={T} E={E}")
            np.testing.assert_array_equal(got_b, w, err_msg=f"{name} vs oracle T={T} E={E}")


def test_noalloc_rejects_sizes_beyond_the_array(lib, torch_cuda):
    torch = torch_cuda
    T, E = 1024 * 65, 1024  # 65 blocks x 1024 experts > 65536 ints
    buf = torch.zeros(T + E + 1, dtype=torch.int32, device="cuda")
    status = lib.infmoe_expert_count_noalloc(T, E, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), buf.data_ptr(),
                                             stream_ptr(torch))
    assert status == capi.ERR_INVALID_ARGUMENT
    assert b"exceed" in lib.infmoe_last_error()
    # the largest size that fits is taken
    T, E = 1024 * 64, 1024
    assert lib.infmoe_expert_count_scratch_bytes(T, E) == 4 * MAX_INTS
    sel = draw_sel(T, E, 9)
    with_scratch, static = run_both(lib, torch, sel, E)
    for a, b in zip(with_scratch, static):
        np.testing.assert_array_equal(b, a)
