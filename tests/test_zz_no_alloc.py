"""stm_route_plan_static (the entry point that allocates nothing) against stm_route_plan.

Both are called through the C ABI with the same ids; every output must agree bit for bit.
Two calls in a row share the library's static scratch array: the second one is smaller, so
anything it wrongly read from the first call's leftovers would show."""

import pytest
import torch

from steptronoss_amd import _lib
from steptronoss_amd._lib import ptr
from tests.helpers import make_topk_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _plan(entry, ids, n_experts):
    n = ids.numel()
    lib = _lib.load()
    hist = torch.full((n_experts,), -7, device=DEV, dtype=torch.int32)
    offsets = torch.full((n_experts + 1,), -7, device=DEV, dtype=torch.int32)
    pos = torch.full(ids.shape, -7, device=DEV, dtype=torch.int32)
    status = torch.zeros(_lib.STATUS_WORDS, device=DEV, dtype=torch.int32)
    stream = torch.cuda.current_stream().cuda_stream or None
    i64 = int(ids.dtype == torch.int64)
    if entry == "static":
        code = lib.stm_route_plan_static(ptr(ids), i64, n, n_experts, ptr(hist), ptr(offsets), ptr(pos), ptr(status), stream)
    else:
        nbytes = lib.stm_route_workspace_bytes(n, n_experts)
        ws = torch.empty(nbytes, device=DEV, dtype=torch.uint8)
        code = lib.stm_route_plan(
            ptr(ids), i64, n, n_experts, ptr(hist), ptr(offsets), ptr(pos), ptr(status), ptr(ws), nbytes, stream
        )
    torch.cuda.synchronize()
    return code, hist.cpu(), offsets.cpu(), pos.cpu(), status.cpu()


def test_static_route_plan_matches_workspace_form_twice():
    gen = torch.Generator().manual_seed(11)
    # first a large problem (fills 256 KiB of the scratch), then a smaller one with other ids
    cases = [(16384, 8, 128, torch.int64, 0.0), (3000, 3, 40, torch.int32, 0.2)]
    for T, K, E, dtype, inv in cases:
        ids = make_topk_ids(T, K, E, gen=gen, invalid_frac=inv, dtype=dtype).to(DEV)
        want = _plan("workspace", ids, E)
        got = _plan("static", ids, E)
        assert want[0] == 0 and got[0] == 0
        for w, g, name in zip(want[1:], got[1:], ("hist", "offsets", "pos", "status")):
            assert torch.equal(w, g), name
        assert int(got[2][-1]) == int((ids >= 0).sum())


def test_static_route_plan_rejects_what_does_not_fit():
    lib = _lib.load()
    cap = lib.stm_route_plan_static_capacity_bytes()
    E = 4096
    n = (cap // (4 * E) + 2) * 256  # two counter rows more than the array holds
    assert lib.stm_route_workspace_bytes(n, E) > cap
    ids = torch.zeros(n, device=DEV, dtype=torch.int32)
    out = torch.empty(n, device=DEV, dtype=torch.int32)
    offs = torch.empty(E + 1, device=DEV, dtype=torch.int32)
    status = torch.zeros(_lib.STATUS_WORDS, device=DEV, dtype=torch.int32)
    code = lib.stm_route_plan_static(ptr(ids), 0, n, E, None, ptr(offs), ptr(out), ptr(status), None)
    assert code == -5 and "static scratch" in _lib.status_string(code)
