"""sy_sort_by_expert_static (the histograms in the library's static device array, for callers
that cannot allocate) against sy_sort_by_expert with a caller's workspace and the CPU oracle,
through the C ABI. Needs an MI355X."""

import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _choices(N, E, k, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.topk(torch.randn(N, E, generator=g), k, dim=-1).indices.int().to(DEV)
    return idx, torch.rand(N, k, generator=g).half().to(DEV)


def _static_sort(abi, lib, idx, w, E):
    N, k = idx.shape
    M = N * k
    i32 = dict(dtype=torch.int32, device=idx.device)
    counts, offsets = torch.full((E,), -1, **i32), torch.full((E + 1,), -1, **i32)
    token, pos_of = torch.full((M,), -1, **i32), torch.full((M,), -1, **i32)
    wsorted = torch.zeros(M, dtype=w.dtype, device=idx.device)
    rc = lib.sy_sort_by_expert_static(idx.data_ptr(), w.data_ptr(), w.element_size(), N, k, E, counts.data_ptr(),
                                      offsets.data_ptr(), token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(),
                                      abi._stream())
    return rc, [counts, offsets, token, wsorted, pos_of]


def test_static_sort_equals_the_workspace_sort_on_two_calls_in_a_row():
    from switchyard_amd import _abi, kernels

    ext = kernels.ext()
    lib = ext.lib
    # both sizes take the launches over many workgroups (more than 2048 choices), which are the
    # ones that use the histograms; the second call is smaller and finds the first one's there
    for N, E, k, seed in ((40000, 64, 8, 1), (3000, 64, 8, 2), (1500, 128, 8, 3), (100, 64, 8, 4)):
        idx, w = _choices(N, E, k, seed)
        assert (lib.sy_sort_workspace_bytes(N, k, E) > 0) == (N * k > 2048)
        rc, got = _static_sort(_abi, lib, idx, w, E)
        assert rc == 0, lib.sy_last_error().decode()
        want = ext.sort_by_expert(idx, w, E)
        torch.cuda.synchronize()
        for name, a, b in zip(("counts", "offsets", "token", "wsorted", "pos_of"), got, want):
            assert torch.equal(a, b), (N, E, name)
        p = O.plan(idx.cpu().long(), w.cpu(), E)
        assert torch.equal(got[2].cpu().long(), p.token) and torch.equal(got[4].cpu().long(), p.pos_of)
        assert torch.equal(got[1].cpu().long(), p.offsets)


def test_static_sort_refuses_what_its_array_cannot_hold():
    from switchyard_amd import _abi, kernels

    lib = kernels.ext().lib
    N, E, k = 20000, 512, 8          # 160 000 choices over 512 experts: 2.6 MB of histograms
    assert lib.sy_sort_workspace_bytes(N, k, E) > (1 << 20)
    idx, w = _choices(N, E, k, 5)
    rc, _ = _static_sort(_abi, lib, idx, w, E)
    assert rc == 1 and "static" in lib.sy_last_error().decode()


def test_static_sort_under_stream_capture():
    """What the entry point is for: after one call outside a capture (which looks the array's
    address up), a call recorded by a stream capture allocates nothing, so the capture succeeds,
    and every replay leaves the five outputs of the workspace sort."""
    from switchyard_amd import _abi, kernels

    ext = kernels.ext()
    lib = ext.lib
    N, E, k = 3000, 64, 8
    idx, w = _choices(N, E, k, 7)
    rc, _ = _static_sort(_abi, lib, idx, w, E)          # warm-up outside the capture
    assert rc == 0, lib.sy_last_error().decode()
    M = N * k
    i32 = dict(dtype=torch.int32, device=DEV)
    outs = [torch.full((E,), -1, **i32), torch.full((E + 1,), -1, **i32), torch.full((M,), -1, **i32),
            torch.zeros(M, dtype=w.dtype, device=DEV), torch.full((M,), -1, **i32)]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.sy_sort_by_expert_static(idx.data_ptr(), w.data_ptr(), w.element_size(), N, k, E, outs[0].data_ptr(),
                                          outs[1].data_ptr(), outs[2].data_ptr(), outs[3].data_ptr(), outs[4].data_ptr(),
                                          _abi._stream())
    assert rc == 0, lib.sy_last_error().decode()
    for seed in (8, 9):
        new_idx, new_w = _choices(N, E, k, seed)
        idx.copy_(new_idx)
        w.copy_(new_w)
        for t in outs:
            t.fill_(0)
        graph.replay()
        torch.cuda.synchronize()
        want = ext.sort_by_expert(idx, w, E)
        for name, a, b in zip(("counts", "offsets", "token", "wsorted", "pos_of"), outs, want):
            assert torch.equal(a, b), (seed, name)
