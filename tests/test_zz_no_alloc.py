"""rlk_linear_logp_fwd_noalloc on a real MI355X: the entry point that takes no workspace and
allocates nothing must give the bits of rlk_linear_logp_fwd, call after call, also when a smaller
call follows a larger one on the same built-in scratch. Called through the C ABI (ctypes) with
caller-allocated inputs and outputs."""

from __future__ import annotations

import pytest
import torch

import inputs

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _stream() -> int:
    return int(torch.cuda.current_stream().cuda_stream)


def _with_workspace(lib, h, w, t, bias, temp, real):
    n, d = h.shape
    v = w.size(0)
    logp = torch.full((n,), 7.0, dtype=torch.float32, device=DEV)
    lse = torch.full((n,), 7.0, dtype=torch.float32, device=DEV)
    ws_bytes = int(lib.rlk_linear_logp_workspace_bytes(n, v))
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=DEV)
    rc = lib.rlk_linear_logp_fwd(
        h.data_ptr(), h.stride(0), w.data_ptr(), w.stride(0), t.data_ptr(),
        bias.data_ptr() if bias is not None else None, temp.data_ptr() if temp is not None else None,
        logp.data_ptr(), lse.data_ptr(), ws.data_ptr(), ws_bytes, n, d, v, 0, real, 0, _stream(),
    )  # fmt: skip
    assert rc == 0, lib.rlk_last_error().decode()
    return logp, lse


def _no_alloc(lib, h, w, t, bias, temp, real, logp, lse):
    n, d = h.shape
    rc = lib.rlk_linear_logp_fwd_noalloc(
        h.data_ptr(), h.stride(0), w.data_ptr(), w.stride(0), t.data_ptr(),
        bias.data_ptr() if bias is not None else None, temp.data_ptr() if temp is not None else None,
        logp.data_ptr(), lse.data_ptr(), n, d, w.size(0), 0, real, 0, _stream(),
    )  # fmt: skip
    return rc


def _bits(x):
    return x.view(torch.int32)


def test_no_alloc_entry_matches_the_workspace_entry_on_consecutive_calls(rlk_lib):
    lib = rlk_lib
    v, d, real = 9000, 256, 8990
    g = torch.Generator().manual_seed(9100)
    bias = (torch.randn(v, generator=g) * 0.3).to(DEV)
    # (tokens, with bias / temperature / padding): large, then smaller calls on the same scratch; 1300 tokens
    # take the split-per-workgroup grid, the others the stream-group grid with its 17-fold staging
    cases = [(1300, True), (700, True), (33, False), (1, True), (700, False)]
    outputs = {n: (torch.empty(n, dtype=torch.float32, device=DEV), torch.empty(n, dtype=torch.float32, device=DEV)) for n, _ in cases}
    for n, extras in cases:
        h, w, t = inputs.logp_inputs(n, vocab=v, hidden=d, seed=9101, rms_norm=False)
        h, w, t = h.to(DEV), w.to(DEV), (t % real).to(DEV)
        temp = (0.5 + torch.rand(n, generator=g)).to(DEV) if extras else None
        b = bias if extras else None
        r = real if extras else v
        want_logp, want_lse = _with_workspace(lib, h, w, t, b, temp, r)
        logp, lse = outputs[n]
        logp.fill_(-3.0), lse.fill_(-3.0)
        # one warm call (code objects of this size's kernels get loaded on first use), then the call under test:
        # the device's free memory, which sees every hipMalloc of the process and not only torch's allocator,
        # must not move
        assert _no_alloc(lib, h, w, t, b, temp, r, logp, lse) == 0, lib.rlk_last_error().decode()
        logp.fill_(-3.0), lse.fill_(-3.0)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert _no_alloc(lib, h, w, t, b, temp, r, logp, lse) == 0, lib.rlk_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] >= free_before
        assert torch.equal(_bits(logp), _bits(want_logp)) and torch.equal(_bits(lse), _bits(want_lse)), (n, extras)
        assert bool(torch.isfinite(logp).all()) and bool((logp <= 0).all())


def test_no_alloc_entry_runs_under_hip_graph_capture(rlk_lib):
    # an allocating call would fail inside a capture; the replays must give the eager bits every time
    lib = rlk_lib
    n, v, d = 300, 5000, 128
    h, w, t = inputs.logp_inputs(n, vocab=v, hidden=d, seed=9300, rms_norm=False)
    h, w, t = h.to(DEV), w.to(DEV), t.to(DEV)
    want_logp, want_lse = _with_workspace(lib, h, w, t, None, None, v)
    logp = torch.empty(n, dtype=torch.float32, device=DEV)
    lse = torch.empty(n, dtype=torch.float32, device=DEV)
    assert _no_alloc(lib, h, w, t, None, None, v, logp, lse) == 0  # warm: per-device set-up happens here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert _no_alloc(lib, h, w, t, None, None, v, logp, lse) == 0, lib.rlk_last_error().decode()
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        logp.fill_(5.0), lse.fill_(5.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(logp), _bits(want_logp)) and torch.equal(_bits(lse), _bits(want_lse))


def test_no_alloc_entry_rejects_sizes_beyond_its_scratch_and_bad_arguments(rlk_lib):
    from rl_engine import _lib

    lib = rlk_lib
    h, w, t = inputs.logp_inputs(8, vocab=2048, hidden=64, seed=9200, rms_norm=False)
    h, w, t = h.to(DEV), w.to(DEV), t.to(DEV)
    logp = torch.empty(8, dtype=torch.float32, device=DEV)
    lse = torch.empty(8, dtype=torch.float32, device=DEV)
    # sizes only: the pointers are never touched when the size check fails
    too_many = 20000
    assert int(lib.rlk_linear_logp_workspace_bytes(too_many, 151936)) > _lib.NOALLOC_SCRATCH_BYTES
    rc = lib.rlk_linear_logp_fwd_noalloc(
        h.data_ptr(), 4096, w.data_ptr(), 4096, t.data_ptr(), None, None, logp.data_ptr(), lse.data_ptr(),
        too_many, 4096, 151936, 0, 151936, 0, _stream(),
    )  # fmt: skip
    assert rc == _lib.RLK_ERR_INVALID_ARGUMENT and b"scratch" in lib.rlk_last_error()
    assert int(lib.rlk_linear_logp_workspace_bytes(1024, 151936)) <= _lib.NOALLOC_SCRATCH_BYTES
    assert int(lib.rlk_linear_logp_workspace_bytes(18000, 151936)) <= _lib.NOALLOC_SCRATCH_BYTES
    rc = lib.rlk_linear_logp_fwd_noalloc(
        h.data_ptr(), 64, w.data_ptr(), 64, t.data_ptr(), None, None, logp.data_ptr(), lse.data_ptr(),
        8, 64, 2048, 0, 4096, 0, _stream(),
    )  # fmt: skip
    assert rc == _lib.RLK_ERR_INVALID_ARGUMENT and b"real_vocab_end" in lib.rlk_last_error()
    assert _no_alloc(lib, h, w, t, None, None, 2048, logp, lse) == 0
    want, _ = _with_workspace(lib, h, w, t, None, None, 2048)
    assert torch.equal(_bits(logp), _bits(want))
