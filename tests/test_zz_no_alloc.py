"""rb_sample_static: the sampling entry point that allocates nothing, called through ctypes
alone (no binding of the package), against rb_sample with a workspace on the same inputs:
two calls in a row, the second smaller, so that what the first left in the library's own
scratch memory lies beyond and under the second's entries."""
from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

_P, _I = ctypes.c_void_p, ctypes.c_int


def _library():
    from rbitnet_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_built())
    lib.rb_last_error.restype = ctypes.c_char_p
    lib.rb_sample.argtypes = [_P, _I, _I, _P, _P, _P, _P, _P]
    lib.rb_sample_static.argtypes = [_P, _I, _I, _P, _P, _P, _P]
    lib.rb_sample_workspace_bytes.argtypes = [_I, _I]
    for name in ("rb_sample", "rb_sample_static", "rb_sample_workspace_bytes", "rb_sample_static_max_stats"):
        getattr(lib, name).restype = _I
    return lib


def _case(rows: int, vocab: int, seed: int, greedy_rows):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3.0)
    logits[0, vocab // 3] = float("nan")                       # counts as -inf
    temperature = torch.full((rows,), 0.8)
    for r in greedy_rows:
        temperature[r] = 0.0
    u = torch.rand(rows, generator=g)
    return logits.cuda(), temperature.cuda(), u.cuda()


def _both(lib, logits, temperature, u):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    workspace = torch.empty(lib.rb_sample_workspace_bytes(rows, vocab) // 8 + 1, dtype=torch.int64, device="cuda")
    rc = lib.rb_sample(logits.data_ptr(), rows, vocab, temperature.data_ptr(), u.data_ptr(), want.data_ptr(),
                       workspace.data_ptr(), stream)
    assert rc == 0, lib.rb_last_error()
    assert lib.rb_sample_static_max_stats() > 0            # the set-up call: the scratch address is known from here on
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]             # the device's own count: an allocation past torch's would show
    rc = lib.rb_sample_static(logits.data_ptr(), rows, vocab, temperature.data_ptr(), u.data_ptr(), got.data_ptr(),
                              stream)
    assert rc == 0, lib.rb_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return got.cpu(), want.cpu()


def test_static_sampling_equals_the_workspace_one_twice_in_a_row():
    lib = _library()
    print("rb_sample_static: 9 x 128256, then 3 x 5000", flush=True)
    first = _case(9, 128256, 0, greedy_rows=(1, 4))
    got, want = _both(lib, *first)
    assert got.tolist() == want.tolist()
    assert all(0 <= t < 128256 for t in got.tolist())
    # the second call is smaller in both directions: fewer rows and fewer chunks a row, so the
    # entries of row r now lie where row 0's chunks 2r, 2r + 1 lay
    second = _case(3, 5000, 1, greedy_rows=(2,))
    got, want = _both(lib, *second)
    assert got.tolist() == want.tolist()
    # greedy rows are the argmax (NaN as -inf, lowest index)
    logits = second[0].cpu()
    assert got[2].item() == int(torch.nan_to_num(logits[2], nan=float("-inf")).argmax())
    # and the first again: the larger call after the smaller
    got, want = _both(lib, *first)
    assert got.tolist() == want.tolist()


def test_static_sampling_under_stream_capture():
    """Recorded into a graph (what the entry point is for) and replayed with other inputs in the same
    buffers, eager work and synchronisations between the replays: every replay equals rb_sample."""
    lib = _library()
    assert lib.rb_sample_static_max_stats() > 0            # outside the capture: asks for the scratch address
    rows, vocab = 5, 33000
    logits, temperature, u = _case(rows, vocab, 3, greedy_rows=(0,))
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.rb_sample_static(logits.data_ptr(), rows, vocab, temperature.data_ptr(), u.data_ptr(), got.data_ptr(),
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.rb_last_error()
    workspace = torch.empty(lib.rb_sample_workspace_bytes(rows, vocab) // 8 + 1, dtype=torch.int64, device="cuda")
    for replay in range(4):
        new_logits, new_t, new_u = _case(rows, vocab, 10 + replay, greedy_rows=(replay % rows,))
        logits.copy_(new_logits)
        temperature.copy_(new_t)
        u.copy_(new_u)
        got.fill_(-2)
        graph.replay()
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        rc = lib.rb_sample(logits.data_ptr(), rows, vocab, temperature.data_ptr(), u.data_ptr(), want.data_ptr(),
                           workspace.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.rb_last_error()
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist(), f"replay {replay}"
        _ = (torch.ones(4096, device="cuda") * 3).sum().item()          # unrelated eager work between the replays


def test_static_sampling_refuses_what_its_scratch_cannot_hold():
    lib = _library()
    limit = lib.rb_sample_static_max_stats()
    vocab = 128256
    chunks = (vocab + 4095) // 4096
    rows = limit // chunks + 1
    tokens = torch.full((rows,), -5, dtype=torch.int32, device="cuda")
    # refused before any pointer is used: the logits pointer is never read
    rc = lib.rb_sample_static(tokens.data_ptr(), rows, vocab, None, None, tokens.data_ptr(),
                              torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert b"scratch holds" in lib.rb_last_error()
    torch.cuda.synchronize()
    assert tokens.tolist() == [-5] * rows
