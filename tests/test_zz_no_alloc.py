"""The sampling entry point that allocates nothing (``jle_sample_static``), called through
``ctypes`` as a caller outside the package would, against ``jle_sample`` with workspaces."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from jax_llm_examples_amd.ops import build

    lib = ctypes.CDLL(build.library_path())
    vp, i = ctypes.c_void_p, ctypes.c_int
    lib.jle_sample.argtypes = [vp] * 8 + [i, i, i, vp]
    lib.jle_sample.restype = i
    lib.jle_sample_static.argtypes = [vp] * 6 + [i, i, i, vp]
    lib.jle_sample_static.restype = i
    return lib


def _inputs(m, v, seed, dev):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(m, v, generator=g) * 3).to(dev)
    temp = torch.tensor([0.0 if r % 3 == 0 else 0.7 + 0.1 * r for r in range(m)], dtype=torch.float32, device=dev)
    top_k = torch.tensor([0 if r % 2 == 0 else 5 for r in range(m)], dtype=torch.int32, device=dev)
    seeds = torch.arange(m, dtype=torch.int32, device=dev) * 7 + 1
    counters = torch.arange(m, dtype=torch.int32, device=dev) % 4
    return logits, temp, top_k, seeds, counters


def test_sampling_without_allocation_equals_sampling_with_workspaces():
    dev = torch.device("cuda:0")
    lib = _library()
    stream = torch.cuda.current_stream(dev).cuda_stream
    # two calls in a row on the same array, the second with fewer rows and a smaller vocabulary
    for m, v, seed in ((37, 50021, 0), (5, 9001, 1)):
        logits, temp, top_k, seeds, counters = _inputs(m, v, seed, dev)
        chunks = -(-v // 8192)
        part_v = torch.empty(m * chunks, dtype=torch.float32, device=dev)
        part_i = torch.empty(m * chunks, dtype=torch.int32, device=dev)
        want = torch.full((m,), -1, dtype=torch.int32, device=dev)
        got = torch.full((m,), -2, dtype=torch.int32, device=dev)
        p = lambda t: t.data_ptr()
        rc = lib.jle_sample(p(logits), p(temp), p(top_k), p(seeds), p(counters), p(want), p(part_v), p(part_i),
                            m, v, 1, stream)
        assert rc == 0
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        rc = lib.jle_sample_static(p(logits), p(temp), p(top_k), p(seeds), p(counters), p(got), m, v, 1, stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        assert got.tolist() == want.tolist()
        greedy = [r for r in range(m) if r % 3 == 0]
        assert got[greedy].tolist() == logits[greedy].argmax(-1).tolist()


def test_sampling_without_allocation_refuses_what_its_array_cannot_hold():
    dev = torch.device("cuda:0")
    lib = _library()
    stream = torch.cuda.current_stream(dev).cuda_stream
    m, v = 700, 8192 * 24  # 16,800 (row, chunk) pairs: more than the array's 16,384
    z = torch.zeros(m, dtype=torch.int32, device=dev)
    t = torch.zeros(m, dtype=torch.float32, device=dev)
    out = torch.full((m,), -5, dtype=torch.int32, device=dev)
    logits = torch.zeros(1, dtype=torch.float32, device=dev)  # never read: the call is refused before any launch
    rc = lib.jle_sample_static(logits.data_ptr(), t.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                               out.data_ptr(), m, v, 0, stream)
    assert rc < 0
    torch.cuda.synchronize()
    assert out.tolist() == [-5] * m
