"""The entry point that allocates nothing (csrc/mv_noalloc.h), called through ctypes as a caller
without the engine would: its tokens against those of the entry point with a caller's workspace,
on two calls in a row, the second with a smaller input; and its refusal of more rows than its
scratch array holds."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def load():
    from minivllm_amd.csrc import build
    path = build.find_library("bf16") or build.build("bf16")
    dll = ctypes.CDLL(path)
    vp, ci, cl = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    dll.mv_last_error.restype = ctypes.c_char_p
    dll.mv_sample_noalloc.restype = ci
    dll.mv_sample_noalloc.argtypes = [vp, cl, ci, ci, vp, vp, vp, vp, vp, vp]
    dll.mv_sample.restype = ci
    dll.mv_sample.argtypes = [vp, cl, ci, ci, vp, vp, vp, vp, vp, vp, ci, vp]
    return dll


def make_rows(M, V, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(M, V, generator=g) * 3).cuda()
    temperature = torch.tensor([0.0, 0.8, 1.0, 0.7] * (M // 4 + 1))[:M].cuda()
    top_k = torch.tensor([0, 0, 20, 0] * (M // 4 + 1), dtype=torch.int32)[:M].cuda()
    top_p = torch.tensor([1.0, 1.0, 1.0, 0.9] * (M // 4 + 1))[:M].cuda()
    rng = torch.stack([torch.arange(M, dtype=torch.int64) + 1000 * seed, torch.arange(M, dtype=torch.int64) % 7],
                      dim=1).contiguous().cuda()
    return logits, temperature, top_k, top_p, rng


def test_sample_noalloc_matches_the_entry_point_with_a_workspace():
    dll = load()
    stream = torch.cuda.current_stream().cuda_stream
    work = torch.empty(1024 * 32 * 2, dtype=torch.int32, device="cuda")
    for call, (M, V) in enumerate([(37, 5003), (5, 4099)]):         # two calls in a row, the second smaller
        logits, temperature, top_k, top_p, rng = make_rows(M, V, seed=call + 1)
        want = torch.full((M,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((M,), -1, dtype=torch.int32, device="cuda")
        rc = dll.mv_sample(logits.data_ptr(), V, M, V, temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                           rng.data_ptr(), want.data_ptr(), work.data_ptr(), 32, stream)
        assert rc == 0, dll.mv_last_error()
        torch.cuda.synchronize()
        before = (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0])
        rc = dll.mv_sample_noalloc(logits.data_ptr(), V, M, V, temperature.data_ptr(), top_k.data_ptr(),
                                   top_p.data_ptr(), rng.data_ptr(), got.data_ptr(), stream)
        assert rc == 0, dll.mv_last_error()
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]) == before      # the device's free memory too
        assert torch.equal(got, want), (call, got.tolist(), want.tolist())
        assert int(want.min()) >= 0 and int(want.max()) < V
        # greedy rows are the arg-max
        greedy = (temperature == 0).nonzero().flatten()
        assert torch.equal(got[greedy].long(), logits[greedy].argmax(dim=-1))


def test_sample_noalloc_refuses_more_rows_than_its_scratch_holds():
    dll = load()
    M, V = 1025, 64
    logits = torch.zeros(M, V, device="cuda")
    out = torch.full((M,), -7, dtype=torch.int32, device="cuda")
    rc = dll.mv_sample_noalloc(logits.data_ptr(), V, M, V, None, None, None, None, out.data_ptr(),
                               torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b"1024 rows" in dll.mv_last_error()
    torch.cuda.synchronize()
    assert int(out.min()) == -7 and int(out.max()) == -7           # nothing ran
