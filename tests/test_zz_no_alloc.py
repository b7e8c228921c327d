"""The sampling entry point that allocates nothing (``lsa_sample_static``), called through ctypes as a caller
without Python bindings would, against the entry point that takes a workspace (``lsa_sample``): two calls in a row,
the second with fewer rows and a shorter vocabulary, so that the fixed scratch array still holds the first call's
statistics when the second runs."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from llmserver_amd.kernels import build
    path = build.build(["sampling"])["sampling"]
    library = ctypes.CDLL(path)
    pointer, integer = ctypes.c_void_p, ctypes.c_int
    library.lsa_sample.argtypes = [pointer, pointer, pointer, pointer, pointer, integer, integer, pointer]
    library.lsa_sample_static.argtypes = [pointer, pointer, pointer, pointer, integer, integer, pointer]
    library.lsa_sample_chunks.argtypes = [integer]
    library.lsa_sample_static_error.argtypes = [integer]
    library.lsa_sample_static_error.restype = ctypes.c_char_p
    for name in ("lsa_sample", "lsa_sample_static", "lsa_sample_chunks", "lsa_sample_static_max_rows"):
        getattr(library, name).restype = integer
    return library


def _inputs(rows, vocab, seed):
    generator = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=generator) * 3).to("cuda")
    temperature = torch.where(torch.arange(rows) % 3 == 0, torch.zeros(rows), torch.full((rows,), 0.7)).to("cuda")   # greedy rows among sampled ones
    uniform = torch.rand(rows, generator=generator).to("cuda")
    return logits, temperature, uniform


def test_static_sampling_equals_sampling_with_a_workspace_on_two_calls_in_a_row():
    library = _library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for rows, vocab, seed in ((96, 151_936, 1), (5, 3_001, 2)):          # the second call is the smaller one
        logits, temperature, uniform = _inputs(rows, vocab, seed)
        expected = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        workspace = torch.empty(rows * library.lsa_sample_chunks(vocab) * 4, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        print(f"lsa_sample rows={rows} vocab={vocab}", flush=True)
        assert library.lsa_sample(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), expected.data_ptr(),
                                  workspace.data_ptr(), rows, vocab, stream) == 0
        print(f"lsa_sample_static rows={rows} vocab={vocab}", flush=True)
        before = torch.cuda.memory_allocated()
        code = library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert code == 0, library.lsa_sample_static_error(code)
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(got, expected)
        greedy = temperature.cpu() == 0
        assert torch.equal(got.cpu()[greedy].long(), logits.cpu().argmax(dim=-1)[greedy])
        assert int(got.min()) >= 0 and int(got.max()) < vocab


def test_static_sampling_refuses_more_rows_than_its_scratch_holds():
    library = _library()
    most = library.lsa_sample_static_max_rows()
    logits, temperature, uniform = _inputs(2, 64, 3)
    out = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # Refused before anything is read or launched: the pointers only stand for rows that are not there.
    code = library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), out.data_ptr(), most + 1, 64, stream)
    assert code != 0 and b"at most" in library.lsa_sample_static_error(code)
    torch.cuda.synchronize()
    assert out.tolist() == [-7, -7]
    assert library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), out.data_ptr(), 0, 64, stream) == 0
