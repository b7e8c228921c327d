"""The sampling entry point that allocates nothing (``lsa_sample_static``), called through ctypes as a caller
without Python bindings would, against the entry point that takes a workspace (``lsa_sample``): two calls in a row,
the second with fewer rows and a shorter vocabulary, so that the fixed scratch array still holds the first call's
statistics when the second runs; the tokens also against the distribution itself, worked out in float64; the device's
free memory before and after; and recorded into a graph and replayed."""
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


def _check_against_the_distribution(got, logits, temperature, uniform):
    """Every token is the one its row's rule picks, worked out apart from the kernels in float64: greedy rows the first
    maximum; sampled rows a token whose interval of the cumulative distribution of softmax(logits / temperature) holds
    the row's uniform number (give or take what 32-bit running sums over 150,000 terms lose)."""
    got, logits, temperature, uniform = got.cpu().long(), logits.cpu().double(), temperature.cpu().double(), uniform.cpu().double()
    assert int(got.min()) >= 0 and int(got.max()) < logits.shape[1]
    for row in range(logits.shape[0]):
        if float(temperature[row]) == 0:
            assert int(got[row]) == int(logits[row].argmax()), row
            continue
        cumulative = torch.cumsum(torch.softmax(logits[row] / temperature[row], dim=-1), dim=-1)
        token = int(got[row])
        below = float(cumulative[token - 1]) if token else 0.0
        assert below - 2e-5 <= float(uniform[row]) <= float(cumulative[token]) + 2e-5, (row, token, below, float(uniform[row]), float(cumulative[token]))


def test_static_sampling_equals_sampling_with_a_workspace_on_two_calls_in_a_row():
    library = _library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # The first call on a device looks the scratch array's address up; it comes before anything is measured.
    logits, temperature, uniform = _inputs(2, 64, 9)
    warm = torch.empty(2, dtype=torch.int32, device="cuda")
    assert library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), warm.data_ptr(), 2, 64, stream) == 0
    torch.cuda.synchronize()
    for rows, vocab, seed in ((96, 151_936, 1), (5, 3_001, 2)):          # the second call is the smaller one
        logits, temperature, uniform = _inputs(rows, vocab, seed)
        expected = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        workspace = torch.empty(rows * library.lsa_sample_chunks(vocab) * 4, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        print(f"lsa_sample rows={rows} vocab={vocab}", flush=True)
        assert library.lsa_sample(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), expected.data_ptr(),
                                  workspace.data_ptr(), rows, vocab, stream) == 0
        torch.cuda.synchronize()
        print(f"lsa_sample_static rows={rows} vocab={vocab}", flush=True)
        # What the driver has left, not what torch's allocator has handed out: an allocation by the library itself
        # (which torch never sees) would take from it.
        free_before, _ = torch.cuda.mem_get_info()
        code = library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert code == 0, library.lsa_sample_static_error(code)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after >= free_before, f"the call took {free_before - free_after} bytes of device memory"
        assert torch.equal(got, expected)
        _check_against_the_distribution(got, logits, temperature, uniform)


def test_static_sampling_inside_a_captured_graph():
    """What the entry point is for: recorded into a graph (while a stream captures, an allocation is an error, and this
    capture is in the mode that forbids them for every thread), then replayed, with the inputs changed and eager
    work between the replays; every replay gives what the distribution demands and what the eager call gives."""
    library = _library()
    rows, vocab = 40, 20_011
    logits, temperature, uniform = _inputs(rows, vocab, 5)
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    eager = torch.full((rows,), -1, dtype=torch.int32, device="cuda")

    def call(result):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        code = library.lsa_sample_static(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), result.data_ptr(), rows, vocab, stream)
        assert code == 0, library.lsa_sample_static_error(code)

    call(eager)                                                # (also the first call on the device, before the capture)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, capture_error_mode="global"):
        call(out)
    torch.cuda.synchronize()
    assert out.tolist() == [-1] * rows                         # recorded, not run
    for replay in range(3):
        fresh = _inputs(rows, vocab, 50 + replay)
        for old, new in zip((logits, temperature, uniform), fresh):
            old.copy_(new)
        call(eager)
        torch.cuda.synchronize()
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        print(f"replay {replay}", flush=True)
        assert torch.equal(out, eager)
        _check_against_the_distribution(out, logits, temperature, uniform)


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
