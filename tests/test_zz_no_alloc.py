"""The sampling entry point that allocates nothing, called through ctypes as a caller without
torch's allocator would: its tokens must be those of ``ra_sample`` (which takes the caller's
scratch buffers), on two calls in a row that share the GPU's scratch array, the second smaller."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(rows, vocab, seed, device):
    g = torch.Generator(device="cpu").manual_seed(seed)
    logits = (torch.randn((rows, vocab), generator=g) * 3.0).to(device)
    logits[0, vocab // 3] = float("inf")            # never wins
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.7 + 0.1 * (r % 5) for r in range(rows)],
                               dtype=torch.float32, device=device)
    seeds = torch.randint(0, 2 ** 62, (rows,), generator=g, dtype=torch.int64).to(device)
    positions = torch.randint(0, 4000, (rows,), generator=g, dtype=torch.int32).to(device)
    return logits, temperature, seeds, positions


def _both(lib, case):
    logits, temperature, seeds, positions = case
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    slices = lib.ra_sample_slices(vocab)
    val = torch.empty((rows, slices), dtype=torch.float32, device=logits.device)
    idx = torch.empty((rows, slices), dtype=torch.int32, device=logits.device)
    want = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    got = torch.full((rows,), -9, dtype=torch.int32, device=logits.device)
    args = (ctypes.c_void_p(logits.data_ptr()), rows, vocab, logits.stride(0),
            ctypes.c_void_p(temperature.data_ptr()), ctypes.c_void_p(seeds.data_ptr()),
            ctypes.c_void_p(positions.data_ptr()))
    rc = lib.ra_sample(*args, ctypes.c_void_p(val.data_ptr()), ctypes.c_void_p(idx.data_ptr()),
                       ctypes.c_void_p(want.data_ptr()), stream)
    assert rc == 0, lib.ra_last_error()
    rc = lib.ra_sample_static(*args, ctypes.c_void_p(got.data_ptr()), stream)
    assert rc == 0, lib.ra_last_error()
    torch.cuda.synchronize()
    return want.cpu(), got.cpu()


def test_sampling_without_allocation_matches_on_two_calls_in_a_row():
    from reinfer_amd.kernels import library
    lib = library.load()
    device = torch.device("cuda:0")
    with torch.cuda.device(device):
        first = _case(48, 151936, 1, device)             # 48 x 75 slices of the shared array
        want, got = _both(lib, first)
        assert torch.equal(want, got)
        assert (got >= 0).all() and (got < 151936).all()
        assert got[0].item() != 151936 // 3
        second = _case(5, 1000, 2, device)               # smaller: one slice a row, over what the first left
        want2, got2 = _both(lib, second)
        assert torch.equal(want2, got2)
        assert (got2 >= 0).all() and (got2 < 1000).all()
        # the first again: the array now holds the second call's winners in its first entries
        want3, got3 = _both(lib, first)
        assert torch.equal(want3, got) and torch.equal(got3, got)


def test_sampling_without_allocation_refuses_what_the_array_cannot_hold():
    from reinfer_amd.kernels import library
    lib = library.load()
    device = torch.device("cuda:0")
    limit = lib.ra_sample_static_max_pairs()
    vocab = 151936
    rows = limit // lib.ra_sample_slices(vocab) + 1
    t = torch.zeros(8, dtype=torch.int32, device=device)
    p = ctypes.c_void_p(t.data_ptr())
    # refused on the host before any launch: the pointers are never read
    rc = lib.ra_sample_static(p, rows, vocab, vocab, p, p, p, p, ctypes.c_void_p(0))
    assert rc != 0
    assert b"scratch" in lib.ra_last_error()


def test_sampling_without_allocation_inside_a_captured_stream():
    """What the entry point is for: after ``ra_sample_static_prepare()`` (the address lookup, once, outside) it
    is called while the stream captures, the graph is replayed several times with eager work between, each
    replay on fresh logits, and every replay's tokens are those of ``ra_sample``; the device's free memory is the
    same before and after the calls."""
    from reinfer_amd.kernels import library
    lib = library.load()
    device = torch.device("cuda:0")
    with torch.cuda.device(device):
        assert lib.ra_sample_static_prepare() == 0, lib.ra_last_error()
        rows, vocab = 12, 4099
        logits, temperature, seeds, positions = _case(rows, vocab, 5, device)
        got = torch.full((rows,), -9, dtype=torch.int32, device=device)
        args = (ctypes.c_void_p(logits.data_ptr()), rows, vocab, logits.stride(0),
                ctypes.c_void_p(temperature.data_ptr()), ctypes.c_void_p(seeds.data_ptr()),
                ctypes.c_void_p(positions.data_ptr()), ctypes.c_void_p(got.data_ptr()))
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(device)[0]
        rc = lib.ra_sample_static(*args, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.ra_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(device)[0] == free_before, "an eager call changed the device's free memory"
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = lib.ra_sample_static(*args, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.ra_last_error()
        for rep in range(4):
            fresh = _case(rows, vocab, 20 + rep, device)
            for dst, src in zip((logits, temperature, seeds, positions), fresh):
                dst.copy_(src)
            got.fill_(-9)
            graph.replay()
            torch.cuda.synchronize()
            want, eager = _both(lib, (logits, temperature, seeds, positions))     # eager work between the replays
            assert torch.equal(got.cpu(), want), rep
            assert torch.equal(eager, want)
