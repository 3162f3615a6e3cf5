"""The entry point that allocates nothing, retro_kernel_sample_greedy_noalloc, against the entry point it is a
variant of (retro_kernel_sample_prepare with k = 1 for every row), through the C ABI.

The caller owns inputs and outputs (torch tensors on the GPU here); the slice partials live in the library's
static device array. Both entry points cut the vocabulary into the same slices, so argmax, max and the double
sum of exponentials must agree bit for bit. Two calls in a row, the second with fewer rows and a smaller
vocabulary, check that what the first call left in the shared array does not leak into the second."""
import numpy as np
import pytest

from retrograd_amd import engine as E

pytestmark = pytest.mark.gpu


def _both(n_rows, n_vocab, seed, ties=False):
    import torch
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((n_rows, n_vocab)) * 3).astype(np.float32)
    if ties:                                  # the maximum several times per row: the lowest id must win
        for r in range(n_rows):
            top = logits[r].max() + 1.0
            logits[r, rng.integers(0, n_vocab, 5)] = top
    want = E.kernel_sample_prepare(logits, [1] * n_rows)
    d_logits = torch.from_numpy(logits).cuda()
    d_argmax = torch.full((n_rows,), -7, dtype=torch.int32, device="cuda")
    d_max = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    d_sum = torch.zeros(n_rows, dtype=torch.float64, device="cuda")
    stream = torch.cuda.current_stream()
    E.kernel_sample_greedy_noalloc(d_logits.data_ptr(), n_rows, n_vocab, d_argmax.data_ptr(), d_max.data_ptr(),
                                   d_sum.data_ptr(), stream.cuda_stream)
    stream.synchronize()
    got = (d_argmax.cpu().numpy(), d_max.cpu().numpy(), d_sum.cpu().numpy())
    assert np.array_equal(got[0], want[0]), (n_rows, n_vocab, got[0], want[0])
    assert np.array_equal(got[1], want[1])
    assert np.array_equal(got[2], want[2]), (got[2], want[2])
    assert np.array_equal(got[0], logits.argmax(axis=1))
    ref = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True)).sum(axis=1)
    assert np.allclose(got[2], ref, rtol=1e-12)


def test_two_calls_in_a_row_the_second_smaller():
    print("no-alloc greedy scan: 48 x 40000, then 5 x 9000", flush=True)
    _both(48, 40000, 1)
    _both(5, 9000, 2)
    print("no-alloc greedy scan: ties, one row, many rows", flush=True)
    _both(16, 16384, 3, ties=True)
    _both(1, 128256, 4)
    _both(700, 8192, 5)            # more than 512 rows: one slice per row
    _both(3, 8200, 6)


def test_sizes_beyond_the_static_array_are_refused_before_any_launch():
    import torch
    limit = E.load_library().retro_kernel_sample_greedy_noalloc_max_rows()
    assert limit == 4096
    x = torch.zeros(8, dtype=torch.float32, device="cuda")
    with pytest.raises(E.EngineError) as err:
        E.kernel_sample_greedy_noalloc(x.data_ptr(), limit + 1, 8192, x.data_ptr(), x.data_ptr(), x.data_ptr(), 0)
    assert "4096" in str(err.value)
    for rows, vocab in ((0, 8192), (4, 0)):
        with pytest.raises(E.EngineError):
            E.kernel_sample_greedy_noalloc(x.data_ptr(), rows, vocab, x.data_ptr(), x.data_ptr(), x.data_ptr(), 0)
    with pytest.raises(E.EngineError):
        E.kernel_sample_greedy_noalloc(0, 4, 8192, x.data_ptr(), x.data_ptr(), x.data_ptr(), 0)


def test_the_call_inside_a_captured_graph_replays_like_the_eager_call():
    # What the entry point is for: callers under stream capture. The address lookup happened before (an engine's
    # creation, or the eager calls of the tests above); the captured region holds the two kernels and nothing else
    # (no memset node). Replayed several times, with eager work and synchronisations in between, over changing
    # logits: every replay must equal the eager call on the same logits.
    import torch
    n_rows, n_vocab = 24, 32000
    rng = np.random.default_rng(9)
    d_logits = torch.zeros((n_rows, n_vocab), dtype=torch.float32, device="cuda")
    d_argmax = torch.full((n_rows,), -7, dtype=torch.int32, device="cuda")
    d_max = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    d_sum = torch.zeros(n_rows, dtype=torch.float64, device="cuda")
    warm = torch.cuda.Stream()
    with torch.cuda.stream(warm):        # one eager call on a side stream first, as torch asks before a capture
        E.kernel_sample_greedy_noalloc(d_logits.data_ptr(), n_rows, n_vocab, d_argmax.data_ptr(), d_max.data_ptr(),
                                       d_sum.data_ptr(), warm.cuda_stream)
    warm.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("no-alloc greedy scan: capture", flush=True)
    with torch.cuda.graph(graph):
        E.kernel_sample_greedy_noalloc(d_logits.data_ptr(), n_rows, n_vocab, d_argmax.data_ptr(), d_max.data_ptr(),
                                       d_sum.data_ptr(), torch.cuda.current_stream().cuda_stream)
    for it in range(4):
        logits = (rng.standard_normal((n_rows, n_vocab)) * 3).astype(np.float32)
        d_logits.copy_(torch.from_numpy(logits))
        d_argmax.fill_(-7)
        torch.cuda.synchronize()
        print("no-alloc greedy scan: replay", it, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        want = E.kernel_sample_prepare(logits, [1] * n_rows)
        assert np.array_equal(d_argmax.cpu().numpy(), want[0]), it
        assert np.array_equal(d_max.cpu().numpy(), want[1]), it
        assert np.array_equal(d_sum.cpu().numpy(), want[2]), it
