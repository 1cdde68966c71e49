"""The histogram entry point that allocates nothing (HipHistogramLaunchNoAlloc: partial
histograms in a static device array) against HipHistogramCommandCreate through an XQueue and
against the CPU oracle, bit for bit: two calls in a row on one stream, the second with a
smaller input (so it finds the first call's contents in the array), then the size limit."""
from ctypes import byref, c_uint64

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

N_BINS = 65536


def _through_xqueue(xs, torch, keys, n, n_bins):
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    stream = torch.cuda.Stream()
    hwq = xs.hip_queue_create(stream.cuda_stream)
    xq = xs.xqueue_create(hwq, xs.kPreemptLevelBlock)
    cmd = c_uint64()
    xs.check(xs.halhip().HipHistogramCommandCreate(byref(cmd), keys.data_ptr(), n, bins.data_ptr(), n_bins, 0))
    xs.check(xs.preempt().XQueueSubmit(xq, cmd.value))
    xs.check(xs.preempt().XQueueWaitAll(xq))
    xs.check(xs.preempt().XQueueDestroy(xq))
    xs.check(xs.preempt().HwQueueDestroy(hwq))
    return bins.cpu().numpy().view(np.uint32)


def test_no_alloc_histogram_matches_the_command_and_the_oracle(xs, gpu):
    torch = gpu
    h = xs.halhip()
    stream = torch.cuda.Stream()
    # first call: the largest input the entry point takes with ragged end (2^26 - 5 keys, Zipf);
    # second call: a smaller one with uniform keys over fewer bins, on the same stream
    cases = [((1 << 26) - 5, N_BINS, "zipf"), ((1 << 20) + 3, 1000, "uniform")]
    inputs = []
    for n, n_bins, kind in cases:
        if kind == "zipf":
            keys_h = oracle.fill_zipf(0, 3, 0, n)
        else:
            keys_h = (np.random.default_rng(9).integers(0, n_bins, size=n)).astype(np.int32)
        inputs.append((n, n_bins, keys_h, torch.from_numpy(keys_h).cuda()))
    torch.cuda.synchronize()

    outs = []
    for n, n_bins, keys_h, keys in inputs:
        bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        print("HipHistogramLaunchNoAlloc n=%d n_bins=%d" % (n, n_bins), flush=True)
        xs.check(h.HipHistogramLaunchNoAlloc(stream.cuda_stream, keys.data_ptr(), n, bins.data_ptr(), n_bins))
        outs.append(bins)
    stream.synchronize()

    for (n, n_bins, keys_h, keys), bins in zip(inputs, outs):
        got = bins.cpu().numpy().view(np.uint32)
        assert np.array_equal(got, oracle.histogram(keys_h, n_bins)), (n, "oracle")
        assert np.array_equal(got, _through_xqueue(xs, torch, keys, n, n_bins)), (n, "command")

    # bins are added to, not cleared: the same call again doubles them
    n, n_bins, keys_h, keys = inputs[1]
    xs.check(h.HipHistogramLaunchNoAlloc(stream.cuda_stream, keys.data_ptr(), n, outs[1].data_ptr(), n_bins))
    stream.synchronize()
    assert np.array_equal(outs[1].cpu().numpy().view(np.uint32), 2 * oracle.histogram(keys_h, n_bins))


def test_no_alloc_histogram_refuses_what_its_array_cannot_hold(xs, gpu):
    torch = gpu
    h = xs.halhip()
    keys = torch.zeros(16, dtype=torch.int32, device="cuda")
    bins = torch.zeros(16, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    assert h.HipHistogramLaunchNoAlloc(s, keys.data_ptr(), (1 << 26) + 1, bins.data_ptr(), 16) == xs.kXSchedErrorInvalidValue
    assert h.HipHistogramLaunchNoAlloc(s, keys.data_ptr(), 16, bins.data_ptr(), 65537) == xs.kXSchedErrorInvalidValue
    assert h.HipHistogramLaunchNoAlloc(s, None, 16, bins.data_ptr(), 16) == xs.kXSchedErrorInvalidValue
    assert h.HipHistogramLaunchNoAlloc(s, keys.data_ptr(), 0, bins.data_ptr(), 16) == xs.kXSchedSuccess
    torch.cuda.synchronize()
    assert int(bins.sum()) == 0


def test_no_alloc_histogram_inside_a_captured_graph(xs, gpu):
    """What the entry point is for: two calls captured into one HIP graph (the capture would
    refuse an allocation), the graph replayed three times with eager work and a
    synchronisation between the replays, the bins after every replay against the oracle. The
    array's address is looked up before the capture begins (here by an eager call)."""
    torch = gpu
    h = xs.halhip()
    n_a, n_b, n_bins = (1 << 22) + 77, (1 << 18) - 3, N_BINS
    keys_a_h = oracle.fill_zipf(0, 5, 0, n_a)
    keys_b_h = (np.random.default_rng(4).integers(0, 4096, size=n_b)).astype(np.int32)
    keys_a, keys_b = torch.from_numpy(keys_a_h).cuda(), torch.from_numpy(keys_b_h).cuda()
    bins = torch.zeros(n_bins, dtype=torch.int32, device="cuda")
    once = oracle.histogram(keys_a_h, n_bins).astype(np.uint64) + oracle.histogram(keys_b_h, n_bins).astype(np.uint64)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        xs.check(h.HipHistogramLaunchNoAlloc(side.cuda_stream, keys_b.data_ptr(), n_b, bins.data_ptr(), n_bins))   # set-up: before the capture
    side.synchronize()
    bins.zero_()
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    print("capturing two HipHistogramLaunchNoAlloc calls", flush=True)
    with torch.cuda.graph(graph, stream=side):
        xs.check(h.HipHistogramLaunchNoAlloc(side.cuda_stream, keys_a.data_ptr(), n_a, bins.data_ptr(), n_bins))
        xs.check(h.HipHistogramLaunchNoAlloc(side.cuda_stream, keys_b.data_ptr(), n_b, bins.data_ptr(), n_bins))
    torch.cuda.synchronize()
    assert int(bins.sum()) == 0, "capturing must not run anything"

    other = torch.zeros(1 << 20, device="cuda")
    for replay in (1, 2, 3):
        print("replay", replay, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        got = bins.cpu().numpy().view(np.uint32).astype(np.uint64)
        assert np.array_equal(got, once * replay), "replay %d" % replay
        other.add_(1.0)                          # the program's own eager work between the replays
        torch.cuda.synchronize()
    assert float(other[0]) == 3.0
