"""Several host threads, each on a stream of its own, calling the library at the same time: the state the library
keeps per process (the kernels' LDS-size registrations, the recorders' ticket slots, the cut table) and per thread
(the last error, the convolution plans) must not leak from one caller into another.  Every thread repeats a mix of
calls and compares each result, bit for bit, with what the same call gave before the threads started."""
import threading

import numpy as np
import pytest
import torch

from nnabla_amd import kernels

pytestmark = pytest.mark.gpu


def _mix(dev, seed):
    """A list of (name, thunk); a thunk runs on the current stream and returns the tensors to compare."""
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn(300, 1000, generator=g, device=dev) * 2
    xa = torch.randn(96, 512, generator=g, device=dev)
    Wa = torch.randn(512, 640, generator=g, device=dev) * 0.05
    xc = torch.randn(2, 32, 9, 9, generator=g, device=dev)
    Wc = torch.randn(40, 32, 3, 3, generator=g, device=dev) * 0.05
    xm = torch.randn(4, 8, 16, 16, generator=g, device=dev).abs()
    q = lambda v: torch.full((1, 8, 1, 1), v, dtype=torch.float32, device=dev)

    def minmax():
        lo, hi = q(-6.0), q(6.0)
        y, scale = kernels.min_max_quantize(xm, lo, hi, q(0.0), q(255.0), 0.999, True, True)
        return y, scale, lo, hi

    def recorder():
        m = torch.zeros(1, device=dev)
        M = torch.zeros(1, device=dev)
        y = kernels.range_recorder(x, m, M, "MinMaxMvaRecorder", 0.99, True)
        return y, m, M

    return [
        ("fixed_point", lambda: (kernels.fixed_point_quantize(x, True, 8, 2.0 ** -4),)),
        ("pow2", lambda: (kernels.pow2_quantize(x, True, True, 4, 1),)),
        ("min_max", minmax),
        ("recorder", recorder),
        ("affine", lambda: kernels.binary_weight_affine(xa, Wa)),
        ("affine_small", lambda: kernels.binary_weight_affine(xa[:4].contiguous(), Wa)),
        ("convolution", lambda: kernels.binary_weight_convolution(xc, Wc, None, (1, 1), (1, 1), (1, 1), 1)),
        ("prune", lambda: (kernels.prune(x, 0.7),)),
    ]


def test_threads_on_their_own_streams_get_their_own_results(dev):
    n_threads, rounds = 4, 25
    mixes = [_mix(dev, 50 + t) for t in range(n_threads)]
    expected = [[tuple(o.clone() for o in thunk()) for _, thunk in mix] for mix in mixes]
    torch.cuda.synchronize()
    failures = []
    start = threading.Barrier(n_threads)

    def work(t):
        try:
            stream = torch.cuda.Stream(device=dev)   # default priority
            with torch.cuda.stream(stream):
                start.wait()
                for r in range(rounds):
                    order = np.random.RandomState(1000 * t + r).permutation(len(mixes[t]))
                    for i in order:
                        name, thunk = mixes[t][i]
                        got = thunk()
                        stream.synchronize()
                        for a, b in zip(got, expected[t][i]):
                            if not torch.equal(a.view(torch.int32), b.view(torch.int32)):
                                failures.append("thread %d round %d %s" % (t, r, name))
                # an error in one thread is this thread's alone
                with pytest.raises(kernels.KernelError):
                    kernels.fixed_point_quantize(mixes[t][0][1]()[0], True, 0, 1.0)
        except Exception as e:   # noqa: BLE001 -- reported below, in the main thread
            failures.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=240)
    assert not any(th.is_alive() for th in threads), "a thread did not finish"
    assert not failures, failures[:5]
