"""Several host threads, each on a stream of its own, run different convolutions through the library at once.

A framework calls the operators from more than one thread (autograd runs backward passes on threads of its own) and
the reference's operations are entered from whichever thread TensorFlow schedules (src/backend/op_collections.hpp:
121-144 keeps its cache behind a mutex).  Here the per-call state (packing session, group steps, addend, kernel
label) is thread-local, the plan cache sits behind a mutex and the per-device set-up is done once: every thread must
get, bit for bit, what the same calls give when they run alone."""
import threading

import pytest
import torch

import phoenix_core_amd as phx
from phoenix_core_amd import capi, ops

pytestmark = pytest.mark.gpu


def Ctx(mode, policy):
    env = {"UPSTRIDE_CONV_FP16_POLICY": policy}
    if mode == 16:
        env["UPSTRIDE_MEMORY_OPTIMIZED"] = "1"
    return phx.Context(env)


# dtype, policy, mode, n, ci, co, h, w, k, stride, groups, channels-last
PROBLEMS = [
    (torch.float16, "full16", 8, 4, 32, 64, 14, 14, 3, 1, 1, False),
    (torch.float16, "full16", 16, 2, 64, 64, 9, 11, 1, 1, 1, False),      # pointwise
    (torch.float16, "full16", 8, 1, 256, 128, 7, 7, 3, 1, 1, False),      # small batch: reduction slices
    (torch.float16, "backward32", 8, 2, 16, 24, 12, 10, 3, 2, 1, False),  # strided, fp32 backward arithmetic
    (torch.float16, "full16", 8, 2, 32, 32, 10, 10, 3, 1, 32, False),     # depthwise: vector-ALU kernels
    (torch.float16, "full16", 8, 2, 32, 32, 9, 8, 3, 1, 8, False),        # merged groups
    (torch.float16, "full16", 8, 3, 16, 40, 8, 8, 3, 1, 1, True),         # channels-last
    (torch.float32, "fp32", 8, 2, 12, 20, 11, 9, 3, 1, 1, False),
    (torch.float32, "fp32", 16, 1, 128, 64, 6, 6, 1, 1, 1, False),        # fp32, sliced
    (torch.float32, "fp32", 8, 2, 8, 8, 13, 13, 5, 2, 1, False),
]


def make(problem, seed):
    dtype, policy, mode, n, ci, co, h, w, k, stride, groups, cl = problem
    gen = torch.Generator(device="cuda").manual_seed(seed)
    scale = 1.0 if dtype == torch.float32 else 0.5
    xs = (4 * n, h, w, ci) if cl else (4 * n, ci, h, w)
    x = (scale * torch.randn(xs, device="cuda", generator=gen)).to(dtype)
    wt = (scale * torch.randn((4, co, ci // groups, k, k), device="cuda", generator=gen) * (2.0 / (k * k * ci // groups)) ** 0.5).to(dtype)
    b = (scale * torch.randn((4, co), device="cuda", generator=gen)).to(dtype)
    desc = phx.Conv2DDescriptor(x.shape, wt.shape, stride, 1, "SAME", groups=groups, use_bias=True, dtype=dtype, context=Ctx(mode, policy),
                                data_format="NHWC" if cl else "NCHW")
    g = (scale * torch.randn(desc.output_shape, device="cuda", generator=gen)).to(dtype)
    return desc, x, wt, b, g


def run(desc, x, wt, b, g):
    y = phx.conv2d_fwd(x, wt, b, desc)
    dw, dx = phx.conv2d_bwd(x, wt, g, desc)
    return y, dw, dx


def test_threads_on_their_own_streams_get_what_the_calls_give_alone():
    capi.init()
    cases = [make(p, 100 + i) for i, p in enumerate(PROBLEMS)]
    want = [run(*c) for c in cases]
    torch.cuda.synchronize()
    nthreads, rounds = 4, 6
    errors = []
    start = threading.Barrier(nthreads)

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            order = [(i * (2 * tid + 1) + tid) % len(cases) for i in range(len(cases))]  # a different order per thread
            start.wait()
            with torch.cuda.stream(stream):
                for r in range(rounds):
                    got = [(i, run(*cases[i])) for i in order]
                    stream.synchronize()
                    for i, outs in got:
                        for name, a, e in zip(("y", "dw", "dx"), outs, want[i]):
                            if not torch.equal(a, e):
                                errors.append("thread %d round %d problem %d: %s differs" % (tid, r, i, name))
        except Exception as exc:  # (an exception in a thread would otherwise pass silently)
            errors.append("thread %d: %r" % (tid, exc))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors[:5]


def test_threads_share_the_plan_cache_while_it_evicts():
    """More distinct problems than the plan cache holds, planned from four threads at once: entries are evicted and
    planned again under the cache's mutex while other threads look theirs up."""
    capi.init()
    shapes = [(1, 8 + 8 * (i % 7), 8 + 8 * (i % 5), 5 + i % 9, 6 + i % 11, 1 + 2 * (i % 2)) for i in range(140)]
    errors = []

    def one(shape, seed):
        n, ci, co, h, w, k = shape
        gen = torch.Generator(device="cuda").manual_seed(seed)
        x = (0.5 * torch.randn((4 * n, ci, h, w), device="cuda", generator=gen)).half()
        wt = (0.5 * torch.randn((4, co, ci, k, k), device="cuda", generator=gen) * (2.0 / (k * k * ci)) ** 0.5).half()
        desc = phx.Conv2DDescriptor(x.shape, wt.shape, 1, 1, "SAME", dtype=torch.float16, context=Ctx(8, "full16"))
        g = (0.5 * torch.randn(desc.output_shape, device="cuda", generator=gen)).half()
        return phx.conv2d_fwd(x, wt, None, desc), ops.conv2d_bwd_data(wt, g, desc), ops.conv2d_bwd_weights(x, g, desc)

    want = [one(s, i) for i, s in enumerate(shapes)]
    torch.cuda.synchronize()

    def worker(tid):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for i in range(tid, len(shapes), 2):  # (every problem is planned by two of the four threads)
                    got = one(shapes[i], i)
                    torch.cuda.current_stream().synchronize()
                    if not all(torch.equal(a, e) for a, e in zip(got, want[i])):
                        errors.append("thread %d problem %d differs" % (tid, i))
        except Exception as exc:
            errors.append("thread %d: %r" % (tid, exc))

    threads = [threading.Thread(target=worker, args=(t % 2,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors[:5]
