"""GPU: the library-owned scratch memory (split-K partial tiles and tickets, expert-layer
intermediates) is per (device, stream) for eager calls and per device for recorded graphs:
host threads on separate streams do not disturb each other, a buffer is never freed under a graph
that uses it, and nothing is allocated while a stream is capturing."""

import threading

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import dtypes
from oracle import torch_ref as tr
from tests.test_gemm_gpu import assert_close_to_f64, make_problem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN_NAMES = "a8w8_blockscale_1x128x128_256x16x64x256_16x16_16x16_1x1_16x16x1_16x16x1_1x16x1x16_4_1x1_intrawave_v1"


def on_device(*ts):
    return [t.to(DEV) for t in ts]


def gemm(a, n, m, split=-1, kernel=""):
    out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(*a, out, splitK=split, kernelName=kernel)
    return out


def test_two_host_threads_on_separate_streams():
    # two shapes whose automatic kernel splits K across workgroups (partial tiles + tickets in scratch)
    shapes = [(16, 1024, 7168), (32, 512, 4096)]
    for m, n, k in shapes:
        assert aiter_amd._ffi.gemm_choice(m, n, k) == "decode_stream"
    problems = [on_device(*make_problem(m, n, k, seed=11 + i)) for i, (m, n, k) in enumerate(shapes)]
    expected = [gemm(p, n, m) for p, (m, n, k) in zip(problems, shapes)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    results = [[], []]
    errors = []

    def worker(i):
        try:
            m, n, k = shapes[i]
            with torch.cuda.stream(streams[i]):
                for _ in range(150):
                    results[i].append(gemm(problems[i], n, m))
            streams[i].synchronize()
        except Exception as e:  # surfaced below: an exception in a thread must fail the test
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for i in range(2):
        want = expected[i].view(torch.int16)
        bad = sum(int(not torch.equal(r.view(torch.int16), want)) for r in results[i])
        assert bad == 0, f"thread {i}: {bad} of {len(results[i])} results differ from the single-threaded one"


def test_same_stream_from_two_threads_is_serialised():
    # the mid_* family uses two launches per call (partial tiles, then their sum): calls of two
    # threads on ONE stream must not interleave them
    shapes = [(128, 512, 2048), (96, 768, 1536)]
    problems = [on_device(*make_problem(m, n, k, seed=21 + i)) for i, (m, n, k) in enumerate(shapes)]
    expected = [gemm(p, n, m, kernel="mid_64x64:s=4") for p, (m, n, k) in zip(problems, shapes)]
    torch.cuda.synchronize()
    results = [[], []]
    errors = []

    def worker(i):
        try:
            m, n, k = shapes[i]
            for _ in range(100):
                results[i].append(gemm(problems[i], n, m, kernel="mid_64x64:s=4"))
        except Exception as e:
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i in range(2):
        want = expected[i].view(torch.int16)
        assert all(torch.equal(r.view(torch.int16), want) for r in results[i])


def test_nothing_is_allocated_under_capture_and_the_capture_survives():
    # 5 K ranges x 2048 x 8192 fp32 = 320 MiB of partial tiles: above what is kept ready for graphs,
    # so recording this call fails whatever ran before -- cleanly, and without harming the capture
    m, n, k = 2048, 8192, 1280
    a = on_device(*make_problem(m, n, k, seed=31))
    eager = gemm(a, n, m, kernel="mid_128x128:s=5")
    small = on_device(*make_problem(16, 1024, 7168, seed=32))
    small_eager = gemm(small, 1024, 16)          # warms the per-device graph scratch for this call
    torch.cuda.synchronize()
    assert_close_to_f64(eager, *[t.cpu() for t in a], "mid_128x128:s=5 eager")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    out_small = torch.zeros(16, 1024, dtype=torch.bfloat16, device=DEV)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            with pytest.raises(RuntimeError, match="capturing"):
                gemm(a, n, m, kernel="mid_128x128:s=5")
            aiter_amd.gemm_a8w8_blockscale_ck(*small, out_small, splitK=-1)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_small.view(torch.int16), small_eager.view(torch.int16))


def test_growth_keeps_recorded_graphs_valid():
    m, n, k = 32, 768, 7168
    a = on_device(*make_problem(m, n, k, seed=41))
    eager = gemm(a, n, m)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    out = torch.zeros(m, n, dtype=torch.bfloat16, device=DEV)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            aiter_amd.gemm_a8w8_blockscale_ck(*a, out, splitK=-1)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), eager.view(torch.int16))
    # eager calls that need ever more scratch make the library replace its buffers (eager and graph side)
    for s, (mm, nn, kk) in ((2, (512, 4096, 1024)), (4, (1024, 4096, 1024)), (6, (1024, 8192, 1024))):
        b = on_device(*make_problem(mm, nn, kk, seed=42 + s))
        big = gemm(b, nn, mm, kernel=f"mid_128x128:s={s}")
        torch.cuda.synchronize()
        assert_close_to_f64(big, *[t.cpu() for t in b], f"mid_128x128:s={s}")
        out.zero_()
        graph.replay()               # still points at the buffers it was recorded with
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16))


def test_forked_streams_of_one_capture_get_scratch_of_their_own():
    # two split-K calls recorded on two forked streams of one capture may run side by side on replay:
    # each stream of the capture gets a lane of the graph scratch to itself, provided as many streams
    # ran scratch-using calls eagerly before (here: the warm-up forks the same way)
    shapes = [(16, 1024, 7168), (32, 512, 4096)]
    problems = [on_device(*make_problem(m, n, k, seed=51 + i)) for i, (m, n, k) in enumerate(shapes)]
    main, side = torch.cuda.Stream(), torch.cuda.Stream()
    eager = []
    for st, p, (m, n, k) in zip((main, side), problems, shapes):
        with torch.cuda.stream(st):
            eager.append(gemm(p, n, m))
    torch.cuda.synchronize()
    outs = [torch.zeros(m, n, dtype=torch.bfloat16, device=DEV) for (m, n, k) in shapes]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(main):
        with torch.cuda.graph(graph, stream=main):
            side.wait_stream(main)
            with torch.cuda.stream(side):
                for _ in range(4):
                    aiter_amd.gemm_a8w8_blockscale_ck(*problems[1], outs[1], splitK=-1)
            for _ in range(4):
                aiter_amd.gemm_a8w8_blockscale_ck(*problems[0], outs[0], splitK=-1)
            main.wait_stream(side)
    for _ in range(20):
        for o in outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, e in zip(outs, eager):
            assert torch.equal(o.view(torch.int16), e.view(torch.int16))
    # a capture that records such calls on more streams than there are lanes is refused with a message,
    # and stays usable
    forks = [torch.cuda.Stream() for _ in range(5)]
    graph2 = torch.cuda.CUDAGraph()
    refused = 0
    with torch.cuda.stream(main):
        with torch.cuda.graph(graph2, stream=main):
            aiter_amd.gemm_a8w8_blockscale_ck(*problems[0], outs[0], splitK=-1)  # takes its lane first
            for f in forks:
                f.wait_stream(main)
                with torch.cuda.stream(f):
                    try:
                        aiter_amd.gemm_a8w8_blockscale_ck(*problems[1], outs[1], splitK=-1)
                    except RuntimeError as e:
                        assert "more streams" in str(e)
                        refused += 1
                main.wait_stream(f)
    assert refused >= 2  # at most four lanes, one of them the first stream's
    outs[0].zero_()
    graph2.replay()
    torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int16), eager[0].view(torch.int16))


def test_eager_growth_beside_another_threads_capture():
    # thread A records a warmed call while thread B, on a stream that never held scratch, makes a call that
    # must allocate: B's allocation happens with the thread's capture mode relaxed, so A's capture (global
    # mode, torch's default) stays valid; should the runtime refuse B all the same, B gets the documented error
    m, n, k = 16, 1024, 7168
    a = on_device(*make_problem(m, n, k, seed=61))
    want_a = gemm(a, n, m)
    mb, nb, kb = 256, 2112, 7168
    b = on_device(*make_problem(mb, nb, kb, seed=62))
    want_b = gemm(b, nb, mb, kernel="mid_64x64:s=7")
    torch.cuda.synchronize()
    out_a = torch.zeros(m, n, dtype=torch.bfloat16, device=DEV)
    out_b = torch.zeros(mb, nb, dtype=torch.bfloat16, device=DEV)
    stream_a, stream_b = torch.cuda.Stream(), torch.cuda.Stream()
    capture_open, b_done = threading.Event(), threading.Event()
    b_error = []

    def thread_b():
        capture_open.wait(timeout=60)
        try:
            with torch.cuda.stream(stream_b):  # a fresh stream: its first scratch-using call allocates
                aiter_amd.gemm_a8w8_blockscale_ck(*b, out_b, splitK=-1, kernelName="mid_64x64:s=7")
        except RuntimeError as e:
            b_error.append(str(e))
        finally:
            b_done.set()

    tb = threading.Thread(target=thread_b)
    tb.start()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream_a):
        with torch.cuda.graph(graph, stream=stream_a):
            capture_open.set()
            assert b_done.wait(timeout=60)
            aiter_amd.gemm_a8w8_blockscale_ck(*a, out_a, splitK=-1)
    tb.join()
    for _ in range(3):
        out_a.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_a.view(torch.int16), want_a.view(torch.int16))
    if b_error:
        assert "another thread captures" in b_error[0], b_error
    else:
        assert torch.equal(out_b.view(torch.int16), want_b.view(torch.int16))


@pytest.mark.parametrize("m,n,k,s", [(1040, 128, 7168, 2), (1934, 128, 7168, 1), (2000, 128, 7168, 2), (3258, 128, 7168, 3)])
def test_tuned_rows_with_split_hint(m, n, k, s):
    # rows of the reference's tuned table with splitK > 0 and M >= 1024, forwarded as its callers do
    a = make_problem(m, n, k, seed=m)
    dev = on_device(*a)
    with_name = gemm(dev, n, m, split=s, kernel=GOLDEN_NAMES)
    bare = gemm(dev, n, m, split=s)
    auto = gemm(dev, n, m)
    torch.cuda.synchronize()
    assert_close_to_f64(with_name, *a, f"{m}x{n}x{k} splitK={s} with the reference's kernel name")
    assert_close_to_f64(bare, *a, f"{m}x{n}x{k} splitK={s}")
    # the reference's name is dropped together with its splitK: same bits as the automatic call
    assert torch.equal(with_name.view(torch.int16), auto.view(torch.int16))


@pytest.mark.parametrize("m,n,k", [(4, 2112, 7168), (200, 1024, 2048), (600, 4096, 1024)])
def test_any_split_hint_is_served(m, n, k):
    a = make_problem(m, n, k, seed=k + m)
    dev = on_device(*a)
    for s in (0, 1, 3, 5, 12, 30):
        for kernel in ("", "prefill_256x256", "tile_64x128"):
            out = gemm(dev, n, m, split=s, kernel=kernel)
            torch.cuda.synchronize()
            assert_close_to_f64(out, *a, f"{m}x{n}x{k} splitK={s} kernel={kernel!r}")
