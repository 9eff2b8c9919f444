"""GPU tests of the call-level behaviour of the C ABI: per-call settings (opencnn_conv_forward_desc),
the split-merge flag sets of streams and captured graphs, the record of transformed filters, and
the report of a hand-over that gave up.  Results are compared with the drop-in call, which
tests/test_parity_gpu.py holds against the oracle."""
import threading

import numpy as np
import pytest

from test_parity_gpu import Runner, check_against_oracle, make_tensors

pytestmark = pytest.mark.gpu

CUT = (64, 16, 40, 40, 128)     # 800 workgroup tiles on a persistent grid: tiles cut between workgroups
FEW = (32, 512, 7, 7, 512)      # fewer tiles than compute units: hand-overs inside the output transforms
EAGER_SETS, GRAPH_SETS = 32, 16


def hip_runtime():
    """The HIP runtime this process has loaded (torch's copy), for raw stream handles: torch hands
    out streams from a pool of 32, which is exactly the number of flag sets."""
    import ctypes
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(paths) == 1, paths
    return ctypes.CDLL(paths.pop())


def prec_of(ocn, name):
    return {"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[name]


def dropin_with(ocn, r, prec):
    try:
        ocn.set_operand_precision(prec)
        return r.dropin()
    finally:
        ocn.set_operand_precision(ocn.F32)


@pytest.mark.parametrize("prec", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(32, 8, 8, 8, 64), CUT, FEW, (33, 20, 9, 12, 100)])
def test_descriptor_call_matches_the_dropin(ocn, torch_gpu, shape, prec):
    print(f"desc {shape} {prec}", flush=True)
    N, C, H, W, K = shape
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    p = prec_of(ocn, prec)
    try:
        ocn.set_operand_precision(p)
        want = r.split()
        kernel = ocn.last_kernel()
    finally:
        ocn.set_operand_precision(ocn.F32)
    r.raw.fill_(float("nan"))
    # the process-wide setting stays fp32: the descriptor alone selects the precision
    ocn.conv_forward_desc(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, precision=p)
    assert ocn.last_kernel() == kernel
    assert np.array_equal(r.result(), want)
    # split API through the descriptor: the filter transform of the call above is still in Ww
    r.raw.fill_(float("nan"))
    ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, precision=p)
    assert np.array_equal(r.result(), want)
    # KCRS filters
    wk = torch_gpu.from_numpy(np.ascontiguousarray(w.transpose(3, 0, 1, 2))).cuda()
    r.raw.fill_(float("nan"))
    ocn.conv_forward_desc(r.xd, wk, r.yd, r.ws, N, C, H, W, K, precision=p, filter_layout=ocn.FILTER_KCRS)
    assert np.array_equal(r.result(), want)


def test_descriptor_rejects_bad_fields(ocn, torch_gpu):
    import ctypes
    x, w = make_tensors(ocn, 32, 8, 8, 8, 64)
    r = Runner(ocn, torch_gpu, x, w)

    def desc(**over):
        d = ocn.ConvDesc()
        d.struct_size = ctypes.sizeof(ocn.ConvDesc)
        d.in_, d.filter, d.out, d.Ww = r.xd.data_ptr(), r.wd.data_ptr(), r.yd.data_ptr(), r.ws.data_ptr()
        d.in_n, d.in_c, d.in_h, d.in_w, d.filt_k = 32, 8, 8, 8, 64
        d.balanced_split = 1
        for k, v in over.items():
            setattr(d, k, v)
        return ocn.lib().opencnn_conv_forward_desc(ctypes.byref(d))

    assert desc() == 0
    for bad in (dict(struct_size=8), dict(in_=None), dict(out=None), dict(Ww=None), dict(in_n=0),
                dict(operand_precision=3), dict(kernel_variant=9), dict(filter_layout=2),
                dict(split_flags=r.ws.data_ptr(), split_flags_bytes=64),
                dict(split_flags=None, split_flags_bytes=1 << 20)):
        assert desc(**bad) == 1, bad
    assert ocn.lib().opencnn_conv_forward_desc(None) == 1
    torch_gpu.cuda.synchronize()


def test_two_threads_with_their_own_streams_and_precisions(ocn, torch_gpu):
    # the process-wide settings cannot serve two threads; the descriptor can: one thread runs
    # fp32 on its stream, the other bf16 on another, at the same time, on layers whose tiles are
    # cut between workgroups.  Each must reproduce its serial result bit for bit.
    print("two threads", flush=True)
    torch = torch_gpu
    jobs = []
    for shape, prec in ((CUT, "f32"), ((64, 32, 56, 56, 64), "bf16")):
        N, C, H, W, K = shape
        x, w = make_tensors(ocn, N, C, H, W, K)
        r = Runner(ocn, torch, x, w)
        jobs.append((r, prec_of(ocn, prec), dropin_with(ocn, r, prec_of(ocn, prec)), torch.cuda.Stream()))
    torch.cuda.synchronize()
    errors = []

    def work(r, prec, want, stream):
        try:
            for rep in range(10):
                with torch.cuda.stream(stream):
                    r.raw.fill_(float("nan"))
                ocn.conv_forward_desc(r.xd, r.wd, r.yd, r.ws, r.N, r.C, r.H, r.W, r.K, precision=prec,
                                      stream=stream)
                assert ocn.last_launch()[1] >= 0, "ran without the split"
                stream.synchronize()
                got = r.raw.cpu().numpy()[r.GUARD:-r.GUARD].reshape(want.shape)
                assert np.array_equal(got, want), f"rep {rep}"
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(e)

    threads = [threading.Thread(target=work, args=j) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    ocn.check_status()


def test_transformed_filter_of_another_precision_is_rejected(ocn, torch_gpu):
    print("Ww record", flush=True)
    N, C, H, W, K = 32, 16, 9, 9, 64
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    want = r.split()
    try:
        ocn.set_operand_precision(ocn.F16)
        ocn.filter_transform(r.wd, r.ws, K, C, ocn.FILTER_CRSK, ocn.WW_MFMA)
    finally:
        ocn.set_operand_precision(ocn.F32)
    with pytest.raises(ocn.OpenCNNError) as e:  # a 2-byte Ww under fp32 operands
        ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
    assert e.value.status == 1 and "precision" in e.value.detail
    with pytest.raises(ocn.OpenCNNError):
        ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, precision=ocn.BF16)
    ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, precision=ocn.F16)  # the matching one
    torch_gpu.cuda.synchronize()
    # the reference layout is not what the fused kernel reads
    ocn.filter_transform(r.wd, r.ws, K, C, ocn.FILTER_CRSK, ocn.WW_REFERENCE)
    with pytest.raises(ocn.OpenCNNError) as e:
        ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
    assert "layout" in e.value.detail
    # another filter shape at the same address
    ocn.filter_transform(r.wd, r.ws, K // 2, C * 2, ocn.FILTER_CRSK, ocn.WW_MFMA)
    with pytest.raises(ocn.OpenCNNError) as e:
        ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
    assert "shape" in e.value.detail
    # a buffer filled by other means: forget the record, the library takes it as it is
    ocn.filter_transform(r.wd, r.ws, K, C, ocn.FILTER_CRSK, ocn.WW_MFMA)
    saved = r.ws.clone()
    ocn.filter_transform(r.wd, r.ws, K, C, ocn.FILTER_CRSK, ocn.WW_REFERENCE)
    r.ws.copy_(saved)
    ocn.forget_workspace(r.ws)
    r.raw.fill_(float("nan"))
    ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
    assert np.array_equal(r.result(), want)


@pytest.mark.parametrize("shape", [CUT, FEW])
def test_split_flags_owned_by_the_caller(ocn, torch_gpu, shape):
    print(f"caller flags {shape}", flush=True)
    torch = torch_gpu
    N, C, H, W, K = shape
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.dropin()
    grid, flag_set = ocn.last_launch()
    assert 0 <= flag_set < EAGER_SETS
    flags = torch.zeros(ocn.split_flags_bytes() // 4, dtype=torch.int32, device="cuda")
    for rep in range(3):  # the flags are back at zero after every launch
        r.raw.fill_(float("nan"))
        ocn.conv_forward_desc(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, split_flags=flags)
        assert ocn.last_launch() == (grid, EAGER_SETS + GRAPH_SETS)
        assert np.array_equal(r.result(), want)
        assert int(flags.abs().sum()) == 0
    # and without the split: another grid, the same tensor up to the association of the sum
    r.raw.fill_(float("nan"))
    ocn.conv_forward_desc(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, balanced_split=False)
    assert ocn.last_launch()[1] == -1
    y = r.result()
    assert np.abs(y - want).max() <= 1e-4 * np.abs(want).max()
    ocn.release_split_flags(flags)  # the library forgets the buffer before it is freed


def test_more_streams_than_flag_sets(ocn, torch_gpu):
    # The library has 32 flag sets for streams and never asks a foreign stream for its state.
    # Once more streams have launched than there are sets, every launch leaves an event behind,
    # and a stream without a set takes over the longest-unused set whose event has completed.
    import ctypes
    print("40 streams", flush=True)
    torch = torch_gpu
    hip = hip_runtime()
    N, C, H, W, K = CUT
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.split()
    grid, _ = ocn.last_launch()

    def make_streams(n):
        out = []
        for _ in range(n):
            h = ctypes.c_void_p()
            assert hip.hipStreamCreateWithFlags(ctypes.byref(h), 1) == 0  # hipStreamNonBlocking
            out.append(h.value)
        return out

    def launch_on(streams):
        sets = []
        for s in streams:
            r.raw.fill_(float("nan"))
            torch.cuda.synchronize()
            ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, stream=s)
            g, flag_set = ocn.last_launch()
            assert (g == grid) == (flag_set >= 0) and flag_set < EAGER_SETS
            y = r.result()
            if flag_set >= 0:
                assert np.array_equal(y, want)
            else:  # without the split: another association of the channel sum
                assert np.abs(y - want).max() <= 1e-4 * np.abs(want).max()
            sets.append(flag_set)
        return sets

    streams = make_streams(40)
    first = launch_on(streams)          # the sets run out: the last streams launch without the split
    assert first[-1] == -1 and len(set(first) - {-1}) == len([s for s in first if s >= 0])
    launch_on(streams)                  # now every launch leaves an event: sets start to change hands
    third = launch_on(streams)
    assert min(third) >= 0, "a stream found no idle set although every launch had completed"
    # streams that no longer exist: their sets are taken over just the same
    torch.cuda.synchronize()
    for s in streams[8:]:
        assert hip.hipStreamDestroy(ctypes.c_void_p(s)) == 0
    fresh = make_streams(40)
    assert min(launch_on(fresh)) >= 0
    # an explicit release: the set is free at once
    before = launch_on(streams[:8])
    for s in streams[:8]:
        ocn.release_stream(s)
    again = launch_on(streams[:8])
    assert min(before) >= 0 and min(again) >= 0
    torch.cuda.synchronize()
    for s in streams[:8] + fresh:
        ocn.release_stream(s)
        assert hip.hipStreamDestroy(ctypes.c_void_p(s)) == 0
    ocn.check_status()


def test_replay_of_a_graph_overlaps_launches_on_its_capture_stream(ocn, torch_gpu):
    # A launch recorded in a capture gets flags of its own (one of the graph sets), not those of
    # the stream it was recorded on: the graph may be replayed on another stream while that stream
    # launches directly.  Both layers have tiles cut between workgroups.
    print("graph next to eager launches", flush=True)
    torch = torch_gpu
    ocn.init()
    N, C, H, W, K = CUT
    x, w = make_tensors(ocn, N, C, H, W, K)
    rg, re = Runner(ocn, torch, x, w), Runner(ocn, torch, x, w)
    want = rg.split()
    re.split()
    s, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    ocn.conv_forward_desc(re.xd, None, re.yd, re.ws, N, C, H, W, K, stream=s)
    eager_set = ocn.last_launch()[1]
    s.synchronize()
    with torch.cuda.graph(g, stream=s):
        ocn.conv_forward_desc(rg.xd, None, rg.yd, rg.ws, N, C, H, W, K, stream=s)
    grid, graph_set = ocn.last_launch()
    assert 0 <= eager_set < EAGER_SETS <= graph_set < EAGER_SETS + GRAPH_SETS
    assert ocn.last_kernel().startswith("wino_f32_asm") and grid == 256
    for rep in range(3):
        rg.raw.fill_(float("nan"))
        re.raw.fill_(float("nan"))
        torch.cuda.synchronize()
        with torch.cuda.stream(s2):
            g.replay()
        for _ in range(3):
            ocn.conv_forward_desc(re.xd, None, re.yd, re.ws, N, C, H, W, K, stream=s)
        with torch.cuda.stream(s2):
            g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(rg.result(), want), f"replay {rep}"
        assert np.array_equal(re.result(), want), f"eager launches next to replay {rep}"
    ocn.check_status()


def test_graph_flag_sets_are_given_back(ocn, torch_gpu):
    # A launch recorded in a stream capture holds one of 16 graph sets until the caller gives it
    # back: a service that captures a graph per shape would otherwise lose the balanced split from
    # its 17th capture on.
    print("graph flag sets", flush=True)
    torch = torch_gpu
    ocn.init()
    N, C, H, W, K = CUT
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.split()
    grid = ocn.last_launch()[0]
    s = torch.cuda.Stream()
    ocn.release_capture(None)  # the graphs of earlier tests are gone

    def capture():
        g = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, stream=s)
        return g, ocn.last_launch()

    def replay_is_right(g):
        r.raw.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        return np.array_equal(r.result(), want)

    # without a release the sets run out, and the counter says so
    held = [capture() for _ in range(GRAPH_SETS)]
    assert sorted(f for _, (_, f) in held) == list(range(EAGER_SETS, EAGER_SETS + GRAPH_SETS))
    assert all(gr == grid for _, (gr, _) in held)
    before = ocn.unsplit_launches()
    g17, (grid17, set17) = capture()
    assert set17 == -1 and grid17 != grid and ocn.unsplit_launches() == before + 1
    y = None
    r.raw.fill_(float("nan"))
    torch.cuda.synchronize()
    g17.replay()
    y = r.result()  # without the split: another association of the channel sum
    assert np.abs(y - want).max() <= 1e-4 * np.abs(want).max()
    assert replay_is_right(held[3][0]) and replay_is_right(held[15][0])
    # one set given back by number: the next capture gets exactly that one
    del g17
    torch.cuda.synchronize()
    ocn.release_capture(None, held[5][1][1])
    g, (gr, f) = capture()
    assert (gr, f) == (grid, held[5][1][1]) and replay_is_right(g)
    # all of this stream's sets given back, then twenty captures in a row, each released
    del held, g
    torch.cuda.synchronize()
    ocn.release_capture(s)
    before = ocn.unsplit_launches()
    for i in range(20):
        g, (gr, f) = capture()
        assert gr == grid and f >= EAGER_SETS, f"capture {i} ran without the split"
        assert replay_is_right(g), f"capture {i}"
        del g
        torch.cuda.synchronize()
        ocn.release_capture(None, f)
    assert ocn.unsplit_launches() == before
    with pytest.raises(ocn.OpenCNNError):
        ocn.release_capture(None, 3)  # a stream's set is not a graph set
    ocn.check_status()


def test_a_launch_that_cuts_no_tile_takes_no_flag_set(ocn, torch_gpu):
    # 256 workgroup tiles on 256 compute units, one tile per workgroup, and the plumbing layer:
    # nothing is handed over, so no set is taken (and none can run out).
    print("no flag set", flush=True)
    torch = torch_gpu
    for shape in ((32, 16, 32, 16, 256), (32, 8, 8, 8, 64)):
        N, C, H, W, K = shape
        x, w = make_tensors(ocn, N, C, H, W, K)
        r = Runner(ocn, torch, x, w)
        before = ocn.unsplit_launches()
        r.split()
        assert ocn.last_launch()[1] == -1, shape
        assert ocn.unsplit_launches() == before


def test_caller_flag_buffers_report_on_their_own(ocn, torch_gpu):
    # Every caller-owned flag buffer has its own status word: a hand-over that gave up on buffer A
    # is reported by the next call that brings A (which also clears A), never by a call on B.
    print("caller buffers, status", flush=True)
    torch = torch_gpu
    N, C, H, W, K = FEW
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.split()
    nwords = ocn.split_flags_bytes() // 4
    A = torch.zeros(nwords, dtype=torch.int32, device="cuda")
    B = torch.zeros(nwords, dtype=torch.int32, device="cuda")

    def call(flags):
        r.raw.fill_(float("nan"))
        ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, split_flags=flags)
        return r.result()

    assert np.array_equal(call(A), want) and np.array_equal(call(B), want)
    gave_up = False
    try:
        ocn.set_wait_limit(1)
        for _ in range(4):
            if not np.array_equal(call(A), want):
                gave_up = True
                break
    except ocn.OpenCNNError as e:
        assert e.status == 719
        pytest.fail("a give-up on A must be reported by the call after it, not by the one that gives up")
    finally:
        ocn.set_wait_limit(0)
    if not gave_up:
        ocn.release_split_flags(A)
        ocn.release_split_flags(B)
        pytest.skip("every hand-over found its partial tile at the first poll")
    # B is clean and says nothing
    assert np.array_equal(call(B), want)
    # A reports once and is cleared by that call; then it works again
    with pytest.raises(ocn.OpenCNNError) as e:
        call(A)
    assert e.value.status == 719 and "gave up" in e.value.detail
    torch.cuda.synchronize()
    assert int(A.abs().sum()) == 0
    assert np.array_equal(call(A), want) and np.array_equal(call(B), want)
    ocn.check_status()
    ocn.release_split_flags(A)
    ocn.release_split_flags(B)


def test_caller_flag_buffers_beyond_the_table_are_refused(ocn, torch_gpu):
    print("caller buffers, table", flush=True)
    torch = torch_gpu
    N, C, H, W, K = CUT
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.split()
    nwords = ocn.split_flags_bytes() // 4
    pool = torch.zeros(65 * nwords, dtype=torch.int32, device="cuda")
    bufs = [pool[i * nwords:(i + 1) * nwords] for i in range(65)]
    try:
        for b in bufs[:64]:
            ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, split_flags=b)
        assert np.array_equal(r.result(), want)
        r.raw.fill_(float("nan"))
        with pytest.raises(ocn.OpenCNNError) as e:
            ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, split_flags=bufs[64])
        assert e.value.status == 1 and "opencnn_release_split_flags" in e.value.detail
        torch.cuda.synchronize()
        assert torch.isnan(r.raw).all(), "a refused call must launch nothing"
        ocn.release_split_flags(bufs[7])
        ocn.conv_forward_desc(r.xd, None, r.yd, r.ws, N, C, H, W, K, split_flags=bufs[64])
        assert np.array_equal(r.result(), want)
    finally:
        torch.cuda.synchronize()
        for b in bufs:
            ocn.release_split_flags(b)


def test_a_wait_that_gives_up_is_reported(ocn, oracle, torch_gpu):
    # Forced from the host: with a limit of one poll, a workgroup that does not find its
    # neighbour's partial tile at once gives up (every wave still ends normally).  The launch's
    # output is then wrong; the status check says so, the next call on the stream fails with
    # hipErrorLaunchFailure and clears the flags, and the call after that is right again.
    print("wait limit", flush=True)
    torch = torch_gpu
    N, C, H, W, K = FEW
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch, x, w)
    want = r.split()
    assert ocn.last_launch()[0] > 64, "the layer's tiles are not cut among workgroups"
    ocn.check_status()
    gave_up = False
    try:
        ocn.set_wait_limit(1)
        for _ in range(4):
            r.raw.fill_(float("nan"))
            try:
                ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
            except ocn.OpenCNNError as e:  # the call after a launch that gave up
                assert e.status == 719 and "gave up" in e.detail
                gave_up = True
                break
            y = r.result()  # synchronises
            if not np.array_equal(y, want):
                # a wrong tile must never go unreported
                with pytest.raises(ocn.OpenCNNError) as e:
                    ocn.check_status()
                assert e.value.status == 719
                gave_up = True
                break
    finally:
        ocn.set_wait_limit(0)
    torch.cuda.synchronize()
    if not gave_up:
        pytest.skip("every hand-over found its partial tile at the first poll")
    ocn.check_status()  # reported once, and the flags are clean again
    for _ in range(3):
        r.raw.fill_(float("nan"))
        ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, N, C, H, W, K)
        assert np.array_equal(r.result(), want)
    ocn.check_status()


def test_timing_entry_point(ocn, oracle, torch_gpu):
    # opencnn_time_forward, the library-side twin of the reference's timing loop
    # (src/openCNN_winograd.cu:426-444): plausible times, only the loops asked for run, and the
    # tensors it leaves behind are the layer's.
    print("time_forward", flush=True)
    N, C, H, W, K = 32, 16, 12, 12, 64
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    total, main, fx = ocn.time_forward(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, warmup=2, iters=20)
    # (three separate passes of 20 calls: plausible magnitudes, no order between them asserted)
    assert 0 < fx < 1.0 and 0 < main < 1.0 and 0 < total < 1.0
    check_against_oracle(oracle, r.result(), x, w)
    only_main = ocn.time_forward(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, warmup=0, iters=5, parts=("main",))
    assert only_main[0] == 0 and only_main[1] > 0 and only_main[2] == 0
    for bad in (dict(iters=0), dict(warmup=-1)):
        with pytest.raises(ocn.OpenCNNError):
            ocn.time_forward(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, **bad)
    try:  # the process-wide precision applies, as for convolutionForward
        ocn.set_operand_precision(ocn.BF16)
        ocn.time_forward(r.xd, r.wd, r.yd, r.ws, N, C, H, W, K, warmup=1, iters=3)
        assert "bf16" in ocn.last_kernel()
    finally:
        ocn.set_operand_precision(ocn.F32)
    torch_gpu.cuda.synchronize()
    ocn.check_status()
