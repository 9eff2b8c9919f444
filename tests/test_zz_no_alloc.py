"""GPU test of opencnn_conv_forward_static, the entry point that allocates nothing: same result,
bit for bit, as convolutionForward (it runs the same two kernels; only the transformed filter
lives in the library's static workspace instead of a caller's buffer), on two calls in a row
that share the workspace, the second with a smaller layer.  And the property it exists for: free
device memory does not move across its first and second call in a fresh process, it can be
recorded into a HIP graph (an allocation under capture would fail the capture), and without
opencnn_init() it refuses and launches nothing.
"""
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu

SEED_X, SEED_W = 0x0C99, 0xF117
GUARD = 4096


def _layer(ocn, torch, N, C, H, K, seed_shift=0):
    x = ocn.synth_input(N, C, H, H, seed=SEED_X + seed_shift)
    w = ocn.synth_filter(K, C, seed=SEED_W + seed_shift)
    dev = torch.device("cuda:0")
    return dict(N=N, C=C, H=H, K=K, xd=torch.from_numpy(x).to(dev), wd=torch.from_numpy(w).to(dev), x=x, w=w)


def _guarded(torch, n):
    raw = torch.full((n + 2 * GUARD,), float("nan"), device="cuda:0")
    return raw, raw[GUARD:GUARD + n]


def _read(torch, raw, shape):
    torch.cuda.synchronize()
    host = raw.cpu().numpy()
    assert np.isnan(host[:GUARD]).all() and np.isnan(host[-GUARD:]).all(), "wrote outside the output"
    return host[GUARD:-GUARD].reshape(shape).copy()


def _dropin(ocn, torch, l):
    """The existing entry point with a caller-owned workspace."""
    N, C, H, K = l["N"], l["C"], l["H"], l["K"]
    ws = torch.full((ocn.workspace_bytes(C, K) // 4,), float("nan"), device="cuda:0")
    raw, yd = _guarded(torch, K * H * H * N)
    td = ocn.tiles_dim(H)
    ocn.convolutionForward(l["xd"], H, H, l["wd"], H, H, N, K, yd, ws, K * N * H * H, td, N, 4, td * 4,
                           C, K, C, 3, 3, 4, 2)
    return _read(torch, raw, (K, H, H, N)), ocn.last_kernel()


def _static(ocn, torch, l):
    N, C, H, K = l["N"], l["C"], l["H"], l["K"]
    raw, yd = _guarded(torch, K * H * H * N)
    ocn.conv_forward_static(l["xd"], l["wd"], yd, N, C, H, H, K)
    return _read(torch, raw, (K, H, H, N)), ocn.last_kernel()


@pytest.mark.parametrize("precision", ["F32", "F16"])
def test_static_workspace_entry_point_matches_convolutionForward(ocn, oracle, torch_gpu, precision):
    torch = torch_gpu
    ocn.init()
    ocn.set_stream(None)
    ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    ocn.set_operand_precision(getattr(ocn, precision))
    try:
        # first a layer whose tiles are cut between workgroups (98 * 2 workgroup tiles on 256 CUs is
        # not a whole number of rounds), then a smaller one: fewer channels, filters, tiles
        big = _layer(ocn, torch, 64, 64, 28, 128)
        small = _layer(ocn, torch, 32, 24, 9, 64, seed_shift=1)
        want_big, kern_big = _dropin(ocn, torch, big)
        want_small, kern_small = _dropin(ocn, torch, small)
        for l, want, kern in ((big, want_big, kern_big), (small, want_small, kern_small)):
            print(f"static workspace {precision} N={l['N']} C={l['C']} H={l['H']} K={l['K']} ({kern})", flush=True)
            got, kern_static = _static(ocn, torch, l)
            assert kern_static == kern
            assert not np.isnan(got).any(), "an output element was never written"
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # ... and the results are right, not merely equal (fp32 bar of the parity tests; the
        # fp16-operand bound against the fp64 direct convolution)
        for l, want in ((big, want_big), (small, want_small)):
            rel64, _, _ = oracle.compare(want, oracle.direct_conv_f64(l["x"], l["w"]))
            assert rel64 <= (1e-3 if precision == "F32" else 2e-3), rel64
        # the big layer once more after the small one: nothing of the small call is left over
        got, _ = _static(ocn, torch, big)
        assert np.array_equal(got.view(np.uint32), want_big.view(np.uint32))
    finally:
        ocn.set_operand_precision(ocn.F32)


def test_static_workspace_rejects_what_does_not_fit(ocn, torch_gpu):
    torch = torch_gpu
    ocn.init()
    limit = ocn.static_workspace_bytes()
    assert limit == 16 << 20
    assert ocn.workspace_bytes(512, 512) == limit      # the largest benchmark layer fits exactly
    C, K, H, N = 520, 512, 4, 32
    assert ocn.workspace_bytes(C, K) > limit
    xd = torch.zeros(C * H * H * N, device="cuda:0")
    wd = torch.zeros(C * 9 * K, device="cuda:0")
    yd = torch.full((K * H * H * N,), float("nan"), device="cuda:0")
    with pytest.raises(ocn.OpenCNNError) as err:
        ocn.conv_forward_static(xd, wd, yd, N, C, H, H, K)
    assert err.value.status == 1 and "static workspace" in err.value.detail
    torch.cuda.synchronize()
    assert torch.isnan(yd).all(), "a rejected call must launch nothing"


# Run in a fresh process, so that the static call is the first thing the library launches there.
CHILD = r"""
import sys
sys.path.insert(0, sys.argv[1])
mode = sys.argv[2]
import numpy as np
import torch
import opencnn_amd as ocn

ocn.load_library()
dev = torch.device("cuda:0")
N, C, H, K = 64, 64, 28, 128   # tiles cut between workgroups: the launch takes a flag set
x = torch.from_numpy(ocn.synth_input(N, C, H, H, seed=0x0C99)).to(dev)
w = torch.from_numpy(ocn.synth_filter(K, C, seed=0xF117)).to(dev)
y = torch.full((K * H * H * N,), float("nan"), device=dev)
small = (32, 24, 9, 64)
x2 = torch.from_numpy(ocn.synth_input(small[0], small[1], small[2], small[2], seed=1)).to(dev)
w2 = torch.from_numpy(ocn.synth_filter(small[3], small[1], seed=2)).to(dev)
y2 = torch.full((small[3] * small[2] * small[2] * small[0],), float("nan"), device=dev)
torch.cuda.synchronize()
if mode == "uninitialised":
    # opencnn_init() never ran in this process: the call must refuse and launch nothing
    rc = ocn.lib().opencnn_conv_forward_static(x.data_ptr(), w.data_ptr(), y.data_ptr(), N, C, H, H, K)
    torch.cuda.synchronize()
    print("rc", rc, "nan", bool(torch.isnan(y).all()), "msg", ocn.lib().opencnn_last_error().decode())
    sys.exit(0)
ocn.init()
torch.cuda.synchronize()
free0 = torch.cuda.mem_get_info()[0]
ocn.conv_forward_static(x, w, y, N, C, H, H, K)
torch.cuda.synchronize()
free1 = torch.cuda.mem_get_info()[0]
ocn.conv_forward_static(x2, w2, y2, small[0], small[1], small[2], small[2], small[3])
torch.cuda.synchronize()
free2 = torch.cuda.mem_get_info()[0]
print("free", free0, free1, free2, "kernel", ocn.last_kernel(), "written", bool(not torch.isnan(y).any() and not torch.isnan(y2).any()))
"""


def _child(mode):
    out = subprocess.run([sys.executable, "-c", CHILD, ROOT, mode], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    return out.stdout.strip().splitlines()[-1].split()


def test_static_call_leaves_free_device_memory_where_it_was(ocn, torch_gpu):
    # first launch of the library in a fresh process (after opencnn_init), then a second, smaller one
    print("static workspace: free memory", flush=True)
    f = _child("measure")
    assert f[0] == "free" and f[5].startswith("wino_f32_asm") and f[7] == "True", f
    free0, free1, free2 = int(f[1]), int(f[2]), int(f[3])
    assert free0 == free1 == free2, (free0, free1, free2)


def test_static_call_without_init_refuses(ocn, torch_gpu):
    print("static workspace: no init", flush=True)
    f = _child("uninitialised")
    assert f[0] == "rc" and int(f[1]) == 3, f     # hipErrorNotInitialized
    assert f[3] == "True", "a refused call must launch nothing"
    assert "opencnn_init" in " ".join(f[5:])


@pytest.mark.parametrize("precision", ["F32", "BF16"])
def test_static_call_replays_from_a_graph(ocn, oracle, torch_gpu, precision):
    # its advertised use: recorded on a stream under capture (where nothing may be allocated),
    # replayed with new inputs, with eager work and synchronisations between the replays
    print(f"static workspace: graph {precision}", flush=True)
    torch = torch_gpu
    ocn.init()
    l = _layer(ocn, torch, 64, 64, 28, 128)
    N, C, H, K = l["N"], l["C"], l["H"], l["K"]
    raw, yd = _guarded(torch, K * H * H * N)
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    try:
        ocn.set_stream(s)
        ocn.set_operand_precision(getattr(ocn, precision))
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        with torch.cuda.graph(g, stream=s):
            ocn.conv_forward_static(l["xd"], l["wd"], yd, N, C, H, H, K)
        assert ocn.last_launch()[1] >= 32, "the captured launch took no graph flag set"
        graph_set = ocn.last_launch()[1]
        for rep in range(3):
            x2, w2 = ocn.synth_input(N, C, H, H, seed=300 + rep), ocn.synth_filter(K, C, seed=400 + rep)
            l["xd"].copy_(torch.from_numpy(x2).to(l["xd"].device))
            l["wd"].copy_(torch.from_numpy(w2).to(l["wd"].device))
            raw.fill_(float("nan"))
            torch.cuda.synchronize()
            g.replay()
            y_graph = _read(torch, raw, (K, H, H, N))
            raw.fill_(float("nan"))
            with torch.cuda.stream(s):
                ocn.conv_forward_static(l["xd"], l["wd"], yd, N, C, H, H, K)
            y_eager = _read(torch, raw, (K, H, H, N))
            assert not np.isnan(y_graph).any()
            assert np.array_equal(y_graph.view(np.uint32), y_eager.view(np.uint32)), f"replay {rep}"
            rel64, _, _ = oracle.compare(y_graph, oracle.direct_conv_f64(x2, w2))
            assert rel64 <= (1e-3 if precision == "F32" else 1.5e-2), rel64
        del g
        torch.cuda.synchronize()
        ocn.release_capture(None, graph_set)
        assert torch.cuda.mem_get_info()[0] >= free0 - (64 << 20)  # (the graph's own bookkeeping aside)
    finally:
        ocn.set_stream(None)
        ocn.set_operand_precision(ocn.F32)
    ocn.check_status()
