"""GPU test of opencnn_conv_forward_static, the entry point that allocates nothing: same result,
bit for bit, as convolutionForward (it runs the same two kernels; only the transformed filter
lives in the library's static workspace instead of a caller's buffer), on two calls in a row
that share the workspace, the second with a smaller layer.
"""
import numpy as np
import pytest

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
