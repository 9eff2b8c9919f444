"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Tolerances (fp32 path): relative L2 <= 1e-5 and max-abs <= 1e-4 * max|y| against the
reference-order fp32 Winograd restatement; relative L2 <= 1e-3 against the fp64 direct
convolution.  Filter transform and exact-integer cases: bit-exact.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_L2_WINOGRAD = 1e-5
MAX_ABS_WINOGRAD = 1e-4  # times max|y|
REL_L2_DIRECT = 1e-3

SEED_X, SEED_W = 0x0C99, 0xF117

# (name, N, C, H, K, input range, filter distribution) — the benchmark configurations
CONFIGS = [
    ("plumbing", 32, 8, 8, 64, (-1.0, 1.0), "uniform"),
    ("resnet_56", 64, 64, 56, 64, (-1.0, 1.0), "he"),
    ("resnet_28", 128, 128, 28, 128, (-1.0, 1.0), "he"),
    ("deep_14", 128, 256, 14, 256, (0.0, 1.0), "he"),
    ("deep_7", 128, 512, 7, 512, (0.0, 1.0), "he"),
]


def make_tensors(ocn, N, C, H, W, K, xr=(-1.0, 1.0), filt="he"):
    x = ocn.synth_input(N, C, H, W, seed=SEED_X, p0=xr[0], p1=xr[1])
    if filt == "he":
        w = ocn.synth_filter(K, C, seed=SEED_W)
    else:
        w = ocn.synth_filter(K, C, seed=SEED_W, dist=ocn.DIST_UNIFORM, p0=-1.0, p1=1.0)
    return x, w


class Runner:
    """Owns device buffers (with guard bands around the output) and calls the C ABI."""

    GUARD = 4096

    def __init__(self, ocn, torch, x, w):
        self.ocn, self.torch = ocn, torch
        self.C, self.H, self.W, self.N = x.shape
        self.K = w.shape[3]
        dev = torch.device("cuda:0")
        self.xd = torch.from_numpy(np.ascontiguousarray(x)).to(dev)
        self.wd = torch.from_numpy(np.ascontiguousarray(w)).to(dev)
        self.ws = torch.empty(ocn.workspace_bytes(self.C, self.K) // 4, device=dev)
        self.n_out = self.K * self.H * self.W * self.N
        self.raw = torch.full((self.n_out + 2 * self.GUARD,), float("nan"), device=dev)
        self.yd = self.raw[self.GUARD:self.GUARD + self.n_out]

    def dropin(self):
        """The reference's call, argument for argument (src/openCNN_winograd.cu:429-431)."""
        o, td = self.ocn, self.ocn.tiles_dim(self.W)
        o.convolutionForward(self.xd, self.H, self.W, self.wd, self.H, self.W, self.N, self.K,
                             self.yd, self.ws, self.n_out, td, self.N, 4, td * 4, self.C,
                             self.K, self.C, 3, 3, 4, 2)
        return self.result()

    def split(self):
        """Filter transform once, then the fused kernel (allows H != W)."""
        o = self.ocn
        o.filter_transform(self.wd, self.ws, self.K, self.C, o.FILTER_CRSK, o.WW_MFMA)
        o.conv_forward_pretransformed(self.xd, self.ws, self.yd, self.N, self.C, self.H,
                                      self.W, self.K)
        return self.result()

    def result(self):
        self.torch.cuda.synchronize()
        raw = self.raw.cpu().numpy()
        g = self.GUARD
        assert np.isnan(raw[:g]).all() and np.isnan(raw[-g:]).all(), "wrote outside the output"
        return raw[g:-g].reshape(self.K, self.H, self.W, self.N).copy()


def check_against_oracle(oracle, y, x, w):
    assert not np.isnan(y).any(), "an output element was never written"
    rel, max_abs, max_ref = oracle.compare(y, oracle.winograd_f32(x, w))
    assert rel <= REL_L2_WINOGRAD, f"rel-L2 vs fp32 Winograd restatement {rel:.3e}"
    assert max_abs <= MAX_ABS_WINOGRAD * max_ref, f"max-abs {max_abs:.3e} vs max|y| {max_ref:.3e}"
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= REL_L2_DIRECT, f"rel-L2 vs fp64 direct convolution {rel64:.3e}"
    return rel, rel64


# ---------------------------------------------------------------- filter transform (FX)

@pytest.mark.parametrize("C,K", [(8, 64), (64, 64), (128, 128), (256, 256), (512, 512), (8, 32), (24, 96),
                                 (1, 1), (3, 40), (12, 48), (21, 130)])
def test_fx_bit_exact(ocn, oracle, torch_gpu, C, K):
    torch = torch_gpu
    print(f"fx C={C} K={K}", flush=True)
    crsk = ocn.synth_filter(K, C, seed=SEED_W)
    kcrs = ocn.synth_filter(K, C, seed=SEED_W, layout=ocn.FILTER_KCRS)
    want = oracle.fx(crsk)
    for host, layout in ((crsk, ocn.FILTER_CRSK), (kcrs, ocn.FILTER_KCRS)):
        wd = torch.from_numpy(host).cuda()
        out = torch.full((C * 16 * K,), float("nan"), device="cuda")
        ocn.filter_transform(wd, out, K, C, layout, ocn.WW_REFERENCE)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().reshape(C, 16, K), want)
        # MFMA-operand order: filters padded to 32, channels to 8, the padding written as zeros
        out = torch.full((ocn.workspace_bytes(C, K) // 4,), float("nan"), device="cuda")
        ocn.filter_transform(wd, out, K, C, layout, ocn.WW_MFMA)
        torch.cuda.synchronize()
        used = (-(-K // 32) * 32) * (-(-C // 8) * 8) * 16  # the workspace also fits the 2-byte layout
        got = out.cpu().numpy()[:used]
        assert np.array_equal(ocn.unswizzle_ww(got, C, K), want)
        assert not np.isnan(got).any()
        assert np.count_nonzero(got) == np.count_nonzero(want)


# ---------------------------------------------------------------- whole path, benchmark sizes

@pytest.mark.parametrize("name,N,C,H,K,xr,filt", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_benchmark_configs(ocn, oracle, torch_gpu, name, N, C, H, K, xr, filt):
    print(f"config {name} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K, xr, filt)
    y = Runner(ocn, torch_gpu, x, w).dropin()
    # the default choice on the benchmark layers is a hand-scheduled kernel (K = 64: two waves
    # share a column tile, else four)
    assert ocn.last_kernel() == ("wino_f32_asm_kw2" if K == 64 else "wino_f32_asm_kw4")
    rel, rel64 = check_against_oracle(oracle, y, x, w)
    print(f"  rel-L2 vs Winograd restatement {rel:.2e}, vs fp64 direct {rel64:.2e}", flush=True)


@pytest.mark.parametrize("N", [32, 64, 96, 128])
def test_reference_sweep_batch_sizes(ocn, oracle, torch_gpu, N):
    # the batch sizes of the reference's sweep (bench/bench.sh:3-21) on its 14x14 layer, C=K cut to 64
    print(f"sweep N={N}", flush=True)
    x, w = make_tensors(ocn, N, 64, 14, 14, 64)
    check_against_oracle(oracle, Runner(ocn, torch_gpu, x, w).dropin(), x, w)


# ---------------------------------------------------------------- edges

@pytest.mark.parametrize("H", [1, 2, 3, 4, 5, 6, 7, 9, 13])
def test_small_square_sizes(ocn, oracle, torch_gpu, H):
    # odd sizes exercise both mask sets of the reference
    # (src/convolutionForward_32x64x8.cu:179-183, src/store_and_transform_output_optSTS64.cuh:65-67)
    print(f"square H={H}", flush=True)
    x, w = make_tensors(ocn, 32, 8, H, H, 32)
    check_against_oracle(oracle, Runner(ocn, torch_gpu, x, w).dropin(), x, w)


@pytest.mark.parametrize("H,W", [(3, 8), (8, 3), (5, 12), (14, 7), (1, 9)])
def test_rectangular_sizes(ocn, oracle, torch_gpu, H, W):
    # beyond the reference (it only models H == W): checked against the fp64 direct convolution
    print(f"rect H={H} W={W}", flush=True)
    x, w = make_tensors(ocn, 32, 16, H, W, 64)
    y = Runner(ocn, torch_gpu, x, w).split()
    assert not np.isnan(y).any()
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= 1e-5


def test_ragged_column_blocks(ocn, oracle, torch_gpu):
    # 25 tiles x 1 batch group = 25 wave tiles: the last workgroup has idle waves
    print("ragged", flush=True)
    x, w = make_tensors(ocn, 32, 8, 10, 10, 96)
    check_against_oracle(oracle, Runner(ocn, torch_gpu, x, w).dropin(), x, w)


# ---------------------------------------------------------------- exact and structural properties

def test_integer_tensors_bit_exact(ocn, oracle, torch_gpu):
    # x in {-2..2}, g in {-2,0,2}: every summation order gives the same fp32 result, so the
    # MFMA path must equal the fp64 direct convolution bit for bit (odd size: masks included)
    print("integers", flush=True)
    rng = np.random.default_rng(7)
    N, C, K, H = 64, 64, 64, 7
    x = rng.integers(-2, 3, (C, H, H, N)).astype(np.float32)
    w = (2 * rng.integers(-1, 2, (C, 3, 3, K))).astype(np.float32)
    y = Runner(ocn, torch_gpu, x, w).dropin()
    assert np.array_equal(y.astype(np.float64), oracle.direct_conv_f64(x, w))
    assert np.array_equal(y, oracle.winograd_f32(x, w))


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GOLDEN_CASES = sorted(f[:-4] for f in os.listdir(GOLDEN) if f.endswith(".npz"))


@pytest.mark.parametrize("family", ["auto", "hip", "register"])
@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_known_answer_vectors_bit_exact(ocn, torch_gpu, name, family):
    # committed integer tensors with their exact convolution (tests/golden/make_vectors.py, numpy
    # only): every kernel family must reproduce them bit for bit, whatever its summation order
    print(f"golden {name} {family}", flush=True)
    v = np.load(os.path.join(GOLDEN, name + ".npz"))
    x, w, want = v["x"].astype(np.float32), v["w"].astype(np.float32), v["y"].astype(np.float32)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_kernel_variant({"auto": ocn.KERNEL_AUTO, "hip": ocn.KERNEL_HIP, "register": ocn.KERNEL_REGISTER}[family])
        y = r.split()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    assert np.array_equal(y, want)


@pytest.mark.parametrize("prec", ["f16", "bf16"])
@pytest.mark.parametrize("family", ["auto", "hip"])
def test_known_answer_vector_bit_exact_with_reduced_operands(ocn, torch_gpu, family, prec):
    # small integers survive the fp16 / bf16 roundings of U and V unchanged (|U| <= 18, |V| <= 16),
    # so the reduced-precision kernels must reproduce the committed vector bit for bit as well
    name = "int_n32_c32_h7_w7_k128"
    print(f"golden {name} {family} {prec}", flush=True)
    v = np.load(os.path.join(GOLDEN, name + ".npz"))
    x, w, want = v["x"].astype(np.float32), v["w"].astype(np.float32), v["y"].astype(np.float32)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_operand_precision(ocn.F16 if prec == "f16" else ocn.BF16)
        ocn.set_kernel_variant(ocn.KERNEL_AUTO if family == "auto" else ocn.KERNEL_HIP)
        y = r.split()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        ocn.set_operand_precision(ocn.F32)
    assert np.array_equal(y, want)


def test_impulse_reproduces_filter_taps(ocn, torch_gpu):
    # one non-zero input pixel: y[:, h0-(r-1), w0-(s-1), n0] = g[c0][r][s][:]; pins all strides
    print("impulse", flush=True)
    N, C, K, H = 32, 8, 32, 6
    w = ocn.synth_filter(K, C, seed=SEED_W)
    for (c0, h0, w0, n0) in [(0, 0, 0, 0), (7, 5, 5, 31), (3, 2, 4, 17)]:
        x = np.zeros((C, H, H, N), np.float32)
        x[c0, h0, w0, n0] = 1.0
        y = Runner(ocn, torch_gpu, x, w).dropin()
        want = np.zeros_like(y)
        for r in range(3):
            for s in range(3):
                hh, ww = h0 - (r - 1), w0 - (s - 1)
                if 0 <= hh < H and 0 <= ww < H:
                    want[:, hh, ww, n0] = w[c0, r, s, :]
        np.testing.assert_allclose(y, want, rtol=0, atol=2e-7)


def test_linearity_at_full_size(ocn, torch_gpu):
    # size-independent property on the 28x28 benchmark layer: conv(2a-3b) = 2conv(a)-3conv(b)
    print("linearity", flush=True)
    N, C, H, K = 128, 128, 28, 128
    a = ocn.synth_input(N, C, H, H, seed=11)
    b = ocn.synth_input(N, C, H, H, seed=12)
    w = ocn.synth_filter(K, C, seed=SEED_W)
    ya = Runner(ocn, torch_gpu, a, w).dropin()
    yb = Runner(ocn, torch_gpu, b, w).dropin()
    yc = Runner(ocn, torch_gpu, 2 * a - 3 * b, w).dropin()
    want = 2 * ya.astype(np.float64) - 3 * yb.astype(np.float64)
    err = np.linalg.norm((yc - want).ravel()) / np.linalg.norm(want.ravel())
    assert err <= 1e-6, err


def test_repeated_calls_are_identical_and_split_matches_dropin(ocn, torch_gpu):
    print("repeat", flush=True)
    x, w = make_tensors(ocn, 64, 64, 14, 14, 128)
    r = Runner(ocn, torch_gpu, x, w)
    y1 = r.dropin()
    y2 = r.dropin()  # same Ww scratch, back to back (stream ordered)
    assert np.array_equal(y1, y2)
    assert np.array_equal(y1, r.split())


@pytest.mark.parametrize("variant", ["register", "lds"])
@pytest.mark.parametrize("N,C,H,K", [(64, 64, 14, 64), (32, 24, 7, 128), (128, 128, 28, 128), (96, 8, 9, 256)])
def test_both_kernel_variants(ocn, oracle, torch_gpu, variant, N, C, H, K):
    # the register variant (every wave transforms its own patches) and the LDS variant (the
    # waves of a workgroup share the transform) must both meet the bar on the same tensors
    print(f"variant {variant} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_REGISTER if variant == "register" else ocn.KERNEL_LDS)
        y = Runner(ocn, torch_gpu, x, w).dropin()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    check_against_oracle(oracle, y, x, w)


def test_lds_variant_rejects_k_not_multiple_of_64(ocn, torch_gpu):
    x, w = make_tensors(ocn, 32, 8, 6, 6, 96)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_LDS)
        with pytest.raises(ocn.OpenCNNError):
            r.dropin()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)


@pytest.mark.parametrize("family", ["asm", "hip"])
@pytest.mark.parametrize("N,C,H,K", [(64, 16, 40, 128), (32, 64, 45, 64), (96, 8, 33, 128)])
def test_balanced_split_matches_plain_launch(ocn, oracle, torch_gpu, N, C, H, K, family):
    # more workgroup tiles than CUs and not a whole number of rounds: the persistent,
    # evenly split launch merges tiles cut between two workgroups.  It must meet the bar,
    # repeat bit for bit (the merge does not depend on timing), and stay within rounding of the
    # plain one-tile-per-workgroup launch.  Both kernel families implement it.
    print(f"balanced {family} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_ASM if family == "asm" else ocn.KERNEL_HIP)
        y1 = r.dropin()
        y2 = r.dropin()
        ocn.set_kernel_variant(ocn.KERNEL_HIP)
        ocn.set_balanced_split(False)
        y0 = r.dropin()
    finally:
        ocn.set_balanced_split(True)
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    assert np.array_equal(y1, y2)
    check_against_oracle(oracle, y1, x, w)
    check_against_oracle(oracle, y0, x, w)
    np.testing.assert_allclose(y1, y0, rtol=0, atol=2e-6 * np.abs(y0).max())


# (N, C, H, W, K): whole tiles per workgroup, tiles cut between workgroups, odd sizes, a missing
# column tile in the last workgroup (odd number of column tiles), one and many chunks
ASM_SHAPES = [(32, 8, 8, 8, 64), (64, 64, 8, 8, 64), (64, 16, 7, 15, 64), (32, 8, 7, 15, 256),
              (64, 32, 16, 16, 128), (64, 24, 31, 31, 64), (32, 40, 45, 45, 64), (32, 16, 63, 5, 128),
              (32, 8, 1, 1, 64), (32, 16, 3, 5, 128), (96, 40, 21, 27, 64), (32, 8, 112, 112, 64),
              (32, 1024, 7, 7, 1024), (256, 64, 28, 28, 64),
              # 3, 5, 7, 9 filter groups: the last filter block has waves without filters
              (32, 8, 6, 6, 96), (64, 96, 28, 28, 96), (64, 40, 14, 14, 160), (64, 32, 20, 20, 224),
              (32, 24, 30, 30, 288),
              # the same with nothing dividing
              (40, 20, 9, 9, 70), (33, 9, 11, 11, 130)]


@pytest.mark.parametrize("N,C,H,W,K", ASM_SHAPES)
def test_assembly_kernels(ocn, oracle, torch_gpu, N, C, H, W, K):
    # the hand-scheduled kernels selected explicitly (an unsupported shape would raise, not fall
    # back), against the fp64 direct convolution and bit for bit against a second call
    print(f"asm N={N} C={C} H={H} W={W} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        y = r.split()
        y2 = r.split()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    assert not np.isnan(y).any(), "an output element was never written"
    assert np.array_equal(y, y2)
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= 1e-5, f"rel-L2 vs fp64 direct {rel64:.3e}"
    if H == W:
        check_against_oracle(oracle, y, x, w)


@pytest.mark.parametrize("name,N,C,H,K,xr,filt", CONFIGS[1:], ids=[c[0] for c in CONFIGS[1:]])
def test_benchmark_configs_on_hip_kernels(ocn, oracle, torch_gpu, name, N, C, H, K, xr, filt):
    # test_benchmark_configs runs the default choice (the assembly kernels on these layers); the
    # HIP C++ kernels stay the path for every shape the assembly does not take
    print(f"hip config {name}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K, xr, filt)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_HIP)
        y = Runner(ocn, torch_gpu, x, w).dropin()
        assert ocn.last_kernel() in ("wino_f32_fused_lds", "wino_f32_stream")
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
    check_against_oracle(oracle, y, x, w)


# layers with fewer tiles than compute units: the units are dealt to more workgroups than tiles,
# the parts of a tile's channel sum handed over through the output tensor in the output
# transforms.  fp32 kernels: equal ranges of at least 8 units over the line of all units (a range
# may cross a tile boundary); fp16 / bf16 kernels: 2 or 4 equal pieces per tile of at least 8 of
# their 16-channel units.  The flags: whether the fp32 / the fp16 and bf16 kernels cut the layer.
FEW_TILES = [(32, 512, 7, 7, 512, True, True), (32, 256, 14, 14, 256, True, True),
             (64, 128, 7, 7, 128, True, False), (32, 64, 8, 8, 64, False, False),
             (32, 136, 5, 9, 96, True, False), (8, 256, 14, 14, 256, True, True),
             (20, 200, 6, 6, 250, True, False), (1, 1024, 7, 7, 1024, True, True),
             (32, 384, 9, 5, 320, True, True), (96, 512, 7, 7, 512, True, False),
             (64, 256, 14, 14, 256, True, False), (32, 72, 10, 10, 128, False, False),
             (32, 160, 10, 10, 128, True, False)]


@pytest.mark.parametrize("prec", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("N,C,H,W,K,cut_f32,cut_h16", FEW_TILES)
def test_few_tiles_cut_among_workgroups(ocn, oracle, torch_gpu, prec, N, C, H, W, K, cut_f32, cut_h16):
    print(f"few tiles {prec} N={N} C={C} H={H} W={W} K={K}", flush=True)
    cut = cut_f32 if prec == "f32" else cut_h16
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[prec])
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        y = r.split()
        y2 = r.split()
        ocn.set_balanced_split(False)  # one workgroup per tile: nothing is handed over
        y1 = r.split()
    finally:
        ocn.set_balanced_split(True)
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        ocn.set_operand_precision(ocn.F32)
    assert not np.isnan(y).any(), "an output element was never written"
    assert np.array_equal(y, y2)
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= {"f32": 1e-5, "f16": 2e-3, "bf16": 1.5e-2}[prec], f"rel-L2 vs fp64 direct {rel64:.3e}"
    rel1, _, _ = oracle.compare(y, y1)
    # cut tiles: another association of the channel sum (fp32 roundings of up to 1024 addends);
    # else the same launch
    assert (0 < rel1 <= 3e-6) if cut else rel1 == 0, f"rel-L2 vs one workgroup per tile {rel1:.3e}"
    if H == W and prec == "f32":
        check_against_oracle(oracle, y, x, w)


def test_assembly_variant_rejects_launches_it_does_not_take(ocn, torch_gpu):
    # 450 workgroup tiles on 256 compute units need the balanced split, which is switched off
    x, w = make_tensors(ocn, 32, 8, 60, 60, 64)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        ocn.set_balanced_split(False)
        with pytest.raises(ocn.OpenCNNError):
            r.dropin()
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        assert not np.isnan(r.dropin()).any()
    finally:
        ocn.set_balanced_split(True)
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)


@pytest.mark.parametrize("family", ["auto", "hip"])
@pytest.mark.parametrize("prec", ["f32", "f16"])
@pytest.mark.parametrize("N,C,H,K", [(64, 64, 14, 64), (128, 64, 20, 128), (33, 20, 9, 100)])
def test_buffers_need_only_float_alignment(ocn, oracle, torch_gpu, family, prec, N, C, H, K):
    # sub-tensors of a larger allocation: every pointer 4, 8 or 12 bytes past a 16-byte boundary
    # (the kernels' wide loads and stores must not assume more than the element's alignment)
    torch = torch_gpu
    x, w = make_tensors(ocn, N, C, H, H, K)
    ref = oracle.direct_conv_f64(x, w)
    n_out, n_ws = K * H * H * N, ocn.workspace_bytes(C, K) // 4
    for off in (1, 2, 3):
        print(f"alignment {family} {prec} N={N} C={C} H={H} K={K} offset {off}", flush=True)
        xd = torch.zeros(x.size + 8, device="cuda")[off:off + x.size]
        xd.copy_(torch.from_numpy(x.ravel()))
        wd = torch.zeros(w.size + 8, device="cuda")[off:off + w.size]
        wd.copy_(torch.from_numpy(w.ravel()))
        raw = torch.full((n_out + 8,), float("nan"), device="cuda")
        ws = torch.zeros(n_ws + 8, device="cuda")[off:off + n_ws]
        try:
            ocn.set_kernel_variant(ocn.KERNEL_AUTO if family == "auto" else ocn.KERNEL_HIP)
            ocn.set_operand_precision(ocn.F32 if prec == "f32" else ocn.F16)
            ocn.filter_transform(wd, ws, K, C, ocn.FILTER_CRSK, ocn.WW_MFMA)
            ocn.conv_forward_pretransformed(xd, ws, raw[off:off + n_out], N, C, H, H, K)
            torch.cuda.synchronize()
        finally:
            ocn.set_kernel_variant(ocn.KERNEL_AUTO)
            ocn.set_operand_precision(ocn.F32)
        r = raw.cpu().numpy()
        assert np.isnan(r[:off]).all() and np.isnan(r[off + n_out:]).all(), "wrote outside the output"
        rel, _, _ = oracle.compare(r[off:off + n_out].reshape(K, H, H, N), ref)
        assert rel <= (1e-5 if prec == "f32" else 2e-3), f"rel-L2 vs fp64 direct {rel:.3e}"


# batches that are no multiple of 32: the assembly kernels cut their column tiles from the line of
# all (spatial tile, batch element) pairs, so a column tile holds several tiles or parts of two.
# The library packs when an eighth of the columns would be empty and the layer has more workgroup
# tiles than compute units, or when fewer tiles can be cut into more pieces (N = 8 on the deep
# layer: with fp32 units only); the other three of the last four shapes stay on the unpacked
# _ragged kernels.
PACKED_SHAPES = [(1, 8, 64, 64, 64, True), (2, 16, 47, 39, 128, True), (3, 8, 45, 45, 64, True),
                 (5, 24, 33, 37, 100, True), (7, 3, 41, 50, 40, True), (9, 40, 36, 36, 250, True),
                 (12, 20, 40, 30, 160, True), (16, 64, 56, 56, 64, True), (17, 16, 50, 50, 64, True),
                 (20, 8, 36, 44, 128, True), (33, 24, 23, 23, 96, True), (40, 16, 28, 28, 128, True),
                 (48, 32, 40, 40, 64, True), (100, 128, 28, 28, 128, True), (70, 8, 30, 30, 64, True),
                 (1, 16, 112, 112, 64, True),
                 (1, 64, 14, 14, 64, False), (8, 256, 14, 14, 256, "f32"), (60, 8, 40, 40, 64, False),
                 (127, 16, 25, 25, 256, False)]


@pytest.mark.parametrize("prec", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("N,C,H,W,K,packed", PACKED_SHAPES)
def test_batches_on_packed_column_tiles(ocn, oracle, torch_gpu, prec, N, C, H, W, K, packed):
    # the assembly kernels selected explicitly; against the fp64 direct convolution, the HIP C++
    # kernels (which leave the columns of missing batch elements empty) and a second call
    print(f"packed {prec} N={N} C={C} H={H} W={W} K={K}", flush=True)
    if isinstance(packed, str):
        packed = packed == prec
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[prec])
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        y = r.split()
        kernel = ocn.last_kernel()
        y2 = r.split()
        ocn.set_kernel_variant(ocn.KERNEL_HIP)
        y_hip = r.split()
        assert "_asm_" not in ocn.last_kernel()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        ocn.set_operand_precision(ocn.F32)
    assert kernel.startswith(f"wino_{prec}_asm_kw")
    assert kernel.endswith("_packed" if packed else "_ragged"), kernel
    assert not np.isnan(y).any(), "an output element was never written"
    assert np.array_equal(y, y2)
    bound = {"f32": 1e-5, "f16": 2e-3, "bf16": 1.5e-2}[prec]
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= bound, f"rel-L2 vs fp64 direct {rel64:.3e}"
    # same products, same fp32 sums per output (the split between workgroups may differ)
    rel_hip, _, _ = oracle.compare(y, y_hip)
    assert rel_hip <= 1e-6, f"rel-L2 vs the HIP kernel {rel_hip:.3e}"


# ---------------------------------------------------------------- shapes outside the reference's tiling

RAGGED = [
    # N, C, H, W, K
    (1, 1, 1, 1, 1),        # one of everything
    (1, 3, 9, 9, 8),        # a single image
    (7, 5, 6, 6, 40),       # nothing aligned
    (33, 8, 8, 8, 64),      # batch tail only
    (48, 12, 7, 7, 64),     # batch and channel tails, odd image
    (32, 9, 10, 10, 32),    # odd channel count only
    (32, 8, 8, 8, 72),      # filter tail only
    (50, 20, 13, 13, 100),
    (64, 30, 5, 11, 136),   # H != W through the split entry points
]


@pytest.mark.parametrize("N,C,H,W,K", RAGGED)
def test_shapes_outside_reference_tiling(ocn, oracle, torch_gpu, N, C, H, W, K):
    # The reference needs N % 32 == 0, K % 64 == 0, C % 8 == 0 and mis-computes silently
    # otherwise (src/openCNN_winograd.cu:212-218); here groups are rounded up and the lanes,
    # channels and filters that do not exist are predicated.  Guard bands around the output
    # catch a store from a lane that should have been off.
    print(f"ragged N={N} C={C} H={H} W={W} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, W, K, filt="uniform")
    r = Runner(ocn, torch_gpu, x, w)
    y = r.split()
    assert not np.isnan(y).any(), "an output element was never written"
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= 1e-5, f"rel-L2 vs fp64 direct {rel64:.3e}"
    if H == W:
        check_against_oracle(oracle, y, x, w)
        assert np.array_equal(r.dropin(), y)


@pytest.mark.parametrize("N,C,H,K", [(48, 12, 7, 64), (100, 20, 13, 100), (33, 8, 30, 128), (7, 5, 6, 40)])
def test_ragged_shape_on_every_kernel_family(ocn, oracle, torch_gpu, N, C, H, K):
    # an even number of filter groups: the assembly kernels by default, the HIP LDS and register
    # kernels on request
    print(f"ragged variants N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K, filt="uniform")
    r = Runner(ocn, torch_gpu, x, w)
    try:
        for variant in (ocn.KERNEL_ASM, ocn.KERNEL_HIP, ocn.KERNEL_REGISTER):
            ocn.set_kernel_variant(variant)
            check_against_oracle(oracle, r.dropin(), x, w)
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)


@pytest.mark.parametrize("prec", ["f32", "f16", "bf16"])
def test_padded_channels_do_not_leak_non_finite_values(ocn, oracle, torch_gpu, prec):
    # C = 5 runs one chunk of 8 (fp16 / bf16: 16) channels; the padded channels multiply zeros on
    # BOTH operands, so an infinity in the last real channel must stay confined to the outputs it
    # reaches: the batch element it sits in
    print(f"ragged inf {prec}", flush=True)
    # K = 32: register kernel (fp32); K = 64: assembly kernel; N = 3 on 40x40: packed column tiles,
    # where the lanes next to the infinity's belong to other spatial tiles
    for N, H, K, n_inf in ((32, 6, 32, 3), (32, 6, 64, 3), (3, 40, 64, 1)):
        C = 5
        x, w = make_tensors(ocn, N, C, H, H, K, filt="uniform")
        x[C - 1, 2, 2, n_inf] = np.inf
        try:
            ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[prec])
            y = Runner(ocn, torch_gpu, x, w).split()
        finally:
            ocn.set_operand_precision(ocn.F32)
        bad = ~np.isfinite(y)
        assert bad[:, :, :, n_inf].any()
        assert not bad[:, 5:, :, n_inf].any() and not bad[:, :, 5:, n_inf].any()  # a 3x3 filter's reach
        bad[:, :, :, n_inf] = False
        assert not bad.any()


@pytest.mark.parametrize("prec", ["f32", "f16"])
@pytest.mark.parametrize("N,C,H,K", [(64, 64, 56, 64), (64, 16, 12, 128), (20, 12, 9, 40), (32, 512, 7, 512)])
def test_non_finite_inputs_spread_as_in_the_reference_arithmetic(ocn, oracle, torch_gpu, prec, N, C, H, K):
    # An infinity or a NaN in the input reaches, through the 4x4 patches, whole 2x2 output tiles
    # of every filter (inf - inf in the output transform), not only the 3x3 neighbourhood of a
    # direct convolution: the restatement of the reference's arithmetic says where, and the
    # kernels - tiles cut between workgroups and merged included - must agree element by element.
    print(f"non-finite {prec} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K)
    x[1, 0, 0, 0] = np.inf                     # a corner: part of one patch only
    x[C - 1, H // 2, H // 2, N - 1] = -np.inf  # an odd / even boundary: up to four patches
    x[C // 2, H - 1, 1, N // 2] = np.nan
    quant = {"f32": 0, "f16": 1}[prec]
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16}[prec])
        y = Runner(ocn, torch_gpu, x, w).split()
    finally:
        ocn.set_operand_precision(ocn.F32)
    want = oracle.winograd_f32(x, w, quant)
    assert np.isnan(want).any() and np.isinf(want).any()
    assert np.array_equal(np.isnan(y), np.isnan(want))
    assert np.array_equal(np.isposinf(y), np.isposinf(want)) and np.array_equal(np.isneginf(y), np.isneginf(want))
    ok = np.isfinite(want)
    rel, max_abs, max_ref = oracle.compare(np.where(ok, y, 0.0), np.where(ok, want, 0.0))
    assert rel <= {"f32": REL_L2_WINOGRAD, "f16": 2e-5}[prec], rel


@pytest.mark.parametrize("variant", ["auto", "hip"])
@pytest.mark.parametrize("N,C,H,K", [(32, 8, 8, 64), (64, 16, 12, 128), (32, 8, 6, 32)])
def test_denormal_operands_and_products_are_not_flushed(ocn, oracle, torch_gpu, variant, N, C, H, K):
    # The reference is compiled without flush-to-zero: denormal inputs, transformed filters,
    # products and sums keep their bits.  Here: MFMA and vector ALU in the same mode (the
    # kernels' descriptors ask for fp32 denormals), checked on tensors whose products lie below
    # the smallest normal number.
    print(f"denormals {variant} N={N} C={C} H={H} K={K}", flush=True)
    rng = np.random.default_rng(7)
    for sx, sw in ((1e-19, 1e-19), (1e-38, 1.0), (1.0, 1e-38), (1e-41, 1.0)):
        x = (rng.uniform(-1, 1, (C, H, H, N)) * sx).astype(np.float32)
        w = (rng.normal(size=(C, 3, 3, K)) * sw).astype(np.float32)
        try:
            ocn.set_kernel_variant(ocn.KERNEL_HIP if variant == "hip" else ocn.KERNEL_AUTO)
            y = Runner(ocn, torch_gpu, x, w).split()
        finally:
            ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        want = oracle.winograd_f32(x, w)
        assert np.abs(want).max() < 1e-36 and (want != 0).mean() > 0.99
        assert (y != 0).mean() == (want != 0).mean()
        rel, _, _ = oracle.compare(y, want)
        assert rel <= REL_L2_WINOGRAD, (sx, sw, rel)


# ---------------------------------------------------------------- layout shims

@pytest.mark.parametrize("N,C,H,W,K", [(32, 8, 8, 8, 64), (64, 64, 56, 56, 64), (96, 1030, 5, 3, 33), (1, 1, 1, 1, 1),
                                       (2, 3, 224, 224, 128)])  # K*H*W beyond 65535 rows of 64
def test_layout_shims_are_exact_permutations(ocn, torch_gpu, N, C, H, W, K):
    # the reference's data_cpy transposes (src/openCNN_winograd.cu:147-153,230,235): bit-exact,
    # checked against numpy; C = 1030 is beyond data_cpy's C <= 1024 launch limit
    print(f"shims N={N} C={C} H={H} W={W} K={K}", flush=True)
    torch = torch_gpu
    nchw = ocn.synth_input(N, C, H, W, seed=5, layout=ocn.INPUT_NCHW)
    src = torch.from_numpy(nchw).cuda()
    dst = torch.full((C, H, W, N), float("nan"), device="cuda")
    ocn.nchw_to_chwn(src, dst, N, C, H, W)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), nchw.transpose(1, 2, 3, 0))
    assert np.array_equal(dst.cpu().numpy(), ocn.synth_input(N, C, H, W, seed=5))
    back = torch.full((N, C, H, W), float("nan"), device="cuda")
    ocn.khwn_to_nkhw(dst, back, N, C, H, W)  # a CHWN tensor is a KHWN tensor with K = C
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy(), nchw)
    kc = min(C, 64)
    kcrs = ocn.synth_filter(K, kc, seed=6, layout=ocn.FILTER_KCRS)
    fsrc = torch.from_numpy(kcrs).cuda()
    fdst = torch.full((kc, 3, 3, K), float("nan"), device="cuda")
    ocn.kcrs_to_crsk(fsrc, fdst, K, kc)
    torch.cuda.synchronize()
    assert np.array_equal(fdst.cpu().numpy(), ocn.synth_filter(K, kc, seed=6))


def test_nchw_pipeline_end_to_end(ocn, oracle, torch_gpu):
    # the reference bench's data flow: NCHW / KCRS tensors -> shims -> convolutionForward -> NCHW
    print("nchw pipeline", flush=True)
    torch = torch_gpu
    N, C, H, K = 64, 32, 12, 64
    nchw = ocn.synth_input(N, C, H, H, seed=SEED_X, layout=ocn.INPUT_NCHW)
    kcrs = ocn.synth_filter(K, C, seed=SEED_W, layout=ocn.FILTER_KCRS)
    xs, ws_ = torch.from_numpy(nchw).cuda(), torch.from_numpy(kcrs).cuda()
    xd, wd = torch.empty(C * H * H * N, device="cuda"), torch.empty(C * 9 * K, device="cuda")
    yd, yn = torch.empty(K * H * H * N, device="cuda"), torch.empty((N, K, H, H), device="cuda")
    wsp = torch.empty(C * 16 * K, device="cuda")
    ocn.nchw_to_chwn(xs, xd, N, C, H, H)
    ocn.kcrs_to_crsk(ws_, wd, K, C)
    td = ocn.tiles_dim(H)
    ocn.convolutionForward(xd, H, H, wd, H, H, N, K, yd, wsp, K * N * H * H, td, N, 4, td * 4, C, K, C, 3, 3, 4, 2)
    ocn.khwn_to_nkhw(yd, yn, N, K, H, H)
    torch.cuda.synchronize()
    want = oracle.direct_conv_f64(nchw.transpose(1, 2, 3, 0), kcrs.transpose(1, 2, 3, 0)).transpose(3, 0, 1, 2)
    rel, _, _ = oracle.compare(yn.cpu().numpy(), np.ascontiguousarray(want))
    assert rel <= 1e-5


# ---------------------------------------------------------------- fp16 / bf16 GEMM operands

# bounds against the fp64 direct convolution: unit round-offs 2^-11 (fp16) and 2^-8 (bf16) on
# both GEMM operands; against the oracle's quantised restatement (same roundings, fp32 chain)
# only the summation order differs
REL_L2_DIRECT_REDUCED = {"f16": 2e-3, "bf16": 1.5e-2}
REL_L2_QUANTISED_RESTATEMENT = 2e-5


@pytest.mark.parametrize("prec", ["f16", "bf16"])
@pytest.mark.parametrize("N,C,H,K,xr", [
    (128, 256, 14, 256, (-1.0, 1.0)),  # the reduced-precision benchmark configuration
    (32, 16, 7, 64, (-1.0, 1.0)),      # odd size, two waves per column tile
    (64, 48, 9, 128, (0.0, 1.0)),      # odd number of 16-channel chunks
    (32, 32, 4, 192, (-1.0, 1.0)),
    (64, 32, 40, 128, (-1.0, 1.0)),    # 800 workgroup tiles of two chunks: tiles cut between workgroups
    (32, 48, 45, 64, (-1.0, 1.0)),     # the same with a missing column tile and three chunks
])
def test_reduced_precision_operands(ocn, oracle, torch_gpu, prec, N, C, H, K, xr):
    print(f"reduced {prec} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K, xr)
    quant = 1 if prec == "f16" else 2
    try:
        ocn.set_operand_precision(ocn.F16 if prec == "f16" else ocn.BF16)
        r = Runner(ocn, torch_gpu, x, w)
        y = r.dropin()
        y2 = r.dropin()
    finally:
        ocn.set_operand_precision(ocn.F32)
    assert not np.isnan(y).any()
    assert np.array_equal(y, y2)
    rel, max_abs, max_ref = oracle.compare(y, oracle.winograd_f32(x, w, quant))
    assert rel <= REL_L2_QUANTISED_RESTATEMENT, f"rel-L2 vs quantised restatement {rel:.3e}"
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert 1e-5 < rel64 <= REL_L2_DIRECT_REDUCED[prec], f"rel-L2 vs fp64 direct {rel64:.3e}"
    print(f"  rel-L2 vs quantised restatement {rel:.2e}, vs fp64 direct {rel64:.2e}", flush=True)


# (N, C, H, W, K) for the hand-scheduled fp16 / bf16 kernels (any shape):
# the benchmark configuration (two filter blocks in lockstep); one tile per workgroup; one
# 16-channel chunk; three filter blocks and an 8 MB transformed filter (one filter-block-major
# line of units); tiles cut between workgroups with one, two and four filter blocks; odd sizes
H16_ASM_SHAPES = [(128, 256, 14, 14, 256), (32, 32, 6, 6, 128), (32, 16, 9, 9, 256), (64, 48, 9, 9, 384),
                  (32, 512, 5, 5, 512), (64, 32, 40, 40, 128), (64, 64, 21, 21, 256), (32, 32, 30, 30, 512),
                  (32, 32, 31, 9, 128), (96, 48, 1, 1, 128),
                  # filter counts of 64, 192 and 320: the last filter block holds two filter groups
                  (64, 64, 56, 56, 64), (32, 32, 12, 12, 192), (32, 16, 7, 7, 64), (64, 48, 19, 19, 320),
                  # channel counts that are no multiple of 16 (an RGB first layer; odd; one over a chunk)
                  (64, 3, 20, 20, 64), (32, 5, 6, 6, 64), (32, 17, 7, 7, 256), (32, 40, 9, 9, 128),
                  # batch sizes and filter counts outside the tiling: masked lanes and rows
                  (33, 5, 7, 7, 40), (100, 40, 9, 9, 250), (1, 1, 4, 4, 1), (48, 72, 12, 12, 160), (16, 64, 28, 28, 96),
                  (8, 32, 33, 17, 1000)]


@pytest.mark.parametrize("prec", ["f16", "bf16"])
@pytest.mark.parametrize("N,C,H,W,K", H16_ASM_SHAPES)
def test_reduced_precision_assembly_kernels(ocn, oracle, torch_gpu, prec, N, C, H, W, K):
    # selected explicitly (an unsupported shape would raise, not fall back); against the
    # quantised restatement, the fp64 direct convolution, a second call, and the HIP C++ kernel
    print(f"reduced asm {prec} N={N} C={C} H={H} W={W} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_operand_precision(ocn.F16 if prec == "f16" else ocn.BF16)
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        y = r.split()
        y2 = r.split()
        ocn.set_kernel_variant(ocn.KERNEL_HIP)
        y_hip = r.split()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        ocn.set_operand_precision(ocn.F32)
    assert not np.isnan(y).any(), "an output element was never written"
    assert np.array_equal(y, y2)
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= REL_L2_DIRECT_REDUCED[prec], f"rel-L2 vs fp64 direct {rel64:.3e}"
    # same operands, same roundings; only the order of the fp32 sums inside the MFMA chain differs
    rel_hip, _, _ = oracle.compare(y, y_hip)
    assert rel_hip <= REL_L2_QUANTISED_RESTATEMENT, f"rel-L2 vs the HIP kernel {rel_hip:.3e}"
    if H == W:
        rel, _, _ = oracle.compare(y, oracle.winograd_f32(x, w, 1 if prec == "f16" else 2))
        assert rel <= REL_L2_QUANTISED_RESTATEMENT, f"rel-L2 vs quantised restatement {rel:.3e}"


def test_reduced_precision_assembly_variant_needs_the_balanced_split(ocn, torch_gpu):
    # 400 workgroup tiles on 256 compute units: the persistent launch cuts tiles, which the caller
    # has switched off, so the assembly kernel selected explicitly must refuse (no silent fallback)
    x, w = make_tensors(ocn, 32, 16, 40, 40, 128)
    r = Runner(ocn, torch_gpu, x, w)
    try:
        ocn.set_operand_precision(ocn.F16)
        ocn.set_balanced_split(False)
        ocn.set_kernel_variant(ocn.KERNEL_ASM)
        with pytest.raises(ocn.OpenCNNError):
            r.dropin()
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        assert not np.isnan(r.dropin()).any()
    finally:
        ocn.set_kernel_variant(ocn.KERNEL_AUTO)
        ocn.set_balanced_split(True)
        ocn.set_operand_precision(ocn.F32)


@pytest.mark.parametrize("prec", ["f16", "bf16"])
@pytest.mark.parametrize("N,C,H,K", [
    (32, 8, 6, 64),     # half a 16-channel chunk
    (33, 5, 7, 40),     # nothing divides: batch, channels, filters, odd image
    (100, 40, 9, 250),  # two and a half chunks, four filter groups of which the last holds 26
    (1, 1, 4, 1),       # the smallest layer
    (48, 72, 12, 160),  # whole groups, but five of them and 4.5 chunks
])
def test_reduced_precision_on_shapes_outside_the_tiling(ocn, oracle, torch_gpu, prec, N, C, H, K):
    # batch, channel and filter counts that are no multiples of 32 / 16 / 64: rounded-up groups
    # with predicated lanes, zero padding in the transformed filter, as for fp32 operands
    print(f"reduced ragged {prec} N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K)
    try:
        ocn.set_operand_precision(ocn.F16 if prec == "f16" else ocn.BF16)
        r = Runner(ocn, torch_gpu, x, w)
        y = r.dropin()
        y2 = r.dropin()
    finally:
        ocn.set_operand_precision(ocn.F32)
    assert not np.isnan(y).any(), "an output element was never written"
    assert np.array_equal(y, y2)
    rel, _, _ = oracle.compare(y, oracle.winograd_f32(x, w, 1 if prec == "f16" else 2))
    assert rel <= REL_L2_QUANTISED_RESTATEMENT, f"rel-L2 vs quantised restatement {rel:.3e}"
    rel64, _, _ = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel64 <= REL_L2_DIRECT_REDUCED[prec], f"rel-L2 vs fp64 direct {rel64:.3e}"


@pytest.mark.parametrize("prec", ["f32", "f16"])
@pytest.mark.parametrize("N,C,H,W,K", [(128, 64, 14, 14, 256), (64, 16, 41, 41, 128), (96, 32, 13, 22, 64),
                                       (64, 32, 27, 9, 320), (32, 512, 7, 7, 512)])
def test_every_tile_order_computes_the_same_layer(ocn, oracle, torch_gpu, prec, N, C, H, W, K):
    # The order in which the assembly kernels walk through the image (opencnn_set_tile_order: image
    # group or spatial tile fastest, rows or zigzag strips, places by starting time) only changes
    # which tiles are cut between workgroups: every output element is written, inside the tensor,
    # and equals the default order's up to the association of the channel sum.
    print(f"tile orders {prec} N={N} C={C} H={H} W={W} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, W, K)
    r = Runner(ocn, torch_gpu, x, w)
    results = {}
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16}[prec])
        for order in (7, 0, 1, 2, 3, 5):
            ocn.set_tile_order(order)
            r.raw.fill_(float("nan"))
            results[order] = r.split()
            assert "_asm_" in ocn.last_kernel()
    finally:
        ocn.set_tile_order(7)
        ocn.set_operand_precision(ocn.F32)
    want = oracle.direct_conv_f64(x, w)
    for order, y in results.items():
        assert not np.isnan(y).any(), f"order {order}: an output element was never written"
        rel64, _, _ = oracle.compare(y, want)
        assert rel64 <= {"f32": 1e-5, "f16": 2e-3}[prec], f"order {order}: rel-L2 vs fp64 direct {rel64:.3e}"
        rel, _, _ = oracle.compare(y, results[7])
        assert rel <= 3e-6, f"order {order}: rel-L2 vs the default order {rel:.3e}"
    with pytest.raises(ocn.OpenCNNError):
        ocn.set_tile_order(8)


def direct_conv_at(torch, xf, wd, points, C, H, W, N):
    """fp64 direct convolution (pad 1) at the sampled (y, x, n) points, all filters: definition of
    the layer, evaluated on the device by gathering the 3x3xC neighbourhood of every point."""
    ys, xs, ns = points.unbind(1)
    chan = torch.arange(C, device=xf.device, dtype=torch.int64)[None, :]
    acc = torch.zeros(points.shape[0], wd.shape[3], device=xf.device, dtype=torch.float64)
    for r in range(3):
        for s in range(3):
            yy, xx = ys + (r - 1), xs + (s - 1)
            ok = (yy >= 0) & (yy < H) & (xx >= 0) & (xx < W)
            at = ((chan * H + yy.clamp(0, H - 1)[:, None]) * W + xx.clamp(0, W - 1)[:, None]) * N + ns[:, None]
            v = xf[at].double() * ok[:, None]
            acc += v @ wd[:, r, s, :].double()
    return acc


@pytest.mark.parametrize("prec,N,C,H,K,kernel", [
    ("f32", 512, 64, 224, 64, "wino_f32_asm_kw2"),     # 6.6 GB in, 6.6 GB out: 64-bit bases of the assembly kernels
    ("f16", 512, 64, 224, 64, "wino_f16_asm_kw4"),
    ("f32", 4096, 8, 224, 8, "wino_f32_fused"),        # five output rows pass 2^31 bytes: the assembly kernels step aside
])
def test_tensors_beyond_four_gigabytes(ocn, torch_gpu, prec, N, C, H, K, kernel):
    # Largest sizes: both tensors close to the 2^31 - 1 elements the entry points accept (the
    # reference indexes with int as well).  Too large for the CPU oracle, so: every output element
    # written, nothing written outside, and 4000 random points plus the tensor's corners against
    # the fp64 direct convolution evaluated at those points.
    print(f"large tensors {prec} N={N} C={C} H={H} K={K}", flush=True)
    torch = torch_gpu
    dev = torch.device("cuda:0")
    n_in, n_out, guard = C * H * H * N, K * H * H * N, 4096
    assert 2 ** 30 < n_in < 2 ** 31 and 2 ** 30 < n_out < 2 ** 31
    gen = torch.Generator(device=dev)
    gen.manual_seed(SEED_X)
    xd = torch.empty(n_in, device=dev).uniform_(-1.0, 1.0, generator=gen)
    w = ocn.synth_filter(K, C, seed=SEED_W)
    wd = torch.from_numpy(w).to(dev)
    ws = torch.empty(ocn.workspace_bytes(C, K) // 4, device=dev)
    raw = torch.full((n_out + 2 * guard,), float("nan"), device=dev)
    yd = raw[guard:guard + n_out]
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16}[prec])
        ocn.filter_transform(wd, ws, K, C, ocn.FILTER_CRSK, ocn.WW_MFMA)
        ocn.conv_forward_pretransformed(xd, ws, yd, N, C, H, H, K)
        torch.cuda.synchronize()
        assert ocn.last_kernel().startswith(kernel), ocn.last_kernel()
        ocn.check_status()
    finally:
        ocn.set_operand_precision(ocn.F32)
    assert bool(torch.isnan(raw[:guard]).all()) and bool(torch.isnan(raw[-guard:]).all()), "wrote outside the output"
    assert not bool(torch.isnan(yd).any()), "an output element was never written"
    pts = torch.stack([torch.randint(0, H, (4000,), generator=gen, device=dev),
                       torch.randint(0, H, (4000,), generator=gen, device=dev),
                       torch.randint(0, N, (4000,), generator=gen, device=dev)], dim=1)
    corners = torch.tensor([[y, x, n] for y in (0, H - 1) for x in (0, H - 1) for n in (0, N - 1)], device=dev)
    pts = torch.cat([corners, pts]).to(torch.int64)
    want = direct_conv_at(torch, xd, wd, pts, C, H, H, N)
    filt = torch.arange(K, device=dev, dtype=torch.int64)[None, :]
    got = yd[((filt * H + pts[:, 0:1]) * H + pts[:, 1:2]) * N + pts[:, 2:3]].double()
    rel = float((got - want).norm() / want.norm())
    worst = float((got - want).abs().max() / want.abs().max())
    bar = {"f32": (1e-5, 1e-4), "f16": (2e-3, 2e-2)}[prec]
    assert rel <= bar[0] and worst <= bar[1], (rel, worst)
    del xd, raw, yd
    torch.cuda.empty_cache()


@pytest.mark.parametrize("N,C,H,K,kernel", [(32, 64, 56, 64, "wino_f32_asm_kw2"), (48, 64, 56, 64, "wino_f32_asm_kw2_packed"),
                                            (96, 256, 14, 256, "wino_f32_asm_kw4"), (96, 120, 28, 250, "wino_f32_asm_kw4_ragged")])
def test_ranges_cut_on_a_weighted_line_compute_the_same_layer(ocn, oracle, torch_gpu, N, C, H, K, kernel):
    # Balanced split of the fp32 assembly kernels: the library may cut the ranges on a line that
    # weighs every tile's output transform (opencnn_set_range_weight forces a weight in half
    # units), which moves the cuts between workgroups and nothing else.
    print(f"weighted ranges N={N} C={C} H={H} K={K}", flush=True)
    x, w = make_tensors(ocn, N, C, H, H, K)
    r = Runner(ocn, torch_gpu, x, w)
    want = oracle.direct_conv_f64(x, w)
    results = {}
    try:
        for forced in (0, 1, 2, 3, 4, 5, 6, 7):  # 0: the library's choice, 1: equal numbers of units
            ocn.set_range_weight(forced - 1)
            r.raw.fill_(float("nan"))
            results[forced] = r.split()
            assert ocn.last_kernel() == kernel and ocn.last_launch()[0] == 256
    finally:
        ocn.set_range_weight(-1)
    for forced, y in results.items():
        assert not np.isnan(y).any(), f"weight {forced}: an output element was never written"
        rel64, _, _ = oracle.compare(y, want)
        assert rel64 <= 1e-5, f"weight {forced}: rel-L2 vs fp64 direct {rel64:.3e}"
        rel, _, _ = oracle.compare(y, results[1])
        assert rel <= 3e-6, f"weight {forced}: rel-L2 vs the equal split {rel:.3e}"


def test_non_default_stream(ocn, oracle, torch_gpu):
    print("stream", flush=True)
    torch = torch_gpu
    x, w = make_tensors(ocn, 32, 16, 9, 9, 64)
    r = Runner(ocn, torch, x, w)
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    try:
        ocn.set_stream(s)
        y = r.dropin()
    finally:
        ocn.set_stream(None)
    check_against_oracle(oracle, y, x, w)


def test_layers_on_different_streams_may_overlap(ocn, oracle, torch_gpu):
    # two layers whose tiles are cut between workgroups (784 and 800 tiles on 256 CUs), launched
    # back to back on two streams without synchronisation in between, so that they may run at the
    # same time: every stream has split-merge flags of its own, the results are the serial ones,
    # bit for bit.  Ten streams in all.
    print("overlapping streams", flush=True)
    torch = torch_gpu
    shapes = [(64, 32, 56, 56, 64), (64, 32, 40, 40, 128)]
    runners, want = [], []
    for N, C, H, W, K in shapes:
        x, w = make_tensors(ocn, N, C, H, W, K)
        r = Runner(ocn, torch, x, w)
        want.append(r.split())
        runners.append(r)
    streams = [torch.cuda.Stream() for _ in range(10)]
    torch.cuda.synchronize()
    try:
        for rep in range(5):
            for r in runners:
                r.raw.fill_(float("nan"))
            torch.cuda.synchronize()
            for i, r in enumerate(runners):
                ocn.set_stream(streams[(2 * rep + i) % len(streams)])
                ocn.conv_forward_pretransformed(r.xd, r.ws, r.yd, r.N, r.C, r.H, r.W, r.K)
                assert ocn.last_launch()[1] >= 0, "launched without the split"
            torch.cuda.synchronize()
            for r, y in zip(runners, want):
                assert np.array_equal(r.result(), y), f"rep {rep}"
    finally:
        ocn.set_stream(None)


@pytest.mark.parametrize("prec,seed,hmax", [("f32", 20241, 48), ("f32", 20242, 14), ("f16", 20243, 40),
                                            ("bf16", 20244, 14)])
def test_random_shapes_on_every_kernel_family(ocn, oracle, torch_gpu, prec, seed, hmax):
    # seeded sweep over batch sizes, channel and filter counts inside and outside the reference's
    # tiling, square and rectangular images, default / HIP-only kernels, balanced split on / off:
    # every output element written exactly inside the tensor, two calls bit-identical, rel-L2
    # against the fp64 direct convolution.  The sweeps over small images with deep channel
    # counts land in the layers whose tiles are cut among workgroups.
    import random

    torch = torch_gpu
    rng = random.Random(seed)
    guard = 4096
    bound = {"f32": 1e-5, "f16": 2e-3, "bf16": 1.5e-2}[prec]
    for case in range(48):
        N = rng.choice([1, 2, 5, 8, 16, 20, 31, 32, 33, 48, 64, 96, 100, 128])
        C = rng.choice([1, 3, 7, 8, 9, 16, 20, 24, 40, 64, 72, 128, 200, 256, 512])
        H = rng.randint(1, hmax)
        W = rng.choice([H, H, rng.randint(1, hmax)])
        K = rng.choice([8, 32, 40, 64, 64, 96, 100, 128, 128, 192, 250, 256, 512])
        if N * C * H * W * K * 18 > 8e9:
            continue
        variant = rng.choice([ocn.KERNEL_AUTO, ocn.KERNEL_AUTO, ocn.KERNEL_HIP])
        balanced = rng.random() < 0.8
        print(f"random case {prec} {case}: N={N} C={C} H={H} W={W} K={K} variant={variant} balanced={balanced}",
              flush=True)
        x = ocn.synth_input(N, C, H, W, seed=case + 1)
        w = ocn.synth_filter(K, C, seed=case + 1000, dist=ocn.DIST_UNIFORM, p0=-1.0, p1=1.0)
        xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
        raw = torch.full((K * H * W * N + 2 * guard,), float("nan"), device="cuda")
        y = raw[guard:guard + K * H * W * N]
        ws = torch.full((ocn.workspace_bytes(C, K) // 4,), float("nan"), device="cuda")
        runs = []
        try:
            ocn.set_kernel_variant(variant)
            ocn.set_balanced_split(balanced)
            ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[prec])
            ocn.filter_transform(wd, ws, K, C, ocn.FILTER_CRSK, ocn.WW_MFMA)
            for _ in range(2):
                raw.fill_(float("nan"))
                ocn.conv_forward_pretransformed(xd, ws, y, N, C, H, W, K)
                torch.cuda.synchronize()
                runs.append(raw.cpu().numpy().copy())
        finally:
            ocn.set_kernel_variant(ocn.KERNEL_AUTO)
            ocn.set_balanced_split(True)
            ocn.set_operand_precision(ocn.F32)
        assert np.isnan(runs[0][:guard]).all() and np.isnan(runs[0][-guard:]).all(), "wrote outside the output"
        got = runs[0][guard:-guard]
        assert not np.isnan(got).any(), "an output element was never written"
        assert np.array_equal(got, runs[1][guard:-guard])
        rel64, _, _ = oracle.compare(got.reshape(K, H, W, N), oracle.direct_conv_f64(x, w))
        assert rel64 <= bound, f"rel-L2 vs fp64 direct {rel64:.3e}"


@pytest.mark.parametrize("N,C,H,K", [(32, 8, 8, 64), (64, 16, 40, 128), (32, 256, 7, 256), (8, 128, 28, 128)])
def test_call_replays_from_a_captured_graph(ocn, oracle, torch_gpu, N, C, H, K):
    # The drop-in call only launches kernels (no allocation, no memset, its device state resets
    # itself), so it can be captured; the second shape has tiles cut between workgroups, the third
    # has fewer tiles than compute units (hand-overs in the output transforms), the fourth packed
    # column tiles on top of that.  Replays
    # with new inputs, eager launches and synchronisations in between, each checked.
    print(f"graph N={N} C={C} H={H} K={K}", flush=True)
    torch = torch_gpu
    ocn.init()  # loads the assembly kernels' code object outside the capture
    x, w = make_tensors(ocn, N, C, H, H, K)
    r = Runner(ocn, torch, x, w)
    td = ocn.tiles_dim(H)

    def launch():
        ocn.convolutionForward(r.xd, H, H, r.wd, H, H, N, K, r.yd, r.ws, r.n_out, td, N, 4, td * 4,
                               C, K, C, 3, 3, 4, 2)

    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    try:
        ocn.set_stream(s)
        with torch.cuda.stream(s):
            launch()
            s.synchronize()
            eager = (ocn.last_kernel(), ocn.last_launch()[0])
            with torch.cuda.graph(g, stream=s):
                launch()
        # the captured launch is the eager one (same kernel, same grid) on a flag set of its own
        assert (ocn.last_kernel(), ocn.last_launch()[0]) == eager
        if (N, C, H, K) == (32, 8, 8, 64):
            assert ocn.last_launch()[1] == -1, "a launch that cuts no tile took a flag set"
        else:
            assert ocn.last_launch()[1] >= 32, "the captured launch shares flags with direct launches"
            assert ocn.last_kernel().startswith("wino_f32_asm") and ocn.last_launch()[0] > 64
        for rep in range(3):
            x2, w2 = ocn.synth_input(N, C, H, H, seed=100 + rep), ocn.synth_filter(K, C, seed=200 + rep)
            r.xd.copy_(torch.from_numpy(x2).to(r.xd.device))
            r.wd.copy_(torch.from_numpy(w2).to(r.wd.device))
            r.raw.fill_(float("nan"))
            torch.cuda.synchronize()
            g.replay()
            y_graph = r.result()
            with torch.cuda.stream(s):
                launch()
            y_eager = r.result()
            assert np.array_equal(y_graph, y_eager)
            check_against_oracle(oracle, y_graph, x2, w2)
    finally:
        ocn.set_stream(None)


def test_timeline_buffer_records_monotone_stamps(ocn, oracle, torch_gpu):
    # bench support of the assembly kernels: every workgroup's first wave records the realtime
    # counter at its start, after its prologue and around every output transform; recording must
    # not change the result, and stops when the buffer is taken away
    print("timeline", flush=True)
    torch = torch_gpu
    N, C, H, K = 64, 16, 40, 128  # 800 workgroup tiles on a persistent grid: several tiles per workgroup
    x, w = make_tensors(ocn, N, C, H, H, K)
    r = Runner(ocn, torch, x, w)
    y_plain = r.split()
    buf = torch.zeros(1024 * 64, dtype=torch.int64, device="cuda")
    try:
        ocn.set_timeline_buffer(buf)
        y_rec = r.split()
    finally:
        ocn.set_timeline_buffer(None)
    assert np.array_equal(y_plain, y_rec)
    rec = buf.cpu().numpy().reshape(-1, 64)
    nwg = int((rec[:, 0] > 0).sum())
    assert nwg >= 8 and (rec[:nwg, 0] >= 4).all() and (rec[:nwg, 0] % 2 == 0).all()
    for v in ocn.read_timeline(buf, nwg):
        assert all(b >= a for a, b in zip(v, v[1:])) and 0 <= v[0] and v[-1] < 1e4
    buf.zero_()
    r.split()
    assert int(buf.abs().sum()) == 0


def test_init_accepts_this_device(ocn, torch_gpu):
    ocn.init()
