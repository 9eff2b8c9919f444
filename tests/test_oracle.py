"""Pins the CPU oracle against what the mathematics fixes (the reference ships no tests,
fixtures or golden vectors for this path): closed forms in fp64, textbook matrices,
brute force on tiny inputs, exact-integer cases where every summation order agrees."""
import os
import numpy as np
import pytest

G = np.array([[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]], dtype=np.float64)
BT = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], dtype=np.float64)
AT = np.array([[1, 1, 1, 0], [0, 1, -1, -1]], dtype=np.float64)


def brute_conv(x_chwn, w_crsk):
    """Independent restatement: zero-pad, then einsum over shifted views (fp64)."""
    x = np.asarray(x_chwn, dtype=np.float64)
    w = np.asarray(w_crsk, dtype=np.float64)
    C, H, W, N = x.shape
    xp = np.zeros((C, H + 2, W + 2, N))
    xp[:, 1:-1, 1:-1, :] = x
    y = np.zeros((w.shape[3], H, W, N))
    for r in range(3):
        for s in range(3):
            y += np.einsum("chwn,ck->khwn", xp[:, r:r + H, s:s + W, :], w[:, r, s, :])
    return y


def test_tiles_dim(oracle):
    # ceil(ceil((W+2)/2)-1) for the sizes the reference sweeps (bench/bench.sh) and odd ones
    for w, want in [(56, 28), (28, 14), (14, 7), (7, 4), (8, 4), (5, 3), (4, 2), (1, 1), (2, 1)]:
        assert oracle.tiles_dim(w) == want


def test_fx_closed_form(oracle):
    rng = np.random.default_rng(1)
    for _ in range(50):
        g = rng.uniform(-1, 1, 9).astype(np.float32)
        want = G @ g.reshape(3, 3).astype(np.float64) @ G.T
        got = oracle.fx_one(g).reshape(4, 4)
        np.testing.assert_allclose(got, want, rtol=0, atol=3e-7)


def test_fx_delta_and_ones_exact(oracle):
    # delta filter e_rs -> outer product of G's columns r and s; exact in fp32
    for r in range(3):
        for s in range(3):
            g = np.zeros(9, np.float32)
            g[r * 3 + s] = 1
            want = np.outer(G[:, r], G[:, s]).astype(np.float32)
            assert np.array_equal(oracle.fx_one(g).reshape(4, 4), want)
    v = np.array([1, 1.5, 0.5, 1], np.float32)
    assert np.array_equal(oracle.fx_one(np.ones(9, np.float32)).reshape(4, 4), np.outer(v, v))


def test_fx_is_not_symmetric_under_transpose_mistake(oracle):
    # a transposed operand (G^T g G) or swapped row/column pass would fail this
    g = np.arange(9, dtype=np.float32)
    want = (G @ g.reshape(3, 3).astype(np.float64) @ G.T).astype(np.float32)
    got = oracle.fx_one(g).reshape(4, 4)
    assert np.array_equal(got, want)  # small integers and halves: exact
    assert not np.array_equal(got, got.T)


def test_fx_tensor_layout(oracle):
    rng = np.random.default_rng(2)
    C, K = 8, 32
    w = rng.integers(-4, 5, size=(C, 3, 3, K)).astype(np.float32)
    got = oracle.fx(w)  # [C][16][K]
    want = np.einsum("ir,crsk,js->cijk", G, w.astype(np.float64), G).reshape(C, 16, K)
    assert np.array_equal(got, want.astype(np.float32))


def test_input_transform_exact(oracle):
    rng = np.random.default_rng(3)
    for _ in range(50):
        d = rng.integers(-8, 9, size=16).astype(np.float32)
        want = BT @ d.reshape(4, 4).astype(np.float64) @ BT.T
        assert np.array_equal(oracle.input_transform(d).reshape(4, 4), want.astype(np.float32))


def test_output_transform_exact(oracle):
    rng = np.random.default_rng(4)
    for _ in range(50):
        m = rng.integers(-8, 9, size=16).astype(np.float32)
        want = AT @ m.reshape(4, 4).astype(np.float64) @ AT.T
        assert np.array_equal(oracle.output_transform(m).reshape(2, 2), want.astype(np.float32))


def test_winograd_identity_single_tile():
    # the algebra the three transforms must satisfy together: A^T[(G g G^T).(B^T d B)]A = corr(d,g)
    rng = np.random.default_rng(5)
    d = rng.integers(-3, 4, size=(4, 4)).astype(np.float64)
    g = rng.integers(-3, 4, size=(3, 3)).astype(np.float64)
    y = AT @ ((G @ g @ G.T) * (BT @ d @ BT.T)) @ AT.T
    want = np.array([[np.sum(d[a:a + 3, b:b + 3] * g) for b in range(2)] for a in range(2)])
    np.testing.assert_allclose(y, want, atol=1e-12)


@pytest.mark.parametrize("H,W", [(4, 4), (5, 5), (7, 7), (8, 8), (3, 6), (1, 1)])
def test_direct_conv_vs_bruteforce(oracle, H, W):
    rng = np.random.default_rng(10 + H * 16 + W)
    N, C, K = 4, 5, 6
    x = rng.uniform(-1, 1, (C, H, W, N)).astype(np.float32)
    w = rng.uniform(-1, 1, (C, 3, 3, K)).astype(np.float32)
    np.testing.assert_allclose(oracle.direct_conv_f64(x, w), brute_conv(x, w), rtol=0, atol=1e-12)


def test_direct_conv_impulse(oracle):
    # single input pixel: the output neighbourhood carries the filter taps, index-reversed
    # (cross-correlation: y[h0-(r-1), w0-(s-1)] = g[r][s]); pins every stride of all layouts
    N, C, K, H, W = 3, 4, 5, 6, 7
    rng = np.random.default_rng(6)
    w = rng.uniform(-1, 1, (C, 3, 3, K)).astype(np.float32)
    for (c0, h0, w0, n0) in [(0, 0, 0, 0), (3, 5, 6, 2), (1, 2, 3, 1)]:
        x = np.zeros((C, H, W, N), np.float32)
        x[c0, h0, w0, n0] = 1.0
        y = oracle.direct_conv_f64(x, w)
        want = np.zeros_like(y)
        for r in range(3):
            for s in range(3):
                hh, ww = h0 - (r - 1), w0 - (s - 1)
                if 0 <= hh < H and 0 <= ww < W:
                    want[:, hh, ww, n0] = w[c0, r, s, :]
        assert np.array_equal(y, want)


@pytest.mark.parametrize("H", [4, 5, 7, 8, 14])
def test_winograd_restatement_vs_direct(oracle, H):
    # odd and even sizes: a wrong mask or tile origin gives O(1) border errors
    rng = np.random.default_rng(20 + H)
    N, C, K = 4, 8, 16
    x = rng.uniform(-1, 1, (C, H, H, N)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (9 * C)), (C, 3, 3, K)).astype(np.float32)
    y = oracle.winograd_f32(x, w)
    assert not np.isnan(y).any()  # every output element written
    rel, max_abs, max_ref = oracle.compare(y, oracle.direct_conv_f64(x, w))
    assert rel <= 5e-7 and max_abs <= 1e-6 * max(max_ref, 1.0)


def test_winograd_restatement_exact_on_integers(oracle):
    # x in {-2..2}, g in {-2,0,2}: U is a multiple of 1/2, every partial sum is exactly
    # representable, so the Winograd result equals the direct result bit for bit.
    rng = np.random.default_rng(7)
    N, C, K, H = 4, 8, 8, 7
    x = rng.integers(-2, 3, (C, H, H, N)).astype(np.float32)
    w = (2 * rng.integers(-1, 2, (C, 3, 3, K))).astype(np.float32)
    y = oracle.winograd_f32(x, w)
    assert np.array_equal(y.astype(np.float64), oracle.direct_conv_f64(x, w))


def test_winograd_linearity(oracle):
    rng = np.random.default_rng(8)
    N, C, K, H = 2, 8, 8, 6
    x1 = rng.integers(-2, 3, (C, H, H, N)).astype(np.float32)
    x2 = rng.integers(-2, 3, (C, H, H, N)).astype(np.float32)
    w = (2 * rng.integers(-1, 2, (C, 3, 3, K))).astype(np.float32)
    lhs = oracle.winograd_f32(2 * x1 - 3 * x2, w)
    rhs = 2 * oracle.winograd_f32(x1, w) - 3 * oracle.winograd_f32(x2, w)
    assert np.array_equal(lhs, rhs)


def _rounding_cases():
    """float32 values that separate a correct round-to-nearest-even from its plausible mistakes:
    random values, exact ties (both neighbours' parities), one ulp either side of a tie, carries
    into the exponent, subnormals of the narrow format, overflow to infinity, signed zeros,
    infinities."""
    rng = np.random.default_rng(9)
    bits = rng.integers(0, 1 << 32, 20000, dtype=np.uint64).astype(np.uint32)
    bits = bits[(bits & 0x7F800000) != 0x7F800000]                       # finite
    ties16 = (bits[:5000] & np.uint32(0xFFFF0000)) | np.uint32(0x8000)   # bf16 ties
    ties13 = (rng.integers(0x38800000, 0x47000000, 5000).astype(np.uint32) & np.uint32(0xFFFFE000)) | np.uint32(0x1000)
    near = np.concatenate([ties16 + np.uint32(1), ties16 - np.uint32(1), ties13 + np.uint32(1), ties13 - np.uint32(1)])
    carries = np.array([0x3F7FFFFF, 0x3F7F8000, 0x3F7F7FFF, 0x477FEFFF, 0x477FF000, 0x477FE000, 0x7F7FFFFF,
                        0x7F7F8000, 0x7F7F7FFF, 0x00000001, 0x00008000, 0x00018000, 0x80000000, 0x00000000,
                        0x7F800000, 0xFF800000], dtype=np.uint32)
    sub16 = np.float32(2.0 ** -24) * np.array([0.25, 0.5, 0.75, 1.0, 1.5, 2.5, 3.5, 1023.5, 1024.5], dtype=np.float32)
    small = rng.uniform(-1e-4, 1e-4, 3000).astype(np.float32)             # fp16 subnormal range and around it
    typical = rng.uniform(-4, 4, 3000).astype(np.float32)
    big = np.array([65504.0, 65519.996, 65520.0, 65536.0, 70000.0, -65520.0, -65519.996], dtype=np.float32)
    v = np.concatenate([bits.view(np.float32), ties16.view(np.float32), ties13.view(np.float32),
                        near.view(np.float32), carries.view(np.float32), sub16, -sub16, small, typical, big])
    return v[~np.isnan(v)]


def _nearest_even_on_grid(v: float, mant_bits: int, emin: int, emax: int) -> float:
    """Round-to-nearest-even of a finite double onto the binary format with `mant_bits` stored
    mantissa bits, normal exponents emin..emax and gradual underflow, from the definition (no bit
    tricks): the two neighbouring grid points in exact arithmetic, the nearer one, the one with
    the even significand on a tie; beyond the largest finite value plus half a step: infinity."""
    from fractions import Fraction
    import math
    if v == 0.0 or math.isinf(v):
        return v
    a = Fraction(abs(v))
    e = max(math.floor(math.log2(abs(v))), emin)
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    while e > emin and Fraction(2) ** e > a:
        e -= 1
    step = Fraction(2) ** (e - mant_bits)
    q, r = divmod(a, step)
    if 2 * r > step or (2 * r == step and q % 2 == 1):
        q += 1
    out = q * step
    largest = (Fraction(2) - Fraction(2) ** -mant_bits) * Fraction(2) ** emax
    if out > largest:
        return math.copysign(math.inf, v)
    return math.copysign(float(out), v)


def test_rounding_to_fp16_and_bf16_against_library_casts(oracle):
    # the oracle's RNE helpers against two independent implementations: numpy's float16 cast and
    # torch's CPU bfloat16 / float16 casts
    import torch
    v = _rounding_cases()
    got16 = np.array([oracle.round_operand(x, 1) for x in v], dtype=np.float32)
    got_bf = np.array([oracle.round_operand(x, 2) for x in v], dtype=np.float32)
    with np.errstate(over="ignore"):
        want16_np = v.astype(np.float16).astype(np.float32)
    t = torch.from_numpy(v.copy())
    want16_t = t.to(torch.float16).to(torch.float32).numpy()
    want_bf = t.to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got16.view(np.uint32), want16_np.view(np.uint32))
    assert np.array_equal(got16.view(np.uint32), want16_t.view(np.uint32))
    assert np.array_equal(got_bf.view(np.uint32), want_bf.view(np.uint32))
    # the cases do exercise what they are for
    assert np.isinf(got16[np.isfinite(v)]).any() and (got_bf != v).any() and (got16 != v).any()


def test_rounding_to_fp16_and_bf16_from_the_definition(oracle):
    # ... and against round-to-nearest-even written from its definition in exact rationals
    # (binary16: 10 mantissa bits, exponents -14..15; bfloat16: 7 bits, -126..127)
    v = _rounding_cases()
    rng = np.random.default_rng(10)
    sample = np.concatenate([v[rng.integers(0, v.size, 1500)], v[-40:]])
    for x in sample:
        x = float(x)
        assert oracle.round_operand(x, 1) == _nearest_even_on_grid(x, 10, -14, 15), x
        want = _nearest_even_on_grid(x, 7, -126, 127)
        got = oracle.round_operand(x, 2)
        assert got == want and np.signbit(got) == np.signbit(want), x
    assert oracle.round_operand(1.5, 0) == 1.5 and oracle.round_operand(1.0 + 2.0 ** -20, 0) == 1.0 + 2.0 ** -20


def test_compare_metric_against_numpy(oracle):
    # oracle.compare is the metric every parity verdict goes through: (rel_l2, max_abs, max_ref)
    rng = np.random.default_rng(11)
    for want_dtype in (np.float32, np.float64):
        want = rng.normal(0, 3, (5, 7, 11)).astype(want_dtype)
        got = (want + rng.normal(0, 1e-3, want.shape)).astype(np.float32)
        rel, max_abs, max_ref = oracle.compare(got, want)
        d = got.astype(np.float64) - want.astype(np.float64)
        assert rel == pytest.approx(np.linalg.norm(d.ravel()) / np.linalg.norm(want.astype(np.float64).ravel()), rel=1e-12)
        assert max_abs == pytest.approx(np.abs(d).max(), rel=1e-12)
        assert max_ref == pytest.approx(np.abs(want).max(), rel=1e-12)
        # identical tensors: exactly zero
        same = want.astype(np.float32)
        assert oracle.compare(same, same.astype(want_dtype))[:2] == (0.0, 0.0)
        # one wrong element is seen by both error figures
        bad = same.copy()
        bad[2, 3, 4] += 0.5
        rel1, max1, _ = oracle.compare(bad, same.astype(want_dtype))
        assert max1 == pytest.approx(0.5, rel=1e-6)
        assert rel1 == pytest.approx(0.5 / np.linalg.norm(same.astype(np.float64).ravel()), rel=1e-6)
        # a NaN or an infinity in the result can never pass a bound
        for poison in (np.nan, np.inf, -np.inf):
            p = same.copy()
            p[0, 0, 0] = poison
            rel2, max2, _ = oracle.compare(p, same.astype(want_dtype))
            assert not rel2 <= 1e30 and not max2 <= 1e30


@pytest.mark.parametrize("quant,bound", [(1, 2e-3), (2, 1.5e-2)])
def test_quantised_restatement_vs_direct(oracle, quant, bound):
    # fp16 / bf16 GEMM operands: unit round-offs 2^-11 / 2^-8 on both operands
    rng = np.random.default_rng(30 + quant)
    N, C, K, H = 4, 16, 16, 7
    x = rng.uniform(-1, 1, (C, H, H, N)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (9 * C)), (C, 3, 3, K)).astype(np.float32)
    rel, _, _ = oracle.compare(oracle.winograd_f32(x, w, quant), oracle.direct_conv_f64(x, w))
    assert 1e-6 < rel <= bound  # quantisation visible, inside the stated bound


# ---------------------------------------------------------------- committed known-answer vectors

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GOLDEN_CASES = sorted(f[:-4] for f in os.listdir(GOLDEN) if f.endswith(".npz"))


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_oracle_reproduces_known_answer_vectors(oracle, name):
    # tests/golden/*.npz: integer tensors and their exact int64 convolution (numpy only,
    # tests/golden/make_vectors.py); both oracle paths must hit them bit for bit
    v = np.load(os.path.join(GOLDEN, name + ".npz"))
    x, w, y = v["x"].astype(np.float32), v["w"].astype(np.float32), v["y"]
    assert np.array_equal(oracle.direct_conv_f64(x, w), y.astype(np.float64))
    if x.shape[1] == x.shape[2]:  # the restatement follows the reference: square images only
        assert np.array_equal(oracle.winograd_f32(x, w), y.astype(np.float32))
        # the fp16 / bf16 roundings of the quantised restatement are exact on these values
        # (|U| <= 18, |V| <= 16 are integers), so it must hit the same vectors
        assert np.array_equal(oracle.winograd_f32(x, w, 1), y.astype(np.float32))
        assert np.array_equal(oracle.winograd_f32(x, w, 2), y.astype(np.float32))
