"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, validates arguments before touching a GPU, and the seeded generators behave."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text)) - {"defined"})


def test_header_symbols_exported(ocn):
    api, bench = declared_functions("opencnn_amd.h"), declared_functions("opencnn_amd_bench.h")
    assert "convolutionForward" in api and "opencnn_filter_transform" in api
    # bench and test support lives in its own header, and only there
    assert set(bench) == {"opencnn_time_forward", "opencnn_set_tile_order", "opencnn_set_range_weight",
                          "opencnn_set_wait_limit", "opencnn_set_timeline_buffer", "opencnn_synth_input",
                          "opencnn_synth_filter"}
    assert not set(api) & set(bench)
    handle = ctypes.CDLL(ocn.LIB_PATH)
    for name in api + bench:
        assert hasattr(handle, name), f"{name} declared in include/ but not exported"
    assert sorted(ocn.EXPORTED_SYMBOLS) == sorted(api + bench)  # the binding covers exactly the headers


def test_tiles_dim_and_workspace(ocn, oracle):
    for w in (1, 2, 5, 7, 8, 14, 28, 56, 57, 224):
        assert ocn.tiles_dim(w) == oracle.tiles_dim(w) == (w + 1) // 2
    assert ocn.workspace_bytes(256, 256) == 256 * 256 * 16 * 4
    assert ocn.workspace_bytes(0, 64) == 0
    # shapes outside the reference's tiling: filters padded to 32, channels to 8 (fp32 operands)
    # or to 64 and 16 (2-byte operands), whichever needs more
    assert ocn.workspace_bytes(12, 48) == 16 * 64 * 16 * 4
    assert ocn.workspace_bytes(1, 1) == max(8 * 32 * 16 * 4, 16 * 64 * 16 * 2)
    assert ocn.workspace_bytes(24, 65) == 24 * 96 * 16 * 4


def _call(ocn, **over):
    """convolutionForward with dummy non-null pointers: validation must fail before launch."""
    a = dict(N=32, C=8, H=8, W=8, K=64, R=3, S=3, m=2, alpha=4, tile=4)
    a.update(over)
    td = over.get("tiles_dim", ocn.tiles_dim(a["W"]))
    oh, ow = over.get("out_h", a["H"]), over.get("out_w", a["W"])
    on, oc = over.get("out_n", a["N"]), over.get("out_c", a["K"])
    fc = over.get("filt_c", a["C"])
    ptr = over.get("ptr", 0x1000)
    return ocn.lib().convolutionForward(ptr, a["H"], a["W"], ptr, oh, ow, on, oc, ptr, ptr,
                                        on * oc * oh * ow, td, a["N"], a["tile"], td * 4,
                                        a["C"], a["K"], fc, a["R"], a["S"], a["alpha"], a["m"])


@pytest.mark.parametrize("over", [
    dict(N=0), dict(N=-32), dict(K=0), dict(C=0), dict(R=5), dict(S=1), dict(m=4),
    dict(alpha=6), dict(tile=6), dict(H=8, W=10), dict(out_h=6), dict(out_n=64), dict(out_c=32),
    dict(filt_c=16), dict(tiles_dim=3), dict(ptr=0), dict(N=1 << 20, H=56, W=56),
])
def test_unsupported_arguments_are_rejected(ocn, over):
    # the reference mis-computes or returns garbage here (src/openCNN_winograd.cu:212-218);
    # the drop-in must return hipErrorInvalidValue (1) and launch nothing
    assert _call(ocn, **over) == 1
    assert ocn.lib().opencnn_last_error() != b""


def test_filter_transform_rejects_bad_arguments(ocn):
    f = ocn.lib().opencnn_filter_transform
    assert f(0x1000, 0x1000, 0, 8, 0, 0) == 1
    assert f(0x1000, 0x1000, 64, -8, 0, 0) == 1
    assert f(0x1000, 0x1000, 64, 8, 2, 0) == 1
    assert f(0x1000, 0x1000, 64, 8, 0, 2) == 1
    assert f(0, 0x1000, 64, 8, 0, 0) == 1


def test_descriptor_is_validated_before_any_launch(ocn):
    d = ocn.ConvDesc()
    call = lambda: ocn.lib().opencnn_conv_forward_desc(ctypes.byref(d))
    assert ocn.lib().opencnn_conv_forward_desc(None) == 1
    assert call() == 1  # struct_size 0
    d.struct_size = ctypes.sizeof(ocn.ConvDesc)
    assert ctypes.sizeof(ocn.ConvDesc) == 104  # the layout of opencnn_conv_desc on LP64
    assert call() == 1  # null tensors
    d.in_ = d.out = d.Ww = d.filter = 0x1000
    d.in_n, d.in_c, d.in_h, d.in_w, d.filt_k = 32, 8, 8, 8, 64
    for field, bad in (("operand_precision", 3), ("kernel_variant", 5), ("filter_layout", 2), ("in_c", 0),
                       ("split_flags_bytes", 4096)):
        good = getattr(d, field)
        setattr(d, field, bad)
        assert call() == 1, field
        assert ocn.lib().opencnn_last_error() != b""
        setattr(d, field, good)
    d.split_flags, d.split_flags_bytes = 0x2000, ocn.split_flags_bytes() - 4
    assert call() == 1  # flag storage too small
    d.split_flags, d.split_flags_bytes = 0x2002, ocn.split_flags_bytes()
    assert call() == 1  # misaligned
    assert ocn.split_flags_bytes() == 32768


def test_status_query_without_a_launch(ocn):
    # nothing has run on any device: nothing to report, and nothing that needs a GPU
    assert ocn.lib().opencnn_check_status() == 0
    assert ocn.lib().opencnn_set_wait_limit(0) == 0
    assert ocn.lib().opencnn_forget_workspace(0x1000) == 0
    assert ocn.last_launch() == (0, -1)
    assert ocn.unsplit_launches() == 0
    assert ocn.lib().opencnn_release_capture(None, -1) == 0
    assert ocn.lib().opencnn_release_capture(None, 3) == 1     # not a graph set
    assert ocn.lib().opencnn_release_capture(None, 48) == 1
    assert ocn.lib().opencnn_release_split_flags(0x1000) == 0
    for bad in (-2, 7):
        assert ocn.lib().opencnn_set_range_weight(bad) == 1
    assert ocn.lib().opencnn_set_range_weight(-1) == 0
    assert ocn.lib().opencnn_set_tile_order(8) == 1 and ocn.lib().opencnn_set_tile_order(7) == 0


def test_synth_layouts_agree(ocn):
    N, C, H, W, K = 32, 8, 5, 6, 64
    chwn = ocn.synth_input(N, C, H, W, seed=0x0C99)
    nchw = ocn.synth_input(N, C, H, W, seed=0x0C99, layout=ocn.INPUT_NCHW)
    assert np.array_equal(chwn, nchw.transpose(1, 2, 3, 0))
    crsk = ocn.synth_filter(K, C, seed=0xF117)
    kcrs = ocn.synth_filter(K, C, seed=0xF117, layout=ocn.FILTER_KCRS)
    assert np.array_equal(crsk, kcrs.transpose(1, 2, 3, 0))


def test_synth_distributions(ocn):
    x = ocn.synth_input(64, 16, 14, 14, seed=1)
    assert x.min() >= -1.0 and x.max() < 1.0 and abs(x.mean()) < 0.01
    assert abs(x.var() - 1.0 / 3.0) < 0.01
    relu = ocn.synth_input(64, 16, 14, 14, seed=1, p0=0.0, p1=1.0)
    assert relu.min() >= 0.0 and relu.max() < 1.0
    C = 64
    g = ocn.synth_filter(128, C, seed=2)
    assert abs(g.mean()) < 2e-3 and abs(g.std() / np.sqrt(2.0 / (9 * C)) - 1.0) < 0.02
    assert not np.array_equal(x, ocn.synth_input(64, 16, 14, 14, seed=2))
    assert np.array_equal(x, ocn.synth_input(64, 16, 14, 14, seed=1))


def test_unswizzle_is_a_permutation(ocn):
    C, K = 8, 64
    a = np.arange(C * 16 * K, dtype=np.float32)
    b = ocn.unswizzle_ww(a, C, K)
    assert sorted(b.ravel().tolist()) == a.tolist()
    # element (kg=1, q=1, p/2=1, h=1, k32=5, p%2=1, s=1) is c = 4+2+1 = 7, k = 37, p = 3
    idx = (((((1 * (C // 4) + 1) * 8 + 1) * 2 + 1) * 32 + 5) * 2 + 1) * 2 + 1
    assert b[7, 3, 37] == a[idx]


def test_use_library_swaps_the_library_behind_the_module(ocn, tmp_path):
    """bench.py --library: another build of the same C ABI becomes the library the wrappers call;
    a path without a library is refused."""
    import opencnn_amd.binding as binding

    own = binding.lib()
    try:
        other = ocn.use_library(ocn.LIB_PATH)
        assert binding.lib() is other
        assert other.opencnn_tiles_dim(56) == 28
        with pytest.raises(ImportError):
            ocn.use_library(str(tmp_path / "libopencnn_amd_missing.so"))
        assert binding.lib() is other
    finally:
        binding._lib = own
