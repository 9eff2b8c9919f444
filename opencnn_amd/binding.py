"""ctypes binding of ``libopencnn_amd.so`` (the C ABI declared in ``include/opencnn_amd.h``).

Device buffers are passed as ``torch`` CUDA(ROCm) tensors or raw integer addresses;
torch is only the owner of device memory and streams here.  Every wrapper raises
:class:`OpenCNNError` on a non-zero status.  Nothing in this module computes a
convolution on the CPU: without the built library there is no product path.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libopencnn_amd.so")

# enum values of include/opencnn_amd.h
WW_REFERENCE, WW_MFMA = 0, 1
FILTER_CRSK, FILTER_KCRS = 0, 1
INPUT_CHWN, INPUT_NCHW = 0, 1
DIST_UNIFORM, DIST_NORMAL = 0, 1
KERNEL_AUTO, KERNEL_REGISTER, KERNEL_LDS, KERNEL_ASM, KERNEL_HIP = 0, 1, 2, 3, 4
F32, F16, BF16 = 0, 1, 2

_c_int, _c_float_p, _c_void_p = ctypes.c_int, ctypes.POINTER(ctypes.c_float), ctypes.c_void_p

# name -> (restype, argtypes); one entry per declaration in include/opencnn_amd.h and
# include/opencnn_amd_bench.h
EXPORTED_SYMBOLS = {
    "opencnn_init": (_c_int, []),
    "convolutionForward": (
        _c_int,
        [_c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
         _c_void_p, ctypes.c_uint, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_int],
    ),
    "convolutionForward_32x64x8": (
        _c_int,
        [_c_void_p, _c_int, _c_int, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p,
         _c_void_p, ctypes.c_uint, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int],
    ),
    "opencnn_tiles_dim": (_c_int, [_c_int]),
    "opencnn_workspace_bytes": (ctypes.c_size_t, [_c_int, _c_int]),
    "opencnn_set_stream": (_c_int, [_c_void_p]),
    "opencnn_set_kernel_variant": (_c_int, [_c_int]),
    "opencnn_set_balanced_split": (_c_int, [_c_int]),
    "opencnn_set_timeline_buffer": (_c_int, [_c_void_p, ctypes.c_size_t]),
    "opencnn_set_operand_precision": (_c_int, [_c_int]),
    "opencnn_filter_transform": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int]),
    "opencnn_conv_forward_pretransformed": (
        _c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int]),
    "opencnn_conv_forward_static": (
        _c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int]),
    "opencnn_static_workspace_bytes": (ctypes.c_size_t, []),
    "opencnn_nchw_to_chwn": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int]),
    "opencnn_khwn_to_nkhw": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int]),
    "opencnn_kcrs_to_crsk": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_int]),
    "opencnn_time_forward": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_float_p, _c_float_p, _c_float_p],
    ),
    "opencnn_synth_input": (
        _c_int,
        [_c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, ctypes.c_ulonglong, _c_int,
         ctypes.c_double, ctypes.c_double],
    ),
    "opencnn_synth_filter": (
        _c_int,
        [_c_void_p, _c_int, _c_int, _c_int, ctypes.c_ulonglong, _c_int, ctypes.c_double,
         ctypes.c_double],
    ),
    "opencnn_last_error": (ctypes.c_char_p, []),
    "opencnn_last_kernel": (ctypes.c_char_p, []),
    "opencnn_last_launch": (_c_int, [ctypes.POINTER(_c_int), ctypes.POINTER(_c_int)]),
    "opencnn_check_status": (_c_int, []),
    "opencnn_release_stream": (_c_int, [_c_void_p]),
    "opencnn_set_wait_limit": (_c_int, [ctypes.c_uint]),
    "opencnn_set_tile_order": (_c_int, [_c_int]),
    "opencnn_set_range_weight": (_c_int, [_c_int]),
    "opencnn_release_capture": (_c_int, [_c_void_p, _c_int]),
    "opencnn_release_split_flags": (_c_int, [_c_void_p]),
    "opencnn_unsplit_launches": (ctypes.c_ulonglong, []),
    "opencnn_forget_workspace": (_c_int, [_c_void_p]),
    "opencnn_conv_forward_desc": (_c_int, [_c_void_p]),
    "opencnn_split_flags_bytes": (ctypes.c_size_t, []),
}


class ConvDesc(ctypes.Structure):
    """opencnn_conv_desc of include/opencnn_amd.h."""

    _fields_ = [
        ("struct_size", ctypes.c_size_t),
        ("in_", _c_void_p), ("filter", _c_void_p), ("out", _c_void_p), ("Ww", _c_void_p),
        ("in_n", _c_int), ("in_c", _c_int), ("in_h", _c_int), ("in_w", _c_int), ("filt_k", _c_int),
        ("filter_layout", _c_int), ("operand_precision", _c_int), ("kernel_variant", _c_int),
        ("balanced_split", _c_int),
        ("stream", _c_void_p), ("split_flags", _c_void_p), ("split_flags_bytes", ctypes.c_size_t),
    ]


class OpenCNNError(RuntimeError):
    """A C-ABI call returned a non-zero hipError_t."""

    def __init__(self, func: str, status: int, detail: str = ""):
        self.func, self.status, self.detail = func, status, detail
        msg = f"{func} failed with hipError_t {status}"
        if detail:
            msg += f" (failed check: {detail})"
        super().__init__(msg)


_lib: Optional[ctypes.CDLL] = None


def load_library(path: str = LIB_PATH) -> ctypes.CDLL:
    """Load the built HIP library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None and path == LIB_PATH:
        return _lib
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `make -C opencnn_amd/csrc` "
            "(or __graft_entry__.build()); opencnn_amd has no non-HIP path")
    # One HIP runtime per process: torch ships its own libamdhip64 (same SONAME as ROCm's).
    # Importing torch first makes the dynamic loader resolve this library's dependency to the
    # copy torch already mapped; loaded in the other order the process ends up with two
    # runtimes and the second one reports hipErrorNoDevice.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    handle = ctypes.CDLL(path)
    for name, (restype, argtypes) in EXPORTED_SYMBOLS.items():
        fn = getattr(handle, name)  # AttributeError if the symbol is not exported
        fn.restype, fn.argtypes = restype, argtypes
    if path == LIB_PATH:
        _lib = handle
    return handle


def use_library(path: str) -> ctypes.CDLL:
    """Make another build of the same C ABI the library behind this module for the rest of the
    process (the timing-only builds of `make -C opencnn_amd/csrc diagnostic`)."""
    global _lib
    _lib = load_library(path)
    return _lib


def lib() -> ctypes.CDLL:
    return _lib if _lib is not None else load_library()


def _ptr(buf) -> int:
    """Address of a torch tensor / numpy array / raw int."""
    if isinstance(buf, int):
        return buf
    if isinstance(buf, np.ndarray):
        if not buf.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy buffer must be C-contiguous")
        return buf.ctypes.data
    if hasattr(buf, "data_ptr"):
        if not buf.is_contiguous():
            raise ValueError("tensor must be contiguous")
        return buf.data_ptr()
    raise TypeError(f"cannot take the address of {type(buf)!r}")


def _dev_f32(buf, what: str) -> int:
    if hasattr(buf, "is_cuda"):
        import torch

        if not buf.is_cuda:
            raise ValueError(f"{what} must live in device memory")
        if buf.dtype != torch.float32:
            raise ValueError(f"{what} must be float32")
    return _ptr(buf)


def _check(func: str, status: int) -> None:
    if status != 0:
        # hipErrorInvalidValue, hipErrorNotInitialized, hipErrorLaunchFailure: set by the library itself
        detail = lib().opencnn_last_error().decode() if status in (1, 3, 719) else ""
        raise OpenCNNError(func, status, detail)


def init() -> None:
    _check("opencnn_init", lib().opencnn_init())


def last_kernel() -> str:
    """Name of the fused kernel this thread's last successful launch used."""
    return lib().opencnn_last_kernel().decode()


def last_launch():
    """(workgroups, flag set) of this thread's last successful fused-kernel launch; flag set -1 =
    launched without the split."""
    grid, flag_set = _c_int(0), _c_int(0)
    _check("opencnn_last_launch", lib().opencnn_last_launch(ctypes.byref(grid), ctypes.byref(flag_set)))
    return grid.value, flag_set.value


def check_status() -> None:
    """Raises OpenCNNError (hipErrorLaunchFailure, 719) if a launch on the current device gave up
    waiting for a partial tile since the last check; call after synchronising."""
    _check("opencnn_check_status", lib().opencnn_check_status())


def release_stream(stream) -> None:
    """Wait for `stream` and give its set of split-merge flags back."""
    handle = 0 if stream is None else getattr(stream, "cuda_stream", stream)
    _check("opencnn_release_stream", lib().opencnn_release_stream(handle))


def set_tile_order(bits: int) -> None:
    """Order of the tiles in the image for this thread's later launches (bits 1, 2, 4 of
    opencnn_set_tile_order; default 7)."""
    _check("opencnn_set_tile_order", lib().opencnn_set_tile_order(bits))


def set_range_weight(half_units: int) -> None:
    """How this thread's later launches cut the ranges of the balanced split: -1 the library
    chooses, 0 equal numbers of units, 1 ... 6 half units per tile end."""
    _check("opencnn_set_range_weight", lib().opencnn_set_range_weight(half_units))


def release_capture(stream=None, flag_set: int = -1) -> None:
    """Give graph flag sets back: the set `flag_set`, or every set recorded on `stream` (None: on
    any stream).  The graphs recorded with them must not run again."""
    handle = 0 if stream is None else getattr(stream, "cuda_stream", stream)
    _check("opencnn_release_capture", lib().opencnn_release_capture(handle, flag_set))


def release_split_flags(split_flags) -> None:
    """Forget a caller-owned flag buffer (its status word is free for another buffer)."""
    _check("opencnn_release_split_flags", lib().opencnn_release_split_flags(_ptr(split_flags)))


def unsplit_launches() -> int:
    """Launches so far that wanted to cut tiles between workgroups and found no flag set free."""
    return lib().opencnn_unsplit_launches()


def set_wait_limit(polls: int) -> None:
    """Polls after which a kernel's wait for a partial tile gives up (0: the default)."""
    _check("opencnn_set_wait_limit", lib().opencnn_set_wait_limit(polls))


def split_flags_bytes() -> int:
    return lib().opencnn_split_flags_bytes()


def forget_workspace(Ww) -> None:
    _check("opencnn_forget_workspace", lib().opencnn_forget_workspace(_ptr(Ww)))


def _workspace(buf, filt_c: int, filt_k: int) -> int:
    """Address of a Ww buffer after checking that it holds opencnn_workspace_bytes()."""
    if hasattr(buf, "numel"):
        have, need = buf.numel() * buf.element_size(), workspace_bytes(filt_c, filt_k)
        if have < need:
            raise ValueError(f"workspace holds {have} bytes, opencnn_workspace_bytes({filt_c}, {filt_k}) = {need}")
    return _dev_f32(buf, "workspace")


def conv_forward_desc(x, w, y, Ww, in_n, in_c, in_h, in_w, filt_k, *, filter_layout=FILTER_CRSK,
                      precision=F32, variant=KERNEL_AUTO, balanced_split=True, stream=None,
                      split_flags=None) -> None:
    """opencnn_conv_forward_desc: one call with its own settings.  `w` None = Ww holds a
    transformed filter already; `split_flags` a zeroed CUDA tensor of split_flags_bytes() or None."""
    d = ConvDesc()
    d.struct_size = ctypes.sizeof(ConvDesc)
    d.in_, d.out = _dev_f32(x, "input"), _dev_f32(y, "output")
    d.filter = None if w is None else _dev_f32(w, "filter")
    d.Ww = _workspace(Ww, in_c, filt_k)
    d.in_n, d.in_c, d.in_h, d.in_w, d.filt_k = in_n, in_c, in_h, in_w, filt_k
    d.filter_layout, d.operand_precision, d.kernel_variant = filter_layout, precision, variant
    d.balanced_split = 1 if balanced_split else 0
    d.stream = None if stream is None else getattr(stream, "cuda_stream", stream)
    if split_flags is not None:
        d.split_flags = _ptr(split_flags)
        d.split_flags_bytes = split_flags.numel() * split_flags.element_size()
    _check("opencnn_conv_forward_desc", lib().opencnn_conv_forward_desc(ctypes.byref(d)))


def tiles_dim(in_w: int) -> int:
    return lib().opencnn_tiles_dim(in_w)


def workspace_bytes(filt_c: int, filt_k: int) -> int:
    return lib().opencnn_workspace_bytes(filt_c, filt_k)


def set_stream(stream) -> None:
    """Select the stream of later calls: a torch.cuda.Stream, a raw handle or None."""
    handle = 0 if stream is None else getattr(stream, "cuda_stream", stream)
    _check("opencnn_set_stream", lib().opencnn_set_stream(handle))


def set_kernel_variant(variant: int) -> None:
    """KERNEL_AUTO, KERNEL_REGISTER, KERNEL_LDS, KERNEL_ASM or KERNEL_HIP for later launches."""
    _check("opencnn_set_kernel_variant", lib().opencnn_set_kernel_variant(variant))


def set_balanced_split(enable: bool) -> None:
    """Persistent, evenly split launch of the LDS kernel for tile counts that do not fill
    whole rounds of CUs (default on)."""
    _check("opencnn_set_balanced_split", lib().opencnn_set_balanced_split(1 if enable else 0))


def set_timeline_buffer(buf) -> None:
    """Record the assembly kernels' timeline into `buf` (a CUDA int64 tensor with 64 entries per
    workgroup), or stop recording with None."""
    if buf is None:
        _check("opencnn_set_timeline_buffer", lib().opencnn_set_timeline_buffer(None, 0))
        return
    if not (buf.is_cuda and buf.is_contiguous() and buf.element_size() == 8):
        raise ValueError("timeline buffer must be a contiguous CUDA int64 tensor")
    _check("opencnn_set_timeline_buffer",
           lib().opencnn_set_timeline_buffer(buf.data_ptr(), buf.numel() * 8))


def read_timeline(buf, n_workgroups: int):
    """Host copy of a recorded timeline: list (one entry per workgroup) of microsecond offsets from
    the earliest stamp of the launch."""
    d = buf.cpu().numpy().reshape(-1, 64)[:n_workgroups]
    counts = d[:, 0].astype(int)
    t0 = min(int(d[b, 2]) for b in range(n_workgroups) if counts[b] > 0)
    return [((d[b, 2:2 + counts[b]] - t0) / 100.0).tolist() for b in range(n_workgroups)]


def set_operand_precision(precision: int) -> None:
    """F32 (default), F16 or BF16 GEMM operands for later calls."""
    _check("opencnn_set_operand_precision", lib().opencnn_set_operand_precision(precision))


def convolutionForward(k, in_h, in_w, w, out_h, out_w, out_n, out_c, C, Ww, n, tiles_dim,
                       in_n, tile_size, elems_dim, in_c, filt_k, filt_c, filt_h, filt_w,
                       alpha, m) -> None:
    """The reference's dispatcher, argument for argument (src/openCNN_winograd.cu:204-209):
    ``k`` CHWN input, ``w`` CRSK filters, ``C`` KHWN output, ``Ww`` workspace."""
    _check("convolutionForward", lib().convolutionForward(
        _dev_f32(k, "input"), in_h, in_w, _dev_f32(w, "filter"), out_h, out_w, out_n, out_c,
        _dev_f32(C, "output"), _workspace(Ww, filt_c, filt_k), n, tiles_dim, in_n, tile_size,
        elems_dim, in_c, filt_k, filt_c, filt_h, filt_w, alpha, m))


def filter_transform(w, Ww, filt_k, filt_c, filter_layout=FILTER_CRSK,
                     ww_layout=WW_REFERENCE) -> None:
    ww = _workspace(Ww, filt_c, filt_k) if ww_layout == WW_MFMA else _dev_f32(Ww, "workspace")
    _check("opencnn_filter_transform", lib().opencnn_filter_transform(
        _dev_f32(w, "filter"), ww, filt_k, filt_c, filter_layout, ww_layout))


def conv_forward_pretransformed(x, Ww, y, in_n, in_c, in_h, in_w, filt_k) -> None:
    _check("opencnn_conv_forward_pretransformed", lib().opencnn_conv_forward_pretransformed(
        _dev_f32(x, "input"), _workspace(Ww, in_c, filt_k), _dev_f32(y, "output"), in_n, in_c,
        in_h, in_w, filt_k))


def conv_forward_static(x, w, y, in_n, in_c, in_h, in_w, filt_k) -> None:
    """convolutionForward on the library's static workspace (allocates nothing; needs init())."""
    _check("opencnn_conv_forward_static", lib().opencnn_conv_forward_static(
        _dev_f32(x, "input"), _dev_f32(w, "filter"), _dev_f32(y, "output"), in_n, in_c, in_h,
        in_w, filt_k))


def static_workspace_bytes() -> int:
    return lib().opencnn_static_workspace_bytes()


def nchw_to_chwn(src, dst, n, c, h, w) -> None:
    _check("opencnn_nchw_to_chwn", lib().opencnn_nchw_to_chwn(_dev_f32(src, "src"), _dev_f32(dst, "dst"), n, c, h, w))


def khwn_to_nkhw(src, dst, n, k, h, w) -> None:
    _check("opencnn_khwn_to_nkhw", lib().opencnn_khwn_to_nkhw(_dev_f32(src, "src"), _dev_f32(dst, "dst"), n, k, h, w))


def kcrs_to_crsk(src, dst, k, c) -> None:
    _check("opencnn_kcrs_to_crsk", lib().opencnn_kcrs_to_crsk(_dev_f32(src, "src"), _dev_f32(dst, "dst"), k, c))


def time_forward(x, w, y, Ww, in_n, in_c, in_h, in_w, filt_k, warmup=1, iters=100,
                 parts=("total", "main", "fx")):
    """Mean ms per call: (filter transform + fused kernel, fused kernel, filter transform); only
    the loops named in `parts` run, the others come back as 0."""
    t = [ctypes.c_float(0.0) for _ in range(3)]
    ref = [ctypes.byref(t[i]) if name in parts else None for i, name in enumerate(("total", "main", "fx"))]
    _check("opencnn_time_forward", lib().opencnn_time_forward(
        _dev_f32(x, "input"), _dev_f32(w, "filter"), _dev_f32(y, "output"),
        _workspace(Ww, in_c, filt_k), in_n, in_c, in_h, in_w, filt_k, warmup, iters, *ref))
    return t[0].value, t[1].value, t[2].value


def synth_input(n, c, h, w, seed, layout=INPUT_CHWN, dist=DIST_UNIFORM, p0=-1.0, p1=1.0):
    """Seeded host tensor, shape (c,h,w,n) for CHWN or (n,c,h,w) for NCHW."""
    shape = (c, h, w, n) if layout == INPUT_CHWN else (n, c, h, w)
    out = np.empty(shape, dtype=np.float32)
    _check("opencnn_synth_input", lib().opencnn_synth_input(
        out.ctypes.data, n, c, h, w, layout, seed, dist, p0, p1))
    return out


def synth_filter(k, c, seed, layout=FILTER_CRSK, dist=DIST_NORMAL, p0=0.0, p1=None):
    """Seeded host filters, shape (c,3,3,k) for CRSK or (k,c,3,3) for KCRS.
    Default: He-init normal(0, sqrt(2/(9c)))."""
    if p1 is None:
        p1 = float(np.sqrt(2.0 / (9.0 * c)))
    shape = (c, 3, 3, k) if layout == FILTER_CRSK else (k, c, 3, 3)
    out = np.empty(shape, dtype=np.float32)
    _check("opencnn_synth_filter", lib().opencnn_synth_filter(
        out.ctypes.data, k, c, layout, seed, dist, p0, p1))
    return out


def unswizzle_ww(ww_mfma: np.ndarray, filt_c: int, filt_k: int) -> np.ndarray:
    """Reorder a host copy of an OPENCNN_WW_MFMA buffer ([kp/32][cp/4][8][2][32][2][2], kp / cp =
    filt_k / filt_c rounded up to 32 / 8) into the reference's [c][16][k] order
    (src/FX_m2.cu:84).  Pure permutation, no arithmetic; the zero padding is dropped."""
    kp, cp = -(-filt_k // 32) * 32, -(-filt_c // 8) * 8
    a = np.asarray(ww_mfma, dtype=np.float32).reshape(-1)[:kp * cp * 16]  # a workspace may be larger
    a = a.reshape(kp // 32, cp // 4, 8, 2, 32, 2, 2)
    # axes: kg, q, p/2, h, k32, p%2, s ; c = 4q + 2s + h ; k = 32kg + k32
    a = a.transpose(1, 6, 3, 2, 5, 0, 4)  # q, s, h, p/2, p%2, kg, k32
    return np.ascontiguousarray(a.reshape(cp, 16, kp)[:filt_c, :, :filt_k])
