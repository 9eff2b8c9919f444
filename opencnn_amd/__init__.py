"""opencnn_amd: MI355X (gfx950) Winograd F(2x2,3x3) forward convolution behind a C ABI.

This package is a thin ctypes binding over ``libopencnn_amd.so`` (hand-written HIP
kernels, see ``csrc/``).  There is no fallback of any kind: if the library is missing
or fails to load, importing :mod:`opencnn_amd.binding` symbols that need it raises.

Names mirror the reference's host interface (``convolutionForward`` and the bench's
shape arguments, src/openCNN_winograd.cu:204-219,246-255).
"""
from .binding import (  # noqa: F401
    LIB_PATH,
    OpenCNNError,
    convolutionForward,
    conv_forward_pretransformed,
    conv_forward_static,
    static_workspace_bytes,
    filter_transform,
    init,
    lib,
    load_library,
    set_stream,
    set_kernel_variant,
    set_balanced_split,
    set_timeline_buffer,
    read_timeline,
    nchw_to_chwn,
    khwn_to_nkhw,
    kcrs_to_crsk,
    set_operand_precision,
    F32,
    F16,
    BF16,
    KERNEL_AUTO,
    KERNEL_REGISTER,
    KERNEL_LDS,
    KERNEL_ASM,
    KERNEL_HIP,
    synth_filter,
    synth_input,
    last_kernel,
    tiles_dim,
    time_forward,
    workspace_bytes,
    EXPORTED_SYMBOLS,
    FILTER_CRSK,
    FILTER_KCRS,
    WW_REFERENCE,
    WW_MFMA,
    INPUT_CHWN,
    INPUT_NCHW,
    DIST_UNIFORM,
    DIST_NORMAL,
    unswizzle_ww,
)

__all__ = [
    "LIB_PATH",
    "OpenCNNError",
    "convolutionForward",
    "conv_forward_pretransformed",
    "conv_forward_static",
    "filter_transform",
    "init",
    "last_kernel",
    "lib",
    "load_library",
    "set_stream",
    "synth_filter",
    "synth_input",
    "tiles_dim",
    "time_forward",
    "workspace_bytes",
    "unswizzle_ww",
]
