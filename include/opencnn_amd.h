/*
 * opencnn_amd — C ABI of the MI355X (gfx950) Winograd F(2x2,3x3) forward convolution.
 *
 * Plain C: pointers and sizes only.  Every device pointer is memory the CALLER
 * allocated on the current HIP device (any float-aligned address, e.g. a slice of a larger
 * allocation); the library allocates no tensors or workspaces.  Its
 * state between calls is the process-wide settings of the opencnn_set_* calls below (stream,
 * kernel variant, balanced split, operand precision; opencnn_conv_forward_desc takes all of
 * them per call instead), the code objects of its assembly kernels (embedded in the library,
 * loaded once per device by opencnn_init or the first launch), 1.5 MB of static device memory
 * that the balanced split uses to hand tiles over between workgroups (48 sets of flags and a spare, zero
 * between launches; see opencnn_set_balanced_split), per device 452 bytes of pinned host memory
 * that the kernels report a failed hand-over in (opencnn_check_status) and 32 events, all made by
 * opencnn_init or the first launch on the device, and a host-side record of the transformed
 * filters it wrote (opencnn_filter_transform).
 * Bench and test support (timing loop, timeline, tile order, wait limit, synthetic tensors) is
 * declared in opencnn_amd_bench.h and exported by the same library.
 * All entry points return a hipError_t value as int (0 == hipSuccess); launches are
 * asynchronous on the selected stream, exactly like the reference, which returns
 * cudaGetLastError() right after its two launches
 * (src/convolutionForward_32x64x8.cu:274-283).
 *
 * Tensor layouts (row-major, last index fastest), as in the reference:
 *   input   CHWN  [in_c][in_h][in_w][in_n]      src/openCNN_winograd.cu:149-150,230
 *   filter  CRSK  [filt_c][3][3][filt_k]        src/openCNN_winograd.cu:235, src/FX_m2.cu:56-57
 *   output  KHWN  [out_c][out_h][out_w][out_n]  src/store_and_transform_output_optSTS64.cuh:85-87
 *   Ww      opencnn_workspace_bytes(filt_c, filt_k) bytes of caller-owned scratch, overwritten
 *           by every call: filt_c*16*filt_k floats as in the reference
 *           (src/openCNN_winograd.cu:310-311) on the shapes the reference takes, more on the
 *           others (see opencnn_workspace_bytes).  Its CONTENT is the transformed filter
 *           U = G g G^T in an MFMA-operand order private to this library; use
 *           opencnn_filter_transform(..., OPENCNN_WW_REFERENCE) to obtain the reference's
 *           [filt_c][16][filt_k] order (src/FX_m2.cu:58-59,84).
 */
#ifndef OPENCNN_AMD_H
#define OPENCNN_AMD_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout of the transformed-filter buffer written by opencnn_filter_transform. */
enum {
  OPENCNN_WW_REFERENCE = 0, /* [filt_c][16][filt_k], position p = i*4+j (src/FX_m2.cu:84) */
  OPENCNN_WW_MFMA = 1       /* [kp/32][cp/4][8][2][32][2][2], kp / cp = filt_k / filt_c rounded up to 32 / 8,
                               padding zero: what the fused kernels read */
};

/* Layout of the 3x3 filters handed to the library. */
enum {
  OPENCNN_FILTER_CRSK = 0, /* what the reference's FX reads (src/FX_m2.cu:69) */
  OPENCNN_FILTER_KCRS = 1  /* the cuDNN-side layout of the reference's bench (src/openCNN_winograd.cu:234) */
};

/*
 * GEMM operand precision of later calls (default OPENCNN_F32, the reference's only mode).
 * With OPENCNN_F16 / OPENCNN_BF16 both transforms and the accumulation stay fp32, but the
 * transformed input and the transformed filter are rounded to nearest-even once and the 16
 * batched GEMMs run on fp16 / bf16 MFMA.  Ww then holds 2-byte elements, padded to 64 filters
 * and 16 channels (opencnn_workspace_bytes covers both precisions).  Any in_n, in_c, filt_k.
 * Tensors in HBM stay fp32.
 * opencnn_filter_transform(..., OPENCNN_WW_MFMA) and the fused kernel must run under the same
 * setting: the library remembers what it wrote to a Ww address and the fused kernel returns
 * hipErrorInvalidValue for a buffer written under another precision (see opencnn_filter_transform).
 */
enum { OPENCNN_F32 = 0, OPENCNN_F16 = 1, OPENCNN_BF16 = 2 };
int opencnn_set_operand_precision(int precision);

/*
 * Replaces the reference's hidden set-up: the caller-side cudaMemcpyToSymbol uploads of
 * the fragment-address tables (src/openCNN_winograd.cu:319-331).  This library has no
 * such tables; the call checks that the current device is a gfx950 part (hipErrorInvalidDevice
 * otherwise) and loads the embedded code object of the assembly kernels on it, which the first
 * launch on a device would otherwise do.  Calling it is optional.
 */
int opencnn_init(void);

/*
 * Drop-in for the reference's host dispatcher
 *   cudaError_t convolutionForward(float *k, int in_h, int in_w, float *w, int out_h,
 *       int out_w, int out_n, int out_c, float *C, float *Ww, const unsigned int n,
 *       int tiles_dim, int in_n, int tile_size, int elems_dim, int in_c, int filt_k,
 *       int filt_c, int filt_h, int filt_w, int alpha, int m)
 * (src/openCNN_winograd.cu:204-219): same 22 arguments, same meaning, same layouts.
 * Runs the filter transform and then the fused kernel, stream-ordered, on the stream
 * set by opencnn_set_stream (default: the null stream, as in the reference).
 *
 * Unlike the reference, which mis-computes silently or returns an uninitialised value
 * on shapes it does not support (src/openCNN_winograd.cu:212-218), unsupported
 * arguments return hipErrorInvalidValue and launch nothing.  Supported: filt_h ==
 * filt_w == 3, m == 2, alpha == tile_size == 4, filt_c == in_c, out_* consistent with pad 1 /
 * stride 1, tiles_dim == opencnn_tiles_dim(in_w), in_h == in_w, every tensor below 2^31
 * elements and in_n*in_h*in_w below 2^28.  in_n, in_c and filt_k are free: outside the reference's in_n % 32 == 0,
 * filt_k % 64 == 0, in_c % 8 == 0 the groups are rounded up and the missing lanes, channels
 * and filters predicated (Ww must then hold opencnn_workspace_bytes(), which is more than the
 * reference's filt_k*filt_c*16 floats).
 */
int convolutionForward(float *k, int in_h, int in_w, float *w, int out_h, int out_w,
                       int out_n, int out_c, float *C, float *Ww, const unsigned int n,
                       int tiles_dim, int in_n, int tile_size, int elems_dim, int in_c,
                       int filt_k, int filt_c, int filt_h, int filt_w, int alpha, int m);

/*
 * The reference's launcher behind the dispatcher, same arguments minus elems_dim
 * (src/convolutionForward_32x64x8.cu:264-284).  Kept so code that binds the launcher
 * directly keeps linking; the name's 32x64x8 is the reference's CUDA tile shape and
 * says nothing about the tiling used here.
 */
int convolutionForward_32x64x8(float *k, int in_h, int in_w, float *w, int out_h,
                               int out_w, int out_n, int out_c, float *C, float *Ww,
                               const unsigned int n, int tiles_dim, int in_n,
                               int tile_size, int in_c, int filt_k, int filt_c,
                               int filt_h, int filt_w, int alpha, int m);

/* tiles per image side, ceil(ceil((in_w+2)/2)-1): the caller-side computation at
 * src/openCNN_winograd.cu:286-288. */
int opencnn_tiles_dim(int in_w);

/* Size in bytes of the Ww scratch: 16*sizeof(float) for each of filt_k (rounded up to 32) x
 * filt_c (rounded up to 8) filters.  On the shapes the reference takes this is its caller-side
 * cudaMalloc, filt_k*filt_c*16*sizeof(float) (src/openCNN_winograd.cu:310-311). */
size_t opencnn_workspace_bytes(int filt_c, int filt_k);

/* Stream (a hipStream_t passed as void*) used by every later call from any thread;
 * NULL selects the null stream, which is what the reference launches on
 * (src/convolutionForward_32x64x8.cu:274,281). */
int opencnn_set_stream(void *stream);

/*
 * Which fused kernel later calls launch.  The reference picks its variant at compile time
 * (-DBASE / -DOPTSTS64 / -DOPTSTS64_CMP / -DOPTLDS64, Makefile:3,8); here it is a run-time
 * switch so both can be measured in one process.
 *   OPENCNN_KERNEL_AUTO      the hand-scheduled assembly kernels where they apply (see
 *                            OPENCNN_KERNEL_ASM), else what OPENCNN_KERNEL_HIP selects
 *   OPENCNN_KERNEL_REGISTER  every wave transforms its own input patches; no LDS, no barriers
 *   OPENCNN_KERNEL_LDS       the waves of a workgroup that share a column tile split the input
 *                            transform and exchange it through LDS (needs an even number of
 *                            filter groups, otherwise later launches return
 *                            hipErrorInvalidValue)
 *   OPENCNN_KERNEL_ASM       the LDS scheme as hand-scheduled gfx950 assembly, one persistent
 *                            launch over all (tile, 8-channel chunk) units (batches that are no
 *                            multiple of 32 may share 32-column tiles across spatial tiles).  Needs more than one
 *                            32-wide filter group, i.e. filt_k > 32 (and, for more workgroup
 *                            tiles than compute units that are not a multiple of them, the
 *                            balanced split switched on); otherwise later launches return
 *                            hipErrorInvalidValue.
 *                            With fp16 / bf16 operands (opencnn_set_operand_precision): units of
 *                            16 channels, any shape (the condition on the balanced split
 *                            stays)
 *   OPENCNN_KERNEL_HIP       the HIP C++ kernels only: the LDS variant when the 32-wide filter
 *                            groups (filt_k / 32, rounded up) pair up (as one continuous pipeline
 *                            over all tiles of a workgroup when the balanced split is in use),
 *                            else the register variant
 */
enum {
  OPENCNN_KERNEL_AUTO = 0,
  OPENCNN_KERNEL_REGISTER = 1,
  OPENCNN_KERNEL_LDS = 2,
  OPENCNN_KERNEL_ASM = 3,
  OPENCNN_KERNEL_HIP = 4
};
int opencnn_set_kernel_variant(int variant);

/*
 * Balanced split of the LDS kernel (default on).  When a layer has more workgroup tiles than
 * the GPU has compute units, but not a whole number of rounds of them (784 tiles on 256 CUs =
 * 3.06 rounds, which plain launching rounds up to 4), one persistent workgroup per CU takes an
 * equal share of (tile, 8-channel chunk) units; a tile whose channel range ends up split
 * between two workgroups is merged through the output tensor and two words of library-owned
 * device state per wave.  Results stay independent of timing (two addends commute).  The same
 * hand-over serves layers with tiles for at most half of the compute units (small batches on
 * deep layers): every tile is cut among two or four workgroups, and the parts of
 * its channel sum are passed from workgroup to workgroup in a fixed order.  Pass 0 to turn
 * it off altogether.  No counterpart in the reference, whose grid is one block per tile
 * (src/convolutionForward_32x64x8.cu:281).
 *
 * Launches that may overlap in time must not share that state, so it exists in sets:
 *   - every stream that launches directly holds one of 32 sets.  The library never touches a
 *     stream it is not asked to launch on (its handle may be stale), so a set only changes
 *     hands on the library's own evidence: from the moment a 33rd stream launches, every launch
 *     is followed by an event (hipEventRecord, about a microsecond), and a stream without a set
 *     takes over the set used longest ago whose event has completed.  Until one has, its
 *     launches run without the split (slower, same results; opencnn_last_launch tells).
 *     opencnn_release_stream(stream) waits for a stream and gives its set back at once, e.g.
 *     before the stream is destroyed.
 *   - launches recorded in a stream capture hold one of 16 further sets per (capture, stream),
 *     since the graph may be replayed at any time on any stream; only the caller knows when it
 *     will never run again, so the set stays taken until opencnn_release_capture gives it back.
 *     With all 16 taken, a captured launch runs without the split.  Two executable graphs
 *     instantiated from one capture share its set and must not run at the same time.
 *   - a caller that wants neither limit passes flag storage of its own in
 *     opencnn_conv_desc.split_flags.
 * Only launches that cut a tile between workgroups take a set; a layer whose tiles fill whole
 * rounds of the compute units, or a kernel with one tile per workgroup, takes none.
 *
 * opencnn_release_capture(stream, flag_set): gives graph sets back once the graphs recorded with
 * them will not run again and their last replay has completed (the caller vouches for both).
 * flag_set >= 0: that set, as opencnn_last_launch reported it right after the captured call;
 * flag_set < 0: every graph set whose launches were recorded on `stream` (on any stream when
 * `stream` is NULL).  A service that captures a graph per shape calls it when it drops a graph.
 *
 * opencnn_unsplit_launches(): fused-kernel launches since the process started, on any thread and
 * device, that would have cut tiles between workgroups and ran without the split because no flag
 * set was free (slower, same results): a counter to watch where opencnn_last_launch is too local.
 */
int opencnn_set_balanced_split(int enable);
int opencnn_release_stream(void *stream);
int opencnn_release_capture(void *stream, int flag_set);
unsigned long long opencnn_unsplit_launches(void);

/*
 * What this thread's last successful fused-kernel launch looked like: its number of workgroups
 * and its set of split-merge flags (0..31 a set of a stream, 32..47 a set of a stream capture, 48
 * the caller's storage, -1 none: the split was off, the launch cut no tile between workgroups,
 * or no set was free).
 * Either pointer may be NULL.  For tests and logs; no counterpart in the reference.
 */
int opencnn_last_launch(int *workgroups, int *flag_set);

/*
 * A kernel's wait for another workgroup's partial tile is bounded (about a second), so that
 * no bug and no workgroup that fails to become resident can hang the GPU.  A wave that gives up
 * finishes normally, but its launch's output is wrong; it reports that in a status word of the
 * launch's flag set, in host memory.  The library reads that word (no copy, no
 * synchronisation) at the next call that uses the same flag set: that call launches nothing
 * but a kernel that clears the flags, and returns hipErrorLaunchFailure with opencnn_last_error()
 * saying so; the call after it works again.  opencnn_check_status() does the same check for all
 * flag sets of the current device at once: call it after synchronising (hipDeviceSynchronize
 * or the streams in use) to learn whether every launch so far, graph replays included, handed
 * its tiles over; it returns 0 or hipErrorLaunchFailure (and has then cleared the library's
 * flag sets).
 * What a report covers: the host only sees the word at its next call, so launches that were
 * queued on the same flags between the launch that gave up and the call that reports it (and
 * replays of a graph until somebody asks) ran on flags that may be inconsistent: treat the output
 * of EVERY launch on that stream or graph since the last clean check as invalid.
 * Flag storage of a caller (opencnn_conv_desc.split_flags): every such buffer has a status word
 * of its own (the library tells up to 64 buffers per device apart, by address;
 * opencnn_release_split_flags(buffer) forgets one, e.g. before it is freed, and a 65th buffer is
 * refused with hipErrorInvalidValue).  A give-up on buffer A is reported by the next call that
 * brings A, and by opencnn_check_status, never by a call on another buffer; the library clears A
 * (a kernel on that call's stream) when the next call brings it, not before: the memory is the
 * caller's and may be gone.
 * The reference has no hand-over and no such state (one block per tile,
 * src/convolutionForward_32x64x8.cu:281).
 */
int opencnn_check_status(void);
int opencnn_release_split_flags(const void *split_flags);

/*
 * The reference's FX kernel as a call of its own (src/FX_m2.cu:51-91, launched at
 * src/convolutionForward_32x64x8.cu:274): U = G g G^T for every (c,k).
 *   w              device, filt_c*9*filt_k floats in `filter_layout`
 *   Ww             device, written in `ww_layout`: filt_c*16*filt_k floats for
 *                  OPENCNN_WW_REFERENCE, opencnn_workspace_bytes() for OPENCNN_WW_MFMA
 * OPENCNN_WW_REFERENCE output is bit-identical to the reference's arithmetic order
 * (only additions and multiplications by 0.5).
 *
 * The library remembers, per device and Ww address (the 64 most recent), the layout, operand
 * precision and filter shape of what it wrote there.  The fused kernel checks a Ww it is given
 * against that record and returns hipErrorInvalidValue on a mismatch (a 2-byte Ww read as floats
 * would give garbage without any other sign); an address without a record is taken as it is.
 * A caller that fills such an address by other means (a copy of a transformed filter saved
 * elsewhere) drops the stale record with opencnn_forget_workspace(Ww).
 */
int opencnn_filter_transform(const float *w, float *Ww, int filt_k, int filt_c,
                             int filter_layout, int ww_layout);
int opencnn_forget_workspace(const void *Ww);

/*
 * The reference's Winograd_kernel as a call of its own
 * (src/convolutionForward_32x64x8.cu:169-262, launched at :281): input transform,
 * 16 batched GEMMs and output transform, reading a Ww that
 * opencnn_filter_transform(..., OPENCNN_WW_MFMA) wrote earlier on the same stream.
 * Lets a caller transform the filters once and reuse them, which the reference's
 * dispatcher cannot (it re-runs FX on every call).  in_h and in_w may differ here.
 */
int opencnn_conv_forward_pretransformed(const float *in, const float *Ww, float *out,
                                        int in_n, int in_c, int in_h, int in_w,
                                        int filt_k);

/*
 * One call with all of its settings: what the process-wide opencnn_set_* calls select for the
 * other entry points, per call, so that threads can use different streams, precisions and
 * kernels at the same time.  No counterpart in the reference (one thread, the null stream,
 * src/openCNN_winograd.cu:426-444).
 *   struct_size        sizeof(opencnn_conv_desc) (other values return hipErrorInvalidValue)
 *   in, out            CHWN input, KHWN output; in_h and in_w may differ
 *   filter             3x3 filters in filter_layout, or NULL
 *   Ww                 opencnn_workspace_bytes(in_c, filt_k) bytes.  With a filter: scratch, as
 *                      in convolutionForward (the filter transform runs first).  With
 *                      filter == NULL: a transformed filter that an earlier call on the same
 *                      stream left there under the same operand_precision (the split API).
 *   operand_precision  OPENCNN_F32 / F16 / BF16;  kernel_variant OPENCNN_KERNEL_*;
 *   balanced_split     0 / 1;  stream  a hipStream_t, NULL = the null stream
 *   split_flags        NULL (the library's flag sets, see opencnn_set_balanced_split), or
 *                      split_flags_bytes >= opencnn_split_flags_bytes() of device memory that the
 *                      caller zeroed once: the hand-over state of this call.  Calls that share
 *                      one such buffer must not overlap in time; calls with different buffers may,
 *                      on any number of streams and graphs (see opencnn_check_status for how a
 *                      failed hand-over on such a buffer is reported, and
 *                      opencnn_release_split_flags).
 * A zero-initialised struct with struct_size, the pointers and the shape filled in selects
 * the defaults except for balanced_split, which a caller who wants the default sets to 1.
 */
typedef struct opencnn_conv_desc {
  size_t struct_size;
  const float *in;
  const float *filter;
  float *out;
  void *Ww;
  int in_n, in_c, in_h, in_w, filt_k;
  int filter_layout;
  int operand_precision;
  int kernel_variant;
  int balanced_split;
  void *stream;
  void *split_flags;
  size_t split_flags_bytes;
} opencnn_conv_desc;
int opencnn_conv_forward_desc(const opencnn_conv_desc *desc);
size_t opencnn_split_flags_bytes(void);

/*
 * convolutionForward for callers that cannot allocate device memory and so have no Ww to pass:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference (its caller always allocates Ww, src/openCNN_winograd.cu:310-311).
 * Same filter transform and fused kernel as convolutionForward (in CHWN, w CRSK, out KHWN,
 * in_h == in_w, the selected stream and operand precision), but the transformed filter goes
 * into a workspace inside the library: opencnn_static_workspace_bytes() = 16 MiB of static
 * device memory per GPU, enough for in_c = filt_k = 512.  The call allocates and frees nothing.
 *   - opencnn_init() must have run on the current device (hipErrorNotInitialized otherwise): it
 *     loads the kernels and looks the workspace up, which this call must not do.
 *   - shapes with opencnn_workspace_bytes(in_c, filt_k) above the limit return
 *     hipErrorInvalidValue and launch nothing.
 *   - every call on a GPU uses that GPU's one workspace, whatever the stream: calls on the same
 *     stream are ordered, calls that overlap in time on one GPU (two streams, two threads) race
 *     on it and must not be made.  The workspace keeps the last call's transformed filter;
 *     each call overwrites all of what it reads.
 */
int opencnn_conv_forward_static(const float *in, const float *w, float *out, int in_n,
                                int in_c, int in_h, int in_w, int filt_k);
size_t opencnn_static_workspace_bytes(void);

/*
 * Layout shims on the selected stream, device to device, src != dst: the reference's data_cpy
 * kernel (src/openCNN_winograd.cu:147-153) as used at :230 (NCHW input -> CHWN) and :235 (KCRS
 * filters -> CRSK), plus the way back for the result (KHWN -> NKHW, i.e. NCHW with K channels),
 * which the reference only does implicitly inside its checker's index map (:185-186).
 * data_cpy is limited to C <= 1024 by its launch shape; these take any tensor below 2^31
 * elements.
 */
int opencnn_nchw_to_chwn(const float *src, float *dst, int n, int c, int h, int w);
int opencnn_khwn_to_nkhw(const float *src, float *dst, int n, int k, int h, int w);
int opencnn_kcrs_to_crsk(const float *src, float *dst, int k, int c);

/* Name of the last failing check in this thread ("" if none): a short static string. */
const char *opencnn_last_error(void);

/*
 * Name of the fused kernel that this thread's last successful launch used ("" before the first):
 * a short static string such as "wino_f32_asm_kw2" or "wino_f16_asm_kw4_packed" (the assembly
 * kernels' symbol names) or "wino_f32_fused_lds" (a HIP C++ kernel).  For logs and tests: which
 * kernel family a shape ends up in is the library's choice (see opencnn_set_kernel_variant).
 * No counterpart in the reference, whose single kernel is fixed at compile time.
 */
const char *opencnn_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* OPENCNN_AMD_H */
