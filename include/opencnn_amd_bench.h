/*
 * opencnn_amd_bench — bench and test support of libopencnn_amd.so, declared apart from the C ABI a
 * caller of the reference would bind (opencnn_amd.h): the timing loop of the reference's bench,
 * a timeline of the assembly kernels, the order in which they walk through the image, the weight
 * of the ranges of the balanced split, the poll limit of a hand-over, and seeded synthetic
 * tensors.  The settings here (tile order, range weight, timeline buffer, wait limit) belong to
 * the CALLING THREAD: they change that thread's later launches and nobody else's.  Results never
 * depend on them (a wait limit small enough to make a hand-over give up excepted, which is what
 * it is for).
 */
#ifndef OPENCNN_AMD_BENCH_H
#define OPENCNN_AMD_BENCH_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Bench support, the library-side twin of the reference's timing loop
 * (src/openCNN_winograd.cu:426-444): `warmup` untimed calls, then `iters` back-to-back
 * calls bracketed by HIP events on the selected stream.  Writes mean milliseconds per
 * call of (a) filter transform + fused kernel, the quantity the reference reports,
 * (b) the fused kernel alone, (c) the filter transform alone.  Synchronises the stream.
 */
int opencnn_time_forward(const float *in, const float *w, float *out, float *Ww,
                         int in_n, int in_c, int in_h, int in_w, int filt_k, int warmup,
                         int iters, float *ms_total, float *ms_main, float *ms_fx);

/*
 * Bench support without a counterpart in the reference: the order in which the assembly kernels
 * walk through the tiles of the image, which decides how much of a tile's input patch is found in
 * the L2 of its XCD because a neighbouring tile has just read it.  Results do not depend on it.
 * Bits: 1 = neighbouring column tiles are neighbouring spatial tiles (else: the same spatial tile
 * of the next 32 batch elements), 2 = spatial tiles numbered in zigzag strips of two tile rows
 * (else row by row), 4 = the tiles that an XCD's workgroups start with lie together in the image,
 * the tiles they go on with beside them.  Default 7; 0 is the order of
 * the first version of the kernels, kept for measurements (profiles/).
 */
int opencnn_set_tile_order(int bits);

/*
 * Bench support without a counterpart in the reference: how the assembly kernels' balanced split
 * cuts the line of (tile, chunk) units into one range per workgroup.  -1 (the default): the
 * library chooses (fp32: a cost model of the ranges, fitted to measurements; fp16 / bf16: 4);
 * 0: equal numbers of units; w = 1 ... 6: on a line that adds w half units to every tile for its
 * output transform, so that a range with one more tile end gets fewer units.
 */
int opencnn_set_range_weight(int half_units);

/*
 * The number of polls after which a kernel's wait for another workgroup's partial tile gives up
 * (see opencnn_check_status in opencnn_amd.h), for tests of that path; 0 restores the default of
 * 2^20 polls.
 */
int opencnn_set_wait_limit(unsigned polls);

/*
 * Bench support without a counterpart in the reference: a timeline of the assembly kernels.
 * While a buffer is set, the first wave of workgroup L of every later launch of those kernels
 * writes into device_buffer[L*64 ...]: [0] the number of stamps, [2], [3], ... the GPU's
 * 100 MHz realtime counter at kernel start, after the prologue, and before and after every output
 * transform (at most 62 stamps).  `bytes` is the size of the buffer; launches with more
 * workgroups than it holds records for do not record.  NULL / 0 turns it off (the default).
 */
int opencnn_set_timeline_buffer(long long *device_buffer, size_t bytes);

/* Layout of a synthetic input written by opencnn_synth_input. */
enum { OPENCNN_INPUT_CHWN = 0, OPENCNN_INPUT_NCHW = 1 };
/* Distribution of a synthetic tensor: uniform on [p0,p1) or normal(mean p0, std p1). */
enum { OPENCNN_DIST_UNIFORM = 0, OPENCNN_DIST_NORMAL = 1 };

/*
 * Seeded synthetic tensors in HOST memory (no GPU involved).  They stand in for the
 * reference's unseeded curand fills and data_cpy transposes
 * (src/openCNN_winograd.cu:127-153,221-238): element values depend only on
 * (seed, logical NCHW / KCRS coordinate), so both layouts of a tensor hold the same
 * numbers.  Return 0, or 1 on a bad argument.
 */
int opencnn_synth_input(float *dst, int n, int c, int h, int w, int layout,
                        unsigned long long seed, int dist, double p0, double p1);
int opencnn_synth_filter(float *dst, int k, int c, int layout, unsigned long long seed,
                         int dist, double p0, double p1);

#ifdef __cplusplus
}
#endif
#endif /* OPENCNN_AMD_BENCH_H */
