/*
 * fdx_debug -- measurement aids and test hooks of libfdx.so.  None of these has a counterpart in the reference and no
 * caller of fdeep::load_model / model::predict needs them: bench.py measures with them, the parity tests use them to
 * force kernel forms that the closed rules and the tuner would not pick on small problems.  Process-wide, meant for
 * one thread.
 */
#ifndef FDX_DEBUG_H
#define FDX_DEBUG_H

#include "fdx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* free and total device memory in bytes (hipMemGetInfo): the tests use it to show that an entry point allocates nothing */
fdx_status fdx_dev_mem_info(size_t* free_bytes, size_t* total_bytes);
/* HIP-event stopwatch on the library stream: start, run work, stop returns milliseconds */
fdx_status fdx_timer_start(void);
fdx_status fdx_timer_stop(float* ms);
/* Shader-clock probe, a measurement aid with no counterpart in the reference (the clock of the compute units falls
 * under load, and with it what the matrix cores can deliver): one lane on a stream of its own samples the shader
 * cycle counter against the constant-rate wall counter every period_us (10..100000) while other work runs, and ends
 * by itself after `samples` (2..65536) periods, at most 10 s in all (samples x period_us <= 10^7).  stop waits for it and returns the clock in GHz over the first
 * window_ms milliseconds after the start: the mean, and the lowest and highest single period.  One probe at a time. */
fdx_status fdx_clock_probe_start(int samples, int period_us);
fdx_status fdx_clock_probe_stop(double window_ms, double* mean_ghz, double* min_ghz, double* max_ghz);
/* name and average duration (ms) of the dominant kernel family since the last reset,
 * measured with HIP events around every launch while profiling is enabled */
fdx_status fdx_profile_enable(int on);
fdx_status fdx_profile_reset(void);
fdx_status fdx_profile_get(int index, char* name, size_t name_len, uint64_t* launches, double* total_ms,
    double* flops, double* bytes);
/* the multiply-add work the family's kernels really issued (2 per multiply-add), where that differs from the algorithmic
 * direct-sum count fdx_profile_get reports: the Winograd convolution issues 16 products per 2x2 output tile and
 * channel pair where the direct sum has 36 */
fdx_status fdx_profile_get_executed(int index, double* executed_flops);

/*
 * Test hooks (no counterpart in the reference; process-wide, meant for one thread): the parity tests use them to drive
 * every tile configuration and scheduling form of the convolution / GEMM kernels on small problems, where the tuner
 * would never pick them.
 *   fdx_debug_force_tile: -1 = tuner decides; 0..3 general kernel tiles; 10..18 fast-path tiles; 30 = the row-streaming
 *     kernel for K <= 128 (where it does not apply the tuner decides); + 100 * splits
 *     (every tile cut into `splits` K ranges), + 10000 (only the last partial round is cut), 20000 + tile = stream-K.
 *   fdx_debug_persist_cap: caps the persistent grid at `workgroups` (at least 8; 0 = the resident count).
 *   fdx_debug_force_strips: whole-tile launches of the fast path number their output tiles in this many column strips
 *     (wherever the output has as many column tiles) instead of letting the traffic model decide; 0 = the model decides.
 *   fdx_debug_force_dw_fusion: how plans built from now on run a depthwise 3x3 convolution and the 1x1 convolutions
 *     around it: -1 = the forms are timed once per block shape (the default), 0 = one launch per layer, 1 = depthwise +
 *     projection as one launch wherever the pair qualifies, 2 = expansion + depthwise + projection as one launch
 *     wherever the block qualifies (other blocks as under 1).
 *   fdx_debug_force_winograd: which kernel plans built from now on run a 3x3 stride-1 convolution with: -1 = the direct and
 *     the Winograd kernel are timed once per shape (the default), 0 = always the direct kernel, 1 = the Winograd kernel
 *     wherever it covers the shape.
 */
fdx_status fdx_debug_force_tile(int cfg);
/* a 1x1 convolution that has absorbed the 1x1 convolution of its residual operand (a residual block with a convolution on
 * its shortcut branch): 1 = one GEMM over both inputs' channels (the default), 0 = the two convolutions one after the
 * other, the second adding to the first's result -- the form taken by itself where the one-launch kernel does not apply */
fdx_status fdx_debug_dual_conv(int one_launch);
/* models loaded and plans built from now on: a 1x1 convolution whose result feeds another 1x1 convolution (the tail of one residual block and
 * the head of the next) and that convolution as one launch: -1 = as the environment says (FDX_CHAIN=1: plans with at least
 * 65536 pixels; otherwise never: the launch measured no faster than the two it replaces), 0 = never, 1 = wherever the
 * kernel covers the pair */
fdx_status fdx_debug_force_chain(int mode);
/* models loaded and plans built from now on: 1 = a LayerNormalization over the last axis whose only readers are Dense / self-attention layers
 * is computed inside those layers' GEMMs (row statistics gathered in the K loop, gamma / beta folded into the filters at
 * load); 0 = every LayerNormalization runs as a launch of its own; -1 = as the environment says (FDX_LN_FOLD=1: inside the
 * GEMMs; the default is a launch of its own, which measured 0.7 % faster on the benched encoder) */
fdx_status fdx_debug_force_ln_fold(int mode);
/* decode sessions created from now on: 1 = the token + position embedding launch of a step is folded into the two GEMMs
 * that read its result (measured slower than the launch it saves, hence not the default), 0 = never, -1 = as the
 * environment says (FDX_DECODE_EMBED_FOLD=1) */
fdx_status fdx_debug_decode_embed_fold(int mode);
fdx_status fdx_debug_persist_cap(int workgroups);
fdx_status fdx_debug_force_strips(int strips);
fdx_status fdx_debug_force_dw_fusion(int mode);
fdx_status fdx_debug_force_winograd(int mode);

#ifdef __cplusplus
}
#endif
#endif
