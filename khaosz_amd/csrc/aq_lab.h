/*
 * Measurement and test entry points of libastrai_q_lab.so.  NOT part of the product ABI
 * (include/astrai_q.h) and not linked into libastrai_q.so: the lab library is the product's
 * objects plus these, built for the benchmark's ceiling probes and for the tests that force
 * a GEMM tile shape.  None of them has a counterpart in the reference.
 */
#ifndef AQ_LAB_H
#define AQ_LAB_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Forces the GEMM workgroup tile for every later GEMM call of this process through the lab
 * library: 32 (128 x 32), 33 (64 x 32), 64 (128 x 64), 65 (64 x 64), 128 (128 x 128), 129 (128 x 128 on
 * wavefront pairs that split every K step: lab build only), 256 (256 x 128), 0 = by shape.  Process-wide and
 * unsynchronised -- which is why it does not exist in the product library. */
int aq_lab_set_gemm_tile(int rows);

/* The tile the library would pick for an M x N output on a device of `compute_units` compute units, in the
 * numbering above (a pure function of its arguments: no device is touched). */
int aq_lab_choose_gemm_tile(int64_t M, int64_t N, int compute_units);

/* Clock counters the lab build's tiled GEMM leaves behind (wavefront 0 of workgroup 0 of the LAST GEMM launch that
 * completed): host int64[8].  [0] shader-clock cycles and [1] 100 MHz reference ticks between the kernel's first and
 * last instruction -- their ratio x 100 MHz is the clock the kernel ran at.  [2..7] are filled only by a build with
 * the K-loop stall counters (python -m khaosz_amd.build --stall-counters, which adds -DAQ_LAB_STALL to the lab
 * library's GEMM object): [2] cycles waited at the stage barriers, [3] cycles of the K loop, [4] tile start ->
 * first stage landed, [5] the first K step, [6] accumulator exchange + epilogue, [7] the whole tile. */
int aq_lab_read_clock(long long *host8);

/* The arithmetic of the row SwiGLU quantiser's mid-range path on single bf16 pairs: h[i] = up[i] * silu(gate[i])
 * (fp32), and in_range[i] = 1 where the kernel's range test lets gate[i] take that path.  For the test that puts
 * every bf16 gate pattern through it against the oracle. */
int aq_lab_probe_swiglu_bf16(const uint16_t *up, const uint16_t *gate, int64_t n, float *h, uint8_t *in_range,
                             void *stream);

/* `workgroups` x 4 wavefronts each issue iters x 8 independent MFMAs.
 * kind 0 = i32_32x32x32_i8 (65536 ops each), 1 = i32_16x16x64_i8 (32768), 2 = f32_32x32x64 e4m3 (131072 flops).
 * data 0 = constant operands (no toggling: the clock stays at its maximum), 1 = random bytes, four operand
 * sets cycled between consecutive instructions (what a GEMM's operand stream does to the power budget).
 * clocks (may be NULL): device int64[2] receiving the shader-clock and 100 MHz reference-clock ticks that
 * wavefront 0 spent in the loop -- their ratio x 100 MHz is the clock the loop ran at. */
int aq_lab_probe_mfma(int kind, int data, int workgroups, int iters, int *sink, long long *clocks, void *stream);

/* Streaming copy, 16 bytes per lane, grid-stride: the known-size kernel HBM counters are scaled against. */
int aq_lab_probe_copy(const void *src, void *dst, int64_t bytes, int workgroups, void *stream);

/* Read `bytes` once.  loads_per_lane = 0: grid-stride loop over `workgroups` workgroups of 256 (each lane's
 * loads are serialised by their use).  loads_per_lane = 1, 2, 4, 8, 16: every lane issues that many 16-byte
 * loads before using any; the launch is sized to cover `bytes` exactly (which must divide evenly) and
 * `workgroups` is ignored.  nontemporal != 0 marks the loads as streaming. */
int aq_lab_probe_read(const void *src, int64_t bytes, int loads_per_lane, int workgroups, int nontemporal,
                      int *sink, void *stream);

/* What fragment reads cost the matrix pipe with one wavefront per SIMD (4 per workgroup), by where they are issued:
 * `iters` iterations of 32 MFMAs (i32_32x32x32_i8) and 16 ds_read_b128 in a ping-pong of two register sets (the MFMAs
 * of one half consume what the reads of the other half filled).  variant 0: MFMAs only; 1: one read behind every
 * second MFMA; 2: a half's eight reads first; 3: reads in pairs behind every fourth MFMA.  clocks: device int64[1]
 * receiving the shader-clock cycles wavefront 0 of workgroup 0 spent in the loop (1024 per iteration is the matrix
 * pipe's own time). */
int aq_lab_probe_mfma_lds_issue(int variant, int workgroups, int iters, int *sink, long long *clocks, void *stream);

/* One wavefront that does nothing: the cost of a launch. */
int aq_lab_probe_empty(int *sink, void *stream);

/* aq_quant_tensor_fp8_onepass with the bound on its wait for the other workgroups (polls of their slots) given
 * by the caller.  spin_limit 0: every workgroup gives up at once and takes the maximum of the whole tensor
 * itself -- the path of a device too busy to run all workgroups together -- so a test can run it without one. */
int aq_lab_quant_tensor_fp8_onepass_spin(const void *x, int x_dtype, int64_t numel, uint8_t *q, float *scale,
                                         void *ws, size_t ws_bytes, int spin_limit, void *stream);

/* Where the wavefronts of the matrix-core decode GEMV that quantises its rows leave time stamps (NULL: nowhere,
 * the default): device int64 [workgroup][16 wavefronts][8], 100 MHz ticks.  Slots: 0 rows and epilogue operands
 * requested, 3 rows rounded into LDS, 4 past the barrier, 5 products done, 6 outputs stored.  Process-wide and
 * unsynchronised: lab only.  (The lab library's GEMV is its own compile of gemv.hip with these stamps in it.) */
int aq_lab_set_gemv_timeline(long long *buf);

/* on != 0: the matrix-core decode GEMV that quantises its rows requests no weight bytes at all (its products
 * then multiply zeros): what the launch costs with the token rows, their rounding, the barrier, the products and
 * the stores but WITHOUT the weight stream -- the floor the rounding sets.  Results are wrong while it is on. */
int aq_lab_set_gemv_skip_weights(int on);

#ifdef __cplusplus
}
#endif
#endif /* AQ_LAB_H */
