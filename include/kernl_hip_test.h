/*
 * kernl_hip_test.h — test and tuning hooks of libkernl_hip.so.
 *
 * Kept apart from kernl_hip.h on purpose: every entry point declared there is re-entrant and touches no process-wide
 * state; the three calls below set process-wide switches.
 */
#ifndef KERNL_HIP_TEST_H
#define KERNL_HIP_TEST_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Test and tuning hooks (process-wide, not thread-safe; no counterpart in the reference).  They change which kernel
 * EVERY later call of the process runs, from any thread: a serving process must not call them.  The library's own
 * tests and benchmarks bind them to run every kernel variant on every case.
 *   kernl_linear_force_tile      0 = heuristic (default); output tile of the MFMA linear kernel: 1 = 256x256,
 *                                2 = 256x192, 3 = 128x128, 4 = 256x128 with 32-wide k-tiles; persistent kernel with one
 *                                wave per SIMD: 5 = 256x256, 6 = 256x192; its one-tile-per-workgroup variant with
 *                                three LDS stages: 7 = 128x256, 8 = 128x192 (5..8 take any K the MFMA path takes, with
 *                                a zero-filled last k-tile when K % 64 != 0; gated epilogues take 1, 3 or 5);
 *                                10 .. 15 = the small-problem kernels (one launch of small tiles over the whole K:
 *                                32 x 64 / 64 x 64 tiles shared by the waves, 16 x 32 / 32 x 32 / 64 x 32 tiles with the
 *                                k-tiles dealt to the waves, 15 = 64 x 128 shared tiles); the heuristic takes them where kernl_linear_small_kind
 *                                says so.  With the heuristic, inputs of at most
 *                                64 rows and K % 64 == 0 go to a kernel that streams the weight once (16 output
 *                                columns per workgroup); 9 = that kernel where it applies, the heuristic elsewhere;
 *                                1..8 keep such inputs on the tile kernels.
 *   kernl_attention_force_scalar non-zero routes every attention call through the strided scalar kernel.
 *   kernl_attention_set_variant  0 = heuristic; register budget of the head-size-64 streaming attention kernel: 1 = built
 *                                for 3 waves/SIMD, 2 = built for 2 waves/SIMD; 3 = streaming kernel for every shape,
 *                                4 = software-pipelined kernel wherever it applies (head size 64; no mask, a per-key
 *                                mask of at most 2048 keys, or causal), also below 1024 keys and on large grids;
 *                                5 = the small-grid form of the streaming kernel (32-row workgroups whose waves split
 *                                the key tiles) wherever it applies (head size 64, non-causal, no mask or a per-key
 *                                mask, at most 4096 keys), whatever the grid.
 */
void kernl_linear_force_tile(int which);
void kernl_attention_force_scalar(int on);
void kernl_attention_set_variant(int which);

/*
 * Rate probe (no counterpart in the reference): launches ONE kernel on `stream` that runs a register-only instruction
 * mix or a plain streaming pass, so that a benchmark can state what this GPU sustains next to the published peaks.
 *   kind 0  v_mfma_f32_32x32x16_f16 on random fp16 operands, one wave per SIMD, 256 accumulator registers
 *        1  v_mfma_f32_16x16x32_f16, same geometry
 *        2  kind 0 on all-zero operands
 *        3  per 32x32x16 MFMA two v_exp_f32 and four v_fma_f32 (the attention tile loop's mix); `workgroups` of 256
 *           threads, two of them fit a CU
 *        4  read-only pass over `bytes` bytes at src (16-byte loads)
 *        5  copy of `bytes` bytes from src to dst
 *   iters       loop trips of kinds 0..3: 32 MFMAs (64 of the smaller shape) per trip and wave for kinds 0..2, 16 for 3
 *   workgroups  grid size (256 threads each); kinds 0..2 want one per CU
 *   src         kinds 0..3: a table of at least 16 MiB of fp16 operand values; kinds 4, 5: the buffer to stream
 *   stats       workgroups x 2 uint64: shader-clock ticks and 100 MHz wall-clock ticks of each workgroup's loop
 *   sink        workgroups x 256 floats the kernels write their results to (so that nothing is optimised away)
 * Returns KERNL_OK or a negative error (kernl_last_error_string()); asynchronous, allocates nothing.
 */
int kernl_probe_rate(int kind, int iters, int workgroups, const void *src, void *dst, int64_t bytes, void *stats,
                     void *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KERNL_HIP_TEST_H */
