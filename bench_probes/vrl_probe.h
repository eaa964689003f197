/*
 * vrl_probe.h — C ABI of libvrl_probe.so: measurement aids of bench.py, no part of the scoring library and with no
 * counterpart in the reference. They give the ceilings the kernels of libvrl_hip.so are measured against: what the memory
 * system delivers for the row kernels' access pattern with no arithmetic in the way, and what the matrix cores sustain
 * on register operands with nothing else in the way. Pointers are device pointers unless said otherwise; `stream` is a
 * hipStream_t as void*; status codes are those of vrl.h.
 */
#ifndef VRL_PROBE_H_
#define VRL_PROBE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * One workgroup per "row" of row_bytes (a multiple of 16) streams it with non-temporal 128-bit accesses exactly as
 * vrl_rowscore's kernel does.
 *   mode 0: read only (the data is XOR-folded; *sink is written only if the fold equals a constant)  -> forward ceiling
 *   mode 1: read src, write dst (n_rows * row_bytes each, not overlapping)                           -> backward ceiling
 *   mode 2: the same copy by 512 workgroups walking the buffer as a whole, 8 KiB per wavefront and trip (faster than
 *           mode 1 on MI355X; no bound either: the row-op backward in many short workgroups is faster again)
 *   mode 3: mode 0 with the workgroup shape the forward kernel uses for 32-bit logits (4 wavefronts, 4 loads in flight)
 *   mode 4: mode 0 by 1024 workgroups walking the buffer as a whole (whether one workgroup per row costs a read stream anything)
 */
int vrl_stream_probe(const void* src, void* dst, int64_t n_rows, int64_t row_bytes, int mode, uint32_t* sink,
                     void* stream);

/*
 * n_workgroups workgroups of 8 wavefronts each issue the products of `iters` 64 x 128 x 16 wavefront tiles
 * (2 * 64 * 128 * 16 flops each) on register operands, nothing else. iters is at most VRL_PROBE_MAX_ITERS (a few hundred
 * milliseconds of work; more returns VRL_ERR_ARG).
 * instruction: 32 = v_mfma_f32_32x32x16_bf16, 16 = v_mfma_f32_16x16x32_bf16 (what the LM-head kernels issue; iters even).
 * random_operands != 0: pseudo-random bf16 operands in (-1, 1), otherwise small constants; the part is power-managed and
 * holds a lower clock when the operand bits toggle, so the first is the ceiling the LM-head kernels are measured against
 * and the second shows the nominal rate. clocks (optional, device, 2 x int64): shader clocks and constant-rate wall-clock
 * ticks that wavefront 0 of workgroup 0 spent in its loop; wall_clock_khz (optional, HOST pointer): the rate of that wall
 * clock. sink (device, 1 float) is practically never written.
 */
#define VRL_PROBE_MAX_ITERS 4000000
int vrl_mfma_probe(int64_t n_workgroups, int64_t iters, int instruction, int random_operands, float* sink,
                   int64_t* clocks, int64_t* wall_clock_khz, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VRL_PROBE_H_ */
