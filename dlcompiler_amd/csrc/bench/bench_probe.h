/*
 * bench_probe.h -- C ABI of libdlblas_bench_probe.so: two measurement kernels that bench.py times
 * to report what the chip sustains beside each roofline.  They are not operators, have no
 * counterpart in the reference and are not part of libdlblas_hip.so.
 * Status codes are those of dlblas_hip.h (0 ok, -1 bad argument, -2 unsupported, -3 launch failure,
 * -4 buffer too small).
 */
#ifndef DLBLAS_BENCH_PROBE_H_
#define DLBLAS_BENCH_PROBE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Launches `blocks` workgroups of 512 threads that each issue `iters` rounds of four independent
 * MFMAs per wave (bf16 32x32x16, or fp8 32x32x64 when fp8 != 0) on operand registers loaded once
 * from `operands` -- no memory traffic or LDS in the loop; valu_per_mfma (0, 4, 8 or 16) adds
 * that many independent fp32 multiply-adds of the same wave after every MFMA.  Timed by the
 * caller, it gives the matrix rate this chip sustains on that operand DATA (the clock under
 * matrix load follows the power the data draws) and, with valu_per_mfma > 0, in that
 * instruction mix (vector instructions only partly hide under matrix instructions).  FLOPs = blocks * 8 waves * iters * 4 * (32768
 * for bf16, 131072 for fp8).  operands: at least dlb_probe_mfma_operand_bytes(blocks) bytes,
 * 16-byte aligned, any contents.  sink: device memory of at least DLB_PROBE_SINK_BYTES bytes that
 * the kernels practically never write (it keeps their loops alive); sink_bytes is checked. */
#define DLB_PROBE_SINK_BYTES 2048
int64_t dlb_probe_mfma_operand_bytes(int blocks);
int dlb_probe_mfma_rate(const void* operands, int64_t operand_bytes, void* sink,
                        int64_t sink_bytes, int blocks, int fp8, int iters, int valu_per_mfma,
                        void* stream);

/* Reads `bytes` (a multiple of 16) from src with non-temporal 16-byte loads, eight in flight per
 * lane, and discards them.  Timed by the caller it is the HBM rate a kernel with no arithmetic and
 * no stores reaches on this chip.  sink as above. */
int dlb_probe_hbm_read(const void* src, void* sink, int64_t sink_bytes, int64_t bytes,
                       void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DLBLAS_BENCH_PROBE_H_ */
