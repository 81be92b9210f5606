/* Measurement probes of the autotune harness (engine/test_any_mma --read-floor, --mfma-ceiling).  Not part of the
 * library's interface: the launches below exist so that the harness can time "nothing" and "a plain read" the way it
 * times the GEMMs, and the matrix cores alone. */
#ifndef ABQ_PROBE_H
#define ABQ_PROBE_H

#include "abq_gemm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference.  Launches a kernel that does nothing
 * (ABQ_PROBE_EMPTY; buf and bytes ignored) or one that reads `bytes` of `buf` once with 16-byte loads and
 * computes nothing (ABQ_PROBE_READ).  The harness times them the way it times the GEMMs: the floor a
 * decode GEMM, which is one launch over a few MB of weights, can be compared with.
 * ABQ_PROBE_MFMA_I8 / ABQ_PROBE_MFMA_FP6: a loop of v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x64_f8f6f4 (E2M3) that
 * touches nothing but registers, eight waves on every compute unit; buf holds the 8 KiB of operand bits the loop
 * runs on (the caller's choice: the matrix cores' clock depends on them) and `bytes` is the number of matrix-core
 * instructions per wave (a multiple of 8).  Work of a launch: 2 * CUs * 4 waves * bytes * 65 536 (I8) or
 * 131 072 (FP6) operations. */
typedef enum abq_probe_kind {
    ABQ_PROBE_EMPTY = 0,
    ABQ_PROBE_READ = 1,
    ABQ_PROBE_MFMA_I8 = 2,
    ABQ_PROBE_MFMA_FP6 = 3
} abq_probe_kind;
abq_status abq_probe_launch(int kind, const void *buf, size_t bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* ABQ_PROBE_H */
