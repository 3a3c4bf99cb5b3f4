/*
 * fsw_probe.h -- measurement kernels for the benchmark, in a library of their own (libfsw_probe.so).
 *
 * NOT part of the product ABI of include/fsw.h and not needed by any caller of it: two yardstick kernels that show
 * what this board sustains with nothing else in the way, which bench.py prints beside its roofline fractions. No
 * counterpart in the reference. Conventions as in fsw.h (device pointers, stream as void*, FSW_OK or a negative
 * FSW_E_* code, FSW_E_DEVICE on anything but a gfx950 GPU).
 */
#ifndef FSW_PROBE_H
#define FSW_PROBE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSW_PROBE_API __attribute__((visibility("default")))

/* `workgroups` x 4 waves each issue iters x 64 v_mfma_f32_16x16x32 from registers (the prefill kernel's accumulator
 * shape) = workgroups * 4 * iters * 64 * 16384 FLOP. dtype: 0 = bf16, 1 = fp16. `operands`: 16 KB of device data in
 * the element type (its values set the power draw), 16-byte aligned; `out`: workgroups * 1 KB of device scratch. */
FSW_PROBE_API int fsw_probe_mfma(int dtype, int iters, const void* operands, void* out, int workgroups, void* stream);
/* Streams `bytes` (a multiple of 16) from `src` once with non-temporal 16-byte loads; `out`: 4 bytes. */
FSW_PROBE_API int fsw_probe_read(const void* src, size_t bytes, void* out, int workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FSW_PROBE_H */
