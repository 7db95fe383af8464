/*
 * libxla_amd_selfcheck.so -- aids for this package's own tests and benchmarks.  Not part of the
 * product: nothing here replaces anything in the reference, and unlike libxla_amd_quant.so these
 * entry points may allocate device memory and synchronise.
 */
#ifndef XLA_AMD_SELFCHECK_H_
#define XLA_AMD_SELFCHECK_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XLA_AMD_SELFCHECK_EXPORT __attribute__((visibility("default")))

/* Evaluates the epilogue's tanh -- fused polynomial steps, a quotient by the shortened f32 division
 * sequence, no |x| >= 20 select -- and a spelling with the plain quotient and the explicit select
 * on all 2^32 f32 bit patterns on the current device, and returns how many results differ (0 is the
 * only acceptable answer), or -1 on a HIP error.  Allocates and synchronises. */
XLA_AMD_SELFCHECK_EXPORT long long xla_amd_selfcheck_tanh_division_mismatches(void);

/* Streams `bytes` (a multiple of 16, buffers 16-byte aligned) from `src` on `stream` -- copied to
 * `dst`, or only read when `dst` is null -- with the access shape that reaches the highest HBM rate
 * on MI355X, so that a benchmark can print what a plain stream achieves on the same machine next to
 * a kernel's own rate, and scale profiler byte counters by a copy of known size.  Returns 0, -1 for
 * bad arguments, -2 for a failed launch. */
XLA_AMD_SELFCHECK_EXPORT int xla_amd_selfcheck_stream(void* dst, const void* src, size_t bytes, void* stream);

/* Enqueues `count` launches of a kernel that does nothing (`workgroups` workgroups of one wave) on
 * `stream`: back to back they show the floor under every one-kernel measurement. */
XLA_AMD_SELFCHECK_EXPORT int xla_amd_selfcheck_launch_empty(void* stream, int count, int workgroups);

#ifdef __cplusplus
}
#endif
#endif /* XLA_AMD_SELFCHECK_H_ */
