/*
 * libhipq_probe.so -- measurement aids of the hipq kernels.  Not part of the product library and
 * not part of its ABI: nothing in libhipq.so, the backend plugin or the host library links or loads
 * it.  bench.py loads it for the device ceilings it reports next to the kernels' rates (matrix-core
 * rate on given operand bytes, a compute unit's intake from L2, integer atomics into L2), and the
 * CPU tests load it for the host-side index arithmetic check.  No counterpart in the reference.
 *
 * Every function returns 0 on success; hipq_probe_last_error() describes the last failure of the
 * calling thread.  Pointers are device pointers unless a comment says otherwise; `stream` is a
 * hipStream_t (NULL: the default stream).
 */
#ifndef HIPQ_PROBE_H
#define HIPQ_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPQ_PROBE_API __attribute__((visibility("default")))

HIPQ_PROBE_API const char* hipq_probe_last_error(void);

/* A full-chip launch of dependent v_mfma_i32_32x32x32_i8 chains on register-resident operands
 * (`operands_8k`: 8 sets of 64 lanes x 16 bytes; `sink`: workgroups x 256 ints).  Each of a
 * workgroup's 4 wavefronts issues 64 x iters MFMAs of 65536 operations. */
HIPQ_PROBE_API int hipq_probe_mfma_i8(const void* operands_8k, void* sink, int32_t workgroups, int32_t iters, void* stream);

/* Whether matrix and vector instructions overlap on a SIMD.  Workgroups of eight wavefronts (two a
 * SIMD), `iters` iterations of 16 v_mfma_i32_32x32x32_i8 a wavefront (32 cycles each on its SIMD) and
 * `vector_per_mfma` (4, 8 or 16) independent v_fma_f32 for each of them (4 cycles each):
 *   mode 0: every wavefront issues both, the vector instructions behind each MFMA
 *   mode 1: the MFMAs alone          mode 2: the vector instructions alone
 *   mode 3: four wavefronts of a workgroup issue only the MFMAs, the other four only the vector work
 *           (half of mode 0's work of either kind: compare with half of modes 1 and 2)
 *   mode 4: mode 0 with the accumulators in a[0:31] (the accumulation registers)
 * `operands_2k`: 2 sets of 64 lanes x 16 bytes; `sink`: workgroups x 512 ints. */
HIPQ_PROBE_API int hipq_probe_coissue(const void* operands_2k, void* sink, int32_t workgroups, int32_t iters, int32_t vector_per_mfma, int32_t mode, void* stream);

/* How many bytes a second a compute unit takes in from L2 (or from HBM).  `workgroups` workgroups of
 * 4 wavefronts (`lds_bytes` of dynamic LDS each: the handle on how many share a compute unit) read
 * `steps` x 32 KiB each out of `buf`: 16 bytes a lane and instruction, 8 instructions a wavefront
 * and step, two steps in flight.
 *   shape 0: a wavefront instruction covers 1024 contiguous bytes
 *   shape 1: 8 rows x 128 bytes (rows `pitch` = 4096 bytes apart: whole cache lines)
 *   shape 2: 16 rows x 64 bytes (half lines)
 *   shape 3: 64 rows x 16 bytes, rows 1024 bytes apart (every lane in a line of its own: the MFMA
 *            fragment read of a row-major matrix)
 *   to_lds 0: into registers (xor-reduced into `sink`); 1: straight into LDS (buffer_load ... lds)
 * Addresses wrap inside `window_bytes` (a power of two >= 1 MiB): a window of a few MiB is served
 * by the L2s after the first pass, a window of GiBs with `spread` != 0 (every workgroup starts
 * `steps` x 32 KiB further on) by HBM.  No division or modulo in the address arithmetic.
 * `sink`: workgroups x 256 ints. */
HIPQ_PROBE_API int hipq_probe_intake(const void* buf, size_t buf_bytes, size_t window_bytes, int32_t spread, int32_t shape, int32_t to_lds, int32_t workgroups, int32_t lds_bytes,
                                     int32_t steps, void* sink, void* stream);

/* Integer atomics into L2: every workgroup adds `rounds` tiles of 128 x 128 int32 (64 KiB, what it
 * holds in registers after a 128 x 128 GEMM tile) to tiles of `dst` without waiting for a return
 * value.  `share` workgroups add to the same tile; same_die != 0: they are the workgroups whose ids
 * are congruent modulo 8 (one compute die, one L2), else consecutive ids (eight dies).
 * `dst`: workgroups / share x rounds tiles of 64 KiB, zeroed by the caller. */
HIPQ_PROBE_API int hipq_probe_atomic_tiles(void* dst, size_t dst_bytes, int32_t workgroups, int32_t share, int32_t same_die, int32_t rounds, void* stream);

/* The floor under a sequence of dependent launches: `kernels` launches in a row on `stream` of a
 * kernel that does nothing (`workgroups` workgroups of 256 lanes; touch != 0: lane 0 of each writes a
 * word of `sink`, workgroups ints).  Timed eagerly and as a replayed graph it says what a pass of that
 * many launches costs before any of them computes anything. */
HIPQ_PROBE_API int hipq_probe_empty_chain(void* sink, int32_t kernels, int32_t workgroups, int32_t touch, void* stream);

/* host-only: n / d by the multiply-shift the Quantize kernels use for their scale index
 * (0 <= n < 2^31, 1 <= d < 2^31) */
HIPQ_PROBE_API uint32_t hipq_debug_fastdiv(uint32_t n, uint32_t d);

#ifdef __cplusplus
}
#endif
#endif
