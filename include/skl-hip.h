/*
 * skl-hip.h - runtime shim of the gfx950 SKL library.
 *
 * The SKL kernel entry points (skl-gfx950.h) keep the reference's `void`
 * signatures and caller-owned buffers. Everything a C caller needs around
 * them on a GPU - device selection, device buffers, the stream kernels are
 * launched on, synchronisation and an error channel - is in this header.
 * All functions have C linkage and take only plain pointers and integers.
 *
 * The reference has no counterpart for this header: SKL has no runtime
 * (README.md:9-10 of the reference) because it runs on the calling hart.
 *
 * Pointer convention of every kernel entry point:
 *   - all pointers are device-accessible (device, managed or pinned-host
 *     allocations): the kernel is enqueued on the current stream and the call
 *     returns without waiting;
 *   - all pointers are ordinary host memory: operands are staged through
 *     temporary device buffers and the call returns after the result has been
 *     copied back (a literal drop-in for a CPU caller);
 *   - a mix of both: nothing is done and SKL_HIP_ERR_MIXED_POINTERS is recorded.
 */
#ifndef SKL_HIP_H
#define SKL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes recorded by the library (HIP's own codes are passed through as
 * positive numbers; the library's own are negative). */
#define SKL_HIP_OK 0
#define SKL_HIP_ERR_MIXED_POINTERS (-1)
#define SKL_HIP_ERR_BAD_ARGUMENT (-2)
#define SKL_HIP_ERR_NO_DEVICE (-3)
#define SKL_HIP_ERR_WORKSPACE (-4)
/* Advisory: the calling thread's stream has no scratch slot on this device (32 other streams hold one). The call
 * that recorded it has still completed, on kernels that need no scratch memory (the 4-bit-weight GEMMs, which
 * need a converted copy of their operands for more than 16 rows, through a buffer of their own that is released
 * once the stream has drained: such a call returns after its work is done). See skl_hip_release_stream().
 * SKL_HIP_ERR_WORKSPACE, by contrast, means that C was not written. */
#define SKL_HIP_ERR_STREAM_SLOTS (-5)

/* Pointer-classification modes for skl_hip_set_pointer_mode(). */
#define SKL_HIP_POINTERS_AUTO 0   /* ask the HIP runtime about every pointer (default) */
#define SKL_HIP_POINTERS_DEVICE 1 /* caller promises device-accessible pointers: no queries */

/* Selects `device` for the calling thread and creates the workspace for split
 * reductions of its current stream (scratch memory is kept per stream and
 * device, created at a stream's first call that needs it). Returns 0 or an error. */
int skl_hip_init(int device);
/* Releases every scratch block of every device and stream. Outstanding work is waited for. */
void skl_hip_shutdown(void);
/* Gives back the scratch blocks a stream holds on the current device (up to 64 MiB of workspace, 32.5 MiB of
 * sums and counters, operand copies) and its slot: call it before destroying a stream that made calls into the
 * library. Waits for the stream's work; no call may be issued on the stream meanwhile. A device keeps at most 32
 * streams with scratch of their own - a call on a further stream records SKL_HIP_ERR_STREAM_SLOTS and runs on the
 * kernels that need no scratch memory. Returns 0 or an error. */
int skl_hip_release_stream(void *stream);

void *skl_hip_malloc(size_t bytes);
void skl_hip_free(void *ptr);
int skl_hip_memcpy_h2d(void *dst, const void *src, size_t bytes);
int skl_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);
int skl_hip_memcpy_d2d(void *dst, const void *src, size_t bytes);
int skl_hip_memset(void *dst, int byte, size_t bytes);
/* Zeroes, on the current stream, the static array in which the calls of skl_gemm_i8_i8_i32_noalloc_gfx950 on the
 * current device share their sums. Every such call leaves the array zero again, so this is only needed after calls
 * that overlapped on the device (they race, see that entry point) or did not finish: slots left non-zero would be
 * added to every later result. Allocates nothing; not to be recorded into a graph. Returns 0 or an error. */
int skl_hip_noalloc_reset(void);

/* The stream (a hipStream_t passed as void*) kernels of the calling thread are
 * enqueued on; NULL selects the default stream. */
void skl_hip_set_stream(void *stream);
void *skl_hip_get_stream(void);
/* Waits for the current stream. */
int skl_hip_synchronize(void);

void skl_hip_set_pointer_mode(int mode);
int skl_hip_get_pointer_mode(void);

/* What a GEMM call with beta == 0 does with a floating-point C (per calling thread).
 * SKL_HIP_BETA_ZERO_INITIALISES (default): the call initialises C, which is what the reference gives beta == 0
 *   for (src/gemm/README.md:43, "accumulation (beta=1) and initialization (beta=0)"): the old C is not read,
 *   except where alpha*A*B is an exact zero, whose sign it decides. The result has the bits of the reference's
 *   for every finite C; an Inf or NaN in C - or whatever uninitialised memory holds - is overwritten.
 * SKL_HIP_BETA_ZERO_AS_REFERENCE: beta*C + alpha*A*B is evaluated as the reference's routines evaluate it
 *   (ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21): the old C is read and multiplied by zero, so an Inf or NaN in it
 *   makes the result NaN, exactly where the reference's result is NaN. Costs the read of C (8192^3 fp8: 256 MiB;
 *   looked through under the product on the large tile kernels, about 8 % on top of the call; up to a fifth where
 *   it is read in the epilogue).
 * Integer GEMMs give the same result either way and never read C when beta == 0; f64 GEMMs always read it.
 * A thread that has not called the setter takes the process's default: SKL_HIP_BETA_ZERO_INITIALISES, or, with
 * SKL_HIP_BETA_ZERO=reference in the environment when the library is first asked, SKL_HIP_BETA_ZERO_AS_REFERENCE. */
#define SKL_HIP_BETA_ZERO_INITIALISES 0
#define SKL_HIP_BETA_ZERO_AS_REFERENCE 1
void skl_hip_set_beta_zero_mode(int mode);
int skl_hip_get_beta_zero_mode(void);
/* 1 if `ptr` is device-accessible, 0 if it is ordinary host memory. */
int skl_hip_pointer_is_device(const void *ptr);

/* Thread-local, sticky until read: the only error channel of the `void`
 * kernel entry points. Reading clears it. */
int skl_hip_last_error(void);
const char *skl_hip_last_error_string(void);

/* Edge of the square tile the packed ("ptex1c / p1xte / ptexte") layouts are
 * counted in. The reference reads it from the matrix engine at run time and
 * its tests assume 64; here it is the constant 64 for every element width. */
size_t skl_hip_te(void);

/* Timing helpers on the current stream (hipEvent_t as void*). */
void *skl_hip_event_create(void);
void skl_hip_event_destroy(void *event);
int skl_hip_event_record(void *event);
/* Waits for `stop`, returns milliseconds between the two events (negative on error). */
float skl_hip_event_elapsed_ms(void *start, void *stop);

/* The two ceilings a report prices kernels against, measured on the device (both enqueue one kernel on the
 * current stream; time them with the events above).
 * skl_hip_probe_hbm_read: a plain read of `bytes` (a multiple of 16, 16-byte aligned) with 128-bit non-temporal
 *   loads, eight in flight per lane: what streaming kernels could reach at best on that many bytes.
 * skl_hip_probe_mfma: `iters` rounds of eight independent 32 x 32 matrix-core instructions per wave on register
 *   operands, two workgroups of four waves on every compute unit - kind 0: int8 32x32x32, 1: bf16 32x32x16,
 *   2: fp8 E4M3 32x32x64; random_operands != 0 fills the operand registers with pseudo-random values (the clock
 *   the chip sustains depends on the operand values), else every element is the same value. Returns the number of
 *   operations (two per multiply-add) of the launch, 0 on error. */
int skl_hip_probe_hbm_read(const void *src, size_t bytes);
double skl_hip_probe_mfma(int kind, int random_operands, int iters);

/* Name and compute-unit count of the current device (for reports). */
int skl_hip_device_info(char *name, size_t name_len, int *compute_units, int *clock_mhz);

#ifdef __cplusplus
}
#endif
#endif /* SKL_HIP_H */
