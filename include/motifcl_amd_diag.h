/*
 * motifcl_amd_diag.h -- measurement and test aids of libmotifcl_amd.so.
 *
 * Nothing here has a counterpart in the reference and nothing here is part of
 * the drop-in boundary (that is motifcl_amd.h): a shader-clock probe used by
 * the benchmark to report the clock the kernels ran at, and the knob that lets
 * a test force the bounded device-side wait of the strip-workspace fused step
 * to give up.  Conventions (status codes, mcc_last_error) are those of
 * motifcl_amd.h.
 */
#ifndef MOTIFCL_AMD_DIAG_H
#define MOTIFCL_AMD_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Polls a strip-workspace step spends on one wait before giving up (0
 * restores the default, about four seconds).  For tests of the error path.
 */
void mcc_compact_counter_fused_strip_set_spin_limit(unsigned spins);

/*
 * Shader-clock probe (a measurement aid with no counterpart in the reference).
 * Enqueues a one-wave kernel on `stream` that sleeps for `seconds` (at most 2) of
 * the constant-rate wall clock and writes two 64-bit counts to the device buffer
 * `out`: out[0] wall-clock ticks, out[1] shader cycles over the same stretch.
 * Launched on a side stream while other kernels run it gives the frequency they
 * ran at: MHz = out[1] / out[0] * wall_clock_khz / 1000.  Matrix-core peaks are
 * quoted at the maximum engine clock; under load the power limit holds the clock
 * below it.
 */
int mcc_clock_probe(void* stream, uint64_t* out, size_t out_nbytes, double seconds);
int mcc_wall_clock_khz(int* khz);

#ifdef __cplusplus
}
#endif

#endif /* MOTIFCL_AMD_DIAG_H */
