/*
 * motifcl_amd_diag.h -- measurement and test aids of libmotifcl_amd.so.
 *
 * Nothing here has a counterpart in the reference and nothing here is part of
 * the drop-in boundary (that is motifcl_amd.h): a shader-clock probe used by
 * the benchmark to report the clock the kernels ran at, the generator of the
 * benchmark's synthetic inputs, and the knobs that let a test force the bounded
 * device-side waits to give up or a small layer to take the paths of a large
 * one.  Every knob is a setting of the calling thread: a thread that never
 * touches them runs on the defaults whatever other threads set, and no entry
 * point of motifcl_amd.h changes its answer because of them.  Conventions
 * (status codes, mcc_last_error) are those of motifcl_amd.h.
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
 * Tiles of the strip-workspace step: 0 (default) chosen by shape -- 256 x 256
 * tiles where whole rounds of them keep the device busy, 128 x 128 otherwise --,
 * 1 the 256 x 256 tiles whenever the shape allows them (sides multiples of 256,
 * token count a multiple of 16, 16-byte aligned operands), 2 never.  Both kernels
 * write the same bytes; tests use the switch to compare them on small shapes.
 * grid_cap > 0 holds the 256 x 256 kernel to that many workgroups, so that a
 * small layer runs in several passes of its persistent grid and parks tiles
 * whose strip ends in a later pass; such a step needs the workspace size
 * mcc_compact_counter_fused_strip_workspace_nbytes_for_grid returns for that
 * cap (the slots for parked tiles; the public size query never depends on the
 * cap) and is rejected with a smaller one.  0 restores the device's own capacity.
 */
void mcc_compact_counter_fused_strip_set_tile_mode(int mode, int grid_cap);
size_t mcc_compact_counter_fused_strip_workspace_nbytes_for_grid(size_t in_features, size_t out_features,
                                                                 size_t batch, int grid_cap);

/*
 * The contraction of shapes that are more than two but not a whole number of rounds of
 * 256 x 256 tiles runs as one launch in which neighbouring workgroups hand a partly
 * summed tile on through the output buffer; a workgroup that does not find the tile it
 * is to continue computes it alone.  `polls` is the number of polls (about a
 * microsecond each) before it does so (0xffffffff restores the default); a non-zero
 * `start_first` makes every workgroup look for that tile before its neighbour can have
 * produced it.  With (0, 1) every hand-off takes the fallback; the result is the same
 * bits either way, which is what the test that uses this checks.
 */
void mcc_contraction_spans_set_test_mode(unsigned polls, int start_first);

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

/*
 * Synthetic inputs of the benchmark, generated on the device by a counter-based generator:
 * lowbias32 of the element index and the stream id -> two 24-bit uniforms -> Box-Muller.
 * dst[i] = sigma * z_i for i < n.  The same (stream_id, n) gives the same bytes on every run
 * of this library; the host copies them when the CPU needs the same inputs.
 */
int mcc_fill_normal_f32(void* stream, float* dst, size_t n, uint32_t stream_id, float sigma);

/*
 * Packed counter state (four 6-bit codes per 3 bytes) with every code uniform on
 * [0, n_codes), from the same generator.  dst holds 3 * n_groups bytes.
 */
int mcc_fill_counter_state_u8(void* stream, uint8_t* dst, size_t n_groups, uint32_t stream_id, uint32_t n_codes);

#ifdef __cplusplus
}
#endif

#endif /* MOTIFCL_AMD_DIAG_H */
