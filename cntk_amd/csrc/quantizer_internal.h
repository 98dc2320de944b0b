// Entry points that the shared library exports for its own tests and tuning runs.
// They are not part of the drop-in boundary and may change.
#pragma once

#include "../../include/cntk_amd_quantizer.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Forces kernel choices on a handle:
 *   quantize_path    0 = automatic, 1 = LDS column tile, 2 = tall-column (global re-read),
 *                    3 = one workgroup per column, column in LDS (fp32, rows a multiple of 4 up to 14336),
 *                    4 = one workgroup per column, column in registers, 16-byte accesses (below 32 (fp64: 64) bits; the
 *                        three matrices at the same offset within 16 bytes),
 *                    5 = the same with one element per access: fp32 any alignment, up to 98304 rows; fp64 256 threads per
 *                        column, 1025 to 6144 rows, below 64 bits, the bytes of path 1
 *                    6 = several workgroups per column, a strip of QWords each (below 32 (fp64: 64) bits, any height whose
 *                        strips number at most half of what the device holds of the kernel, any alignment)
 *                    7 = the same in two or three launches, each reading the matrix: any height of two strips or more (the
 *                        bytes of path 6)
 *   tile_gs          0 = automatic, else threads per column in the tile statistics phase (power of two, 8..256)
 *   unq_slots        0 = automatic, else bit positions decoded per thread by the QWord-major unquantize
 *   unq_mode         0 = automatic, 1 = QWord-major decoder with one store per value, 2 = tile decoder wherever it can run,
 *                    3 = automatic without the tile decoder, 4 = row-major decoder (packed column in LDS) wherever it can
 *                    run, 5 = row-major decoder that fetches its QWords itself wherever it can run, 6 = the same for short
 *                    columns (the matrix as one run of 16-byte groups) wherever it can run
 *   tile_stage       -1 = automatic, 0 = tile kernels write the residual straight to memory, 1 = through LDS */
int cntkq_debug_set_tuning(cntkq_quantizer* h, int quantize_path, unsigned tile_gs, unsigned unq_slots,
                           int unq_mode, int tile_stage);

/* How often a lane of a strip kernel (path 6) polls for another workgroup's partial sum before it gives up and raises the
 * error that the next cntkq_wait_quantize_done reports. Zero makes every exchange fail at once while every kernel still
 * runs to its end: the way to test that error path. */
int cntkq_debug_set_strip_spin_limit(cntkq_quantizer* h, unsigned limit);

/* The most strips per column that the strip kernels (path 6) take on the handle's device at this bit width: half of what
 * the device holds of the kernel, as the runtime's occupancy query tells (a column of more strips than half a die holds
 * has them on all eight dies), never more than 8 x 128 (0: unknown, or no strip kernel for the bit width). A strip is
 * 512 / 1024 / 2048 QWords at 1 / 2 / 4 and more bits; of a double matrix 128 / 256 / 512 / 1024 at 1 / 2 / 4 / 8 and more. */
unsigned cntkq_debug_strip_max_strips(cntkq_quantizer* h, size_t nbits, int zero_threshold_for_1bit);
unsigned cntkq_debug_strip_max_strips_f64(cntkq_quantizer* h, size_t nbits, int zero_threshold_for_1bit);

/* Ties caller-owned hipEvent_t objects (either may be NULL) to the NEXT kernel this handle launches: start_event is
 * set when that kernel begins, stop_event when it has finished, by the dispatch itself. Used to time single kernels
 * without putting extra commands into the stream. The stop event also becomes what the matching Wait call waits on,
 * so it must stay alive until then. With a gradient-set call next: start_event at its first launch, stop_event at its
 * last, and the call's own completion event recorded on the stream behind that. */
int cntkq_debug_attach_events(cntkq_quantizer* h, void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
