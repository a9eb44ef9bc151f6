/* Timing diagnostics for the LDS-patch convolution kernel (msnhnet_amd/lib/libmsnh_diag.so, built beside libmsnh_hip.so).
 *
 * Measurement only: no product path loads this library.  It instantiates convPatch8Kernel with its timing switches (the DBG
 * template parameter: parts of the kernel compiled out, shader clock read inside the kernel), which the kernel library itself
 * ships only with every switch off.  No counterpart in the reference.
 */
#ifndef MSNH_HIP_DIAG_H
#define MSNH_HIP_DIAG_H
#include "msnh_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One launch of the float16 3x3 stride-1 pad-1 patch kernel on NHWC x (batch, h, w, c) with packed weights wt (oc, 9, c), per-channel
 * scale / shift, leaky activation, no residual, into y (batch, h, w, oc).
 *   tile     : 46 (64 x 384 tile, twelve wavefronts on 32 x 64 wave tiles) or 52 (the same tile, K split between two groups of six
 *              wavefronts on 64 x 64 wave tiles)
 *   switches : sum of  1 no main-loop loads, 2 no LDS fragment reads, 4 no main-loop barrier, 8 no MFMAs, 16 no epilogue,
 *              32 no prologue loads, 64 clocks: the first wavefront writes the shader-clock ticks and the 100 MHz constant-clock
 *              ticks of its main loop to clocks[0], clocks[1] (device memory, two 64-bit words).  With any of 1..32 set the
 *              output is meaningless; with 0 or 64 it is the library's result.
 * Only the combinations msnh_hip_diag_patch8_switches() lists are instantiated; others return an error.  c must be a multiple of
 * 64, oc of 64; the shape must be one the tile accepts (msnh_hip_conv2d_tile_supported says so for the plain kernel). */
int msnh_hip_diag_patch8(int tile, int switches, int batch, int c, int h, int w, int oc, const void *x, const void *wt, const float *scale,
                     const float *shift, void *y, void *clocks, msnh_stream_t s);

/* the instantiated switch combinations: writes up to cap values to out, returns their number */
int msnh_hip_diag_patch8_switches(int *out, int cap);

/* an empty kernel of the given grid (what a launch costs before it does anything) */
int msnh_hip_diag_empty_launch(int blocks, int threads, msnh_stream_t s);

#ifdef __cplusplus
}
#endif
#endif
