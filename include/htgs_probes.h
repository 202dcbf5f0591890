/*
 * htgs_probes -- measurement probes of the MI355X rasterizer build.  Not part of the drop-in boundary and not in
 * libhtgs_amd.so: a separate library (htgs_amd/diagnostics/libhtgs_probes.so) that only the benchmark loads.
 * No counterpart in the reference.  Return values: 0 = ok, 2 = bad argument, 3 = the launch failed.
 */
#ifndef HTGS_PROBES_H
#define HTGS_PROBES_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* How long one vector instruction holds a SIMD.  Launch number `instruction` (0 .. until htgs_probe_issue_cost_name
 * returns NULL) runs n_blocks workgroups of four waves, each wave `turns` loop turns of 64 copies of that instruction;
 * out receives n_blocks * 256 floats.  Timed by the caller: cycles per instruction and SIMD =
 * time * clock * 1024 SIMDs / (n_blocks * 4 * turns * 64). */
const char *htgs_probe_issue_cost_name(int instruction);
int htgs_probe_issue_cost_launch(int instruction, float *out, int n_blocks, int turns, void *stream);

/* A plain device-to-device copy of n_bytes (multiple of 16) with one 16-byte load and store per thread.  Hardware
 * counters read on it calibrate the same counters read on the rasterizer's kernels. */
int htgs_probe_copy_bytes(void *dst, const void *src, size_t n_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif
