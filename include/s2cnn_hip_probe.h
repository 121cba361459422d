/* Measurement entry point of libs2cnn_probe.so.  NOT part of the drop-in boundary (include/s2cnn_hip.h) and not built
 * with it: `python -m s2cnn_amd.csrc.build --probes` builds the library, `bench.py --floor` is its only caller.
 * No counterpart in the reference.
 *
 * The per-volume kernel of the 64^3 grid alone (direction 0: analysis, x -> records in the workspace; 1: synthesis,
 * records -> y), full spectra, with parts compiled out: probe 0 the kernel as shipped, 1 without the multiply-adds of the
 * Wigner contraction, 2 (analysis) without its table loads as well, 2 (synthesis) with those multiply-adds issued as
 * 4x4x1 matrix instructions instead.  With probe != 0 the results are meaningless: only
 * the time is read.  packed_table: the packed table of s2cnn_so3_pack_table(32, 32, direction); workspace:
 * s2cnn_so3_analysis_workspace(32, 32, nbatch, 0) bytes.  Returns 0 or a code of s2cnn_hip.h.
 */
#ifndef S2CNN_HIP_PROBE_H
#define S2CNN_HIP_PROBE_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif
int s2cnn_so3_fft64_probe(const float *x, float *y, const float *packed_table, void *workspace, size_t workspace_bytes,
                          long nbatch, int direction, int probe, void *stream);
#ifdef __cplusplus
}
#endif
#endif
