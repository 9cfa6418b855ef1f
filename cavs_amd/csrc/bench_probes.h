/*
 * Measurement aids of the kernel benchmark (python -m cavs_amd.kernel_bench): exported by
 * libcavs_hip.so, not part of the product interface in include/cavs_hip.h and with no
 * counterpart in the reference.
 */
#ifndef CAVS_CSRC_BENCH_PROBES_H_
#define CAVS_CSRC_BENCH_PROBES_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One launch in which every wavefront of four workgroups per CU issues iters * 8 independent
 * v_mfma_f32_32x32x2_f32 on register operands and nothing else -- what the matrix pipes sustain
 * at the clocks the device holds under that load, to set beside the nominal peak.  `out` takes
 * 4 * CUs * 256 floats (1024 * 256 on MI355X); *flops receives the launch's FLOP count. */
int cavs_mfma_probe(float *out, size_t out_floats, int iters, double *flops, void *stream);

#ifdef __cplusplus
}
#endif
#endif
