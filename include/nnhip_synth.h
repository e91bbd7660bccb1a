/*
 * nnhip_synth - device-side synthetic weight generator used by bench.py and the GPU tests.
 *
 * It has no counterpart in the reference: NNtrain loads real GGUF files.  The 27B-shape decode benchmark needs
 * 28.7 GB of random-init Q8_0 blocks, which is far quicker to draw on the GPU than on the host.  The generator
 * lives in its own library (libnnhip_synth.so) so that libnnhip.so stays the drop-in boundary and nothing else.
 */
#ifndef NNHIP_SYNTH_H
#define NNHIP_SYNTH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Fills `blocks` Q8_0 blocks at dptr (34 bytes each) on `stream` (a hipStream_t, may be null): per block 32 values
 * w ~ N(0, sigma) from a counter-based generator keyed by (seed, block index), d = max|w| / 127 stored as fp16,
 * q = round(w / d) clipped to +-127 - the quantize_row_q8_0 convention.  Returns 0 or a hipError_t. */
int nnhip_synth_q8_0(void* stream, void* dptr, uint64_t blocks, uint64_t seed, float sigma);

/* Fills `count` floats with N(0, 1) draws keyed by (seed, index).  Returns 0 or a hipError_t. */
int nnhip_synth_normal_f32(void* stream, float* dptr, uint64_t count, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif
