// Host launcher of the MFMA-only measurement kernels (see probe.hip).
#pragma once
#include <hip/hip_runtime.h>

#define MUON_PROBE_BLOCKS 256                     // one workgroup per compute unit
#define MUON_PROBE_OPERAND_BYTES (256L * 12 * 512 * 16)  // 12 fragments of 16 bytes per thread
#define MUON_PROBE_SINK_FLOATS (256L * 512)
#define MUON_PROBE_FLOP_PER_ITER (256.0 * 8 * 16 * 32768.0)

hipError_t launch_mfma_probe(const void* operands, float* sink, int shape, int iters, hipStream_t stream);
