// Host launchers of the multi-tensor kernels (see multi_tensor.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/muon_hip.h"
#include "common.h"

#define MUON_MULTI_CHUNK MUON_HIP_MULTI_CHUNK  // elements per block

// A list of n tensors as device arrays: base pointers, element counts and the index of each
// tensor's first chunk (n + 1 entries; the last one is the number of chunks).
struct MultiTensorList {
    const void* const* ptrs;
    const long* numel;
    const long* chunk_start;
    int n;
    long chunks;
};

hipError_t launch_adamw_multi(const MultiTensorList& l, const void* const* g_ptrs, const void* const* e1_ptrs,
                              const void* const* e2_ptrs, const double* bias1, const double* bias2, int dtype,
                              double lr, double b1, double b2, double eps, double wd, hipStream_t stream);
hipError_t launch_tensor_norms(const MultiTensorList& l, int dtype, double norm_type, float* partials, float* norms,
                               hipStream_t stream);
hipError_t launch_total_norm(const float* norms, int n, int dtype, double norm_type, float* total_f32, void* total_typed,
                             hipStream_t stream);
hipError_t launch_clip_scale_multi(const MultiTensorList& l, int dtype, const float* total_f32, int norm_dtype,
                                   double max_norm, hipStream_t stream);
