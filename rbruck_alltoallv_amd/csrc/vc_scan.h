// vc_scan.h — wavefront-level prefix sums (64 lanes) and their workgroup composition.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vc_common.h"

#define VC_WAVE 64
#define VC_WAVES_PER_BLOCK (VC_THREADS / VC_WAVE)

// Inclusive prefix sum across the 64 lanes of a wavefront.
__device__ __forceinline__ int64_t vc_wave_inclusive_scan(int64_t v) {
    const int lane = threadIdx.x & (VC_WAVE - 1);
#pragma unroll
    for (int o = 1; o < VC_WAVE; o <<= 1) {
        int64_t u = __shfl_up(v, o, VC_WAVE);
        if (lane >= o) v += u;
    }
    return v;
}

// Exclusive prefix sum across a 256-thread workgroup; `total` receives the sum of all
// lanes.  `lds` must hold VC_WAVES_PER_BLOCK int64 and is safe to reuse after return.
__device__ __forceinline__ int64_t vc_block_exclusive_scan(int64_t v, int64_t *lds, int64_t &total) {
    const int lane = threadIdx.x & (VC_WAVE - 1);
    const int wave = threadIdx.x / VC_WAVE;
    int64_t incl = vc_wave_inclusive_scan(v);
    __syncthreads();                       // protects lds from the previous use
    if (lane == VC_WAVE - 1) lds[wave] = incl;
    __syncthreads();
    int64_t before = 0, all = 0;
#pragma unroll
    for (int k = 0; k < VC_WAVES_PER_BLOCK; k++) {
        int64_t t = lds[k];
        if (k < wave) before += t;
        all += t;
    }
    total = all;
    return before + incl - v;
}

// Sum across a 256-thread workgroup (every thread gets the result).
__device__ __forceinline__ int64_t vc_block_sum(int64_t v, int64_t *lds) {
    int64_t total;
    (void)vc_block_exclusive_scan(v, lds, total);
    return total;
}

// Maximum across a 256-thread workgroup (every thread gets the result).
__device__ __forceinline__ int64_t vc_block_max(int64_t v, int64_t *lds) {
#pragma unroll
    for (int o = VC_WAVE / 2; o > 0; o >>= 1) {
        const int64_t u = __shfl_xor(v, o, VC_WAVE);
        v = u > v ? u : v;
    }
    __syncthreads();                       // protects lds from the previous use
    if ((threadIdx.x & (VC_WAVE - 1)) == 0) lds[threadIdx.x / VC_WAVE] = v;
    __syncthreads();
    int64_t m = lds[0];
#pragma unroll
    for (int k = 1; k < VC_WAVES_PER_BLOCK; k++) m = lds[k] > m ? lds[k] : m;
    return m;
}
