// Shared helpers for the gfx950 kernels of libdifflut_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/difflut_hip.h"

#define DL_WAVE 64

static inline int dl_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? DL_OK : (int)e;
}

static inline size_t dl_align256(size_t v) { return (v + 255) & ~(size_t)255; }
static inline int dl_ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// Value of `v` held by lane `src_lane` (0..63) of the same wavefront.
__device__ __forceinline__ float dl_lane_read(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

// Wave-uniform value into a scalar register so that loads addressed by it become scalar loads.
__device__ __forceinline__ int dl_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// MI355X hands the workgroups of a 1-D grid to its 8 XCDs round-robin by block id, and every XCD has
// its own L2.  dl_xcd_map turns the block id into (inner, outer) such that all `inner_count` blocks
// of one outer index run on the same XCD, so what they share is fetched into one L2 once.
// Launch with dl_xcd_grid(inner_count, outer_count) blocks; blocks mapped past the end return false.
#define DL_XCDS 8
// fourth word of a raw buffer descriptor on gfx9 (32-bit data format, range check against num_records)
#define DL_BUFFER_WORD3 0x00020000
static inline int dl_xcd_grid(int inner_count, int outer_count) {
    return DL_XCDS * inner_count * ((outer_count + DL_XCDS - 1) / DL_XCDS);
}
__device__ __forceinline__ bool dl_xcd_map(int inner_count, int outer_count, int &inner, int &outer) {
    const int xcd = blockIdx.x % DL_XCDS, q = blockIdx.x / DL_XCDS;
    inner = q % inner_count;
    outer = (q / inner_count) * DL_XCDS + xcd;
    return outer < outer_count;
}

// Optional per-kernel timing (dl_profile_enable / dl_profile_read): when switched on, every
// launch site records a HIP event before and after its kernel on the launch stream.
void dl_prof_begin(const char *kernel_name, hipStream_t s);
void dl_prof_end(hipStream_t s);
#define DL_TIMED(name, s, ...) \
    do {                       \
        dl_prof_begin(name, s); \
        __VA_ARGS__;           \
        dl_prof_end(s);        \
    } while (0)
