// A small fill kernel: how the host mirror puts sequence lengths into device memory.  It is enqueued on the caller's
// stream like the attention launch that reads the lengths, so a step through the mirror is launches only: no
// host-blocking copy, nothing that races with a previous step still running on that stream, and a step can be
// captured in a HIP graph (a captured step replays at the position it was captured at).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hs {

static __global__ void fill_i32_kernel(int32_t *p, int32_t n, int32_t v) {
    const int32_t i = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i < n) p[i] = v;
}

inline hipError_t fill_i32(int32_t *p, int32_t n, int32_t v, hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    fill_i32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, n, v);
    return hipGetLastError();
}

// fp8 paged batch: the rows of a batch keep their per-kv-head scales in buffers of their own ([2][Hkv], K then V);
// the decode entry point wants them as [n][Hkv] arrays.
static __global__ void gather_head_scales_kernel(const float *const *rows, float *k_out, float *v_out, int32_t n, int32_t hkv) {
    const int32_t i = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i >= n * hkv) return;
    const int32_t r = i / hkv, h = i - r * hkv;
    k_out[i] = rows[r][h];
    v_out[i] = rows[r][hkv + h];
}

inline hipError_t gather_head_scales(const float *const *rows, float *k_out, float *v_out, int32_t n, int32_t hkv, hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    gather_head_scales_kernel<<<(unsigned)((n * hkv + 255) / 256), 256, 0, stream>>>(rows, k_out, v_out, n, hkv);
    return hipGetLastError();
}

}  // namespace hs
