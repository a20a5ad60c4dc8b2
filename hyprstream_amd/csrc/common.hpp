// Shared device helpers for the gfx950 kernels of libhs_attn.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hs_attn.h"

namespace hs {

constexpr int kWave = 64;

// Error plumbing of the C ABI (api.hip owns the thread-local message).
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

// Addressing of the head-major cache layout; block tables resolved per token.
struct KvAddr {
    int64_t code_stride_seq, code_stride_head, scale_stride_seq, scale_stride_head;
    int32_t capacity_tokens, block_table_stride;
    int32_t cap_shift;     // log2(capacity_tokens) when that is a power of two (the usual 256-token blocks), else -1
    const int32_t *table;  // K or V table already chosen; nullptr = not paged
};

inline KvAddr make_addr(const hs_kv_layout &l, int which_table) {
    KvAddr a;
    a.code_stride_seq = l.code_stride_seq;
    a.code_stride_head = l.code_stride_head;
    a.scale_stride_seq = l.scale_stride_seq;
    a.scale_stride_head = l.scale_stride_head;
    a.capacity_tokens = l.capacity_tokens;
    a.block_table_stride = l.block_table_stride;
    a.cap_shift = -1;
    if (l.capacity_tokens > 0 && (l.capacity_tokens & (l.capacity_tokens - 1)) == 0)
        for (int s = 0; s < 31; ++s)
            if ((1 << s) == l.capacity_tokens) a.cap_shift = s;
    a.table = which_table ? l.v_block_table : l.k_block_table;
    return a;
}

// A read of memory that no kernel writes while this one runs (block tables, lengths), through the constant address
// space: with a wavefront-uniform address it is a scalar load even in a kernel that also stores to global memory.
// (An ordinary uniform load there becomes a vector load, whose result waits in line behind every K/V tile load the
// wavefront has in flight.)
__device__ __forceinline__ int32_t load_invariant(const int32_t *p, int64_t i) {
    typedef const int32_t __attribute__((address_space(4))) *cptr;
    return ((cptr)(uintptr_t)p)[i];
}

// Resolve (sequence b, token t) -> (storage unit, slot).  Returns false when t is outside
// what the sequence can hold (unit/slot are then 0/0, a valid but meaningless location).
__device__ __forceinline__ bool resolve(const KvAddr &a, int b, int t, int64_t &unit, int &slot) {
    unit = 0;  // on failure the caller still holds an address inside the buffer
    slot = 0;
    if (t < 0) return false;
    if (a.table) {
        int blk = a.cap_shift >= 0 ? t >> a.cap_shift : t / a.capacity_tokens;
        if (blk >= a.block_table_stride) return false;
        int id = load_invariant(a.table, (int64_t)b * a.block_table_stride + blk);
        if (id < 0) return false;
        unit = id;
        slot = t - blk * a.capacity_tokens;
        return true;
    }
    if (t >= a.capacity_tokens) return false;
    unit = b;
    slot = t;
    return true;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f);
// The attention output as bf16, times the output gate when there is one (Qwen3.5 full-attention layers,
// qwen3_5.rs:1056-1059: ctx * gate.sigmoid() on bf16 tensors -- the sigmoid is rounded to bf16, then the product).
__device__ __forceinline__ uint32_t gated_bf16_bits(float attn, const uint16_t *gate, int64_t i) {
    const uint32_t o = f32_to_bf16_bits(attn);
    if (gate == nullptr) return o;
    const float sg = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-bf16_bits_to_f32(gate[i])))));
    return f32_to_bf16_bits(bf16_bits_to_f32(o) * sg);
}

// fp32 -> bf16 bits, round-to-nearest-even (NaN stays a quiet NaN): gfx950's conversion instruction.  Compared on the
// device with the integer formulation ((u + 0x7fff + ((u >> 16) & 1)) >> 16, NaN -> (u >> 16) | 0x40, which is what
// libtorch and the CPU oracle compute) over all 2^32 inputs: the same bits for every one, NaNs included.  One
// instruction instead of seven matters in the kernels that round after every operation to reproduce bf16 tensor ops.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}

template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        T w = __shfl_xor(v, o, 64);
        v = v > w ? v : w;
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Load E consecutive source elements (E in {1,2,4}) starting at element index `i` as fp32.
template <int E>
__device__ __forceinline__ void load_src(const void *p, int dtype, int64_t i, float (&x)[E]) {
    if (dtype == HS_F32) {
        const float *s = (const float *)p + i;
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = s[e];
    } else {
        const uint16_t *s = (const uint16_t *)p + i;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            uint16_t h = s[e];
            if (dtype == HS_BF16) x[e] = bf16_bits_to_f32(h);
            else {
                _Float16 f;
                __builtin_memcpy(&f, &h, 2);
                x[e] = (float)f;
            }
        }
    }
}

}  // namespace hs
