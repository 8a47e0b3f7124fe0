// The arithmetic of the layer ops, in one place. The plain kernels and the
// kernels that fuse an int8 quantiser behind the same op include this header,
// so that "op, then quantise" and "fused op+quantise" see the same FP16 value
// bit for bit (the contract of the reference's fused quantisers:
// include/vibevoice/device.h:298-317).
#pragma once

#include "vv_common.hpp"

namespace vv {

constexpr int kMaxWgThreads = 1024;
constexpr int kMaxWgWaves = kMaxWgThreads / kWave;

// ── RMSNorm ──────────────────────────────────────────────────────────────

// 1 / sqrt(mean(x^2) + eps) with the hardware reciprocal square root (1 ulp of
// FP32, i.e. ~1e-7 relative against an FP16 result whose own rounding is 5e-4).
// Every lane of every wave of a row evaluates this, so it has to be a handful
// of instructions: the correctly rounded divide + sqrt + divide sequence is
// ~60 and was a measurable share of the VALU time with one chunk per thread.
__device__ __forceinline__ float inv_rms(float sumsq, float inv_n, float eps) {
    return __builtin_amdgcn_rsqf(sumsq * inv_n + eps);
}

// acc += sum of squares of one chunk, element 0 first.
__device__ __forceinline__ float chunk_sumsq(const f32x8& x, float acc) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = fmaf(x[i], x[i], acc);
    return acc;
}

// Sum of `acc` over the whole workgroup: DPP reduction inside each wave, one
// float per wave through `partial` (LDS, kMaxWgWaves floats), one barrier, then
// every thread adds the wave sums in wave order, so all threads hold the same
// bits. `partial` must not be reused before the next barrier.
__device__ __forceinline__ float block_sum(float acc, float* partial) {
    acc = wave_sum(acc);
    if (lane_id() == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    float total = 0.0f;
    const int nwaves = (int)blockDim.x >> 6;
    for (int i = 0; i < nwaves; ++i) total += partial[i];
    return total;
}

// The same for kN independent values at once (kN rows sharing a workgroup): one
// barrier for all of them. `partial` is kN x kMaxWgWaves floats of LDS.
template <int kN>
__device__ __forceinline__ void block_sum_n(float (&acc)[kN], float (*partial)[kMaxWgWaves]) {
#pragma unroll
    for (int r = 0; r < kN; ++r) {
        const float w = wave_sum(acc[r]);
        if (lane_id() == 0) partial[r][threadIdx.x >> 6] = w;
    }
    __syncthreads();
    const int nwaves = (int)blockDim.x >> 6;
#pragma unroll
    for (int r = 0; r < kN; ++r) {
        float total = 0.0f;
        for (int i = 0; i < nwaves; ++i) total += partial[r][i];
        acc[r] = total;
    }
}

template <int kN>
__device__ __forceinline__ void block_max_n(float (&v)[kN], float (*partial)[kMaxWgWaves]) {
#pragma unroll
    for (int r = 0; r < kN; ++r) {
        const float w = wave_max(v[r]);
        if (lane_id() == 0) partial[r][threadIdx.x >> 6] = w;
    }
    __syncthreads();
    const int nwaves = (int)blockDim.x >> 6;
#pragma unroll
    for (int r = 0; r < kN; ++r) {
        float m = 0.0f;
        for (int i = 0; i < nwaves; ++i) m = fmaxf(m, partial[r][i]);
        v[r] = m;
    }
}

// (x * inv) * w per element, two roundings, then one FP16 rounding.
__device__ __forceinline__ Chunk scale_chunk(const Chunk& x16, float inv, const Chunk& w16) {
    f32x8 x = unpack(x16);
    const f32x8 g = unpack(w16);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (x[i] * inv) * g[i];
    return pack(x);
}

// ── RoPE ─────────────────────────────────────────────────────────────────

// The rotation of one (lo, hi) pair in the CPU path's arithmetic: four products,
// one subtraction, one addition, none of them fused, so that the only difference
// from the CPU result is the last bits of sin/cos.
struct Pair {
    float lo, hi;
};
__device__ __forceinline__ Pair rotate(float a, float b, float c, float s) {
#pragma clang fp contract(off)
    const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
    Pair r;
    r.lo = ac - bs;
    r.hi = as + bc;
    return r;
}

// ── SwiGLU ───────────────────────────────────────────────────────────────

// silu(g) * u in the CPU path's association, (g / (1 + e^-g)) * u, with the
// hardware exponential and reciprocal: exp2(-g * log2 e) and rcp are each
// accurate to about 1 ulp of FP32, three orders below the FP16 rounding of the
// result. Large |g| needs no special case: e^-g -> inf gives rcp -> 0 and
// g * 0 = -0 (the CPU path's -65504 / inf), e^-g -> 0 gives g itself.
__device__ __forceinline__ float swiglu1(float g, float u) {
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
    const float silu = g * __builtin_amdgcn_rcpf(1.0f + e);
    return silu * u;
}

__device__ __forceinline__ Chunk swiglu_chunk(const Chunk& gate, const Chunk& up) {
    const f32x8 g = unpack(gate), u = unpack(up);
    f32x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = swiglu1(g[i], u[i]);
    return pack(r);
}

}  // namespace vv
