// Shared device helpers for the gfx950 layer kernels: 16-byte chunk access,
// FP16 <-> FP32 unpacking, and a wave64 all-reduce built on DPP lane permutes.
//
// Everything here assumes wave64 (CDNA) and is compiled for gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/vibevoice_hip.h"

namespace vv {

constexpr int kWave = 64;         // lanes per wavefront
constexpr int kBlock = 256;       // threads per workgroup: 4 waves, one per SIMD
constexpr int kWavesPerBlock = kBlock / kWave;

typedef _Float16 h16;
typedef h16 h16x2 __attribute__((ext_vector_type(2)));
typedef h16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

// One 16-byte chunk = 8 FP16 values = what one lane moves per memory instruction.
struct alignas(16) Chunk {
    uint32_t w[4];
};
static_assert(sizeof(Chunk) == 16, "Chunk must be 16 bytes");

__device__ __forceinline__ Chunk load_chunk(const Chunk* p) { return *p; }
__device__ __forceinline__ void store_chunk(Chunk* p, const Chunk& c) { *p = c; }

// Streaming forms (the "nt" bit on global_load/global_store): the line is
// touched once and should be the first to leave the caches. On MI355X a plain
// copy moves 5.7 TB/s with ordinary accesses and 6.3 TB/s with these, and the
// gap is wider for short launches against a last-level cache that earlier
// kernels left full of written lines (a 2048-row add+norm: 13.5 us with ordinary
// accesses, 11.7 us with these; its stores alone are worth 20 %). The hosts pick
// them from kStreamBytes per launch on; below that (a decode step, a handful of
// rows) ordinary accesses leave the output in L2 for the kernel that consumes it.
constexpr size_t kStreamBytes = (size_t)2 << 20;

__device__ __forceinline__ Chunk load_chunk_stream(const Chunk* p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    Chunk c;
    c.w[0] = v.x; c.w[1] = v.y; c.w[2] = v.z; c.w[3] = v.w;
    return c;
}
__device__ __forceinline__ void store_chunk_stream(Chunk* p, const Chunk& c) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = {c.w[0], c.w[1], c.w[2], c.w[3]};
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

template <bool kStream>
__device__ __forceinline__ Chunk load_chunk_as(const Chunk* p) {
    if constexpr (kStream) return load_chunk_stream(p);
    else return load_chunk(p);
}
template <bool kStream>
__device__ __forceinline__ void store_chunk_as(Chunk* p, const Chunk& c) {
    if constexpr (kStream) store_chunk_stream(p, c);
    else store_chunk(p, c);
}

__device__ __forceinline__ f32x8 unpack(const Chunk& c) {
    const h16x8 h = __builtin_bit_cast(h16x8, c);
    f32x8 f;
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
    return f;
}

// FP32 -> FP16 with round-to-nearest-even (v_cvt_f16_f32 under the default
// rounding mode). The empty asm makes the FP32 value opaque at this point:
// without it the compiler may fold a preceding multiply by a widened FP16
// operand into v_fma_mixlo_f16 with a +0 addend, which turns a product of -0
// into +0 (observed in the 2-byte SwiGLU path).
__device__ __forceinline__ h16 to_half(float v) {
    asm("" : "+v"(v));
    return (h16)v;
}

// Eight of them, packed back into one chunk.
__device__ __forceinline__ Chunk pack(const f32x8& f) {
    h16x8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = to_half(f[i]);
    return __builtin_bit_cast(Chunk, h);
}

// ── wave64 all-reduce ────────────────────────────────────────────────────
// DPP moves data between lanes inside the VALU, with no LDS traffic and no
// barrier. Steps: xor-1 and xor-2 inside each quad, mirror inside each
// half-row (8 lanes) and row (16 lanes); after that every lane of a row holds
// its row's sum, and the four row sums are read out through scalar registers.
// All lanes end with the same bits (each step adds the same two values in
// every lane of a pair, and FP32 addition commutes).
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl,
                                              0xF, 0xF, true);
    return __builtin_bit_cast(float, r);
}

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);   // row_half_mirror
    v += dpp_move<0x140>(v);   // row_mirror
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

// The same butterfly with max instead of +, for row-wise absmax.
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)),
                 fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// Integer sum over each quad of lanes (lanes 4q..4q+3), left in all four.
__device__ __forceinline__ int quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    return v;
}

__device__ __forceinline__ int wave_in_block() {
    return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
}
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63); }

// ── host helpers ─────────────────────────────────────────────────────────
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Streaming accesses for launches of at least kStreamBytes; the environment
// variable VV_HIP_STREAM=0 / 1 forces them off / on (for A/B measurements).
inline bool use_streaming(size_t launch_bytes) {
    static const int forced = [] {
        const char* e = getenv("VV_HIP_STREAM");
        return (e && (e[0] == '0' || e[0] == '1')) ? e[0] - '0' : -1;
    }();
    return forced >= 0 ? forced == 1 : launch_bytes >= kStreamBytes;
}

inline vv_status_t launch_status() {
    return hipGetLastError() == hipSuccess ? VV_OK : VV_ERR_CUDA_LAUNCH;
}

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace vv
