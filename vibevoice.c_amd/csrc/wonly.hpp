// The older weight-only formats (FP16 activations against quantised weights), as
// one rule per format for the eight FP16 weights of a 16-byte output slot. Every
// kernel that needs the FP16 weight (the dequantisers, the small-M MFMA kernel)
// goes through wo_slot, so all of them multiply the same bits:
//   kWoInt8  int8 [N][K], FP32 scale per row:           fp16(float(q) * scale)
//   kWoNf4   4-bit code-book indices [N*K/2], high nibble = even element,
//            FP16 absmax per 64 flat elements:           fp16(book[code] * absmax)
//   kWoAwq   4-bit codes [N][K/2], high nibble = even column, FP16 scale and
//            min per group of 32..256 columns:           fp16(fma(q, scale, min))
#pragma once
#include "vv_common.hpp"

namespace vv {

constexpr int kWoF16 = 0, kWoInt8 = 1, kWoNf4 = 2, kWoAwq = 3;     // the first three: vv_skinny_format_t

typedef uint32_t wo_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t wo_u32x4 __attribute__((ext_vector_type(4)));

// bitsandbytes' NF4 code book.
__device__ const float kNf4Book[16] = {
    -1.0f,                 -0.6961928009986877f,  -0.5250730514526367f,  -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f,  0.16093020141124725f,  0.24611230194568634f,  0.33791524171829224f,
    0.44070982933044434f,  0.5626170039176941f,   0.7229568362236023f,   1.0f};

struct WoSource {
    const void* w;          // the codes
    const void* scales;     // INT8: FP32 [N]; NF4: FP16 [N*K/64]; AWQ: FP16 [N][K >> gshift]
    const void* mins;       // AWQ: FP16 [N][K >> gshift]
    int gshift;             // AWQ: log2 of the group size
};

__device__ __forceinline__ uint32_t wo_pack(float a, float b) {
    const h16x2 v = {to_half(a), to_half(b)};
    return __builtin_bit_cast(uint32_t, v);
}

// Columns 8 slot .. 8 slot + 7 of weight row `row` as eight FP16 values. `book`:
// the NF4 code book in LDS (unused by the other formats). K % 8 == 0.
template <int kFmt>
__device__ __forceinline__ wo_u32x4 wo_slot(const WoSource& s, const float* book, size_t row, int K, int slot) {
    wo_u32x4 out;
    if constexpr (kFmt == kWoF16) {
        out = *(reinterpret_cast<const wo_u32x4*>(static_cast<const h16*>(s.w) + row * K) + slot);
    } else if constexpr (kFmt == kWoInt8) {
        const wo_u32x2 q = *(reinterpret_cast<const wo_u32x2*>(static_cast<const int8_t*>(s.w) + row * K) + slot);
        const float sc = static_cast<const float*>(s.scales)[row];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t word = p < 2 ? q.x : q.y;
            const int a = (int)(int8_t)(word >> (16 * (p & 1)));
            const int b = (int)(int8_t)(word >> (16 * (p & 1) + 8));
            out[p] = wo_pack((float)a * sc, (float)b * sc);
        }
    } else {
        const size_t first = row * K + (size_t)slot * 8;              // flat element index
        const uint32_t bits = static_cast<const uint32_t*>(s.w)[first >> 3];
        if constexpr (kFmt == kWoNf4) {
            const float sc = (float)static_cast<const h16*>(s.scales)[first >> 6];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t byte = (bits >> (8 * p)) & 0xFFu;
                out[p] = wo_pack(book[byte >> 4] * sc, book[byte & 15u] * sc);
            }
        } else {
            const size_t g = row * (size_t)(K >> s.gshift) + (size_t)((slot * 8) >> s.gshift);
            const float sc = (float)static_cast<const h16*>(s.scales)[g];
            const float mn = (float)static_cast<const h16*>(s.mins)[g];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t byte = (bits >> (8 * p)) & 0xFFu;
                // q * scale is exact in FP32 (4 x 11 bits): one rounding with or without the fusion
                out[p] = wo_pack(__builtin_fmaf((float)(byte >> 4), sc, mn), __builtin_fmaf((float)(byte & 15u), sc, mn));
            }
        }
    }
    return out;
}

}  // namespace vv
