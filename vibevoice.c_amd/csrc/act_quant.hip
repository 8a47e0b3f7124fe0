// Per-token int8 activation quantisers, alone and fused behind RMSNorm and
// SwiGLU: the front end of the W8A8 / W4A8 linear layers.
//
// Contract (include/vibevoice/device.h:298-317 of the reference): per row,
// sx = max|v| / 127 and xq = clamp(round-half-even(v * (127 / max|v|)), +-127),
// where v is THE FP16 VALUE THE UNFUSED OP WOULD HAVE WRITTEN, so a fused row
// is bit-identical to "op, then vv_act_quant_dev" and to the CPU quantiser on
// those values. That is obtained by construction: the FP16 value comes from the
// same inline functions (row_math.hpp), in the same thread-to-chunk mapping and
// reduction order, as vv_rmsnorm_dev and vv_swiglu_dev.
//
// Shape: one workgroup per row, one 16-byte chunk (8 columns) per thread, the
// FP16 row kept in registers from the op to the quantiser (no shared-memory
// copy of the row, no second read). Two workgroup reductions (sum of squares
// for the norm, absmax for the scale); four consecutive threads cover one run
// of 32 columns, so the per-run sum `xsum` is a DPP quad reduction. For the
// permuted layouts a thread's 8 bytes are placed through LDS inside its own
// quad, so the global store is one 8-byte coalesced store per thread in every
// layout.
#include "row_math.hpp"

namespace vv {
namespace {

enum QuantSrc : int { kQPlain = 0, kQNorm = 1, kQSwiglu = 2 };

constexpr int kMaxQuantK = 22528;   // VV_ACT_QUANT_MAX_K (device.h:312)
constexpr int kMinNormQuantK = 256; // VV_ACT_QUANT_MIN_K (device.h:314)

// Where column j (0..31) of a 32-column run is stored (q8.h:56-66 of the reference).
__device__ __forceinline__ int q8_pos(int layout, int j) {
    const int odd = j & 1, word = (j >> 1) & 3, slot = (j >> 3) + 4 * odd;
    switch (layout) {
        case 1:  return odd ? 16 + (j >> 1) : (j >> 1);           // nibble: evens, then odds
        case 2:  return 8 * word + 4 * (slot & 1) + (slot >> 1);  // W4 GEMV
        case 3:  return 16 * odd + 4 * word + (slot & 3);         // W4 MMA
        default: return j;
    }
}

// max |v| over the 8 halves of a chunk, in packed FP16 (exact: max and abs do
// not round): 4 masks + 3 v_pk_max_f16 instead of 8 conversions and 8 maxima.
__device__ __forceinline__ float chunk_absmax(const Chunk& c) {
    h16x2 m[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) m[i] = __builtin_bit_cast(h16x2, c.w[i] & 0x7FFF7FFFu);
    const h16x2 a = __builtin_elementwise_max(__builtin_elementwise_max(m[0], m[1]),
                                              __builtin_elementwise_max(m[2], m[3]));
    return fmaxf((float)a[0], (float)a[1]);
}

// Quantise one chunk: q_i = round-half-even(v_i * to_q), |q_i| <= 127 for every
// finite row (|v| <= amax and to_q = RN(127/amax) keep the product below 127.5).
// The product is rounded to FP32 first, as on the CPU, and the rounding to an
// integer is the FP32 addition of 1.5 * 2^23: its result carries q in its low
// mantissa bits (two's complement in the low byte), and subtracting the
// constant again gives q as an exact float for the per-run sum. No step may be
// fused into an FMA (that would remove the product's rounding).
__device__ __forceinline__ void quantise_chunk(const Chunk& h, float to_q, uint32_t& lo,
                                               uint32_t& hi, float& total) {
#pragma clang fp contract(off)
    constexpr float kRound = 12582912.0f;   // 1.5 * 2^23
    const f32x8 v = unpack(h);
    uint32_t bits[8];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float scaled = v[i] * to_q;
        const float shifted = scaled + kRound;
        bits[i] = __builtin_bit_cast(uint32_t, shifted);
        sum = sum + (shifted - kRound);
    }
    total = sum;
    // low byte of each of bits[0..3] -> lo, of bits[4..7] -> hi (v_perm_b32)
    const uint32_t p01 = __builtin_amdgcn_perm(bits[1], bits[0], 0x0c0c0400u);
    const uint32_t p23 = __builtin_amdgcn_perm(bits[3], bits[2], 0x0c0c0400u);
    const uint32_t p45 = __builtin_amdgcn_perm(bits[5], bits[4], 0x0c0c0400u);
    const uint32_t p67 = __builtin_amdgcn_perm(bits[7], bits[6], 0x0c0c0400u);
    lo = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
    hi = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
}

// One workgroup per row (kRows = 1 in every launch; several rows per workgroup
// were measured and bought nothing: these kernels are bound by instruction
// issue, not by loads in flight), kCpt chunks per thread.
template <int kCpt, int kRows, int kSrc, bool kStream>
__global__ __launch_bounds__(kMaxWgThreads) void quant_rows_wg(
    const Chunk* a_in, const Chunk* __restrict__ b_in, int rows, int nchunks, float inv_n,
    float eps, int layout, int8_t* __restrict__ xq, float* __restrict__ sx,
    int32_t* __restrict__ xsum) {
    __shared__ float partial_sum[kRows][kMaxWgWaves];
    __shared__ float partial_max[kRows][kMaxWgWaves];
    __shared__ __attribute__((aligned(8))) unsigned char stage[kMaxWgThreads * 8];

    const int t = (int)threadIdx.x;
    const int nthreads = (int)blockDim.x;
    const int row0 = (int)blockIdx.x * kRows;

    // ── the op: FP16 values h[][] exactly as the unfused kernel would store them ──
    Chunk h[kRows][kCpt], b[kRows][kCpt];
    bool live_row[kRows];
    size_t row_of[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        live_row[r] = kRows == 1 || row0 + r < rows;
        row_of[r] = (size_t)(live_row[r] ? row0 + r : rows - 1);   // a dead row re-reads the last one
        const size_t in_base = row_of[r] * (size_t)nchunks;
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            if (c < nchunks) {
                h[r][j] = load_chunk_as<kStream>(a_in + in_base + c);
                if (kSrc == kQNorm) b[r][j] = load_chunk(b_in + c);                        // weight
                if (kSrc == kQSwiglu) b[r][j] = load_chunk_as<kStream>(b_in + in_base + c);  // up
            }
        }
    }
    if (kSrc == kQNorm) {
        float acc[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            acc[r] = 0.0f;
#pragma unroll
            for (int j = 0; j < kCpt; ++j)
                if (j * nthreads + t < nchunks) acc[r] = chunk_sumsq(unpack(h[r][j]), acc[r]);
        }
        block_sum_n<kRows>(acc, partial_sum);
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            const float inv = inv_rms(acc[r], inv_n, eps);
#pragma unroll
            for (int j = 0; j < kCpt; ++j)
                if (j * nthreads + t < nchunks) h[r][j] = scale_chunk(h[r][j], inv, b[r][j]);
        }
    } else if (kSrc == kQSwiglu) {
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int j = 0; j < kCpt; ++j)
                if (j * nthreads + t < nchunks) h[r][j] = swiglu_chunk(h[r][j], b[r][j]);
    }

    // ── the scale: absmax over each row ──
    float amax[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        amax[r] = 0.0f;
#pragma unroll
        for (int j = 0; j < kCpt; ++j)
            if (j * nthreads + t < nchunks) amax[r] = fmaxf(amax[r], chunk_absmax(h[r][j]));
    }
    block_max_n<kRows>(amax, partial_max);

    // ── quantise, sum per run of 32, place, store ──
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        const float to_q = amax[r] > 0.0f ? 127.0f / amax[r] : 0.0f;   // correctly rounded
        if (t == 0 && live_row[r]) sx[row_of[r]] = amax[r] / 127.0f;    // divisions, as on the CPU
        int8_t* out_row = xq + row_of[r] * (size_t)nchunks * 8u;
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            const bool live = c < nchunks && live_row[r];   // a quad is live or dead as a whole
            uint32_t lo = 0, hi = 0;
            float run_part = 0.0f;
            if (c < nchunks) quantise_chunk(h[r][j], to_q, lo, hi, run_part);
            const int total = quad_sum((int)run_part);
            if (live && xsum && (t & 3) == 0)
                xsum[row_of[r] * (size_t)(nchunks >> 2) + (size_t)(c >> 2)] = total;
            if (layout != 0) {
                // Exchange inside the quad through LDS: byte i of this chunk is column
                // 8*(t&3)+i of its run and belongs at q8_pos of that; then each thread
                // takes back the 8 consecutive bytes it will store. Same wave, in-order
                // LDS queue: no barrier.
                unsigned char* run = stage + (t >> 2) * 32;
                const int j0 = (t & 3) * 8;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t word = i < 4 ? lo : hi;
                    run[q8_pos(layout, j0 + i)] = (unsigned char)(word >> (8 * (i & 3)));
                }
                const uint2 placed = *reinterpret_cast<const uint2*>(stage + t * 8);
                lo = placed.x;
                hi = placed.y;
            }
            if (live) {
                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                const u32x2 v = {lo, hi};
                u32x2* dst = reinterpret_cast<u32x2*>(out_row + (size_t)c * 8u);
                if (kStream) __builtin_nontemporal_store(v, dst);
                else *dst = v;
            }
        }
    }
}

// ── RMSNorm + quantise for rows of at most 512 chunks: one wave per row ───
// The quantiser's arithmetic is fixed cost per THREAD (two reductions, two
// divisions, addressing) plus ~10 VALU operations per element, against only
// 3 bytes of traffic per element: with one chunk per thread the kernel is
// bound by instruction issue, not by HBM (46.8 us at 14449 x 3584, the plain
// quantiser 35.5 us against 27.9 us with four chunks per thread). Here a lane
// holds kCpl chunks — chunk j*64 + lane, exactly the chunk that lane `lane` of
// wave j holds in vv_rmsnorm_dev's workgroup — so the sum of squares can be
// formed in vv_rmsnorm_dev's order (per chunk, then the same DPP tree per group
// of 64 chunks, then the groups in order) without LDS or barriers, and the FP16
// values stay bit-identical to the unfused op's.
template <int kCpl, bool kStream>
__global__ __launch_bounds__(kBlock) void quant_norm_wave(
    const Chunk* __restrict__ x, const Chunk* __restrict__ weight, int rows, int nchunks,
    float inv_n, float eps, int layout, int8_t* __restrict__ xq, float* __restrict__ sx,
    int32_t* __restrict__ xsum) {
    __shared__ __attribute__((aligned(8))) unsigned char stage[kWavesPerBlock][kWave * 8];
    const int wave = wave_in_block();
    const int row = (int)blockIdx.x * kWavesPerBlock + wave;
    if (row >= rows) return;
    const int lane = lane_id();
    const size_t in_base = (size_t)row * (size_t)nchunks;

    Chunk h[kCpl], w[kCpl];
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (c < nchunks) {
            h[j] = load_chunk_as<kStream>(x + in_base + c);
            w[j] = load_chunk(weight + c);
        }
    }
    float total = 0.0f;
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        const float acc = c < nchunks ? chunk_sumsq(unpack(h[j]), 0.0f) : 0.0f;
        total += wave_sum(acc);          // group j = wave j of the unfused kernel, added in order
    }
    const float inv = inv_rms(total, inv_n, eps);
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        if (j * kWave + lane < nchunks) {
            h[j] = scale_chunk(h[j], inv, w[j]);
            amax = fmaxf(amax, chunk_absmax(h[j]));
        }
    }
    amax = wave_max(amax);
    const float to_q = amax > 0.0f ? 127.0f / amax : 0.0f;
    if (lane == 0) sx[row] = amax / 127.0f;

    int8_t* out_row = xq + (size_t)row * (size_t)nchunks * 8u;
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        const bool live = c < nchunks;
        uint32_t lo = 0, hi = 0;
        float run_part = 0.0f;
        if (live) quantise_chunk(h[j], to_q, lo, hi, run_part);
        const int total_q = quad_sum((int)run_part);
        if (live && xsum && (lane & 3) == 0)
            xsum[(size_t)row * (size_t)(nchunks >> 2) + (size_t)(c >> 2)] = total_q;
        if (layout != 0) {               // place the bytes inside the quad through LDS (see above)
            unsigned char* run = stage[wave] + (lane >> 2) * 32;
            const int j0 = (lane & 3) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t word = i < 4 ? lo : hi;
                run[q8_pos(layout, j0 + i)] = (unsigned char)(word >> (8 * (i & 3)));
            }
            const uint2 placed = *reinterpret_cast<const uint2*>(stage[wave] + lane * 8);
            lo = placed.x;
            hi = placed.y;
        }
        if (live) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const u32x2 v = {lo, hi};
            u32x2* dst = reinterpret_cast<u32x2*>(out_row + (size_t)c * 8u);
            if (kStream) __builtin_nontemporal_store(v, dst);
            else *dst = v;
        }
    }
}

vv_status_t check_args(int M, int K, const void* a, const void* b, bool need_b, const int8_t* xq,
                       const float* sx, int layout) {
    if (!a || !xq || !sx || (need_b && !b)) return VV_ERR_NULL_PTR;
    if (M <= 0 || K <= 0) return VV_ERR_INVALID_ARG;
    if ((K & 31) != 0 || K > kMaxQuantK) return VV_ERR_UNSUPPORTED;
    if (layout < 0 || layout > 3) return VV_ERR_INVALID_ARG;
    // vector accesses: 16-byte aligned inputs, 8-byte aligned output
    if (!aligned16(a) || (need_b && !aligned16(b)) || (reinterpret_cast<uintptr_t>(xq) & 7u))
        return VV_ERR_UNSUPPORTED;
    return VV_OK;
}

template <int kSrc>
vv_status_t launch_quant(const void* a, const void* b, int M, int K, float eps, int layout,
                         int8_t* xq, float* sx, int32_t* xsum, hipStream_t st) {
    const int nchunks = K / 8;
    static const bool light_norm = getenv("VV_Q8_LIGHT_NORM") != nullptr;   // A/B switch, read once
    if (kSrc == kQNorm && nchunks <= 8 * kWave && !light_norm) {
        const float inv_k = 1.0f / (float)K;
        const bool nt = use_streaming((size_t)M * (size_t)K * 3u);
        const dim3 g((unsigned)((M + kWavesPerBlock - 1) / kWavesPerBlock));
        const Chunk* px = static_cast<const Chunk*>(a);
        const Chunk* pw = static_cast<const Chunk*>(b);
#define VV_QN(C)                                                                                  \
    case C:                                                                                       \
        if (nt) quant_norm_wave<C, true><<<g, kBlock, 0, st>>>(px, pw, M, nchunks, inv_k, eps, layout, \
                                                               xq, sx, xsum);                     \
        else quant_norm_wave<C, false><<<g, kBlock, 0, st>>>(px, pw, M, nchunks, inv_k, eps, layout,   \
                                                             xq, sx, xsum);                       \
        break;
        switch ((nchunks + kWave - 1) / kWave) {
            VV_QN(1) VV_QN(2) VV_QN(3) VV_QN(4) VV_QN(5) VV_QN(6) VV_QN(7) VV_QN(8)
        }
#undef VV_QN
        return launch_status();
    }
    // chunks per thread: VV_Q8_CPT forces (A/B aid), else the smallest that fits 1024 threads
    static const int forced_cpt = getenv("VV_Q8_CPT") ? atoi(getenv("VV_Q8_CPT")) : 0;
    int cpt = (nchunks + kMaxWgThreads - 1) / kMaxWgThreads;            // 1..3
    // Without a reduction inside the op the mapping is free: four chunks per thread
    // amortise the per-thread cost (plain quantiser 35.5 -> 27.9 us at 14449 x 3584).
    // The fused norm must keep vv_rmsnorm_dev's mapping (same summation order).
    if (kSrc == kQPlain && cpt < 4 && nchunks >= 4 * kWave) cpt = 4;
    if (forced_cpt > cpt && kSrc != kQNorm) cpt = forced_cpt;
    if (cpt == 5 || cpt == 6) cpt = 7;
    if (cpt > 8) cpt = 8;
    const int threads = ((nchunks + cpt - 1) / cpt + kWave - 1) / kWave * kWave;
    const float inv_n = 1.0f / (float)K;
    const size_t in_tensors = kSrc == kQSwiglu ? 2 : 1;
    const bool stream = use_streaming((size_t)M * (size_t)K * (in_tensors * 2u + 1u));
    const Chunk* pa = static_cast<const Chunk*>(a);
    const Chunk* pb = static_cast<const Chunk*>(b);
    const dim3 grid((unsigned)M);
#define VV_Q_LAUNCH(C, R, S)                                                                   \
    quant_rows_wg<C, R, kSrc, S><<<grid, threads, 0, st>>>(pa, pb, M, nchunks, inv_n, eps, layout, \
                                                          xq, sx, xsum)
#define VV_Q_PICK(C, R) do { if (stream) VV_Q_LAUNCH(C, R, true); else VV_Q_LAUNCH(C, R, false); } while (0)
    switch (cpt) {
        case 1: VV_Q_PICK(1, 1); break;
        case 2: VV_Q_PICK(2, 1); break;
        case 3: VV_Q_PICK(3, 1); break;
        case 4: VV_Q_PICK(4, 1); break;
        case 7: VV_Q_PICK(7, 1); break;
        default: VV_Q_PICK(8, 1); break;
    }
#undef VV_Q_PICK
#undef VV_Q_LAUNCH
    return launch_status();
}

// acc[k] = max(acc[k], max_m |x[m,k]|): one thread per column, rows split over
// blockIdx.y; non-negative floats order like their bit patterns, so the running
// maximum is an unsigned atomic max (exact in any order).
__global__ __launch_bounds__(kBlock) void col_absmax_kernel(const h16* __restrict__ x, int M, int K,
                                                            float* acc, int rows_per_group) {
    const int k = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (k >= K) return;
    const int m0 = (int)blockIdx.y * rows_per_group;
    const int m1 = min(M, m0 + rows_per_group);
    float best = 0.0f;
    for (int m = m0; m < m1; ++m) best = fmaxf(best, fabsf((float)x[(size_t)m * (size_t)K + k]));
    atomicMax(reinterpret_cast<unsigned int*>(acc) + k, __float_as_uint(best));
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_act_quant_dev(const void* x, int M, int K, int layout, int8_t* xq, float* sx,
                             int32_t* xsum, void* stream) {
    const vv_status_t s = vv::check_args(M, K, x, nullptr, false, xq, sx, layout);
    if (s != VV_OK) return s;
    return vv::launch_quant<vv::kQPlain>(x, nullptr, M, K, 0.0f, layout, xq, sx, xsum,
                                         vv::as_stream(stream));
}

vv_status_t vv_rmsnorm_q8_dev(const void* x, const void* weight, int M, int K, float eps,
                              int layout, int8_t* xq, float* sx, int32_t* xsum, void* stream) {
    const vv_status_t s = vv::check_args(M, K, x, weight, true, xq, sx, layout);
    if (s != VV_OK) return s;
    if (K < vv::kMinNormQuantK) return VV_ERR_UNSUPPORTED;
    return vv::launch_quant<vv::kQNorm>(x, weight, M, K, eps, layout, xq, sx, xsum,
                                        vv::as_stream(stream));
}

vv_status_t vv_swiglu_q8_dev(const void* gate, const void* up, int M, int K, int layout,
                             int8_t* xq, float* sx, int32_t* xsum, void* stream) {
    const vv_status_t s = vv::check_args(M, K, gate, up, true, xq, sx, layout);
    if (s != VV_OK) return s;
    return vv::launch_quant<vv::kQSwiglu>(gate, up, M, K, 0.0f, layout, xq, sx, xsum,
                                          vv::as_stream(stream));
}

vv_status_t vv_col_absmax_dev(const void* x, int M, int K, float* acc, void* stream) {
    if (!x || !acc) return VV_ERR_NULL_PTR;
    if (M <= 0 || K <= 0) return VV_ERR_INVALID_ARG;
    const int groups = M < 64 ? 1 : (M + 63) / 64 > 1024 ? 1024 : (M + 63) / 64;
    const int rows_per_group = (M + groups - 1) / groups;
    const dim3 grid((unsigned)((K + vv::kBlock - 1) / vv::kBlock), (unsigned)groups);
    vv::col_absmax_kernel<<<grid, vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<const vv::h16*>(x), M, K, acc, rows_per_group);
    return vv::launch_status();
}

}  // extern "C"
