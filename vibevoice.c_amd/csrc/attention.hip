// Causal grouped-query attention over an FP16 KV cache: the prefill form
// (q_len rows against the first kv_len positions) and the decode form (one
// row per head against the whole cache), plus the FP16 cache store.
//
// Q, O are [rows][n_q_heads][head_dim]; the cache is [row][n_kv_heads]
// [head_dim], row = position, or, with a page table, page_table[t / 64] * 64
// + t % 64. Every kernel keeps the softmax online (running maximum and
// denominator in FP32, in the base-2 domain: v_exp_f32 is 2^x).
//
//   prefill128   head_dim 128 on the matrix cores. A workgroup owns 128
//                query rows of one head, a wave 32 of them; keys come in
//                tiles of 64 through LDS. The products are computed
//                TRANSPOSED: S^T = K Q^T puts one query row in each lane
//                (lane % 32) with 32 of the tile's keys in its registers, so
//                the row maximum and sum are register reductions plus one
//                exchange with lane ^ 32, the rescale of O is one factor per
//                lane, and the probabilities, rounded to FP16, are already
//                laid out as the B operand of O^T = V^T P^T. V is transposed
//                on its way into LDS (four keys of one channel per 8-byte
//                slot) so the A operand of that product is two 8-byte reads.
//   decode128    one query row per head: bound by the cache bytes. The same
//                pieces with the query heads that share a KV head in the
//                place of the query rows, so a slice of K and V is read once
//                for the whole group; one wave per (slice, KV head). Slices
//                leave (max, sum, unnormalised O) in the caller's scratch
//                and decode_merge folds them.
//   rows_generic any head_dim <= 256, any alignment: one wave per (row, head).
#include <algorithm>
#include <atomic>

#include "vv_common.hpp"

namespace vv {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef h16 h16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kPage = 64;            // positions per page (include/vibevoice/kv_quant.h:52)
constexpr int kFormatFp16 = 0;       // VV_KV_FP16
constexpr int kMaxParts = 256;       // decode slices per KV head
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
// The slack of a row's reference exponent below its running maximum, in base-2 exponents (RowState).
constexpr float kMaxSlack = 8.0f;
// A value and its partner's, 32 (or 16) lanes away, combined in the vector ALU: the gfx950 lane swaps exchange
// the odd rows of one register with the even rows of another (rows of 32 or 16 lanes), so from two copies of v
// one register ends up with the lower row's values in both rows of a pair and the other with the upper row's.
// No trip through the LDS crossbar and no counter to wait for; max and + commute, so every lane gets the bits
// that v (op) shuffle-xor(v) gave it. (As instructions: the compiler's builtin for them hands back the first
// register twice. The two wait states are what it puts between a vector write and a swap that reads it.)
__device__ __forceinline__ void swap_rows32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float max_xor32(float v) {
    float a = v, b = v;
    swap_rows32(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float sum_xor32(float v) {
    float a = v, b = v;
    swap_rows32(a, b);
    return a + b;
}
__device__ __forceinline__ float max_xor16(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float sum_xor16(float v) {
    float a = v, b = v;
    swap_rows16(a, b);
    return a + b;
}

__device__ __forceinline__ int cache_row(const int* page_table, int t) {
    return page_table ? page_table[t / kPage] * kPage + t % kPage : t;
}

// ── head_dim 128 on the matrix cores: the pieces both forms share ─────────
constexpr int kD = 128;
constexpr int kPartFloats = kD + 4;        // a partial state: 128 channels, max, sum, 2 unused (16-byte rows)
constexpr int kPrefillSplitRows = 2048;    // (rows x key runs) of a split prefill the caller's scratch holds per query head
constexpr int kQTile = 128;          // query rows per prefill workgroup (32 per wave)
constexpr int kKeyTile = 64;         // keys per LDS tile
constexpr int kVtStride = kKeyTile + 4;   // halves per transposed-V row: 136 B

struct KvTile {
    Chunk k[kKeyTile * (kD / 8)];                 // [key][16 slots], slot ^ (key & 15)
    __align__(16) h16 vt[kD * kVtStride];         // [channel][key]
    float lev[16];                                // TurboQuant caches: the format's level table
};

// Per-lane state of one query row (lane % 32) over the keys seen so far: O^T register 4g + r of tile t is
// channel 32t + 8g + 4*(lane / 32) + r. o and l are on the scale 2^-m_use, and l is THIS LANE's share of the
// row's sum (its keys of every tile; the two halves of a wave are added once, at the end: row_sum).
// The reference exponent m_use of the online softmax need not be the running maximum: with any value not far
// below it the probabilities stay inside FP16 and the FP32 sums, and the quotient O / l does not depend on it. So
// a tile's probabilities are formed with the reference AS IT STANDS, with no look at the tile's maximum, and each
// lane compares the sum of its 32 against a bar (thr): none of them can be larger than their sum. Only where a
// sum passes the bar - or a row has seen no key yet (thr < 0: any sum passes) - are the rows' maxima taken and
// exchanged, the reference moved up where a row's maximum is more than kMaxSlack above it, O and l rescaled, and
// the tile's probabilities formed again (settle; the raw scores are still there). After a row's first tile that
// almost never happens, where a reference that follows the maximum moves in nearly half of all tiles on random
// scores (some one of a wave's 32 rows finds a new maximum): a tile costs no maximum, no exchange between lanes
// and no arithmetic on the state. A row's rule depends on that row's scores alone.
constexpr float kSumBar = 32768.0f;               // 2^15: a lane's 32 probabilities of a tile, each below FP16's 65504
struct RowState {
    f32x16 o[kD / 32];
    float thr, m_use, l;                          // thr < 0: the row has seen no key (then m_use = 0), else kSumBar
    __device__ __forceinline__ void reset() {
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[t][r] = 0.0f;
        thr = -1.0f;
        m_use = 0.0f;
        l = 0.0f;
    }
    // mx: this lane's raw maximum of the tile at hand. Called by the whole wave.
    __device__ __forceinline__ void settle(float mx, float scale_log2) {
        mx = max_xor32(mx);
        const bool unseen = thr < 0.0f;
        const float top = mx * scale_log2;
        const bool moves = unseen ? mx > -INFINITY : top > m_use + kMaxSlack;
        const float use = moves ? top : m_use;
        const float alpha = unseen ? 0.0f : exp2_fast(m_use - use);                   // exactly 1 where nothing moves
        l *= alpha;
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
        m_use = use;
        thr = unseen && !moves ? -1.0f : kSumBar;
    }
    __device__ __forceinline__ float reference() const { return thr < 0.0f ? -INFINITY : m_use; }
    __device__ __forceinline__ float row_sum() const { return sum_xor32(l); }
};
// A lane's 32 scores of a tile -> probabilities on the reference m_use, rounded to FP16 two per conversion
// (v_cvt_pk_f16_f32) into the B operand's slots (score q of the tile: slot q % 8 of key step q / 8), and their
// FP32 sum in this order.
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void probabilities(const f32x16 (&s)[2], float scale_log2, float m_use, h16x8 (&pf)[4],
                                              float& sum) {
    sum = 0.0f;
#pragma unroll
    for (int q = 0; q < 32; q += 2) {
        const f32x2 two = {exp2_fast(fmaf(s[q >> 4][q & 15], scale_log2, -m_use)),
                           exp2_fast(fmaf(s[q >> 4][(q & 15) + 1], scale_log2, -m_use))};
        sum += two[0];
        sum += two[1];
        const h16x2 h = __builtin_convertvector(two, h16x2);
        pf[q >> 3][q & 7] = h[0];
        pf[q >> 3][(q & 7) + 1] = h[1];
    }
}
__device__ __forceinline__ float lane_max(const f32x16 (&s)[2]) {
    float mx = -INFINITY;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[a][r]);
    return mx;
}

// Keys t0 .. t0+63 of KV head kvh, first into registers (fetch: issued a tile
// ahead, so the loads fly while the previous tile is computed), then into LDS
// (commit). Rows past last_key repeat it: they are masked, but must hold finite
// values. K keeps its layout; V is transposed: a thread takes four consecutive
// keys of one 8-channel chunk and writes, per channel, the four keys as 8 bytes.
template <int kThreads>
struct TileRegs {
    static constexpr int kIter = kKeyTile * (kD / 8) / kThreads;   // chunks per thread, K and V each
    Chunk k[kIter], v[kIter];
};

// Cache formats the matrix-core kernels read (include/vibevoice/kv_quant.h:34-36).
// The FP8 ones are widened to FP16 on their way into the registers: every
// E4M3 / E5M2 value is an FP16 value, so from there on the tile is the tile of
// an FP16 cache that holds the decoded values.
constexpr int kFmtFp16 = 0, kFmtE4M3 = 1, kFmtE5M2 = 2;
// TurboQuant (kv_quant.h:37-40): 4, 3, 2 or 1.5 bits per value as one little-endian
// bit stream per vector, value d at bit d * bits (pair P at bit 3 P for 1.5 bits),
// each code an index into a table of Lloyd-Max levels of a unit Gaussian, times
// the vector's own RMS (FP16, one per vector, beside the store). The vectors are
// stored rotated; the caller rotates Q and un-rotates O (vv_kv_rotate_dev).
constexpr int kFmtTq4 = 3, kFmtTq3 = 4, kFmtTq2 = 5, kFmtTq15 = 6;

__device__ const float kTqLevels[4][16] = {
    {-2.725112f, -2.065280f, -1.613787f, -1.251845f, -0.938657f, -0.654379f, -0.386970f, -0.127960f,
     +0.127960f, +0.386970f, +0.654379f, +0.938657f, +1.251845f, +1.613787f, +2.065280f, +2.725112f},
    {-2.150300f, -1.343258f, -0.755588f, -0.244756f, +0.244756f, +0.755588f, +1.343258f, +2.150300f},
    {-1.511418f, -0.452456f, +0.452456f, +1.511418f},
    // 1.5 bits: eight 2-D code words, a pair of values shares one 3-bit index
    {-1.500251f, +0.674678f, -1.127883f, -0.787015f, -0.283251f, +0.390133f, -0.103102f, +1.624620f,
     +0.100120f, -1.618563f, +0.286482f, -0.379555f, +1.134227f, +0.790368f, +1.496572f, -0.666578f}};

template <int kFmt> struct KvFormat {
    static constexpr bool kTq = kFmt >= kFmtTq4;
    // bytes per 128-value vector; bits one 8-channel slot takes; bits per code; values per code
    static constexpr int kBytes = kFmt == kFmtFp16 ? 256 : kFmt <= kFmtE5M2 ? 128
                                : kFmt == kFmtTq4 ? 64 : kFmt == kFmtTq3 ? 48 : kFmt == kFmtTq2 ? 32 : 24;
    static constexpr int kCodeBits = kFmt == kFmtTq4 ? 4 : kFmt == kFmtTq2 ? 2 : 3;
    static constexpr int kPerCode = kFmt == kFmtTq15 ? 2 : 1;
    static constexpr int kSlotBits = 8 / kPerCode * kCodeBits;
};

// Four FP8 codes (the bytes of `codes`) as two half2 words, lanes in byte order.
template <int kFmt>
__device__ __forceinline__ void widen4(uint32_t codes, uint32_t& lo, uint32_t& hi) {
    // byte b -> 16-bit lane b << 8: an E5M2 code IS the top byte of the FP16 value
    lo = __builtin_amdgcn_perm(0u, codes, 0x010C000Cu);
    hi = __builtin_amdgcn_perm(0u, codes, 0x030C020Cu);
    if constexpr (kFmt == kFmtE4M3) {
        // sign stays, exponent and mantissa move down one bit (FP16 has five exponent bits):
        // that reads 2^-8 too small (bias 15 against 7), subnormals included, so scale by 256
        typedef h16 h16x2v __attribute__((ext_vector_type(2)));
        const h16x2v k256 = {(h16)256.0f, (h16)256.0f};
        const uint32_t l = ((lo >> 1) & 0x3F803F80u) | (lo & 0x80008000u);
        const uint32_t h = ((hi >> 1) & 0x3F803F80u) | (hi & 0x80008000u);
        lo = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2v, l) * k256);
        hi = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2v, h) * k256);
    }
}

// `count` bits at bit `offset` of a vector of `nwords` 32-bit words.
__device__ __forceinline__ uint32_t stream_bits(const uint32_t* __restrict__ words, int nwords, int offset,
                                                int count) {
    const int wi = offset >> 5, sh = offset & 31;
    const uint32_t lo = words[wi], hi = words[min(wi + 1, nwords - 1)];
    const uint32_t v = sh ? ((lo >> sh) | (hi << (32 - sh))) : lo;
    return count == 32 ? v : v & ((1u << count) - 1u);
}

// The eight channels of slot `slot` of a TurboQuant vector in FP32: RMS times level.
template <int kFmt>
__device__ __forceinline__ void tq_slot_values(const void* __restrict__ cache, const h16* __restrict__ meta,
                                               const float* lev, size_t vec, int slot, float (&val)[8]) {
    typedef KvFormat<kFmt> F;
    const uint32_t* words = reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(cache) + vec * F::kBytes);
    const uint32_t bits = stream_bits(words, F::kBytes / 4, slot * F::kSlotBits, F::kSlotBits);
    const float sigma = (float)meta[vec];
#pragma unroll
    for (int c = 0; c < 8 / F::kPerCode; ++c) {
        const uint32_t code = (bits >> (F::kCodeBits * c)) & ((1u << F::kCodeBits) - 1u);
        if constexpr (F::kPerCode == 1) {
            val[c] = sigma * lev[code];
        } else {
            val[2 * c] = sigma * lev[2 * code];
            val[2 * c + 1] = sigma * lev[2 * code + 1];
        }
    }
}

// Slot `slot` (eight channels) of vector `vec` (= cache row * n_kv_heads + KV head) as FP16.
// `meta` (per-vector RMS) and `lev` (the level table, in LDS) serve the TurboQuant formats.
template <int kFmt>
__device__ __forceinline__ Chunk load_slot(const void* __restrict__ cache, const h16* __restrict__ meta,
                                           const float* lev, size_t vec, int slot) {
    if constexpr (kFmt == kFmtFp16) {
        return load_chunk(static_cast<const Chunk*>(cache) + vec * (kD / 8) + slot);
    } else if constexpr (KvFormat<kFmt>::kTq) {
        float val[8];
        tq_slot_values<kFmt>(cache, meta, lev, vec, slot, val);
        h16x8 out;
#pragma unroll
        for (int c = 0; c < 8; ++c) out[c] = to_half(val[c]);
        return __builtin_bit_cast(Chunk, out);
    } else {
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
        const u32x2 codes = *(static_cast<const u32x2*>(cache) + vec * (kD / 8) + slot);
        u32x4v w;
        uint32_t a, b, c, d;
        widen4<kFmt>(codes.x, a, b);
        widen4<kFmt>(codes.y, c, d);
        w.x = a; w.y = b; w.z = c; w.w = d;
        return __builtin_bit_cast(Chunk, w);
    }
}

struct KvSource {
    const void* k;
    const void* v;
    const h16* k_meta;
    const h16* v_meta;
    const int* page_table;
};

// The format's level table into the tile (TurboQuant only); every thread of the workgroup calls it.
template <int kFmt>
__device__ __forceinline__ void load_levels(KvTile& tile, int tid) {
    if constexpr (KvFormat<kFmt>::kTq) {
        if (tid < 16) tile.lev[tid] = kTqLevels[kFmt - kFmtTq4][tid];
        __syncthreads();
    }
}

template <int kThreads, int kFmt>
__device__ __forceinline__ void fetch_tile(TileRegs<kThreads>& regs, const KvSource& src, const float* lev,
                                           int n_kv_heads, int kvh, int t0, int last_key, int tid) {
    const void* __restrict__ Kc = src.k;
    const void* __restrict__ Vc = src.v;
    const int* __restrict__ page_table = src.page_table;
    constexpr int kIter = TileRegs<kThreads>::kIter;
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
        const int q = tid + i * kThreads, r = q >> 4, slot = q & 15;
        const int row = cache_row(page_table, min(t0 + r, last_key));
        regs.k[i] = load_slot<kFmt>(Kc, src.k_meta, lev, (size_t)row * n_kv_heads + kvh, slot);
    }
#pragma unroll
    for (int i = 0; i < kIter / 4; ++i) {
        const int q = tid + i * kThreads, dchunk = q & 15, kg = q >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = cache_row(page_table, min(t0 + 4 * kg + j, last_key));
            regs.v[4 * i + j] = load_slot<kFmt>(Vc, src.v_meta, lev, (size_t)row * n_kv_heads + kvh, dchunk);
        }
    }
}

template <int kThreads>
__device__ __forceinline__ void commit_tile(KvTile& tile, const TileRegs<kThreads>& regs, int tid) {
    constexpr int kIter = TileRegs<kThreads>::kIter;
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
        const int q = tid + i * kThreads, r = q >> 4, slot = q & 15;
        tile.k[r * 16 + (slot ^ (r & 15))] = regs.k[i];
    }
#pragma unroll
    for (int i = 0; i < kIter / 4; ++i) {
        const int q = tid + i * kThreads, dchunk = q & 15, kg = q >> 4;
        h16x8 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = __builtin_bit_cast(h16x8, regs.v[4 * i + j]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const h16x4 w = {v[0][e], v[1][e], v[2][e], v[3][e]};
            *reinterpret_cast<h16x4*>(&tile.vt[(8 * dchunk + e) * kVtStride + 4 * kg]) = w;
        }
    }
}

// S^T = K Q^T for the tile: register 4g + r of s[a] is key 32a + 8g + 4*half + r
// of the tile, for this lane's query row.
__device__ __forceinline__ void tile_scores(const KvTile& tile, const h16x8 (&qf)[kD / 16],
                                            int col, int half, f32x16 (&s)[2]) {
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[a][r] = 0.0f;
#pragma unroll
        for (int st = 0; st < kD / 16; ++st) {
            const int row = 32 * a + col, slot = 2 * st + half;
            const h16x8 kf = __builtin_bit_cast(h16x8, tile.k[row * 16 + (slot ^ (row & 15))]);
            s[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[st], s[a], 0, 0, 0);
        }
    }
}

// s holds the raw scores (-inf where unseen); scale_log2 = log2(e) / sqrt(d) > 0
// turns them into base-2 exponents inside one fused multiply-add per value.
// Online-softmax update of the row state, then O^T += V^T P^T over the tile's
// four 16-key steps. Slot e of this lane in step (a, sp) is register 8*sp + e
// of s[a], i.e. key 32a + 16sp + 8(e / 4) + 4*half + e % 4: the two 8-byte
// reads of V^T below. O is rescaled only when some row's reference exponent
// moves (RowState::settle).
__device__ __forceinline__ void tile_update(const KvTile& tile, const f32x16 (&s)[2], RowState& st,
                                            int col, int half, float scale_log2) {
    h16x8 pf[4];
    float sum;
    probabilities(s, scale_log2, st.m_use, pf, sum);
    if (__builtin_amdgcn_ballot_w64(sum > st.thr) != 0) {
        st.settle(lane_max(s), scale_log2);
        probabilities(s, scale_log2, st.m_use, pf, sum);
    }
    st.l += sum;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int a = u >> 1, sp = u & 1;
#pragma unroll
        for (int t = 0; t < kD / 32; ++t) {
            const h16* base = &tile.vt[(32 * t + col) * kVtStride + 32 * a + 16 * sp + 4 * half];
            const h16x4 lo = *reinterpret_cast<const h16x4*>(base);
            const h16x4 hi = *reinterpret_cast<const h16x4*>(base + 8);
            const h16x8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            st.o[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[u], st.o[t], 0, 0, 0);
        }
    }
}

__device__ __forceinline__ void load_query(h16x8 (&qf)[kD / 16], const h16* qp, int half) {
#pragma unroll
    for (int s = 0; s < kD / 16; ++s)
        qf[s] = __builtin_bit_cast(h16x8, load_chunk(reinterpret_cast<const Chunk*>(qp) + 2 * s + half));
}

// ── prefill ──────────────────────────────────────────────────────────────
template <int kFmt>
__global__ __launch_bounds__(kBlock, 2) void prefill128(
    const h16* __restrict__ Q, KvSource src, h16* __restrict__ O, int n_q_heads, int n_kv_heads,
    int q_len, int q_offset, int kv_len, int causal, float scale_log2) {
    __shared__ KvTile tile;

    const int tid = (int)threadIdx.x;
    load_levels<kFmt>(tile, tid);
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;        // this lane's query row inside the wave's 32
    const int half = lane >> 5;
    const int head = (int)blockIdx.y;
    const int kvh = head / (n_q_heads / n_kv_heads);
    // Causal rows late in the prompt see the most keys: launch those first.
    const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * kQTile;
    const int qw0 = q0 + wave * 32;
    const int qrow = qw0 + col;
    const int q_abs = q_offset + qrow;

    // Keys any row of the workgroup / of this wave may see.
    int wg_limit = kv_len, wave_limit = qw0 < q_len ? kv_len : 0;
    if (causal) {
        wg_limit = min(kv_len, q_offset + min(q0 + kQTile, q_len));
        wave_limit = qw0 < q_len ? min(kv_len, q_offset + min(qw0 + 32, q_len)) : 0;
    }

    h16x8 qf[kD / 16];
    load_query(qf, Q + ((size_t)min(qrow, q_len - 1) * n_q_heads + head) * kD, half);
    RowState st;
    st.reset();

    TileRegs<kBlock> regs;
    if (wg_limit > 0) fetch_tile<kBlock, kFmt>(regs, src, tile.lev, n_kv_heads, kvh, 0, kv_len - 1, tid);
    for (int t0 = 0; t0 < wg_limit; t0 += kKeyTile) {
        __syncthreads();
        commit_tile<kBlock>(tile, regs, tid);
        __syncthreads();
        if (t0 + kKeyTile < wg_limit)
            fetch_tile<kBlock, kFmt>(regs, src, tile.lev, n_kv_heads, kvh, t0 + kKeyTile, kv_len - 1, tid);
        if (t0 >= wave_limit) continue;
        f32x16 s[2];
        tile_scores(tile, qf, col, half, s);
        // Only a tile that reaches past the cache end or past the wave's first
        // row's position has anything to hide.
        if (t0 + kKeyTile > kv_len || (causal && t0 + kKeyTile - 1 > q_offset + qw0)) {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = t0 + 32 * a + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool seen = key < kv_len && (!causal || key <= q_abs);
                    s[a][r] = seen ? s[a][r] : -INFINITY;
                }
        }
        tile_update(tile, s, st, col, half, scale_log2);
    }

    if (qrow < q_len) {
        const float l_row = st.row_sum();
        const float inv = l_row > 0.0f ? 1.0f / l_row : 0.0f;
        h16* op = O + ((size_t)qrow * n_q_heads + head) * kD;
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = to_half(st.o[t][4 * g + r] * inv);
                *reinterpret_cast<h16x4*>(op + 32 * t + 8 * g + 4 * half) = o;
            }
    }
}

// ── prefill over an FP16 cache, head_dim 128: the same arithmetic as prefill128, pipelined ─────
// A wave issues in order, so a tile done as "all the score MFMAs, then the softmax, then all the
// O MFMAs" leaves the matrix pipe idle through the softmax and the vector ALU idle through the
// MFMAs; measured, the softmax of a tile costs about what its 32 MFMAs cost. Here the loop is
// skewed by one tile: while the vector ALU turns tile j's scores into probabilities, the matrix
// pipe computes tile j + 1's scores, a slice of the one issued behind each MFMA of the other; then
// the O^T += V^T P^T MFMAs of tile j run. K and V both go from global memory straight into LDS, row
// major as they lie in the cache (two buffers each, no registers, no commit, one barrier per tile):
// the V^T operand is transposed on its way OUT of LDS (ds_read_b64_tr_b16: four keys of sixteen
// channels per group of sixteen lanes, two reads per fragment), which takes the tile's transposition -
// four loads, sixteen byte permutes and eight LDS writes per thread and tile - off the vector ALU
// that bounds this kernel (1812 -> 1691 us at 14449 rows). A key's 64-byte quarters rotate with the
// key, so the four keys of a transposing read lie in four quarters of the banks. A lane multiplies
// the keys in the order in which its probabilities leave the score MFMAs. The values and their order
// of summation are those of prefill128: the same bits.
// The loop is unrolled by two so that the buffers are compile-time constants (LDS addresses are a
// per-lane offset plus an immediate) and the two score sets swap roles without a copy; contiguous
// caches are addressed as a uniform base per tile plus a per-lane offset that never changes; the
// probabilities are converted two at a time. What is left is bound by the vector ALU: about 180
// vector instructions and 33 exponentials per tile and wave against 32 MFMAs. The softmax block runs
// at a higher wave priority than the V^T P^T block (the SIMD's other wave belongs to the compute
// unit's other workgroup and is in any phase to this one), and the two exchanges between the halves
// of a wave are lane swaps in the vector ALU (max_xor32, sum_xor32); the row maximum of the next tile
// is taken behind the first V^T P^T MFMAs, so that the exponentials spread over all sixteen score
// MFMAs: 1691 -> 1501 us together.
// Workgroups are ordered heaviest first across ALL heads, which alone is worth 12 % of a causal 14k
// prompt over "heaviest first per head"; the query heads of one KV head share an XCD (see the kernel).
template <int kValue> struct Parity { static constexpr int value = kValue; };
struct PipeTiles {
    Chunk k[2][kKeyTile * 16];                   // [buffer][key][16 slots], slot ^ (key & 15)
    Chunk v[2][kKeyTile * 16];                   // [buffer][key][16 slots], slot + 4 (key & 3) mod 16
};
// Four keys of sixteen channels, transposed on the way out of LDS: lane t of each group of sixteen lanes
// points at four consecutive halves, and lane j of the group receives element j % 4 of lanes j / 4, j / 4 + 4,
// j / 4 + 8, j / 4 + 12. With lane t at channels 4 (t % 4) .. + 3 of key t / 4, lane j gets channel j of keys 0 .. 3.
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ s16x4 lds_read_transposed(const char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p));
}
__device__ __forceinline__ void copy16_to_lds(const void* gptr, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_byte_addr), "v"(gptr) : "memory", "m0");
}
// kSplit: the keys are cut into `n_runs` runs of `tiles_per_part` tiles (an even number); a workgroup takes one run
// of what it would have taken alone and leaves each row's state - 128 unnormalised channels, the
// scaled maximum, the sum - in `parts` as record (row, head, run) for prefill_merge. For a few rows against a long
// cache: one row tile is 28 workgroups that each walk the whole cache, tile after tile, on a chip of 256 units.
template <bool kSplit>
__global__ __launch_bounds__(kBlock, 2) void prefill_pipe(
    const h16* __restrict__ Q, const h16* __restrict__ K, const h16* __restrict__ V, const int* __restrict__ page_table,
    h16* __restrict__ O, int n_q_heads, int n_kv_heads, int q_len, int q_offset, int kv_len, int causal, float scale_log2,
    float* __restrict__ parts, int n_runs, int tiles_per_part) {
    __shared__ PipeTiles tiles;
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, half = lane >> 5;
    // Workgroup i runs on XCD i % 8 as that XCD's (i / 8)-th. The query heads of one KV head that work on the same
    // rows read the same K and V tiles at the same time: such a group is kept on ONE XCD (one L2), its members next
    // to each other in that XCD's order, and the groups are dealt to the XCDs heaviest rows first.
    const int group_heads = n_q_heads / n_kv_heads;
    const int n_row_tiles = (q_len + kQTile - 1) / kQTile;
    const int xcd = (int)blockIdx.x & 7, nth = (int)blockIdx.x >> 3;
    int group = (nth / group_heads) * 8 + xcd;                    // (row tile, KV head), heaviest first
    int run = 0;                                                  // kSplit: (run, row tile, KV head) dealt the same way
    if (kSplit) {
        run = group / (n_row_tiles * n_kv_heads);
        group -= run * (n_row_tiles * n_kv_heads);
        if (run >= n_runs) return;
    }
    if (group >= n_row_tiles * n_kv_heads) return;                // the whole workgroup, before any barrier
    const int kvh = group % n_kv_heads;
    const int head = kvh * group_heads + nth % group_heads;
    const int q0 = (n_row_tiles - 1 - group / n_kv_heads) * kQTile;
    const int qw0 = q0 + wave * 32;
    const int qrow = qw0 + col;
    const int q_abs = q_offset + qrow;
    // A wave whose 32 rows all lie past the chunk's end (a chunk of a few rows against a long cache: three of a
    // workgroup's four waves) copies its share of every tile and keeps the barriers, and computes nothing.
    const bool idle = qw0 >= q_len;
    int wg_limit = kv_len;
    if (causal) wg_limit = min(kv_len, q_offset + min(q0 + kQTile, q_len));
    int ntiles = (wg_limit + kKeyTile - 1) / kKeyTile;
    const int last_key = kv_len - 1;
    const size_t row_halves = (size_t)n_kv_heads * kD;
    const uint32_t lds_k0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)&tiles.k[0][0]);
    int tile0 = 0;                                                // first key tile of this workgroup's run
    if (kSplit) {
        tile0 = run * tiles_per_part;
        ntiles = min(tiles_per_part, ntiles - tile0);
        if (ntiles <= 0) {                                        // nothing the rows may see in this run: empty states
            if (qrow < q_len) {
                float* rec = parts + (((size_t)qrow * n_q_heads + head) * n_runs + run) * kPartFloats;
                for (int i = half; i < kPartFloats; i += 2) rec[i] = i == kD ? -INFINITY : 0.0f;
            }
            return;                                               // the whole workgroup, before any barrier
        }
    }

    h16x8 qf[kD / 16];
    load_query(qf, Q + ((size_t)min(qrow, q_len - 1) * n_q_heads + head) * kD, half);
    RowState st;
    st.reset();

    // K tile j -> buffer j & 1, straight into LDS: copy c of this wave fills slots 64 (4 wave + c) .. + 63:
    // keys 4 (4 wave + c) .. + 3, the lane owning (key, physical slot) and fetching the logical slot.
    // Contiguous cache, tile wholly inside it: a uniform base per tile plus a 32-bit offset per lane that never
    // changes, so a copy costs no vector instruction. Otherwise (pages, the cache's last rows): an address per lane.
    uint32_t k_off[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int key = 4 * (4 * wave + c) + (lane >> 4), phys = lane & 15;
        k_off[c] = (uint32_t)(((size_t)key * row_halves + (size_t)kvh * kD) * 2u) + (uint32_t)((phys ^ (key & 15)) * 16);
    }
    auto request_k = [&](int j) {
        const int t0 = (tile0 + j) * kKeyTile;
        const uint32_t lds_at = lds_k0 + (uint32_t)(j & 1) * (kKeyTile * 256u) + (uint32_t)(4 * wave) * 1024u;
        if (!page_table && t0 + kKeyTile <= kv_len) {
            const char* base = reinterpret_cast<const char*>(K) + (size_t)t0 * row_halves * 2u;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             : : "s"(lds_at + (uint32_t)c * 1024u), "v"(k_off[c]), "s"(base) : "memory", "m0");
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int key = 4 * (4 * wave + c) + (lane >> 4), phys = lane & 15;
                const int row = cache_row(page_table, min(t0 + key, last_key));
                const Chunk* g = reinterpret_cast<const Chunk*>(K + (size_t)row * row_halves + (size_t)kvh * kD) + (phys ^ (key & 15));
                copy16_to_lds(g, lds_at + (uint32_t)c * 1024u);
            }
        }
    };
    // V tile j -> buffer j & 1 the same way (the cache rows of K and V have one layout); the lane owning (key,
    // physical slot p) fetches logical slot p - 4 (key % 4): a key's 64-byte quarters rotate with the key, so the
    // four keys a transposing read gathers lie in four different quarters of the banks.
    const uint32_t lds_v0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)&tiles.v[0][0]);
    uint32_t v_off[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int key = 4 * (4 * wave + c) + (lane >> 4), phys = lane & 15;
        v_off[c] = (uint32_t)(((size_t)key * row_halves + (size_t)kvh * kD) * 2u) + (uint32_t)(((phys - 4 * (key & 3)) & 15) * 16);
    }
    auto request_v = [&](int j) {
        const int t0 = (tile0 + j) * kKeyTile;
        const uint32_t lds_at = lds_v0 + (uint32_t)(j & 1) * (kKeyTile * 256u) + (uint32_t)(4 * wave) * 1024u;
        if (!page_table && t0 + kKeyTile <= kv_len) {
            const char* base = reinterpret_cast<const char*>(V) + (size_t)t0 * row_halves * 2u;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             : : "s"(lds_at + (uint32_t)c * 1024u), "v"(v_off[c]), "s"(base) : "memory", "m0");
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int key = 4 * (4 * wave + c) + (lane >> 4), phys = lane & 15;
                const int row = cache_row(page_table, min(t0 + key, last_key));
                const Chunk* g = reinterpret_cast<const Chunk*>(V + (size_t)row * row_halves + (size_t)kvh * kD) + ((phys - 4 * (key & 3)) & 15);
                copy16_to_lds(g, lds_at + (uint32_t)c * 1024u);
            }
        }
    };
    auto scores = [&](int j, f32x16 (&s)[2]) {
        const Chunk* kb = tiles.k[j & 1];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[a][r] = 0.0f;
#pragma unroll
            for (int s8 = 0; s8 < kD / 16; ++s8) {
                const int row = 32 * a + col, slot = 2 * s8 + half;
                const h16x8 kf = __builtin_bit_cast(h16x8, kb[row * 16 + (slot ^ (row & 15))]);
                s[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s8], s[a], 0, 0, 0);
            }
        }
    };

    // (q_len, kv_len > 0: every workgroup has at least one tile. The prologue is unconditional so that the
    // compiler knows the query loads have been waited for when the loop starts; on a path around it, it
    // would wait for them - and with them for every copy in flight - inside the loop.)
    request_k(0);
    request_k(1);
    request_v(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // K 0, K 1 and V 0 landed
    __syncthreads();
    // a lane's fragment positions inside a tile never change: row col (+ 32 a) of K, slot 2 s8 + half swizzled;
    // row col (+ 32 t) of V^T, unit 2 u + half swizzled ((32 t + col) / 2 % 8 = col / 2 % 8)
    int kf_idx[8];
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) kf_idx[s8] = col * 16 + ((2 * s8 + half) ^ (col & 15));
    f32x16 s_pp[2][2];                        // the scores of the tile in hand and of the next, by tile parity
    if (!idle) scores(0, s_pp[0]);
    __syncthreads();                                          // K 0 is read: its buffer may take K 2

    // Byte offsets of this lane's fragments from the start of a K / V^T buffer: with the buffer a compile-time
    // constant (the loop is unrolled by two) the rest of an LDS address is an immediate.
    uint32_t kf_byte[8], vt_byte[4];
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) kf_byte[s8] = (uint32_t)kf_idx[s8] * 16u;
    // V^T fragments: channel tile t (32 channels), key step u (16 keys). A lane multiplies, in this order, keys
    // 16 u + 4 half + 0 .. 3 and 16 u + 8 + 4 half + 0 .. 3 (where its probabilities sit after the score MFMAs):
    // two transposing reads of four keys each. In its group of sixteen lanes, lane t points at key t / 4 of the
    // four and at channels 32 t' + 16 (group % 2) + 4 (t % 4) .. + 3; the key's quarter rotation depends on t / 4
    // alone, so the address is one register per channel tile plus an immediate for (u, which four, buffer).
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int tin = lane & 15, kk = tin >> 2;
        const int slot = 4 * ((t + kk) & 3) + 2 * ((lane >> 4) & 1) + ((tin & 3) >> 1);
        vt_byte[t] = (uint32_t)((4 * half + kk) * 256 + slot * 16 + (tin & 1) * 8);
    }
    // Tile j's scores lose what the row may not see: only a tile that reaches past the cache end or past the
    // wave's first row's position has anything to hide.
    auto hide = [&](int j, f32x16 (&sc)[2]) {
        const int t0 = (tile0 + j) * kKeyTile;
        if (t0 + kKeyTile > kv_len || (causal && t0 + kKeyTile - 1 > q_offset + qw0)) {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = t0 + 32 * a + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool seen = key < kv_len && (!causal || key <= q_abs);
                    sc[a][r] = seen ? sc[a][r] : -INFINITY;
                }
        }
    };
    // The row maximum (scaled) of the tile in hand: taken while the vector ALU has nothing else to do, behind the
    // first V^T P^T MFMAs of the tile before (behind the first scores in the prologue).
    if (!idle) hide(0, s_pp[0]);
    // one tile: P = j & 1 names the buffers and which of the two score sets is "this tile"
    auto body = [&](int j, auto parity_c) {
        constexpr int P = decltype(parity_c)::value;
        f32x16 (&s_cur)[2] = s_pp[P];
        f32x16 (&s_next)[2] = s_pp[P ^ 1];
        request_k(j + 2);                                     // into the buffer tile j's K has left
        request_v(j + 1);                                     // into the buffer tile j - 1's V has left
        if (idle) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            return;
        }
        const char* kb = reinterpret_cast<const char*>(&tiles.k[P ^ 1][0]);
        auto k_frag = [&](int k) {                            // step k = 8 a + s8
            return __builtin_bit_cast(h16x8, *reinterpret_cast<const Chunk*>(kb + (k >> 3) * 8192 + kf_byte[k & 7]));
        };
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) s_next[a][r] = 0.0f;
        h16x8 kf[3];
        kf[0] = k_frag(0);
        kf[1] = k_frag(1);
        h16x8 pf[4];
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            __builtin_amdgcn_sched_barrier(0);
            if (k + 2 < 16) kf[(k + 2) % 3] = k_frag(k + 2);
            s_next[k >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[k % 3], qf[k & 7], s_next[k >> 3], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            {                                                 // scores 2 k, 2 k + 1: as in probabilities()
                const int q = 2 * k;
                const f32x2 two = {exp2_fast(fmaf(s_cur[q >> 4][q & 15], scale_log2, -st.m_use)),
                                   exp2_fast(fmaf(s_cur[q >> 4][(q & 15) + 1], scale_log2, -st.m_use))};
                sum += two[0];
                sum += two[1];
                const h16x2 h = __builtin_convertvector(two, h16x2);
                pf[q >> 3][q & 7] = h[0];
                pf[q >> 3][(q & 7) + 1] = h[1];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // (the compiler would sink the conversions past the branches below to their first use, out from under the
        // MFMAs they were placed behind: their results are pinned here)
        asm volatile("" : "+v"(pf[0]), "+v"(pf[1]), "+v"(pf[2]), "+v"(pf[3]), "+v"(sum));
        if (__builtin_amdgcn_ballot_w64(sum > st.thr) != 0) {     // rare (RowState): the reference settles, the tile again
            st.settle(lane_max(s_cur), scale_log2);
            probabilities(s_cur, scale_log2, st.m_use, pf, sum);
        }
        st.l += sum;
        // block 2: O^T += V^T P^T on the matrix pipe, the V^T fragments transposed out of the row-major tile
        const char* vb = reinterpret_cast<const char*>(&tiles.v[P][0]);
        auto v_frag = [&](int k) {                            // step k = 4 u + t
            const char* at = vb + vt_byte[k & 3] + (k >> 2) * 4096;
            const s16x4 lo = lds_read_transposed(at), hi = lds_read_transposed(at + 2048);
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(h16x8, both);
        };
        h16x8 vf[3];
        vf[0] = v_frag(0);
        vf[1] = v_frag(1);
        // Block 2 is matrix work alone and block 1 is bound by its vector work: where the SIMD's other wave
        // (of the compute unit's second workgroup) is in block 1, it goes first, and these MFMAs fill the
        // matrix pipe under its softmax (1.5-2 % at 14449 rows).
        __builtin_amdgcn_s_setprio(0);
        hide(j + 1, s_next);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            __builtin_amdgcn_sched_barrier(0);
            if (k + 2 < 16) vf[(k + 2) % 3] = v_frag(k + 2);
            st.o[k & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[k % 3], pf[k >> 2], st.o[k & 3], 0, 0, 0);
        }
        __builtin_amdgcn_s_setprio(1);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // K j+2 and V j+1 landed
        __syncthreads();
    };
    // An odd tile count is rounded up: the extra tile lies wholly past the keys the workgroup may see, so it
    // is masked, its probabilities are zeros and the state does not move.
    __builtin_amdgcn_s_setprio(1);                            // block 1's priority; block 2 lowers it for itself
    for (int j = 0; j < ntiles; j += 2) {
        body(j, Parity<0>{});
        body(j + 1, Parity<1>{});
    }

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // no copy may land after the workgroup has gone
    const float l_row = st.row_sum();
    if (kSplit) {
        if (qrow < q_len) {
            float* rec = parts + (((size_t)qrow * n_q_heads + head) * n_runs + run) * kPartFloats;
            // register 4 g + r of tile t is channel 32 t + 8 g + 4 half + r
#pragma unroll
            for (int t = 0; t < kD / 32; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    *reinterpret_cast<float4*>(rec + 32 * t + 8 * g + 4 * half) =
                        float4{st.o[t][4 * g], st.o[t][4 * g + 1], st.o[t][4 * g + 2], st.o[t][4 * g + 3]};
            if (half == 0) *reinterpret_cast<float2*>(rec + kD) = float2{st.reference(), l_row};
        }
        return;
    }
    if (qrow < q_len) {
        const float inv = l_row > 0.0f ? 1.0f / l_row : 0.0f;
        h16* op = O + ((size_t)qrow * n_q_heads + head) * kD;
        // register 4 g + r of tile t is channel 32 t + 8 g + 4 half + r
        typedef h16 h16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                h16x4 o4;
#pragma unroll
                for (int r = 0; r < 4; ++r) o4[r] = to_half(st.o[t][4 * g + r] * inv);
                *reinterpret_cast<h16x4*>(op + 32 * t + 8 * g + 4 * half) = o4;
            }
    }
}


// The runs of a split prefill folded: one wave per (row, head), two channels per lane, the runs in order. A run's
// record is 128 unnormalised channels, its scaled maximum and its sum; a run that saw no key has maximum -inf.
__global__ __launch_bounds__(kBlock) void prefill_merge(const float* __restrict__ parts, h16* __restrict__ O,
                                                        int rows_heads, int n_parts) {
    constexpr int kMostRuns = 16;                          // what vv_attn_prefill cuts a prefill into at most
    const int item = (int)blockIdx.x * kWavesPerBlock + wave_in_block();
    if (item >= rows_heads) return;
    const int lane = lane_id();
    const float* rec = parts + (size_t)item * n_parts * kPartFloats;
    // every run's values are asked for before the first is used: one trip to memory
    float m[kMostRuns], l[kMostRuns];
    float2 v[kMostRuns];
#pragma unroll
    for (int p = 0; p < kMostRuns; ++p) {
        const float* r = rec + (size_t)min(p, n_parts - 1) * kPartFloats;
        m[p] = p < n_parts ? r[kD] : -INFINITY;
        l[p] = r[kD + 1];
        v[p] = *reinterpret_cast<const float2*>(r + 2 * lane);
    }
    float m_all = -INFINITY;
#pragma unroll
    for (int p = 0; p < kMostRuns; ++p) m_all = fmaxf(m_all, m[p]);
    float o0 = 0.0f, o1 = 0.0f, l_all = 0.0f;
#pragma unroll
    for (int p = 0; p < kMostRuns; ++p) {
        const float f = m[p] == -INFINITY ? 0.0f : exp2_fast(m[p] - m_all);
        o0 = fmaf(v[p].x, f, o0);
        o1 = fmaf(v[p].y, f, o1);
        l_all = fmaf(l[p], f, l_all);
    }
    const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
    typedef h16 h16x2v __attribute__((ext_vector_type(2)));
    const h16x2v out = {to_half(o0 * inv), to_half(o1 * inv)};
    *reinterpret_cast<h16x2v*>(O + (size_t)item * kD + 2 * lane) = out;
}

// ── any head_dim <= 256: one wave per (query row, head) ──────────────────
__global__ __launch_bounds__(kWave) void rows_generic(
    const h16* Q, const h16* Kc, const h16* Vc, const int* page_table, h16* O, int n_q_heads,
    int n_kv_heads, int head_dim, int q_len, int q_offset, int kv_len, const int* d_kv_len,
    int causal, float scale_log2) {
    const int qrow = (int)blockIdx.x, head = (int)blockIdx.y;
    const int lane = lane_id();
    const int kvh = head / (n_q_heads / n_kv_heads);
    if (d_kv_len) kv_len = *d_kv_len;
    int limit = kv_len;
    if (causal) limit = min(kv_len, q_offset + qrow + 1);
    const h16* qp = Q + ((size_t)qrow * n_q_heads + head) * head_dim;
    float q[4], acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        q[j] = d < head_dim ? (float)qp[d] * scale_log2 : 0.0f;
        acc[j] = 0.0f;
    }
    float m_run = -INFINITY, l_run = 0.0f;
    for (int t = 0; t < limit; ++t) {
        const size_t off = ((size_t)cache_row(page_table, t) * n_kv_heads + kvh) * head_dim;
        float part = 0.0f, v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            part += d < head_dim ? q[j] * (float)Kc[off + d] : 0.0f;
            v[j] = d < head_dim ? (float)Vc[off + d] : 0.0f;
        }
        const float x = wave_sum(part);
        const float m_new = fmaxf(m_run, x);
        const float alpha = exp2_fast(m_run - m_new);
        const float p = exp2_fast(x - m_new);
        l_run = l_run * alpha + p;
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = acc[j] * alpha + p * v[j];
    }
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    h16* op = O + ((size_t)qrow * n_q_heads + head) * head_dim;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        if (d < head_dim) op[d] = to_half(acc[j] * inv);
    }
}

// ── decode, head_dim 128 ─────────────────────────────────────────────────
// One wave per (slice of the positions, KV head, 32 query heads of its group):
// the heads sharing a KV head take the place of the prefill's query rows, so
// the slice's K and V are read once for all of them. n_parts == 1 writes O;
// otherwise each slice leaves (max, sum, unnormalised O) per head in `parts`.

template <int kFmt>
__global__ __launch_bounds__(kWave) void decode128(
    const h16* __restrict__ Q, KvSource src, h16* __restrict__ O, float* __restrict__ parts,
    int n_q_heads, int n_kv_heads, int cache_len, const int* __restrict__ d_cache_len,
    int n_parts, float scale_log2) {
    __shared__ KvTile tile;

    const int lane = (int)threadIdx.x;
    load_levels<kFmt>(tile, lane);
    const int col = lane & 31, half = lane >> 5;
    const int part = (int)blockIdx.x;
    const int kvh = (int)blockIdx.y;
    const int group = n_q_heads / n_kv_heads;
    const int g = (int)blockIdx.z * 32 + col;                 // this lane's head inside the group
    const int head = kvh * group + min(g, group - 1);
    const int len = d_cache_len ? *d_cache_len : cache_len;
    const int per = (((len + n_parts - 1) / n_parts) + kKeyTile - 1) & ~(kKeyTile - 1);
    const int begin = part * per, end = min(len, begin + per);

    h16x8 qf[kD / 16];
    load_query(qf, Q + (size_t)head * kD, half);
    RowState st;
    st.reset();

    TileRegs<kWave> regs;
    if (begin < end) fetch_tile<kWave, kFmt>(regs, src, tile.lev, n_kv_heads, kvh, begin, end - 1, lane);
    for (int t0 = begin; t0 < end; t0 += kKeyTile) {
        __syncthreads();
        commit_tile<kWave>(tile, regs, lane);
        __syncthreads();
        if (t0 + kKeyTile < end)
            fetch_tile<kWave, kFmt>(regs, src, tile.lev, n_kv_heads, kvh, t0 + kKeyTile, end - 1, lane);
        f32x16 s[2];
        tile_scores(tile, qf, col, half, s);
        if (t0 + kKeyTile > end) {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = t0 + 32 * a + 8 * (r >> 2) + 4 * half + (r & 3);
                    s[a][r] = key < end ? s[a][r] : -INFINITY;
                }
        }
        tile_update(tile, s, st, col, half, scale_log2);
    }

    if (g >= group) return;
    if (n_parts == 1) {
        const float l_row = st.row_sum();
        const float inv = l_row > 0.0f ? 1.0f / l_row : 0.0f;
        h16* op = O + (size_t)head * kD;
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = to_half(st.o[t][4 * q + r] * inv);
                *reinterpret_cast<h16x4*>(op + 32 * t + 8 * q + 4 * half) = o;
            }
    } else {
        float* dst = parts + ((size_t)head * n_parts + part) * kPartFloats;
        const float l_row = st.row_sum();
        if (half == 0) { dst[kD] = st.reference(); dst[kD + 1] = l_row; }
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 o = {st.o[t][4 * q], st.o[t][4 * q + 1], st.o[t][4 * q + 2], st.o[t][4 * q + 3]};
                *reinterpret_cast<f32x4*>(dst + 32 * t + 8 * q + 4 * half) = o;
            }
    }
}

// ── decode over an FP16 cache, head_dim 128, groups of up to 16 query heads ───
// The decode is a stream of the cache: 512 bytes per position and KV head, used once,
// and a launch lives for a few microseconds, so what counts is that every byte is
// requested at once and that a wave has little code to run when its bytes arrive (a
// wave's first pass over its code is a chain of instruction-cache misses). A
// workgroup of sixteen waves owns a slice of the positions of one KV head; wave w
// takes the 16-key blocks w, w + 16, ... of the slice, one block at a time with the
// next block's eight loads (16 bytes per lane each) in flight. At 14k positions a
// wave has exactly one block: the whole cache is in flight from the first
// microsecond, 2048 short waves per KV head. Both products run on the matrix cores
// with the group's query heads in the place of rows:
//   scores   S^T = K Q^T (16x16x32): the K rows go from global memory straight into
//            the A operand - lane (key l % 16, j = l / 16) holds channels
//            32 s + 8 j .. + 7 in step s, the query fragment the same channels - and
//            lane (head l % 16, j) ends up with keys 4 j .. 4 j + 3 of the block.
//   softmax  online per head in FP32, base-2 domain; maximum and sum cross the four
//            j groups by lane exchange. The probabilities, rounded to FP16, are
//            already the B operand of the second product (16x16x16, k = key).
//   O^T      = V^T P^T: lane (chunk c = l % 16, j) loads keys 4 j .. 4 j + 3 of chunk c as stored; element e of
//            those four rows are the four keys of channel 8 c + e, which is exactly this lane's share of the A
//            operand of the tile "channels {8 c + e}" (row c, keys 4 j .. + 3): the transposition costs a pick
//            of halves, no LDS. Lane (head l % 16, j') accumulates channels 32 j' + 8 r + e in FP32.
// Nothing passes through LDS in the loop. The waves' states meet in LDS once and the workgroup leaves one (max,
// sum, unnormalised O) record per head in `parts`, for decode_merge.
constexpr int kStreamWaves = 16;
constexpr int kStreamThreads = kStreamWaves * kWave;
constexpr int kStreamOStride = kD + 1;          // floats per head in the waves' exchange (odd: spreads banks)
// A wave's LDS: its O for kHeads heads.
constexpr int stream_tile_bytes(int heads) { return (heads * kStreamOStride * 4 + 15) / 16 * 16; }

// Where channel ch of a head sits in the waves' exchange: the upper two of the four 32-channel blocks turned by 16, so
// that the four lanes that hold one (e, r) of the same head in their four blocks write four different banks
// (with a plain layout blocks j and j + 2 are 64 floats apart: every store a two-way conflict).
__device__ __forceinline__ int stream_o_slot(int ch) { return (ch & ~31) | ((ch + ((ch >> 2) & 16)) & 31); }

template <int kHeads>      // the group's query heads, padded: 8 or 16
__global__ __launch_bounds__(kStreamThreads) void decode_stream(
    const h16* __restrict__ Q, const h16* __restrict__ K, const h16* __restrict__ V,
    const int* __restrict__ page_table, float* __restrict__ parts, int n_q_heads, int n_kv_heads,
    int cache_len, const int* __restrict__ d_cache_len, int n_parts, float scale_log2) {
    // Per wave: its O after the loop, [head][kStreamOStride] floats.
    __shared__ __attribute__((aligned(16))) char tile_lds[kStreamWaves][stream_tile_bytes(kHeads)];
    __shared__ float m_lds[kStreamWaves][16], l_lds[kStreamWaves][16];
    auto o_of = [&](int w) { return reinterpret_cast<float*>(tile_lds[w]); };

    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = wave_in_block();
    const int c = lane & 15, j = lane >> 4;        // c: key (scores) / head (softmax, O) / chunk (V loads)
    const int part = (int)blockIdx.x, kvh = (int)blockIdx.y;
    const int group = n_q_heads / n_kv_heads;
    const int len = d_cache_len ? *d_cache_len : cache_len;
    const int per = (((len + n_parts - 1) / n_parts) + 15) & ~15;
    const int begin = part * per, end = min(len, begin + per);
    const size_t row_halves = (size_t)n_kv_heads * kD;

    // Block n of this wave starts at key begin + 16 (wave + 16 n). Keys past the slice repeat its last
    // key (finite values; their scores are masked).
    Chunk kr[4], vr[4];
    auto fetch = [&](int key0) {
        const int tk = min(key0 + c, end - 1);
        const Chunk* kp = reinterpret_cast<const Chunk*>(K + (size_t)cache_row(page_table, tk) * row_halves +
                                                         (size_t)kvh * kD);
#pragma unroll
        for (int s = 0; s < 4; ++s) kr[s] = load_chunk_stream(kp + 4 * s + j);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tv = min(key0 + 4 * j + i, end - 1);
            vr[i] = load_chunk_stream(reinterpret_cast<const Chunk*>(
                V + (size_t)cache_row(page_table, tv) * row_halves + (size_t)kvh * kD) + c);
        }
    };
    int key0 = begin + 16 * wave;
    if (key0 < end) fetch(key0);

    // The query fragments of this lane's head: channels 32 s + 8 j .. + 7 of step s.
    h16x8 qf[4];
    {
        const Chunk* qp = reinterpret_cast<const Chunk*>(Q + (size_t)(kvh * group + min(c, group - 1)) * kD);
#pragma unroll
        for (int s = 0; s < 4; ++s) qf[s] = __builtin_bit_cast(h16x8, load_chunk(qp + 4 * s + j));
    }

    f32x4 o[8];                                    // o[e][r]: channel 32 j + 8 r + e of head c
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;

    for (; key0 < end; key0 += 16 * kStreamWaves) {
        // scores: lane (head c, j) gets keys key0 + 4 j + r
        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, kr[s]), qf[s], sc, 0, 0, 0);
        h16x8 v4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v4[i] = __builtin_bit_cast(h16x8, vr[i]);
        const int next = key0 + 16 * kStreamWaves;
        if (next < end) fetch(next);               // the same for the whole wave

        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            sc[r] = key0 + 4 * j + r < end ? sc[r] : -INFINITY;
            mx = fmaxf(mx, sc[r]);
        }
        mx = max_xor32(max_xor16(mx)) * scale_log2;
        const float m_new = fmaxf(m, mx);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        if (__builtin_amdgcn_ballot_w64(m_new > m && m > -INFINITY) != 0) {
            const float alpha = exp2_fast(m - m_use);
            l *= alpha;
#pragma unroll
            for (int e = 0; e < 8; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[e][r] *= alpha;
        }
        m = m_new;

        h16x4 pf;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = exp2_fast(fmaf(sc[r], scale_log2, -m_use));
            l += p;
            pf[r] = (h16)p;
        }
        // V^T P^T: lane (chunk c, j) holds keys 4 j .. 4 j + 3 of channels 8 c .. 8 c + 7 as they were stored; the four
        // keys of ONE channel 8 c + e are this lane's part of the A operand of tile e (row c = channel 8 c + e, keys
        // 4 j .. + 3), so the transposition is a pick of element e from the four rows: no trip through LDS.
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const h16x4 vf = {v4[0][e], v4[1][e], v4[2][e], v4[3][e]};
            o[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(vf, pf, o[e], 0, 0, 0);
        }
    }

    // the wave's denominators meet across the four j groups; then the waves
    l = sum_xor32(sum_xor16(l));
    if (j == 0) {
        m_lds[wave][c] = m;
        l_lds[wave][c] = l;
    }
    if (c < group) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_of(wave)[c * kStreamOStride + stream_o_slot(32 * j + 8 * r + e)] = o[e][r];
    }
    __syncthreads();
    for (int idx = tid; idx < group * kD; idx += kStreamThreads) {
        const int h = idx >> 7, ch = idx & (kD - 1);
        float m_all = -INFINITY;
#pragma unroll 4
        for (int w = 0; w < kStreamWaves; ++w) m_all = fmaxf(m_all, m_lds[w][h]);
        float ov = 0.0f, l_all = 0.0f;
#pragma unroll 4
        for (int w = 0; w < kStreamWaves; ++w) {
            const float mw = m_lds[w][h];
            const float f = mw == -INFINITY ? 0.0f : exp2_fast(mw - m_all);
            ov = fmaf(o_of(w)[h * kStreamOStride + stream_o_slot(ch)], f, ov);
            l_all = fmaf(l_lds[w][h], f, l_all);
        }
        float* dst = parts + ((size_t)(kvh * group + h) * n_parts + part) * kPartFloats;
        dst[ch] = ov;
        if (ch == 0) { dst[kD] = m_all; dst[kD + 1] = l_all; }
    }
}

// Folds the slices of one head. The first n_parts threads turn the slices'
// maxima into weights 2^(m_p - m_all) (kept in LDS) and sum the weighted
// denominators; then 8 groups of 128 threads take every 8th slice for one
// channel each, so a thread's loads are few and independent.
constexpr int kMergeGroups = 8;
constexpr int kMergeThreads = kD * kMergeGroups;

__global__ __launch_bounds__(kMergeThreads) void decode_merge(const float* __restrict__ parts,
                                                              h16* __restrict__ O, int n_parts) {
    __shared__ float s_f[kMaxParts];
    __shared__ float s_red[2][kMergeThreads / kWave];
    __shared__ float s_o[kMergeGroups][kD];
    const int head = (int)blockIdx.x, tid = (int)threadIdx.x;
    const int d = tid % kD, grp = tid / kD;
    const float* src = parts + (size_t)head * n_parts * kPartFloats;

    // The first 64 slices' values are requested before the maxima are exchanged: one trip to memory, not two.
    float v0[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int p = grp + u * kMergeGroups;
        v0[u] = p < n_parts ? src[p * kPartFloats + d] : 0.0f;
    }
    const bool mine = tid < n_parts;
    const float m = mine ? src[tid * kPartFloats + kD] : -INFINITY;
    const float l = mine ? src[tid * kPartFloats + kD + 1] : 0.0f;
    const float wm = wave_max(m);
    if ((tid & 63) == 0) s_red[0][tid >> 6] = wm;
    __syncthreads();
    float m_all = -INFINITY;
#pragma unroll
    for (int w = 0; w < kMergeThreads / kWave; ++w) m_all = fmaxf(m_all, s_red[0][w]);
    const float f = m == -INFINITY ? 0.0f : exp2_fast(m - m_all);
    if (mine) s_f[tid] = f;
    const float wl = wave_sum(l * f);
    if ((tid & 63) == 0) s_red[1][tid >> 6] = wl;
    __syncthreads();
    float l_all = 0.0f;
#pragma unroll
    for (int w = 0; w < kMergeThreads / kWave; ++w) l_all += s_red[1][w];

    float o = 0.0f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int p = grp + u * kMergeGroups;
        if (p < n_parts) o = fmaf(v0[u], s_f[p], o);
    }
    for (int p0 = grp + 8 * kMergeGroups; p0 < n_parts; p0 += 8 * kMergeGroups) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + u * kMergeGroups;
            v[u] = p < n_parts ? src[p * kPartFloats + d] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + u * kMergeGroups;
            if (p < n_parts) o = fmaf(v[u], s_f[p], o);
        }
    }
    s_o[grp][d] = o;
    __syncthreads();
    if (grp == 0) {
        float total = 0.0f;
#pragma unroll
        for (int g = 0; g < kMergeGroups; ++g) total += s_o[g][d];
        O[(size_t)head * kD + d] = to_half(l_all > 0.0f ? total / l_all : 0.0f);
    }
}

// ── FP16 cache store ─────────────────────────────────────────────────────
__global__ __launch_bounds__(kBlock) void kv_store_fp16(
    const h16* __restrict__ k, const h16* __restrict__ v, h16* __restrict__ k_store,
    h16* __restrict__ v_store, int row_halves, int pos, const int* __restrict__ d_pos,
    int n_positions, const int* __restrict__ page_table) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (size_t)n_positions * row_halves) return;
    const int p = (int)(i / row_halves), e = (int)(i % row_halves);
    const int t = (d_pos ? *d_pos : pos) + p;
    const size_t dst = (size_t)cache_row(page_table, t) * row_halves + e;
    k_store[dst] = k[i];
    v_store[dst] = v[i];
}

// The same in 16-byte chunks, for rows that are whole chunks at aligned addresses (any n_kv_heads x 128): a thread
// asks for its K and V chunks before it reads the position and the page, so a decode step's store is three trips
// to memory in a row (arguments; position, K and V together; page), not five, and a prefill's moves 16 bytes an access.
__global__ __launch_bounds__(kBlock) void kv_store_fp16_chunks(
    const Chunk* __restrict__ k, const Chunk* __restrict__ v, Chunk* __restrict__ k_store,
    Chunk* __restrict__ v_store, int row_chunks, int pos, const int* __restrict__ d_pos, int n_chunks,
    const int* __restrict__ page_table) {
    const int i = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (i >= n_chunks) return;
    const Chunk kc = load_chunk(k + i), vc = load_chunk(v + i);
    const int p = i / row_chunks, e = i - p * row_chunks;
    const int t = (d_pos ? *d_pos : pos) + p;
    const size_t dst = (size_t)cache_row(page_table, t) * row_chunks + e;
    store_chunk(k_store + dst, kc);
    store_chunk(v_store + dst, vc);
}

// ── FP8 cache store (src/cuda/kv_quant.cu:57-84, kv_codec.cuh:66-128) ──────
// One value to E4M3 (bias 7, largest finite 448 = 0x7E) or E5M2 (bias 15,
// largest finite 57344 = 0x7B) in integer arithmetic: zero and NaN give a signed
// zero, magnitudes from half a step above the largest finite value saturate to
// it, below the smallest normal the value is a count of subnormal steps rounded
// half up, else round to nearest even on the FP32 mantissa with the carry going
// into the exponent.
template <bool kE5M2>
__device__ __forceinline__ uint32_t fp8_encode(float f) {
    constexpr int kMant = kE5M2 ? 2 : 3, kBias = kE5M2 ? 15 : 7, kDrop = 23 - kMant;
    constexpr uint32_t kMaxCode = kE5M2 ? 0x7Bu : 0x7Eu;
    const uint32_t b = __builtin_bit_cast(uint32_t, f);
    const uint32_t sign = (b >> 24) & 0x80u;
    const float a = fabsf(f);
    if (!(a > 0.0f)) return sign;
    if (a >= (kE5M2 ? 61440.0f : 464.0f)) return sign | kMaxCode;
    int e = (int)((b >> 23) & 0xFFu) - 127;
    if (e < 1 - kBias) {
        int q = (int)(a * (kE5M2 ? 65536.0f : 512.0f) + 0.5f);
        q = min(q, 1 << kMant);                       // rolls into the smallest normal
        return sign | (uint32_t)q;
    }
    const uint32_t m = b & 0x7FFFFFu;
    uint32_t mm = m >> kDrop;
    const uint32_t rem = m & ((1u << kDrop) - 1u), half_way = 1u << (kDrop - 1);
    if (rem > half_way || (rem == half_way && (mm & 1u))) {
        if (++mm == (1u << kMant)) { mm = 0; ++e; }
    }
    if (e > (kE5M2 ? 15 : 8)) return sign | kMaxCode;
    return sign | ((uint32_t)(e + kBias) << kMant) | mm;
}

// Per head and channel the FP32 mean of the run's keys, positions in order.
__global__ void kv_build_ref(const h16* __restrict__ k, h16* __restrict__ ref, int n_kv_heads, int n_pos) {
    const int h = (int)blockIdx.x, d = (int)threadIdx.x;
    float acc = 0.0f;
    for (int p = 0; p < n_pos; ++p) acc += (float)k[((size_t)p * n_kv_heads + h) * kD + d];
    ref[(size_t)h * kD + d] = to_half(acc / (float)n_pos);
}

// blockIdx.y = 0: keys (minus the head's reference key when there is one), 1: values.
// A thread encodes eight channels.
template <bool kE5M2>
__global__ __launch_bounds__(kBlock) void kv_store_fp8(
    const h16* __restrict__ k, const h16* __restrict__ v, uint8_t* __restrict__ k_store,
    uint8_t* __restrict__ v_store, const h16* __restrict__ k_ref, int n_kv_heads, int pos,
    const int* __restrict__ d_pos, int n_positions, const int* __restrict__ page_table) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;         // (position, head, slot)
    const int slots_per_pos = n_kv_heads * (kD / 8);
    if (i >= (size_t)n_positions * slots_per_pos) return;
    const bool keys = blockIdx.y == 0;
    const int p = (int)(i / slots_per_pos), e = (int)(i % slots_per_pos);
    const int head = e / (kD / 8), slot = e % (kD / 8);
    const h16x8 src = *(reinterpret_cast<const h16x8*>(keys ? k : v) + i);
    h16x8 ref = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool centred = keys && k_ref != nullptr;
    if (centred) ref = *(reinterpret_cast<const h16x8*>(k_ref) + head * (kD / 8) + slot);
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        float val = (float)src[c];
        if (centred) val -= (float)ref[c];
        w[c >> 2] |= fp8_encode<kE5M2>(val) << (8 * (c & 3));
    }
    const int t = (d_pos ? *d_pos : pos) + p;
    const size_t dst = (size_t)cache_row(page_table, t) * slots_per_pos + e;
    *(reinterpret_cast<u32x2*>(keys ? k_store : v_store) + dst) = u32x2{w[0], w[1]};
}

// ── TurboQuant store, unpack and rotation (src/cuda/kv_quant.cu:86-119, 171-199;
//    kv_codec.cuh:130-165, 228-285) ──────────────────────────────────────────
// 32 lanes per vector (two vectors per wave), four consecutive channels per lane,
// FP32 additions in exactly this order: strides 1 and 2 inside a lane, then lane
// strides 1 .. 16, the upper partner taking (other - own).
constexpr float kWhtNorm = 0.0883883476f;      // 1 / sqrt(128)

__device__ __forceinline__ float tq_sign(int d) {     // the fixed +-1 pattern of the transform
    uint32_t h = (uint32_t)d * 2654435761u + 0x9E3779B9u;
    h ^= h >> 15; h *= 0x85EBCA6Bu; h ^= h >> 13;
    return (h & 1u) ? -1.0f : 1.0f;
}

__device__ __forceinline__ void wht128(float (&v)[4], int lane32) {
    float a;
    a = v[0] + v[1]; v[1] = v[0] - v[1]; v[0] = a;
    a = v[2] + v[3]; v[3] = v[2] - v[3]; v[2] = a;
    a = v[0] + v[2]; v[2] = v[0] - v[2]; v[0] = a;
    a = v[1] + v[3]; v[3] = v[1] - v[3]; v[1] = a;
#pragma unroll
    for (int m = 1; m < 32; m <<= 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float o = __shfl_xor(v[i], m);
            v[i] = (lane32 & m) ? o - v[i] : v[i] + o;
        }
    }
}

__device__ __forceinline__ void tq_rotate(float (&v)[4], int lane32, bool inverse) {
    if (!inverse) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= tq_sign(4 * lane32 + i);
        wht128(v, lane32);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= kWhtNorm;
    } else {
        wht128(v, lane32);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= kWhtNorm * tq_sign(4 * lane32 + i);
    }
}

__global__ __launch_bounds__(kBlock) void kv_rotate(h16* __restrict__ x, int n_vectors, int inverse) {
    const int vec = (int)blockIdx.x * (kBlock / 32) + (int)threadIdx.x / 32;
    const int lane32 = (int)threadIdx.x & 31;
    h16* p = x + (size_t)min(vec, n_vectors - 1) * kD + 4 * lane32;
    const h16x4 in = *reinterpret_cast<const h16x4*>(p);
    float v[4] = {(float)in[0], (float)in[1], (float)in[2], (float)in[3]};
    tq_rotate(v, lane32, inverse != 0);
    if (vec < n_vectors) *reinterpret_cast<h16x4*>(p) = h16x4{to_half(v[0]), to_half(v[1]), to_half(v[2]), to_half(v[3])};
}

// The packed code of a lane's four values: per value the number of mid-points
// between neighbouring levels it exceeds; 1.5 bits: the nearest of eight 2-D
// code words per pair, the first winning ties.
template <int kFmt>
__device__ __forceinline__ uint32_t tq_pack4(const float (&y)[4], float inv_sigma) {
#pragma clang fp contract(off)
    typedef KvFormat<kFmt> F;
    const float* lev = kTqLevels[kFmt - kFmtTq4];
    uint32_t bits = 0;
    if constexpr (kFmt == kFmtTq15) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const float a = y[2 * p] * inv_sigma, b = y[2 * p + 1] * inv_sigma;
            uint32_t best = 0;
            float bd = 3.402823466e+38f;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float da = a - lev[2 * c], db = b - lev[2 * c + 1];
                const float d = da * da + db * db;
                if (d < bd) { bd = d; best = (uint32_t)c; }
            }
            bits |= best << (3 * p);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float t = y[i] * inv_sigma;
            uint32_t c = 0;
#pragma unroll
            for (int j = 0; j + 1 < (1 << F::kCodeBits); ++j) c += (t > 0.5f * (lev[j] + lev[j + 1])) ? 1u : 0u;
            bits |= c << (F::kCodeBits * i);
        }
    }
    return bits;
}

// blockIdx.y = 0: keys (minus the head's reference key when there is one), 1: values.
template <int kFmt>
__global__ __launch_bounds__(kBlock) void kv_store_tq(
    const h16* __restrict__ k, const h16* __restrict__ v, uint8_t* __restrict__ k_store,
    uint8_t* __restrict__ v_store, h16* __restrict__ k_meta, h16* __restrict__ v_meta,
    const h16* __restrict__ k_ref, int n_kv_heads, int pos, const int* __restrict__ d_pos, int n_positions,
    const int* __restrict__ page_table) {
    typedef KvFormat<kFmt> F;
    constexpr int kLaneBits = 4 / F::kPerCode * F::kCodeBits;      // 16, 12, 8, 6
    __shared__ uint32_t pack[kBlock / 32][16];
    const int slot = (int)threadIdx.x / 32, lane32 = (int)threadIdx.x & 31;
    const int total = n_positions * n_kv_heads;
    const int idx = (int)blockIdx.x * (kBlock / 32) + slot;
    const int vec = min(idx, total - 1);
    const bool keys = blockIdx.y == 0;
    const int p = vec / n_kv_heads, head = vec % n_kv_heads;
    const h16x4 in = *reinterpret_cast<const h16x4*>((keys ? k : v) + (size_t)vec * kD + 4 * lane32);
    float val[4] = {(float)in[0], (float)in[1], (float)in[2], (float)in[3]};
    if (keys && k_ref) {
        const h16x4 r = *reinterpret_cast<const h16x4*>(k_ref + (size_t)head * kD + 4 * lane32);
#pragma unroll
        for (int i = 0; i < 4; ++i) val[i] -= (float)r[i];
    }
    tq_rotate(val, lane32, false);
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) ss = fmaf(val[i], val[i], ss);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float sigma = sqrtf(fmaxf(ss / (float)kD, 1e-12f));
    const uint32_t bits = tq_pack4<kFmt>(val, 1.0f / sigma);

    // lanes own overlapping words: assemble the vector's bit stream in LDS
    if (lane32 < 16) pack[slot][lane32] = 0u;
    __syncthreads();
    const int bit = kLaneBits * lane32;
    atomicOr(&pack[slot][bit >> 5], bits << (bit & 31));
    if ((bit & 31) + kLaneBits > 32) atomicOr(&pack[slot][(bit >> 5) + 1], bits >> (32 - (bit & 31)));
    __syncthreads();
    if (idx >= total) return;
    const int t = (d_pos ? *d_pos : pos) + p;
    const size_t row_vec = (size_t)cache_row(page_table, t) * n_kv_heads + head;
    uint32_t* dst = reinterpret_cast<uint32_t*>((keys ? k_store : v_store) + row_vec * F::kBytes);
    if (lane32 < F::kBytes / 4) dst[lane32] = pack[slot][lane32];
    h16* meta = keys ? k_meta : v_meta;
    if (lane32 == 0 && meta) meta[row_vec] = to_half(sigma);
}

// An FP8 store back to FP16, plus the reference key when given. A thread unpacks eight channels.
template <int kFmt>
__global__ __launch_bounds__(kBlock) void kv_dequant(const void* __restrict__ store, const h16* __restrict__ meta,
                                                     const h16* __restrict__ ref, h16* __restrict__ out,
                                                     int n_kv_heads, size_t n_slots) {
    static_assert(!KvFormat<kFmt>::kTq, "TurboQuant stores unpack through kv_dequant_tq");
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_slots) return;
    // FP32 until the one rounding of the output (an FP8 value is exact in FP16 either way)
    float f[8];
    const h16x8 h = __builtin_bit_cast(h16x8, load_slot<kFmt>(store, meta, nullptr, i / (kD / 8), (int)(i % (kD / 8))));
#pragma unroll
    for (int c = 0; c < 8; ++c) f[c] = (float)h[c];
    if (ref) {
        const int head = (int)((i / (kD / 8)) % n_kv_heads), slot = (int)(i % (kD / 8));
        const h16x8 r = *(reinterpret_cast<const h16x8*>(ref) + head * (kD / 8) + slot);
#pragma unroll
        for (int c = 0; c < 8; ++c) f[c] += (float)r[c];
    }
    h16x8 val;
#pragma unroll
    for (int c = 0; c < 8; ++c) val[c] = to_half(f[c]);
    *(reinterpret_cast<h16x8*>(out) + i) = val;
}

// A TurboQuant store back to FP16 in the ORIGINAL space: RMS times level, the
// inverse rotation, plus the reference key when given, one rounding at the end
// (kv_quant.cu:311-338). 32 lanes share a vector, four channels each, as in the store.
template <int kFmt>
__global__ __launch_bounds__(kBlock) void kv_dequant_tq(const void* __restrict__ store, const h16* __restrict__ meta,
                                                        const h16* __restrict__ ref, h16* __restrict__ out,
                                                        int n_kv_heads, size_t n_vectors) {
    typedef KvFormat<kFmt> F;
    __shared__ float lev[16];
    if (threadIdx.x < 16) lev[threadIdx.x] = kTqLevels[kFmt - kFmtTq4][threadIdx.x];
    __syncthreads();
    const size_t at = (size_t)blockIdx.x * (kBlock / 32) + threadIdx.x / 32;
    const size_t vec = at < n_vectors ? at : n_vectors - 1;          // every lane takes part in the exchange
    const int lane32 = (int)threadIdx.x & 31;
    constexpr int kLaneBits = F::kSlotBits / 2;
    const uint32_t* words = reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(store) + vec * F::kBytes);
    const uint32_t bits = stream_bits(words, F::kBytes / 4, lane32 * kLaneBits, kLaneBits);
    const float sigma = (float)meta[vec];
    float v[4];
#pragma unroll
    for (int c = 0; c < 4 / F::kPerCode; ++c) {
#pragma clang fp contract(off)       // rounded products: the butterfly's first additions must not fuse with them
        const uint32_t code = (bits >> (F::kCodeBits * c)) & ((1u << F::kCodeBits) - 1u);
        if constexpr (F::kPerCode == 1) {
            v[c] = sigma * lev[code];
        } else {
            v[2 * c] = sigma * lev[2 * code];
            v[2 * c + 1] = sigma * lev[2 * code + 1];
        }
    }
    tq_rotate(v, lane32, true);
    if (ref) {
        const h16x4 r = *reinterpret_cast<const h16x4*>(ref + (vec % n_kv_heads) * kD + 4 * lane32);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] += (float)r[c];
    }
    if (at < n_vectors)
        *reinterpret_cast<h16x4*>(out + vec * kD + 4 * lane32) =
            h16x4{to_half(v[0]), to_half(v[1]), to_half(v[2]), to_half(v[3])};
}

struct PageIds { int id[32]; };
__global__ void page_map(int* table, int first, int n, PageIds ids) {
    const int i = (int)threadIdx.x;
    if (i < n) table[first + i] = ids.id[i];
}

// Slices of the decode: one per 64 keys, rounded up to a power of two between 16 and 256. The
// floor of 16 keeps the launch shape still over the first 1024 positions (a captured decode step
// is re-made when the shape moves; the reference's shape moves every 1024 positions too, and its
// own test of the device-side length holds a backend to that, tests/test_decode_position.c:213-218).
constexpr int kMinParts = 16;
int decode_parts(int cache_len) {
    int want = (cache_len + kKeyTile - 1) / kKeyTile, n = kMinParts;
    while (n < want && n < kMaxParts) n *= 2;
    return n;
}

// Slices of the streaming decode (FP16 caches): as many workgroups as the chip has compute units
// (one slice per 64 keys until then), never more slices than the packed formats' kernel would use, so
// the partial-state buffer of vv_attn_scratch_bytes() holds either.
int stream_parts(int cache_len, int n_kv_heads) {
    static const int wgs = [] {
        const char* e = getenv("VV_DEC_WGS");
        const int v = e ? atoi(e) : 0;
        return v > 0 ? v : 256;
    }();
    int most = kMinParts;
    while (most * n_kv_heads < wgs && most < kMaxParts) most *= 2;
    const int n = decode_parts(cache_len);
    return n < most ? n : most;
}

bool fp8_format(int kv_format) { return kv_format == kFmtE4M3 || kv_format == kFmtE5M2; }
bool tq_format(int kv_format) { return kv_format >= kFmtTq4 && kv_format <= kFmtTq15; }
bool packed_format(int kv_format) { return fp8_format(kv_format) || tq_format(kv_format); }
bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

// One kernel instance per packed cache format.
#define VV_FOR_PACKED_FORMAT(fmt, CALL)                 \
    switch (fmt) {                                      \
        case kFmtE4M3: CALL(kFmtE4M3); break;           \
        case kFmtE5M2: CALL(kFmtE5M2); break;           \
        case kFmtTq4: CALL(kFmtTq4); break;             \
        case kFmtTq3: CALL(kFmtTq3); break;             \
        case kFmtTq2: CALL(kFmtTq2); break;             \
        default: CALL(kFmtTq15); break;                 \
    }

// What a packed format needs of a view: head_dim 128, 16-byte aligned Q / O, stores aligned to
// their unit (8 bytes of FP8 codes per slot, 32-bit words of TurboQuant codes) and, for
// TurboQuant, the per-vector RMS arrays.
bool packed_view_ok(const vv_kv_view_t* kv) {
    if (kv->head_dim != kD) return false;
    if (fp8_format(kv->format)) return aligned8(kv->k) && aligned8(kv->v);
    return aligned4(kv->k) && aligned4(kv->v) && kv->k_meta && kv->v_meta;
}

bool shape_ok(int n_q_heads, int n_kv_heads, int head_dim) {
    return n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0 && head_dim > 0 &&
           head_dim <= 256;
}

// Whether a decode over this view runs decode128 (and, past 1024 positions, needs the
// partial-state buffer) rather than the wave-per-head kernel.
bool decode_on_matrix_cores(const void* q, const vv_kv_view_t* kv) {
    return packed_format(kv->format) ||
           (kv->head_dim == kD && aligned16(q) && aligned16(kv->k) && aligned16(kv->v));
}

}  // namespace
}  // namespace vv

extern "C" {

/* One implementation serves every backend name: what differs between fa1,
 * fa2 and flashinfer on the reference's CUDA side is how the card is used,
 * not the result. FP16 caches, and FP8 / TurboQuant ones at head_dim 128,
 * contiguous or paged. */
int vv_attn_resolve(int requested, int kv_format, bool paged, int n_q_heads, int n_kv_heads,
                    int head_dim) {
    enum { kAuto = 0, kFa1 = 1, kFa2 = 2, kFlashinfer = 3 };
    const bool served = kv_format == vv::kFormatFp16 || (vv::packed_format(kv_format) && head_dim == vv::kD);
    if (!served || !vv::shape_ok(n_q_heads, n_kv_heads, head_dim)) return kFa1;
    if (requested == kFlashinfer) return kFlashinfer;
    if (requested == kFa1 && !paged) return kFa1;
    return kFa2;
}

size_t vv_attn_scratch_bytes(int n_q_heads, int n_kv_heads, int head_dim) {
    (void)n_kv_heads;
    if (n_q_heads <= 0 || head_dim <= 0) return 0;
    // per query head: the decode's slices, or the (rows x key runs) of a short prefill split over the keys
    constexpr size_t kRecords = vv::kMaxParts > vv::kPrefillSplitRows ? vv::kMaxParts : vv::kPrefillSplitRows;
    return (size_t)n_q_heads * kRecords * ((size_t)head_dim + 4) * sizeof(float);
}

int vv_attn_decode_shape(int backend, int n_q_heads, int n_kv_heads, int cache_len) {
    (void)backend; (void)n_q_heads; (void)n_kv_heads;
    return vv::decode_parts(cache_len);
}

vv_status_t vv_attn_prefill(int backend, const void* q, const vv_kv_view_t* kv, void* out,
                            int n_q_heads, int q_len, int q_offset, int kv_len, bool causal,
                            void* scratch, void* stream) {
    (void)backend;
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (q_len <= 0 || kv_len <= 0) return VV_OK;
    if (!kv->k || !kv->v) return VV_ERR_NULL_PTR;
    const bool packed = vv::packed_format(kv->format);
    if (kv->format != vv::kFormatFp16 && !packed) return VV_ERR_UNSUPPORTED;
    if (!vv::shape_ok(n_q_heads, kv->n_kv_heads, kv->head_dim)) return VV_ERR_UNSUPPORTED;
    if (packed && (!vv::packed_view_ok(kv) || !vv::aligned16(q) || !vv::aligned16(out))) return VV_ERR_UNSUPPORTED;
    if (q_offset < 0) return VV_ERR_INVALID_ARG;
    hipStream_t st = vv::as_stream(stream);
    const float scale_log2 = vv::kLog2e / sqrtf((float)kv->head_dim);
    const vv::h16* Q = static_cast<const vv::h16*>(q);
    const vv::h16* K = static_cast<const vv::h16*>(kv->k);
    const vv::h16* V = static_cast<const vv::h16*>(kv->v);
    vv::h16* O = static_cast<vv::h16*>(out);
    const vv::KvSource src = {kv->k, kv->v, static_cast<const vv::h16*>(kv->k_meta),
                              static_cast<const vv::h16*>(kv->v_meta), kv->page_table};
    // A/B aid for the parity tests: the plain tile kernel on an FP16 cache (same bits as the pipelined one).
    const char* force_tile = getenv("VV_ATTN_PREFILL_TILE");
    const bool tile_fp16 = !packed && force_tile && force_tile[0] == '1' && kv->head_dim == vv::kD &&
                           vv::aligned16(q) && vv::aligned16(kv->k) && vv::aligned16(kv->v) && vv::aligned16(out);
    if (tile_fp16) {
        const dim3 grid((unsigned)((q_len + vv::kQTile - 1) / vv::kQTile), (unsigned)n_q_heads);
        vv::prefill128<vv::kFmtFp16><<<grid, vv::kBlock, 0, st>>>(Q, src, O, n_q_heads, kv->n_kv_heads, q_len,
                                                                  q_offset, kv_len, causal ? 1 : 0, scale_log2);
    } else if (packed) {
        const dim3 grid((unsigned)((q_len + vv::kQTile - 1) / vv::kQTile), (unsigned)n_q_heads);
#define VV_PREFILL(F)                                                                                          \
    vv::prefill128<vv::F><<<grid, vv::kBlock, 0, st>>>(Q, src, O, n_q_heads, kv->n_kv_heads, q_len, q_offset, \
                                                       kv_len, causal ? 1 : 0, scale_log2)
        using namespace vv;
        VV_FOR_PACKED_FORMAT(kv->format, VV_PREFILL)
#undef VV_PREFILL
    } else if (kv->head_dim == vv::kD && vv::aligned16(q) && vv::aligned16(kv->k) && vv::aligned16(kv->v) &&
               vv::aligned16(out)) {
        const int row_tiles = (q_len + vv::kQTile - 1) / vv::kQTile;
        const int groups = kv->n_kv_heads * row_tiles;                                   // see the kernel's numbering
        const unsigned gx = (unsigned)(8 * ((groups + 7) / 8) * (n_q_heads / kv->n_kv_heads));
        // Few rows against many keys: the keys are cut into runs, as many as give every compute unit two
        // workgroups, as the caller's scratch holds, and as leave a run eight tiles or more.
        const int key_tiles = ((causal ? std::min(kv_len, q_offset + q_len) : kv_len) + vv::kKeyTile - 1) / vv::kKeyTile;
        int runs = 1;
        if (scratch && vv::aligned16(scratch) && q_len <= vv::kPrefillSplitRows)
            runs = std::min(std::min(512 / (row_tiles * n_q_heads), 16),
                            std::min(vv::kPrefillSplitRows / q_len, key_tiles / 8));
        if (runs >= 2) {
            int per = (key_tiles + runs - 1) / runs;
            per += per & 1;                                        // whole pairs of tiles: the loop is unrolled by two
            runs = (key_tiles + per - 1) / per;
            float* parts = static_cast<float*>(scratch);
            const unsigned gsplit = (unsigned)(8 * ((groups * runs + 7) / 8) * (n_q_heads / kv->n_kv_heads));
            vv::prefill_pipe<true><<<dim3(gsplit), vv::kBlock, 0, st>>>(
                Q, K, V, kv->page_table, O, n_q_heads, kv->n_kv_heads, q_len, q_offset, kv_len, causal ? 1 : 0,
                scale_log2, parts, runs, per);
            if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
            const int items = q_len * n_q_heads;
            vv::prefill_merge<<<dim3((unsigned)((items + vv::kWavesPerBlock - 1) / vv::kWavesPerBlock)), vv::kBlock, 0,
                                st>>>(parts, O, items, runs);
        } else {
            vv::prefill_pipe<false><<<dim3(gx), vv::kBlock, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads,
                                                                     kv->n_kv_heads, q_len, q_offset, kv_len,
                                                                     causal ? 1 : 0, scale_log2, nullptr, 1, 0);
        }
    } else {
        const dim3 grid((unsigned)q_len, (unsigned)n_q_heads);
        vv::rows_generic<<<grid, vv::kWave, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads,
                                                     kv->n_kv_heads, kv->head_dim, q_len, q_offset,
                                                     kv_len, nullptr, causal ? 1 : 0, scale_log2);
    }
    return vv::launch_status();
}

}  // extern "C" (reopened below)

namespace vv {
namespace {

// The split decode: decode128 over the slices, then decode_merge. `parts` holds
// the slices' partial states (vv_attn_scratch_bytes() of device memory); every
// (head, slice) record the merge reads is written by decode128 in the same call,
// empty slices included, so the buffer needs no clearing between calls.
vv_status_t attn_decode_launch(const void* q, const vv_kv_view_t* kv, void* out, int n_q_heads,
                               int cache_len, const int* d_cache_len, float* parts,
                               hipStream_t st) {
    const bool packed = packed_format(kv->format);
    const float scale_log2 = kLog2e / sqrtf((float)kv->head_dim);
    const h16* Q = static_cast<const h16*>(q);
    const h16* K = static_cast<const h16*>(kv->k);
    const h16* V = static_cast<const h16*>(kv->v);
    h16* O = static_cast<h16*>(out);
    const KvSource src = {kv->k, kv->v, static_cast<const h16*>(kv->k_meta),
                          static_cast<const h16*>(kv->v_meta), kv->page_table};
    const int q_group = n_q_heads / kv->n_kv_heads;
    if (!packed && q_group <= 16 && decode_on_matrix_cores(q, kv)) {
        if (!parts) return VV_ERR_NULL_PTR;
        const int n_parts = stream_parts(cache_len, kv->n_kv_heads);
        const dim3 grid((unsigned)n_parts, (unsigned)kv->n_kv_heads);
        if (q_group <= 8)
            decode_stream<8><<<grid, kStreamThreads, 0, st>>>(Q, K, V, kv->page_table, parts, n_q_heads, kv->n_kv_heads,
                                                             cache_len, d_cache_len, n_parts, scale_log2);
        else
            decode_stream<16><<<grid, kStreamThreads, 0, st>>>(Q, K, V, kv->page_table, parts, n_q_heads, kv->n_kv_heads,
                                                              cache_len, d_cache_len, n_parts, scale_log2);
        if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
        decode_merge<<<dim3((unsigned)n_q_heads), kMergeThreads, 0, st>>>(parts, O, n_parts);
    } else if (decode_on_matrix_cores(q, kv)) {
        const int n_parts = decode_parts(cache_len);
        if (n_parts > 1 && !parts) return VV_ERR_NULL_PTR;
        const int group = n_q_heads / kv->n_kv_heads;
        const dim3 grid((unsigned)n_parts, (unsigned)kv->n_kv_heads, (unsigned)((group + 31) / 32));
#define VV_DECODE(F)                                                                                  \
    decode128<F><<<grid, kWave, 0, st>>>(Q, src, O, parts, n_q_heads, kv->n_kv_heads, cache_len,     \
                                         d_cache_len, n_parts, scale_log2)
        if (packed) {
            VV_FOR_PACKED_FORMAT(kv->format, VV_DECODE)
        } else {
            VV_DECODE(kFmtFp16);
        }
#undef VV_DECODE
        if (n_parts > 1) {
            if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
            decode_merge<<<dim3((unsigned)n_q_heads), kMergeThreads, 0, st>>>(parts, O, n_parts);
        }
    } else {
        // One row: position cache_len - 1 sees everything, so no mask is needed.
        const dim3 grid(1u, (unsigned)n_q_heads);
        rows_generic<<<grid, kWave, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads, kv->n_kv_heads,
                                             kv->head_dim, 1, 0, cache_len, d_cache_len, 0, scale_log2);
    }
    return launch_status();
}

// Argument checks shared by the two decode entry points; VV_OK means "launch".
vv_status_t attn_decode_check(const void* q, const vv_kv_view_t* kv, const void* out, int n_q_heads) {
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (!kv->k || !kv->v) return VV_ERR_NULL_PTR;
    const bool packed = packed_format(kv->format);
    if (kv->format != kFormatFp16 && !packed) return VV_ERR_UNSUPPORTED;
    if (!shape_ok(n_q_heads, kv->n_kv_heads, kv->head_dim)) return VV_ERR_UNSUPPORTED;
    if (packed && (!packed_view_ok(kv) || !aligned16(q))) return VV_ERR_UNSUPPORTED;
    return VV_OK;
}

// ── the library's own partial-state buffer, for callers that cannot allocate ──
// One array per GPU the library runs on, held until the process ends. In host
// code the array's name is only a handle for hipGetSymbolAddress: the device
// address is looked up once per device (with that device current) and only that
// address is ever handed to a kernel.
constexpr int kStaticMaxQHeads = VV_ATTN_DECODE_STATIC_MAX_Q_HEADS;
constexpr size_t kStaticFloats = (size_t)kStaticMaxQHeads * kMaxParts * kPartFloats;   // 8.25 MiB
static __device__ __align__(256) float scratch[kStaticFloats];

constexpr int kMaxDevices = 64;
std::atomic<float*> g_scratch_ptr[kMaxDevices];

// The array of the device the stream belongs to (the current device for the default stream), which must be the
// current device: a symbol's address can only be asked of the current device.
float* static_scratch(hipStream_t st) {
    int dev = -1, stream_dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    if (st && hipStreamGetDevice(st, &stream_dev) == hipSuccess && stream_dev != dev) return nullptr;
    float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
            (void)hipGetLastError();
            return nullptr;
        }
        p = static_cast<float*>(sym);      // every thread that races here finds the same address
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    return p;
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_attn_decode(int backend, const void* q, const vv_kv_view_t* kv, void* out,
                           int n_q_heads, int cache_len, const int* d_cache_len, void* scratch,
                           void* stream) {
    (void)backend;
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (cache_len <= 0) return VV_OK;
    const vv_status_t rc = vv::attn_decode_check(q, kv, out, n_q_heads);
    if (rc != VV_OK) return rc;
    return vv::attn_decode_launch(q, kv, out, n_q_heads, cache_len, d_cache_len,
                                  static_cast<float*>(scratch), vv::as_stream(stream));
}

/* vv_attn_decode with the slices' partial states in the library's own
 * file-scope device array instead of a caller's buffer: no hipMalloc, hipFree
 * or other allocating call, here or below. */
vv_status_t vv_attn_decode_static(int backend, const void* q, const vv_kv_view_t* kv, void* out,
                                  int n_q_heads, int cache_len, const int* d_cache_len,
                                  void* stream) {
    (void)backend;
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (cache_len <= 0) return VV_OK;
    const vv_status_t rc = vv::attn_decode_check(q, kv, out, n_q_heads);
    if (rc != VV_OK) return rc;
    float* parts = nullptr;
    if (vv::decode_on_matrix_cores(q, kv) && vv::decode_parts(cache_len) > 1) {
        // the partial states are [n_q_heads][slices][head_dim + 4] floats, head_dim 128 on this path
        if (n_q_heads > vv::kStaticMaxQHeads) return VV_ERR_INVALID_ARG;
        parts = vv::static_scratch(vv::as_stream(stream));
        if (!parts) return VV_ERR_CUDA;
    }
    return vv::attn_decode_launch(q, kv, out, n_q_heads, cache_len, d_cache_len, parts,
                                  vv::as_stream(stream));
}

/* The older entry points for raw FP16 caches (device.h:621-655): the same
 * kernels, the cache given as two pointers instead of a view. */
size_t vv_gqa_decode_scratch_bytes(int n_q_heads, int head_dim) {      // the decode's slices alone
    if (n_q_heads <= 0 || head_dim <= 0) return 0;
    return (size_t)n_q_heads * vv::kMaxParts * ((size_t)head_dim + 4) * sizeof(float);
}

int vv_gqa_decode_shape(int cache_len) { return vv::decode_parts(cache_len); }

vv_status_t vv_gqa_attention_decode_dev(const void* q, const void* k_cache, const void* v_cache,
                                        void* output, int n_q_heads, int n_kv_heads, int head_dim,
                                        int cache_len, const int* d_cache_len, void* scratch,
                                        void* stream) {
    const vv_kv_view_t view = {k_cache, v_cache, nullptr, nullptr, nullptr, vv::kFormatFp16, n_kv_heads,
                               head_dim};
    return vv_attn_decode(2, q, &view, output, n_q_heads, cache_len, d_cache_len, scratch, stream);
}

vv_status_t vv_gqa_attention_prefill_cached_dev(const void* q, const void* k_cache, const void* v_cache,
                                                void* output, int n_q_heads, int n_kv_heads,
                                                int head_dim, int q_len, int q_offset, int kv_len,
                                                bool causal, void* stream) {
    const vv_kv_view_t view = {k_cache, v_cache, nullptr, nullptr, nullptr, vv::kFormatFp16, n_kv_heads,
                               head_dim};
    return vv_attn_prefill(2, q, &view, output, n_q_heads, q_len, q_offset, kv_len, causal, nullptr,
                           stream);
}

vv_status_t vv_gqa_attention_prefill_dev(const void* q, const void* k, const void* v, void* output,
                                         int n_q_heads, int n_kv_heads, int head_dim, int seq_len,
                                         bool causal, void* stream) {
    return vv_gqa_attention_prefill_cached_dev(q, k, v, output, n_q_heads, n_kv_heads, head_dim, seq_len,
                                               0, seq_len, causal, stream);
}

vv_status_t vv_kv_store_dev(const void* k_fp16, const void* v_fp16, void* k_store, void* v_store,
                            void* k_meta, void* v_meta, void* k_ref, bool build_ref,
                            int n_kv_heads, int head_dim, int pos, const int* d_pos,
                            int n_positions, int kv_format, const int* page_table, void* stream) {
    if (!k_fp16 || !v_fp16 || !k_store || !v_store) return VV_ERR_NULL_PTR;
    if (kv_format != vv::kFormatFp16 && !vv::packed_format(kv_format)) return VV_ERR_UNSUPPORTED;
    if (n_kv_heads <= 0 || head_dim <= 0 || pos < 0) return VV_ERR_INVALID_ARG;
    if (n_positions <= 0) return VV_OK;
    if (vv::packed_format(kv_format)) {
        if (head_dim != vv::kD || !vv::aligned16(k_fp16) || !vv::aligned16(v_fp16) || (k_ref && !vv::aligned16(k_ref)))
            return VV_ERR_UNSUPPORTED;
        if (vv::fp8_format(kv_format) ? !(vv::aligned8(k_store) && vv::aligned8(v_store))
                                      : !(vv::aligned4(k_store) && vv::aligned4(v_store)))
            return VV_ERR_UNSUPPORTED;
        hipStream_t st = vv::as_stream(stream);
        if (k_ref && build_ref) {
            vv::kv_build_ref<<<dim3((unsigned)n_kv_heads), vv::kD, 0, st>>>(static_cast<const vv::h16*>(k_fp16),
                                                                           static_cast<vv::h16*>(k_ref), n_kv_heads,
                                                                           n_positions);
            if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
        }
        const size_t slots = (size_t)n_positions * n_kv_heads * (vv::kD / 8);
        const dim3 grid((unsigned)((slots + vv::kBlock - 1) / vv::kBlock), 2u);
        const vv::h16* K = static_cast<const vv::h16*>(k_fp16);
        const vv::h16* V = static_cast<const vv::h16*>(v_fp16);
        uint8_t* KS = static_cast<uint8_t*>(k_store);
        uint8_t* VS = static_cast<uint8_t*>(v_store);
        const vv::h16* R = static_cast<const vv::h16*>(k_ref);
        if (vv::tq_format(kv_format)) {
            constexpr int kPerBlock = vv::kBlock / 32;
            const dim3 tq_grid((unsigned)((n_positions * n_kv_heads + kPerBlock - 1) / kPerBlock), 2u);
            vv::h16* KM = static_cast<vv::h16*>(k_meta);
            vv::h16* VM = static_cast<vv::h16*>(v_meta);
#define VV_STORE(F)                                                                                            \
    vv::kv_store_tq<vv::F><<<tq_grid, vv::kBlock, 0, st>>>(K, V, KS, VS, KM, VM, R, n_kv_heads, pos, d_pos,     \
                                                           n_positions, page_table)
            switch (kv_format) {
                case vv::kFmtTq4: VV_STORE(kFmtTq4); break;
                case vv::kFmtTq3: VV_STORE(kFmtTq3); break;
                case vv::kFmtTq2: VV_STORE(kFmtTq2); break;
                default: VV_STORE(kFmtTq15); break;
            }
#undef VV_STORE
            return vv::launch_status();
        }
        if (kv_format == vv::kFmtE5M2)
            vv::kv_store_fp8<true><<<grid, vv::kBlock, 0, st>>>(K, V, KS, VS, R, n_kv_heads, pos, d_pos, n_positions,
                                                                page_table);
        else
            vv::kv_store_fp8<false><<<grid, vv::kBlock, 0, st>>>(K, V, KS, VS, R, n_kv_heads, pos, d_pos, n_positions,
                                                                 page_table);
        return vv::launch_status();
    }
    const int row = n_kv_heads * head_dim;
    const size_t n = (size_t)n_positions * row;
    if (row % 8 == 0 && n / 8 <= 0x7fffffffu && vv::aligned16(k_fp16) && vv::aligned16(v_fp16) &&
        vv::aligned16(k_store) && vv::aligned16(v_store)) {
        const int n_chunks = (int)(n / 8);
        vv::kv_store_fp16_chunks<<<dim3((unsigned)((n_chunks + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                                   vv::as_stream(stream)>>>(
            static_cast<const vv::Chunk*>(k_fp16), static_cast<const vv::Chunk*>(v_fp16),
            static_cast<vv::Chunk*>(k_store), static_cast<vv::Chunk*>(v_store), row / 8, pos, d_pos, n_chunks,
            page_table);
        return vv::launch_status();
    }
    vv::kv_store_fp16<<<dim3((unsigned)((n + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                        vv::as_stream(stream)>>>(
        static_cast<const vv::h16*>(k_fp16), static_cast<const vv::h16*>(v_fp16),
        static_cast<vv::h16*>(k_store), static_cast<vv::h16*>(v_store), row, pos, d_pos,
        n_positions, page_table);
    return vv::launch_status();
}

vv_status_t vv_kv_quant_store_dev(const void* k_fp16, const void* v_fp16, void* k_store, void* v_store,
                                  void* k_meta, void* v_meta, void* k_ref, bool build_ref, int n_kv_heads,
                                  int head_dim, int pos, const int* d_pos, int n_positions, int kv_format,
                                  void* stream) {
    if (kv_format == vv::kFormatFp16) return VV_ERR_UNSUPPORTED;
    return vv_kv_store_dev(k_fp16, v_fp16, k_store, v_store, k_meta, v_meta, k_ref, build_ref, n_kv_heads,
                           head_dim, pos, d_pos, n_positions, kv_format, nullptr, stream);
}

vv_status_t vv_kv_dequant_dev(const void* store, const void* meta, const void* ref, void* out_fp16,
                              int n_kv_heads, int head_dim, int n_pos, int kv_format, void* stream) {
    if (!store || !out_fp16) return VV_ERR_NULL_PTR;
    if (head_dim != vv::kD || !vv::packed_format(kv_format) || n_kv_heads <= 0) return VV_ERR_UNSUPPORTED;
    if (vv::tq_format(kv_format) && !meta) return VV_ERR_NULL_PTR;
    if (!(vv::fp8_format(kv_format) ? vv::aligned8(store) : vv::aligned4(store)) || !vv::aligned16(out_fp16) ||
        (ref && !vv::aligned16(ref)))
        return VV_ERR_UNSUPPORTED;
    if (n_pos <= 0) return VV_OK;
    hipStream_t st = vv::as_stream(stream);
    const vv::h16* M = static_cast<const vv::h16*>(meta);
    const vv::h16* R = static_cast<const vv::h16*>(ref);
    vv::h16* O = static_cast<vv::h16*>(out_fp16);
    const size_t vectors = (size_t)n_pos * n_kv_heads, slots = vectors * (vv::kD / 8);
    if (vv::tq_format(kv_format)) {
        const dim3 grid((unsigned)((vectors + vv::kBlock / 32 - 1) / (vv::kBlock / 32)));
        switch (kv_format) {
            case vv::kFmtTq4: vv::kv_dequant_tq<vv::kFmtTq4><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, vectors); break;
            case vv::kFmtTq3: vv::kv_dequant_tq<vv::kFmtTq3><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, vectors); break;
            case vv::kFmtTq2: vv::kv_dequant_tq<vv::kFmtTq2><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, vectors); break;
            default: vv::kv_dequant_tq<vv::kFmtTq15><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, vectors); break;
        }
    } else {
        const dim3 grid((unsigned)((slots + vv::kBlock - 1) / vv::kBlock));
        if (kv_format == vv::kFmtE4M3) vv::kv_dequant<vv::kFmtE4M3><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, slots);
        else vv::kv_dequant<vv::kFmtE5M2><<<grid, vv::kBlock, 0, st>>>(store, M, R, O, n_kv_heads, slots);
    }
    return vv::launch_status();
}

/* In-place randomised Hadamard transform of [rows][n_heads][128] FP16 (Q before attention over
 * a TurboQuant cache) and its inverse (O after it). */
static vv_status_t kv_rotate_entry(void* x_fp16, int n_heads, int head_dim, int rows, int inverse, void* stream) {
    if (!x_fp16) return VV_ERR_NULL_PTR;
    if (head_dim != vv::kD || !vv::aligned8(x_fp16)) return VV_ERR_UNSUPPORTED;
    if (n_heads <= 0 || rows <= 0) return VV_OK;
    const int n = rows * n_heads;
    constexpr int kPerBlock = vv::kBlock / 32;
    vv::kv_rotate<<<dim3((unsigned)((n + kPerBlock - 1) / kPerBlock)), vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<vv::h16*>(x_fp16), n, inverse);
    return vv::launch_status();
}

vv_status_t vv_kv_rotate_dev(void* x_fp16, int n_heads, int head_dim, int rows, void* stream) {
    return kv_rotate_entry(x_fp16, n_heads, head_dim, rows, 0, stream);
}

vv_status_t vv_kv_unrotate_dev(void* x_fp16, int n_heads, int head_dim, int rows, void* stream) {
    return kv_rotate_entry(x_fp16, n_heads, head_dim, rows, 1, stream);
}

vv_status_t vv_gqa_attention_decode_q_dev(const void* q, const void* k_store, const void* v_store,
                                          const void* k_meta, const void* v_meta, void* output,
                                          int n_q_heads, int n_kv_heads, int head_dim, int cache_len,
                                          const int* d_cache_len, int kv_format, void* scratch, void* stream) {
    if (!q || !k_store || !v_store || !output || !scratch) return VV_ERR_NULL_PTR;
    if (cache_len == 0) return VV_OK;
    if (head_dim != vv::kD || !vv::packed_format(kv_format)) return VV_ERR_UNSUPPORTED;
    const vv_kv_view_t view = {k_store, v_store, k_meta, v_meta, nullptr, kv_format, n_kv_heads, head_dim};
    return vv_attn_decode(2, q, &view, output, n_q_heads, cache_len, d_cache_len, scratch, stream);
}

vv_status_t vv_gqa_attention_prefill_q_dev(const void* q, const void* k_store, const void* v_store,
                                           const void* k_meta, const void* v_meta, void* output,
                                           int n_q_heads, int n_kv_heads, int head_dim, int q_len,
                                           int q_offset, int kv_len, bool causal, int kv_format, void* stream) {
    if (!q || !k_store || !v_store || !output) return VV_ERR_NULL_PTR;
    if (q_len == 0 || kv_len == 0) return VV_OK;
    if (head_dim != vv::kD || !vv::packed_format(kv_format)) return VV_ERR_UNSUPPORTED;
    const vv_kv_view_t view = {k_store, v_store, k_meta, v_meta, nullptr, kv_format, n_kv_heads, head_dim};
    return vv_attn_prefill(2, q, &view, output, n_q_heads, q_len, q_offset, kv_len, causal, nullptr, stream);
}

vv_status_t vv_kv_page_map_dev(int* page_table, int first, int n, const int* pages, void* stream) {
    if (n <= 0) return VV_OK;
    if (!page_table || !pages) return VV_ERR_NULL_PTR;
    if (first < 0) return VV_ERR_INVALID_ARG;
    // The ids travel as kernel arguments, 32 a launch: the host array is read
    // before this returns and the writes are ordered on the stream.
    for (int done = 0; done < n; done += 32) {
        vv::PageIds ids;
        const int m = n - done < 32 ? n - done : 32;
        for (int i = 0; i < 32; ++i) ids.id[i] = i < m ? pages[done + i] : 0;
        vv::page_map<<<1, 32, 0, vv::as_stream(stream)>>>(page_table, first + done, m, ids);
        if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
    }
    return VV_OK;
}

}  // extern "C"
