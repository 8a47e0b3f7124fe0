// Rotary position embedding (rotate-half pairing) on Q and K, in place.
//
// What is shared and what is streamed:
//   - cos/sin depend only on (position, pair index), not on the head. A
//     workgroup owns kPosPerBlock consecutive positions; its 256 threads first
//     compute those positions' head_dim/2 cosines and sines once into LDS
//     (LDS is justified here: every head of Q and K at that position reuses
//     the same 2 x 64 values), then stream the heads through.
//   - head_dim = 128 is 16 chunks; the pair (d, d+64) is chunk c with chunk
//     c+8, so a lane that loads chunks c and c+8 of one head rotates 8 pairs
//     without talking to any other lane. 28 Q heads + 4 K heads = 256 such
//     lane tasks per position: one per thread of the workgroup.
//   - frequencies: inv_freq[i] = powf(theta, -2i/head_dim) is computed on the
//     HOST with the C library's powf and passed by value in the kernel
//     arguments. The angle (float)pos * inv_freq reaches ~1e4 rad at long
//     prompts, where one FP32 ulp of the angle is ~1e-3 rad, so a frequency
//     that differs by one ulp from the CPU path's would be visible; the host
//     value is bit-identical to what the CPU kernels compute. The device then
//     forms the angle with one FP32 multiply and calls the full-range sincosf
//     (never the fast intrinsics, whose error grows with |angle|).
#include <math.h>

#include "row_math.hpp"

namespace vv {
namespace {

constexpr int kMaxPairs = 128;      // head_dim <= 256
constexpr int kPosPerBlock = 4;     // positions per workgroup in the head_dim-128 kernel

struct FreqTable {
    float f[kMaxPairs];
};

struct RopeArgs {
    h16* q;                 // [rows, nq, head_dim] or nullptr
    h16* k;                 // [rows, nk, head_dim] or nullptr
    const h16* q_bias;      // [nq * head_dim] or nullptr
    const h16* k_bias;      // [nk * head_dim] or nullptr
    const int* d_position;  // device int with the first row's position, or nullptr
    int rows, nq, nk, head_dim, position_offset;
};

__device__ __forceinline__ Chunk add_bias(const Chunk& v, const Chunk& b) {
    const f32x8 x = unpack(v), y = unpack(b);
    f32x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = x[i] + y[i];
    return pack(r);      // rounded to FP16 before the rotation, as bias_add then rope would
}

// head_dim == 128, 16-byte aligned tensors, at most kMaxFastHeads heads in all.
//
// A workgroup owns `posb` consecutive positions. Work item = (position, head,
// chunk pair); thread t takes items t, t+256, ... — kItems of them. For the
// 32 heads of Qwen2-7B's Q+K that is one position per workgroup and ONE item
// per thread: measured at T = 14449, 1 / 2 / 4 items per thread give 38.3 /
// 39.4 / 40.9 us — the memory system rewards many light workgroups — so more
// items per thread are used only when a position has more than 256 of them. Order inside the kernel: issue every global load of the
// thread's items first, THEN compute the cos/sin table (one (position, pair)
// per thread, full-range sincosf) and cross the barrier, so the memory latency
// runs under the transcendental work; then rotate and store.
constexpr int kMaxItems = 4;
constexpr int kMaxFastHeads = kMaxItems * kBlock / 8;   // 128: one position per workgroup

template <bool kBias, bool kStream, bool kExact, int kItems>   // kExact: 32 heads, 256 items per position
__global__ __launch_bounds__(kBlock) void rope128(RopeArgs a, FreqTable freqs, int posb) {
    __shared__ __attribute__((aligned(16))) float cs_cos[kPosPerBlock][64];
    __shared__ __attribute__((aligned(16))) float cs_sin[kPosPerBlock][64];

    const int first = a.d_position ? *a.d_position : a.position_offset;
    const int row0 = (int)blockIdx.x * posb;
    const int tasks = (a.nq + a.nk) * 8;            // (head, chunk pair) per position
    const int items = min(posb, a.rows - row0) * tasks;
    // Fetched before the tensor loads are issued: memory returns in issue order,
    // so waiting for this value later does not wait for the tensor data.
    float my_freq = freqs.f[threadIdx.x & 63];

    // Loads are unconditional (an item past the end re-reads the last valid
    // one and is simply not stored): straight-line code lets the compiler count
    // outstanding loads exactly instead of draining them all at the first use.
    Chunk* lo_p[kItems];
    Chunk lo[kItems], hi[kItems];
    int p_of[kItems], c_of[kItems];
    bool live[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int want = (int)threadIdx.x + k * kBlock;
        live[k] = want < items;
        const int item = live[k] ? want : items - 1;
        const int p = kExact ? item >> 8 : item / tasks;
        const int t = kExact ? item & 255 : item - p * tasks;
        const int head = t >> 3, c = t & 7;
        const size_t row = (size_t)(row0 + p);
        h16* base = head < a.nq
            ? a.q + (row * (size_t)a.nq + (size_t)head) * 128u
            : a.k + (row * (size_t)a.nk + (size_t)(head - a.nq)) * 128u;
        lo_p[k] = reinterpret_cast<Chunk*>(base) + c;
        lo[k] = load_chunk_as<kStream>(lo_p[k]);
        hi[k] = load_chunk_as<kStream>(lo_p[k] + 8);
        p_of[k] = p;
        c_of[k] = c;
        if (kBias) {
            const h16* bias = head < a.nq
                ? (a.q_bias ? a.q_bias + (size_t)head * 128u : nullptr)
                : (a.k_bias ? a.k_bias + (size_t)(head - a.nq) * 128u : nullptr);
            if (bias) {
                const Chunk* bp = reinterpret_cast<const Chunk*>(bias) + c;
                lo[k] = add_bias(lo[k], load_chunk(bp));
                hi[k] = add_bias(hi[k], load_chunk(bp + 8));
            }
        }
    }

    // Use point of my_freq, outside any branch, so its load stays where it was
    // written (ahead of the tensor loads) and only it is waited for here.
    asm volatile("" : "+v"(my_freq));

    if ((int)threadIdx.x < posb * 64) {      // thread t -> (position t / 64, pair t % 64)
        const int p = (int)threadIdx.x >> 6, i = (int)threadIdx.x & 63;
        const int pos = first + row0 + p;
        const float ang = (float)pos * my_freq;
        float s, c;
        sincosf(ang, &s, &c);
        cs_cos[p][i] = c;
        cs_sin[p][i] = s;
    }
    __syncthreads();

#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (live[k]) {
            const f32x8 x0 = unpack(lo[k]), x1 = unpack(hi[k]);
            const f32x8 cv = *reinterpret_cast<const f32x8*>(&cs_cos[p_of[k]][c_of[k] * 8]);
            const f32x8 sv = *reinterpret_cast<const f32x8*>(&cs_sin[p_of[k]][c_of[k] * 8]);
            f32x8 y0, y1;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const Pair r = rotate(x0[i], x1[i], cv[i], sv[i]);
                y0[i] = r.lo;
                y1[i] = r.hi;
            }
            store_chunk_as<kStream>(lo_p[k], pack(y0));
            store_chunk_as<kStream>(lo_p[k] + 8, pack(y1));
        }
    }
}

// head_dim == 128, at most 32 heads in all: ONE WAVE PER POSITION, for launches
// of a few thousand positions. With a workgroup per position a 2048-row prefill
// chunk is a bit more than one round of workgroups on the chip, each a
// load -> barrier -> store chain; here it is 2048 independent waves, all
// resident at once, with no LDS and no barrier. Lane l is (chunk pair c = l % 8,
// head group l / 8) and takes heads l / 8, l / 8 + 8, ... (four items for 32
// heads): its eight loads go out first; then the lane computes the cosine and
// sine of ONE pair index (l, of 64) and collects the eight it needs, pairs
// 8c .. 8c + 7, from lanes 8c .. 8c + 7 by cross-lane reads. Same angle, same
// sincosf, same unfused rotation as rope128: the same bits.
constexpr int kWaveItems = 4;

template <bool kBias, bool kStream>
__global__ __launch_bounds__(kBlock) void rope128_wave(RopeArgs a, FreqTable freqs) {
    const int row = (int)blockIdx.x * ((int)blockDim.x >> 6) + wave_in_block();
    if (row >= a.rows) return;                    // whole waves leave; nothing below synchronises
    const int lane = lane_id(), c = lane & 7, hg = lane >> 3;
    const int heads = a.nq + a.nk;
    const int first = a.d_position ? *a.d_position : a.position_offset;
    float my_freq = freqs.f[lane];

    Chunk* lo_p[kWaveItems];
    Chunk lo[kWaveItems], hi[kWaveItems];
    bool live[kWaveItems];
#pragma unroll
    for (int k = 0; k < kWaveItems; ++k) {
        const int want = hg + 8 * k;
        live[k] = want < heads;
        const int head = live[k] ? want : heads - 1;
        h16* base = head < a.nq
            ? a.q + ((size_t)row * (size_t)a.nq + (size_t)head) * 128u
            : a.k + ((size_t)row * (size_t)a.nk + (size_t)(head - a.nq)) * 128u;
        lo_p[k] = reinterpret_cast<Chunk*>(base) + c;
        lo[k] = load_chunk_as<kStream>(lo_p[k]);
        hi[k] = load_chunk_as<kStream>(lo_p[k] + 8);
        if (kBias) {
            const h16* bias = head < a.nq
                ? (a.q_bias ? a.q_bias + (size_t)head * 128u : nullptr)
                : (a.k_bias ? a.k_bias + (size_t)(head - a.nq) * 128u : nullptr);
            if (bias) {
                const Chunk* bp = reinterpret_cast<const Chunk*>(bias) + c;
                lo[k] = add_bias(lo[k], load_chunk(bp));
                hi[k] = add_bias(hi[k], load_chunk(bp + 8));
            }
        }
    }
    asm volatile("" : "+v"(my_freq));             // the frequency is waited for here, not the tensor data

    float my_s, my_c;
    sincosf((float)(first + row) * my_freq, &my_s, &my_c);
    f32x8 cv, sv;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        cv[i] = __shfl(my_c, 8 * c + i);
        sv[i] = __shfl(my_s, 8 * c + i);
    }
#pragma unroll
    for (int k = 0; k < kWaveItems; ++k) {
        if (live[k]) {
            const f32x8 x0 = unpack(lo[k]), x1 = unpack(hi[k]);
            f32x8 y0, y1;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const Pair r = rotate(x0[i], x1[i], cv[i], sv[i]);
                y0[i] = r.lo;
                y1[i] = r.hi;
            }
            store_chunk_as<kStream>(lo_p[k], pack(y0));
            store_chunk_as<kStream>(lo_p[k] + 8, pack(y1));
        }
    }
}

// Any even head_dim <= 256, any alignment: one workgroup per position,
// 2-byte accesses.
__global__ __launch_bounds__(kBlock) void rope_generic(RopeArgs a, FreqTable freqs) {
    __shared__ float cs_cos[kMaxPairs];
    __shared__ float cs_sin[kMaxPairs];
    const int half = a.head_dim / 2;
    const int first = a.d_position ? *a.d_position : a.position_offset;
    const size_t row = blockIdx.x;
    const int pos = first + (int)row;
    for (int i = (int)threadIdx.x; i < half; i += kBlock) {
        const float ang = (float)pos * freqs.f[i];
        float s, c;
        sincosf(ang, &s, &c);
        cs_cos[i] = c;
        cs_sin[i] = s;
    }
    __syncthreads();
    const int heads = a.nq + a.nk;
    const int tasks = heads * half;
    for (int t = (int)threadIdx.x; t < tasks; t += kBlock) {
        const int head = t / half, i = t - head * half;
        h16* v;
        const h16* bias = nullptr;
        if (head < a.nq) {
            v = a.q + (row * (size_t)a.nq + (size_t)head) * (size_t)a.head_dim;
            if (a.q_bias) bias = a.q_bias + (size_t)head * (size_t)a.head_dim;
        } else {
            v = a.k + (row * (size_t)a.nk + (size_t)(head - a.nq)) * (size_t)a.head_dim;
            if (a.k_bias) bias = a.k_bias + (size_t)(head - a.nq) * (size_t)a.head_dim;
        }
        h16 h0 = v[i], h1 = v[i + half];
        if (bias) {
            h0 = to_half((float)h0 + (float)bias[i]);
            h1 = to_half((float)h1 + (float)bias[i + half]);
        }
        const float x0 = (float)h0, x1 = (float)h1;
        const float c = cs_cos[i], s = cs_sin[i];
        const Pair r = rotate(x0, x1, c, s);
        v[i] = to_half(r.lo);
        v[i + half] = to_half(r.hi);
    }
}

// The cosines and sines of a run of positions, once for every layer that rotates at those
// positions: table[row][i] = {cos, sin}((float)(first + row) * inv_freq[i]), i < head_dim / 2 -
// the angle and the sincosf of the rope kernels, so a rotation that reads the table gives their bits.
__global__ __launch_bounds__(kBlock) void rope_table(float2* __restrict__ table, int rows, int half,
                                                     int position_offset, const int* __restrict__ d_position,
                                                     FreqTable freqs) {
    const int idx = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (idx >= rows * half) return;
    const int row = idx / half, i = idx - row * half;
    const int first = d_position ? *d_position : position_offset;
    float s, c;
    sincosf((float)(first + row) * freqs.f[i], &s, &c);
    table[idx] = make_float2(c, s);
}

// x[row][head][:] = rope(x (+ bias)) with cos/sin read from such a table: the form of
// vv_bias_rope_qk_dev for callers that hold one. One thread per (row, head, chunk pair), head_dim 128.
__global__ __launch_bounds__(kBlock) void rope128_from_table(h16* __restrict__ x, const h16* __restrict__ bias,
                                                             const float2* __restrict__ table, int rows,
                                                             int heads) {
    const size_t item = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (item >= (size_t)rows * heads * 8) return;
    const int c = (int)(item & 7);
    const size_t rh = item >> 3;
    const int head = (int)(rh % heads);
    const size_t row = rh / heads;
    Chunk* lo_p = reinterpret_cast<Chunk*>(x + rh * 128u) + c;
    Chunk lo = load_chunk(lo_p), hi = load_chunk(lo_p + 8);
    if (bias) {
        const Chunk* bp = reinterpret_cast<const Chunk*>(bias + (size_t)head * 128u) + c;
        lo = add_bias(lo, load_chunk(bp));
        hi = add_bias(hi, load_chunk(bp + 8));
    }
    const float2* t = table + row * 64 + c * 8;
    const f32x8 x0 = unpack(lo), x1 = unpack(hi);
    f32x8 y0, y1;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float2 cs = t[i];
        const Pair r = rotate(x0[i], x1[i], cs.x, cs.y);
        y0[i] = r.lo;
        y1[i] = r.hi;
    }
    store_chunk(lo_p, pack(y0));
    store_chunk(lo_p + 8, pack(y1));
}

// The same rotation of two tensors in one launch (the q and k rows of a chunk): head h < heads_a is a's, the rest b's.
__global__ __launch_bounds__(kBlock) void rope128_pair_from_table(h16* __restrict__ a, h16* __restrict__ b,
                                                                  const float2* __restrict__ table, int rows,
                                                                  int heads_a, int heads_b) {
    const size_t item = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const int heads = heads_a + heads_b;
    if (item >= (size_t)rows * heads * 8) return;
    const int c = (int)(item & 7);
    const size_t rh = item >> 3;
    const int head = (int)(rh % heads);
    const size_t row = rh / heads;
    h16* x = head < heads_a ? a + (row * heads_a + head) * 128u : b + (row * heads_b + (head - heads_a)) * 128u;
    Chunk* lo_p = reinterpret_cast<Chunk*>(x) + c;
    const Chunk lo = load_chunk(lo_p), hi = load_chunk(lo_p + 8);
    const float2* t = table + row * 64 + c * 8;
    const f32x8 x0 = unpack(lo), x1 = unpack(hi);
    f32x8 y0, y1;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float2 cs = t[i];
        const Pair r = rotate(x0[i], x1[i], cs.x, cs.y);
        y0[i] = r.lo;
        y1[i] = r.hi;
    }
    store_chunk(lo_p, pack(y0));
    store_chunk(lo_p + 8, pack(y1));
}

// The table depends only on (theta, head_dim); each host thread remembers the
// last one it built (thread-local, so concurrent callers never share state).
const FreqTable& host_freqs(float theta, int head_dim) {
    thread_local FreqTable table;
    thread_local float cached_theta = 0.0f;
    thread_local int cached_dim = 0;
    if (cached_dim != head_dim || cached_theta != theta) {
        const int half = head_dim / 2;
        for (int i = 0; i < kMaxPairs; ++i)
            table.f[i] = i < half ? powf(theta, -2.0f * (float)i / (float)head_dim) : 0.0f;
        cached_theta = theta;
        cached_dim = head_dim;
    }
    return table;
}

vv_status_t launch_rope(void* q, void* k, const void* q_bias, const void* k_bias, int rows,
                        int nq, int nk, int head_dim, int position_offset,
                        const int* d_position, float theta, hipStream_t st) {
    if (!q) nq = 0;
    if (!k) nk = 0;
    if (nq < 0 || nk < 0) return VV_ERR_INVALID_ARG;
    if (rows <= 0 || nq + nk == 0 || head_dim <= 0) return VV_OK;
    if ((head_dim & 1) || head_dim > 2 * kMaxPairs) return VV_ERR_UNSUPPORTED;

    RopeArgs a;
    a.q = nq ? static_cast<h16*>(q) : nullptr;
    a.k = nk ? static_cast<h16*>(k) : nullptr;
    a.q_bias = nq ? static_cast<const h16*>(q_bias) : nullptr;
    a.k_bias = nk ? static_cast<const h16*>(k_bias) : nullptr;
    a.d_position = d_position;
    a.rows = rows; a.nq = nq; a.nk = nk; a.head_dim = head_dim;
    a.position_offset = position_offset;
    const FreqTable& freqs = host_freqs(theta, head_dim);
    const bool has_bias = a.q_bias || a.k_bias;

    const bool fast = head_dim == 128 && nq + nk <= kMaxFastHeads &&
                      (!a.q || aligned16(a.q)) && (!a.k || aligned16(a.k)) &&
                      (!a.q_bias || aligned16(a.q_bias)) && (!a.k_bias || aligned16(a.k_bias));
    if (fast) {
        // items per thread: enough for one position, then as many positions per
        // workgroup as fit (at most kPosPerBlock); VV_ROPE_ITEMS=1|2|4 forces (A/B aid)
        static const int forced_items = [] {
            const char* e = getenv("VV_ROPE_ITEMS");
            const int v = e ? atoi(e) : 0;
            return (v == 1 || v == 2 || v == 4) ? v : 0;       // anything else: not forced
        }();
        const int tasks = (nq + nk) * 8;
        int items = forced_items ? forced_items : 1;
        while (items * kBlock < tasks) items *= 2;          // <= kMaxItems by the head limit
        if (items == 3) items = 4;
        int posb = items * kBlock / tasks;
        if (posb > kPosPerBlock) posb = kPosPerBlock;
        if (posb < 1) posb = 1;
        const dim3 grid((unsigned)((rows + posb - 1) / posb));
        const bool stream = use_streaming(2u * (size_t)rows * (size_t)(nq + nk) * 128u * 2u);
        const bool exact = (nq + nk) * 8 == kBlock;
        // A wave per position for launches that would otherwise be one to three rounds of
        // workgroups: measured cold at 28 + 4 heads, workgroup / wave per position:
        // 1024 rows 4.7 / 4.3 us, 2048 rows 7.7 / 7.1 us, 4096 rows 12.8 / 12.8 us,
        // 14449 rows 38.5 / 40.3 us. VV_ROPE_WAVE=0|1 forces.
        static const int forced_wave = [] {
            const char* e = getenv("VV_ROPE_WAVE");
            return (e && (e[0] == '0' || e[0] == '1')) ? e[0] - '0' : -1;
        }();
        const long eq_rows = (long)rows * (nq + nk) / 32;
        bool wave = eq_rows >= 768 && eq_rows <= 3584;
        if (forced_wave >= 0) wave = forced_wave == 1;
        if (wave && nq + nk <= 8 * kWaveItems && !forced_items) {
            const dim3 wgrid((unsigned)((rows + kWavesPerBlock - 1) / kWavesPerBlock));
            if (has_bias && stream)  rope128_wave<true, true><<<wgrid, kBlock, 0, st>>>(a, freqs);
            else if (has_bias)       rope128_wave<true, false><<<wgrid, kBlock, 0, st>>>(a, freqs);
            else if (stream)         rope128_wave<false, true><<<wgrid, kBlock, 0, st>>>(a, freqs);
            else                     rope128_wave<false, false><<<wgrid, kBlock, 0, st>>>(a, freqs);
            return launch_status();
        }
#define VV_ROPE_LAUNCH(B, S, E, I) rope128<B, S, E, I><<<grid, kBlock, 0, st>>>(a, freqs, posb)
#define VV_ROPE_ITEMS(B, S, E)                          \
    do {                                                \
        if (items == 1)      VV_ROPE_LAUNCH(B, S, E, 1); \
        else if (items == 2) VV_ROPE_LAUNCH(B, S, E, 2); \
        else                 VV_ROPE_LAUNCH(B, S, E, 4); \
    } while (0)
#define VV_ROPE_PICK(B, S) \
    do { if (exact) VV_ROPE_ITEMS(B, S, true); else VV_ROPE_ITEMS(B, S, false); } while (0)
        if (has_bias && stream)  VV_ROPE_PICK(true, true);
        else if (has_bias)       VV_ROPE_PICK(true, false);
        else if (stream)         VV_ROPE_PICK(false, true);
        else                     VV_ROPE_PICK(false, false);
#undef VV_ROPE_PICK
#undef VV_ROPE_ITEMS
#undef VV_ROPE_LAUNCH
    } else {
        rope_generic<<<dim3((unsigned)rows), kBlock, 0, st>>>(a, freqs);
    }
    return launch_status();
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_rope_dev(void* x, int seq_len, int n_heads, int head_dim, int position_offset,
                        const int* d_position, float theta, void* stream) {
    if (!x) return VV_ERR_NULL_PTR;
    return vv::launch_rope(x, nullptr, nullptr, nullptr, seq_len, n_heads, 0, head_dim,
                           position_offset, d_position, theta, vv::as_stream(stream));
}

vv_status_t vv_rope_qk_dev(void* q, void* k, int seq_len, int n_q_heads, int n_kv_heads,
                           int head_dim, int position_offset, const int* d_position, float theta,
                           void* stream) {
    if (!q && !k) return VV_ERR_NULL_PTR;
    return vv::launch_rope(q, k, nullptr, nullptr, seq_len, n_q_heads, n_kv_heads, head_dim,
                           position_offset, d_position, theta, vv::as_stream(stream));
}

vv_status_t vv_bias_rope_qk_dev(void* q, void* k, const void* q_bias, const void* k_bias,
                                int seq_len, int n_q_heads, int n_kv_heads, int head_dim,
                                int position_offset, const int* d_position, float theta,
                                void* stream) {
    if (!q && !k) return VV_ERR_NULL_PTR;
    return vv::launch_rope(q, k, q_bias, k_bias, seq_len, n_q_heads, n_kv_heads, head_dim,
                           position_offset, d_position, theta, vv::as_stream(stream));
}

vv_status_t vv_rope_table_dev(void* table, int seq_len, int head_dim, int position_offset,
                              const int* d_position, float theta, void* stream) {
    if (!table) return VV_ERR_NULL_PTR;
    if (seq_len <= 0 || head_dim <= 0) return VV_OK;
    if ((head_dim & 1) || head_dim > 2 * vv::kMaxPairs) return VV_ERR_UNSUPPORTED;
    if (reinterpret_cast<uintptr_t>(table) & 15u) return VV_ERR_UNSUPPORTED;    // its readers load 16 bytes at a time
    const int half = head_dim / 2;
    const size_t n = (size_t)seq_len * (size_t)half;
    vv::rope_table<<<dim3((unsigned)((n + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<float2*>(table), seq_len, half, position_offset, d_position, vv::host_freqs(theta, head_dim));
    return vv::launch_status();
}

}  // extern "C"

// For gemm.hip: a[rows][heads_a][128] and b[rows][heads_b][128] rotated in place in one launch, cos/sin from a
// vv_rope_table_dev table (16-byte aligned tensors, table rows 0 .. rows - 1).
__attribute__((visibility("hidden")))
vv_status_t vv_rope128_pair_from_table(void* a, void* b, const void* table, int rows, int heads_a, int heads_b,
                                       void* stream) {
    const size_t items = (size_t)rows * (size_t)(heads_a + heads_b) * 8u;
    vv::rope128_pair_from_table<<<dim3((unsigned)((items + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                                  vv::as_stream(stream)>>>(static_cast<vv::h16*>(a), static_cast<vv::h16*>(b),
                                                           static_cast<const float2*>(table), rows, heads_a, heads_b);
    return vv::launch_status();
}

// For gemm.hip: x[rows][heads][128] = rope(x + bias) with cos/sin from a vv_rope_table_dev table
// (16-byte aligned x and bias, table rows 0 .. rows - 1).
__attribute__((visibility("hidden")))
vv_status_t vv_rope128_from_table(void* x, const void* bias, const void* table, int rows, int heads, void* stream) {
    const size_t items = (size_t)rows * (size_t)heads * 8u;
    vv::rope128_from_table<<<dim3((unsigned)((items + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                             vv::as_stream(stream)>>>(static_cast<vv::h16*>(x), static_cast<const vv::h16*>(bias),
                                                      static_cast<const float2*>(table), rows, heads);
    return vv::launch_status();
}
