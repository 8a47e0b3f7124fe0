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
__device__ __forceinline__ float other_half(float v) { return __shfl_xor(v, 32); }

__device__ __forceinline__ int cache_row(const int* page_table, int t) {
    return page_table ? page_table[t / kPage] * kPage + t % kPage : t;
}

// ── head_dim 128 on the matrix cores: the pieces both forms share ─────────
constexpr int kD = 128;
constexpr int kQTile = 128;          // query rows per prefill workgroup (32 per wave)
constexpr int kKeyTile = 64;         // keys per LDS tile
constexpr int kVtStride = kKeyTile + 4;   // halves per transposed-V row: 136 B

struct KvTile {
    Chunk k[kKeyTile * (kD / 8)];                 // [key][16 slots], slot ^ (key & 15)
    __align__(16) h16 vt[kD * kVtStride];         // [channel][key]
};

// Per-lane state of one query row (lane % 32) over the keys seen so far: O^T
// register 4g + r of tile t is channel 32t + 8g + 4*(lane / 32) + r.
struct RowState {
    f32x16 o[kD / 32];
    float m, l;                                   // running max (base-2 domain) and sum
    __device__ __forceinline__ void reset() {
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[t][r] = 0.0f;
        m = -INFINITY;
        l = 0.0f;
    }
};

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

template <int kThreads>
__device__ __forceinline__ void fetch_tile(TileRegs<kThreads>& regs, const h16* __restrict__ Kc,
                                           const h16* __restrict__ Vc,
                                           const int* __restrict__ page_table, size_t kv_stride,
                                           int kvh, int t0, int last_key, int tid) {
    constexpr int kIter = TileRegs<kThreads>::kIter;
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
        const int q = tid + i * kThreads, r = q >> 4, slot = q & 15;
        const int row = cache_row(page_table, min(t0 + r, last_key));
        regs.k[i] = load_chunk(reinterpret_cast<const Chunk*>(Kc + (size_t)row * kv_stride + kvh * kD) + slot);
    }
#pragma unroll
    for (int i = 0; i < kIter / 4; ++i) {
        const int q = tid + i * kThreads, dchunk = q & 15, kg = q >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = cache_row(page_table, min(t0 + 4 * kg + j, last_key));
            regs.v[4 * i + j] =
                load_chunk(reinterpret_cast<const Chunk*>(Vc + (size_t)row * kv_stride + kvh * kD) + dchunk);
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
// reads of V^T below. O is rescaled only when some row's maximum moved (after
// the first few tiles it rarely does): the factor is exactly 1 otherwise.
__device__ __forceinline__ void tile_update(const KvTile& tile, f32x16 (&s)[2], RowState& st,
                                            int col, int half, float scale_log2) {
    float mx = -INFINITY;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[a][r]);
    mx = fmaxf(mx, other_half(mx)) * scale_log2;
    const float m_new = fmaxf(st.m, mx);
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;
    float sum = 0.0f;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = exp2_fast(fmaf(s[a][r], scale_log2, -m_use));
            s[a][r] = p;
            sum += p;
        }
    sum += other_half(sum);
    if (__builtin_amdgcn_ballot_w64(m_new > st.m) != 0) {
        const float alpha = exp2_fast(st.m - m_use);
        st.l *= alpha;
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) st.o[t][r] *= alpha;
    }
    st.l += sum;
    st.m = m_new;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int a = u >> 1, sp = u & 1;
        h16x8 pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) pf[e] = (h16)s[a][8 * sp + e];
#pragma unroll
        for (int t = 0; t < kD / 32; ++t) {
            const h16* base = &tile.vt[(32 * t + col) * kVtStride + 32 * a + 16 * sp + 4 * half];
            const h16x4 lo = *reinterpret_cast<const h16x4*>(base);
            const h16x4 hi = *reinterpret_cast<const h16x4*>(base + 8);
            const h16x8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            st.o[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, st.o[t], 0, 0, 0);
        }
    }
}

__device__ __forceinline__ void load_query(h16x8 (&qf)[kD / 16], const h16* qp, int half) {
#pragma unroll
    for (int s = 0; s < kD / 16; ++s)
        qf[s] = __builtin_bit_cast(h16x8, load_chunk(reinterpret_cast<const Chunk*>(qp) + 2 * s + half));
}

// ── prefill ──────────────────────────────────────────────────────────────
__global__ __launch_bounds__(kBlock, 2) void prefill128(
    const h16* __restrict__ Q, const h16* __restrict__ Kc, const h16* __restrict__ Vc,
    const int* __restrict__ page_table, h16* __restrict__ O, int n_q_heads, int n_kv_heads,
    int q_len, int q_offset, int kv_len, int causal, float scale_log2) {
    __shared__ KvTile tile;

    const int tid = (int)threadIdx.x;
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
    const size_t kv_stride = (size_t)n_kv_heads * kD;

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
    if (wg_limit > 0) fetch_tile<kBlock>(regs, Kc, Vc, page_table, kv_stride, kvh, 0, kv_len - 1, tid);
    for (int t0 = 0; t0 < wg_limit; t0 += kKeyTile) {
        __syncthreads();
        commit_tile<kBlock>(tile, regs, tid);
        __syncthreads();
        if (t0 + kKeyTile < wg_limit)
            fetch_tile<kBlock>(regs, Kc, Vc, page_table, kv_stride, kvh, t0 + kKeyTile, kv_len - 1, tid);
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
        const float inv = st.l > 0.0f ? 1.0f / st.l : 0.0f;
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
constexpr int kPartFloats = kD + 4;        // per (head, slice): 128 channels, max, sum, 2 unused (16-byte rows)

__global__ __launch_bounds__(kWave) void decode128(
    const h16* __restrict__ Q, const h16* __restrict__ Kc, const h16* __restrict__ Vc,
    const int* __restrict__ page_table, h16* __restrict__ O, float* __restrict__ parts,
    int n_q_heads, int n_kv_heads, int cache_len, const int* __restrict__ d_cache_len,
    int n_parts, float scale_log2) {
    __shared__ KvTile tile;

    const int lane = (int)threadIdx.x;
    const int col = lane & 31, half = lane >> 5;
    const int part = (int)blockIdx.x;
    const int kvh = (int)blockIdx.y;
    const int group = n_q_heads / n_kv_heads;
    const int g = (int)blockIdx.z * 32 + col;                 // this lane's head inside the group
    const int head = kvh * group + min(g, group - 1);
    const int len = d_cache_len ? *d_cache_len : cache_len;
    const int per = (((len + n_parts - 1) / n_parts) + kKeyTile - 1) & ~(kKeyTile - 1);
    const int begin = part * per, end = min(len, begin + per);
    const size_t kv_stride = (size_t)n_kv_heads * kD;

    h16x8 qf[kD / 16];
    load_query(qf, Q + (size_t)head * kD, half);
    RowState st;
    st.reset();

    TileRegs<kWave> regs;
    if (begin < end) fetch_tile<kWave>(regs, Kc, Vc, page_table, kv_stride, kvh, begin, end - 1, lane);
    for (int t0 = begin; t0 < end; t0 += kKeyTile) {
        __syncthreads();
        commit_tile<kWave>(tile, regs, lane);
        __syncthreads();
        if (t0 + kKeyTile < end)
            fetch_tile<kWave>(regs, Kc, Vc, page_table, kv_stride, kvh, t0 + kKeyTile, end - 1, lane);
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
        const float inv = st.l > 0.0f ? 1.0f / st.l : 0.0f;
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
        if (half == 0) { dst[kD] = st.m; dst[kD + 1] = st.l; }
#pragma unroll
        for (int t = 0; t < kD / 32; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 o = {st.o[t][4 * q], st.o[t][4 * q + 1], st.o[t][4 * q + 2], st.o[t][4 * q + 3]};
                *reinterpret_cast<f32x4*>(dst + 32 * t + 8 * q + 4 * half) = o;
            }
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
    for (int p0 = grp; p0 < n_parts; p0 += 8 * kMergeGroups) {
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

struct PageIds { int id[32]; };
__global__ void page_map(int* table, int first, int n, PageIds ids) {
    const int i = (int)threadIdx.x;
    if (i < n) table[first + i] = ids.id[i];
}

int decode_parts(int cache_len) {
    int want = (cache_len + kKeyTile - 1) / kKeyTile, n = 1;
    while (n < want && n < kMaxParts) n *= 2;
    return n;
}

bool shape_ok(int n_q_heads, int n_kv_heads, int head_dim) {
    return n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0 && head_dim > 0 &&
           head_dim <= 256;
}

}  // namespace
}  // namespace vv

extern "C" {

/* One implementation serves every backend name: what differs between fa1,
 * fa2 and flashinfer on the reference's CUDA side is how the card is used,
 * not the result. FP16 caches only, contiguous or paged. */
int vv_attn_resolve(int requested, int kv_format, bool paged, int n_q_heads, int n_kv_heads,
                    int head_dim) {
    enum { kAuto = 0, kFa1 = 1, kFa2 = 2, kFlashinfer = 3 };
    if (kv_format != vv::kFormatFp16 || !vv::shape_ok(n_q_heads, n_kv_heads, head_dim)) return kFa1;
    if (requested == kFlashinfer) return kFlashinfer;
    if (requested == kFa1 && !paged) return kFa1;
    return kFa2;
}

size_t vv_attn_scratch_bytes(int n_q_heads, int n_kv_heads, int head_dim) {
    (void)n_kv_heads;
    if (n_q_heads <= 0 || head_dim <= 0) return 0;
    return (size_t)n_q_heads * vv::kMaxParts * ((size_t)head_dim + 4) * sizeof(float);
}

int vv_attn_decode_shape(int backend, int n_q_heads, int n_kv_heads, int cache_len) {
    (void)backend; (void)n_q_heads; (void)n_kv_heads;
    return vv::decode_parts(cache_len);
}

vv_status_t vv_attn_prefill(int backend, const void* q, const vv_kv_view_t* kv, void* out,
                            int n_q_heads, int q_len, int q_offset, int kv_len, bool causal,
                            void* scratch, void* stream) {
    (void)backend; (void)scratch;
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (q_len <= 0 || kv_len <= 0) return VV_OK;
    if (!kv->k || !kv->v) return VV_ERR_NULL_PTR;
    if (kv->format != vv::kFormatFp16) return VV_ERR_UNSUPPORTED;
    if (!vv::shape_ok(n_q_heads, kv->n_kv_heads, kv->head_dim)) return VV_ERR_UNSUPPORTED;
    if (q_offset < 0) return VV_ERR_INVALID_ARG;
    hipStream_t st = vv::as_stream(stream);
    const float scale_log2 = vv::kLog2e / sqrtf((float)kv->head_dim);
    const vv::h16* Q = static_cast<const vv::h16*>(q);
    const vv::h16* K = static_cast<const vv::h16*>(kv->k);
    const vv::h16* V = static_cast<const vv::h16*>(kv->v);
    vv::h16* O = static_cast<vv::h16*>(out);
    if (kv->head_dim == vv::kD && vv::aligned16(q) && vv::aligned16(kv->k) && vv::aligned16(kv->v) &&
        vv::aligned16(out)) {
        const dim3 grid((unsigned)((q_len + vv::kQTile - 1) / vv::kQTile), (unsigned)n_q_heads);
        vv::prefill128<<<grid, vv::kBlock, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads,
                                                    kv->n_kv_heads, q_len, q_offset, kv_len,
                                                    causal ? 1 : 0, scale_log2);
    } else {
        const dim3 grid((unsigned)q_len, (unsigned)n_q_heads);
        vv::rows_generic<<<grid, vv::kWave, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads,
                                                     kv->n_kv_heads, kv->head_dim, q_len, q_offset,
                                                     kv_len, nullptr, causal ? 1 : 0, scale_log2);
    }
    return vv::launch_status();
}

vv_status_t vv_attn_decode(int backend, const void* q, const vv_kv_view_t* kv, void* out,
                           int n_q_heads, int cache_len, const int* d_cache_len, void* scratch,
                           void* stream) {
    (void)backend;
    if (!q || !kv || !out) return VV_ERR_NULL_PTR;
    if (cache_len <= 0) return VV_OK;
    if (!kv->k || !kv->v) return VV_ERR_NULL_PTR;
    if (kv->format != vv::kFormatFp16) return VV_ERR_UNSUPPORTED;
    if (!vv::shape_ok(n_q_heads, kv->n_kv_heads, kv->head_dim)) return VV_ERR_UNSUPPORTED;
    hipStream_t st = vv::as_stream(stream);
    const float scale_log2 = vv::kLog2e / sqrtf((float)kv->head_dim);
    const vv::h16* Q = static_cast<const vv::h16*>(q);
    const vv::h16* K = static_cast<const vv::h16*>(kv->k);
    const vv::h16* V = static_cast<const vv::h16*>(kv->v);
    vv::h16* O = static_cast<vv::h16*>(out);
    if (kv->head_dim == vv::kD && vv::aligned16(q) && vv::aligned16(kv->k) && vv::aligned16(kv->v)) {
        const int n_parts = vv::decode_parts(cache_len);
        if (n_parts > 1 && !scratch) return VV_ERR_NULL_PTR;
        const int group = n_q_heads / kv->n_kv_heads;
        const dim3 grid((unsigned)n_parts, (unsigned)kv->n_kv_heads, (unsigned)((group + 31) / 32));
        vv::decode128<<<grid, vv::kWave, 0, st>>>(Q, K, V, kv->page_table, O,
                                                     static_cast<float*>(scratch), n_q_heads,
                                                     kv->n_kv_heads, cache_len, d_cache_len,
                                                     n_parts, scale_log2);
        if (n_parts > 1) {
            if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
            vv::decode_merge<<<dim3((unsigned)n_q_heads), vv::kMergeThreads, 0, st>>>(
                static_cast<const float*>(scratch), O, n_parts);
        }
    } else {
        // One row: position cache_len - 1 sees everything, so no mask is needed.
        const dim3 grid(1u, (unsigned)n_q_heads);
        vv::rows_generic<<<grid, vv::kWave, 0, st>>>(Q, K, V, kv->page_table, O, n_q_heads,
                                                     kv->n_kv_heads, kv->head_dim, 1, 0, cache_len,
                                                     d_cache_len, 0, scale_log2);
    }
    return vv::launch_status();
}

/* The older entry points for raw FP16 caches (device.h:621-655): the same
 * kernels, the cache given as two pointers instead of a view. */
size_t vv_gqa_decode_scratch_bytes(int n_q_heads, int head_dim) {
    return vv_attn_scratch_bytes(n_q_heads, 1, head_dim);
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
    (void)k_meta; (void)v_meta; (void)k_ref; (void)build_ref;
    if (!k_fp16 || !v_fp16 || !k_store || !v_store) return VV_ERR_NULL_PTR;
    if (kv_format != vv::kFormatFp16) return VV_ERR_UNSUPPORTED;
    if (n_kv_heads <= 0 || head_dim <= 0 || pos < 0) return VV_ERR_INVALID_ARG;
    if (n_positions <= 0) return VV_OK;
    const int row = n_kv_heads * head_dim;
    const size_t n = (size_t)n_positions * row;
    vv::kv_store_fp16<<<dim3((unsigned)((n + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                        vv::as_stream(stream)>>>(
        static_cast<const vv::h16*>(k_fp16), static_cast<const vv::h16*>(v_fp16),
        static_cast<vv::h16*>(k_store), static_cast<vv::h16*>(v_store), row, pos, d_pos,
        n_positions, page_table);
    return vv::launch_status();
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
