// Row kernels: RMSNorm, residual-add + RMSNorm, embedding gather (+ RMSNorm).
//
// All of them stream [rows, hidden] FP16 once and are bound by HBM bandwidth.
// Layout of the fast path: ONE WAVE OWNS ONE ROW and keeps it in registers
// (hidden = 3584 is 448 16-byte chunks = 7 per lane), so the row is read from
// memory exactly once, the sum of squares is reduced across the 64 lanes with
// DPP permutes, and no LDS and no barrier are involved. A 256-thread workgroup
// is four independent rows. Rows that do not fit that shape (hidden not a
// multiple of 8, wider than 4096, or unaligned pointers) take a
// workgroup-per-row kernel with a two-pass loop.
#include "vv_common.hpp"

namespace vv {
namespace {

enum RowMode : int {
    kPlain = 0,    // normed = rmsnorm(src)
    kAdd = 1,      // state = half(state + src); normed = rmsnorm(state)
    kGather = 2,   // state = src[ids[row]];      normed = rmsnorm(state)
    kGatherOnly = 3  // state = src[ids[row]]
};

// 1 / sqrt(mean(x^2) + eps) with the hardware reciprocal square root (1 ulp of
// FP32, i.e. ~1e-7 relative against an FP16 result whose own rounding is 5e-4).
// Every lane of every wave of a row evaluates this, so it has to be a handful
// of instructions: the correctly rounded divide + sqrt + divide sequence is
// ~60 and was a measurable share of the VALU time with one chunk per thread.
__device__ __forceinline__ float inv_rms(float sumsq, float inv_n, float eps) {
    return __builtin_amdgcn_rsqf(sumsq * inv_n + eps);
}

// ── one wave per row, row held in registers ──────────────────────────────
// kCpl = chunks per lane (row width <= 512 * kCpl halves); kFull = the row is
// exactly 64 * kCpl chunks, so no lane is ever idle and loads are unpredicated.
template <int kCpl, int kMode, bool kFull, bool kStream>
__global__ __launch_bounds__(kBlock) void norm_rows_wave(
    const Chunk* src, Chunk* state, const int32_t* __restrict__ ids,
    const Chunk* __restrict__ weight, Chunk* normed, int rows, int nchunks, float inv_n,
    float eps) {
    const int row = (int)blockIdx.x * kWavesPerBlock + wave_in_block();
    if (row >= rows) return;
    const int lane = lane_id();

    size_t src_row = (size_t)row;
    if (kMode == kGather || kMode == kGatherOnly)
        src_row = (size_t)__builtin_amdgcn_readfirstlane(ids[row]);
    const Chunk* s = src + src_row * (size_t)nchunks;
    const size_t out_base = (size_t)row * (size_t)nchunks;

    // Issue every load of the row before the first use: kCpl (or 2*kCpl)
    // independent 16-byte loads in flight per lane. Gathered table rows are
    // read with ordinary loads even in streaming launches: measured on MI355X,
    // a row gather with streaming loads runs 10 % slower (5.3 vs 5.9 TB/s for
    // gather + two outputs), and a table row may well be needed again.
    constexpr bool kStreamSrc = kStream && !(kMode == kGather || kMode == kGatherOnly);
    Chunk a[kCpl];
    Chunk b[kCpl];
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (kFull || c < nchunks) {
            a[j] = load_chunk_as<kStreamSrc>(s + c);
            if (kMode == kAdd) b[j] = load_chunk_as<kStream>(state + out_base + c);
        }
    }

    if (kMode == kGatherOnly) {
#pragma unroll
        for (int j = 0; j < kCpl; ++j) {
            const int c = j * kWave + lane;
            if (kFull || c < nchunks) store_chunk_as<kStream>(state + out_base + c, a[j]);
        }
        return;
    }

    Chunk w[kCpl];
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (kFull || c < nchunks) w[j] = load_chunk(weight + c);
    }

    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (kFull || c < nchunks) {
            f32x8 x = unpack(a[j]);
            if (kMode == kAdd) {
                const f32x8 r = unpack(b[j]);
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = r[i] + x[i];
                // The stored residual is the FP16 rounding of the sum, and the
                // norm reads that rounded value (what add-then-norm would see).
                a[j] = pack(x);
                x = unpack(a[j]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(x[i], x[i], acc);
        }
    }
    if (kMode == kAdd || kMode == kGather) {
#pragma unroll
        for (int j = 0; j < kCpl; ++j) {
            const int c = j * kWave + lane;
            if (kFull || c < nchunks) store_chunk_as<kStream>(state + out_base + c, a[j]);
        }
    }

    const float inv = inv_rms(wave_sum(acc), inv_n, eps);

#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (kFull || c < nchunks) {
            f32x8 x = unpack(a[j]);
            const f32x8 g = unpack(w[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (x[i] * inv) * g[i];
            store_chunk_as<kStream>(normed + out_base + c, pack(x));
        }
    }
}

// ── one workgroup per row, one chunk per thread ──────────────────────────
// blockDim = the row's chunk count rounded up to whole waves (448 threads = 7
// waves for hidden 3584), kCpt chunks per thread for rows wider than 1024
// chunks. Every wave is light (one or two 16-byte loads per lane), which is the
// shape the memory system rewards: a pure copy with this structure moves
// 6.4 TB/s for the add+norm traffic pattern against 5.8 TB/s with one wave per
// row. Sum of squares: DPP reduction inside each wave, then one float per wave
// through LDS and a single barrier.
constexpr int kMaxWgThreads = 1024;

template <int kCpt, int kMode, bool kStream, bool kFull>   // kFull: nchunks == kCpt * blockDim.x
__global__ __launch_bounds__(kMaxWgThreads) void norm_rows_wg(
    const Chunk* src, Chunk* state, const int32_t* __restrict__ ids,
    const Chunk* __restrict__ weight, Chunk* normed, int nchunks, float inv_n, float eps) {
    __shared__ float partial[kMaxWgThreads / kWave];
    const size_t row = blockIdx.x;
    const int t = (int)threadIdx.x;
    const int nthreads = (int)blockDim.x;

    size_t src_row = row;
    if (kMode == kGather || kMode == kGatherOnly) src_row = (size_t)ids[row];
    const Chunk* s = src + src_row * (size_t)nchunks;
    const size_t out_base = row * (size_t)nchunks;
    constexpr bool kStreamSrc = kStream && !(kMode == kGather || kMode == kGatherOnly);

    Chunk a[kCpt], b[kCpt], w[kCpt];
#pragma unroll
    for (int j = 0; j < kCpt; ++j) {
        const int c = j * nthreads + t;
        if (kFull || c < nchunks) {
            a[j] = load_chunk_as<kStreamSrc>(s + c);
            if (kMode == kAdd) b[j] = load_chunk_as<kStream>(state + out_base + c);
            if (kMode != kGatherOnly) w[j] = load_chunk(weight + c);
        }
    }
    if (kMode == kGatherOnly) {
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            if (kFull || c < nchunks) store_chunk_as<kStream>(state + out_base + c, a[j]);
        }
        return;
    }

    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < kCpt; ++j) {
        const int c = j * nthreads + t;
        if (kFull || c < nchunks) {
            f32x8 x = unpack(a[j]);
            if (kMode == kAdd) {
                const f32x8 r = unpack(b[j]);
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = r[i] + x[i];
                // stored residual = FP16 rounding of the sum; the norm reads that value
                a[j] = pack(x);
                x = unpack(a[j]);
            }
            if (kMode == kAdd || kMode == kGather)
                store_chunk_as<kStream>(state + out_base + c, a[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(x[i], x[i], acc);
        }
    }

    acc = wave_sum(acc);
    if (lane_id() == 0) partial[t >> 6] = acc;
    __syncthreads();
    float total = 0.0f;
    const int nwaves = nthreads >> 6;
    for (int i = 0; i < nwaves; ++i) total += partial[i];
    const float inv = inv_rms(total, inv_n, eps);

#pragma unroll
    for (int j = 0; j < kCpt; ++j) {
        const int c = j * nthreads + t;
        if (kFull || c < nchunks) {
            f32x8 x = unpack(a[j]);
            const f32x8 g = unpack(w[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (x[i] * inv) * g[i];
            store_chunk_as<kStream>(normed + out_base + c, pack(x));
        }
    }
}

// ── one workgroup per row, any width, any alignment ──────────────────────
// Two passes; the second re-reads what the first one left in `state` (kAdd,
// kGather) or the source row (kPlain), which the caches still hold. Thread t
// touches the same elements in both passes, so `normed` may alias `src`.
template <int kMode, typename T>   // T = Chunk (8 halves at a time) or h16
__global__ __launch_bounds__(kBlock) void norm_rows_block(
    const T* src, T* state, const int32_t* __restrict__ ids, const T* __restrict__ weight,
    T* normed, int units, float inv_n, float eps) {
    __shared__ float partial[kWavesPerBlock];
    const int row = (int)blockIdx.x;
    size_t src_row = (size_t)row;
    if (kMode == kGather || kMode == kGatherOnly) src_row = (size_t)ids[row];
    const T* s = src + src_row * (size_t)units;
    T* st = state + (size_t)row * (size_t)units;
    T* out = normed + (size_t)row * (size_t)units;

    float acc = 0.0f;
    for (int c = (int)threadIdx.x; c < units; c += kBlock) {
        if constexpr (sizeof(T) == 16) {
            Chunk v = load_chunk(s + c);
            f32x8 x = unpack(v);
            if (kMode == kAdd) {
                const f32x8 r = unpack(load_chunk(st + c));
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = r[i] + x[i];
                v = pack(x);
                x = unpack(v);
            }
            if (kMode != kPlain) store_chunk(st + c, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(x[i], x[i], acc);
        } else {
            h16 v = s[c];
            if (kMode == kAdd) v = to_half((float)st[c] + (float)v);
            if (kMode != kPlain) st[c] = v;
            acc = fmaf((float)v, (float)v, acc);
        }
    }
    if (kMode == kGatherOnly) return;

    acc = wave_sum(acc);
    if (lane_id() == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
    const float inv = inv_rms(total, inv_n, eps);

    const T* again = (kMode == kPlain) ? s : st;
    for (int c = (int)threadIdx.x; c < units; c += kBlock) {
        if constexpr (sizeof(T) == 16) {
            f32x8 x = unpack(load_chunk(again + c));
            const f32x8 g = unpack(load_chunk(weight + c));
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (x[i] * inv) * g[i];
            store_chunk(out + c, pack(x));
        } else {
            out[c] = to_half(((float)again[c] * inv) * (float)weight[c]);
        }
    }
}

template <int kMode>
vv_status_t launch_rows(const void* src, void* state, const int32_t* ids, const void* weight,
                        void* normed, int rows, int hidden, float eps, hipStream_t st) {
    if (rows <= 0 || hidden <= 0) return VV_OK;
    const bool vec = (hidden % 8 == 0) && aligned16(src) && aligned16(state) &&
                     aligned16(weight) && aligned16(normed);
    const int nchunks = hidden / 8;
    const float inv_n = 1.0f / (float)hidden;
    static const bool use_wave = [] {
        const char* e = getenv("VV_HIP_ROWS");
        return e && e[0] == 'w' && e[1] == 'a';       // VV_HIP_ROWS=wave: A/B aid
    }();
    if (vec && !use_wave && nchunks <= 3 * kMaxWgThreads) {
        const int cpt = (nchunks + kMaxWgThreads - 1) / kMaxWgThreads;
        int threads = ((nchunks + cpt - 1) / cpt + kWave - 1) / kWave * kWave;
        const size_t tensors = kMode == kAdd ? 4 : (kMode == kGather ? 3 : 2);
        const bool stream = use_streaming(tensors * (size_t)rows * (size_t)hidden * 2u);
        const Chunk* s = static_cast<const Chunk*>(src);
        Chunk* stt = static_cast<Chunk*>(state);
        const Chunk* w = static_cast<const Chunk*>(weight);
        Chunk* o = static_cast<Chunk*>(normed);
        const dim3 grid((unsigned)rows);
        const bool full = nchunks == cpt * threads;
#define VV_WG_LAUNCH(C, S, F) \
    norm_rows_wg<C, kMode, S, F><<<grid, threads, 0, st>>>(s, stt, ids, w, o, nchunks, inv_n, eps)
#define VV_WG_CASE(C)                                        \
    case C:                                                  \
        if (stream && full)  VV_WG_LAUNCH(C, true, true);    \
        else if (stream)     VV_WG_LAUNCH(C, true, false);   \
        else if (full)       VV_WG_LAUNCH(C, false, true);   \
        else                 VV_WG_LAUNCH(C, false, false);  \
        break;
        switch (cpt) { VV_WG_CASE(1) VV_WG_CASE(2) VV_WG_CASE(3) }
#undef VV_WG_CASE
#undef VV_WG_LAUNCH
        return launch_status();
    }
    if (vec && nchunks <= 8 * kWave) {
        const Chunk* s = static_cast<const Chunk*>(src);
        Chunk* stt = static_cast<Chunk*>(state);
        const Chunk* w = static_cast<const Chunk*>(weight);
        Chunk* o = static_cast<Chunk*>(normed);
        const dim3 grid((unsigned)((rows + kWavesPerBlock - 1) / kWavesPerBlock));
        const int cpl = (nchunks + kWave - 1) / kWave;
        const bool full = nchunks == cpl * kWave;
        // bytes this launch streams: 2 tensors (plain, gather-only), 3 (gather+norm), 4 (add+norm)
        const size_t tensors = kMode == kAdd ? 4 : (kMode == kGather ? 3 : 2);
        const bool stream = use_streaming(tensors * (size_t)rows * (size_t)hidden * 2u);
#define VV_ROWS_LAUNCH(N, F, S) \
    norm_rows_wave<N, kMode, F, S><<<grid, kBlock, 0, st>>>(s, stt, ids, w, o, rows, nchunks, inv_n, eps)
#define VV_ROWS_CASE(N)                                       \
    case N:                                                   \
        if (full && stream)       VV_ROWS_LAUNCH(N, true, true);   \
        else if (full)            VV_ROWS_LAUNCH(N, true, false);  \
        else if (stream)          VV_ROWS_LAUNCH(N, false, true);  \
        else                      VV_ROWS_LAUNCH(N, false, false); \
        break;
        switch (cpl) {
            VV_ROWS_CASE(1) VV_ROWS_CASE(2) VV_ROWS_CASE(3) VV_ROWS_CASE(4)
            VV_ROWS_CASE(5) VV_ROWS_CASE(6) VV_ROWS_CASE(7) VV_ROWS_CASE(8)
        }
#undef VV_ROWS_CASE
#undef VV_ROWS_LAUNCH
        return launch_status();
    }
    if (vec) {
        norm_rows_block<kMode, Chunk><<<dim3((unsigned)rows), kBlock, 0, st>>>(
            static_cast<const Chunk*>(src), static_cast<Chunk*>(state), ids,
            static_cast<const Chunk*>(weight), static_cast<Chunk*>(normed), nchunks, inv_n, eps);
    } else {
        norm_rows_block<kMode, h16><<<dim3((unsigned)rows), kBlock, 0, st>>>(
            static_cast<const h16*>(src), static_cast<h16*>(state), ids,
            static_cast<const h16*>(weight), static_cast<h16*>(normed), hidden, inv_n, eps);
    }
    return launch_status();
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_rmsnorm_dev(const void* input, const void* weight, void* output, int seq_len,
                           int hidden_size, float eps, void* stream) {
    if (!input || !weight || !output) return VV_ERR_NULL_PTR;
    // `state` is unused in this mode; pass an aligned non-null placeholder.
    return vv::launch_rows<vv::kPlain>(input, output, nullptr, weight, output, seq_len,
                                       hidden_size, eps, vv::as_stream(stream));
}

vv_status_t vv_add_rmsnorm_dev(void* residual, const void* x, const void* weight, void* normed,
                               int seq_len, int hidden_size, float eps, void* stream) {
    if (!residual || !x || !weight || !normed) return VV_ERR_NULL_PTR;
    return vv::launch_rows<vv::kAdd>(x, residual, nullptr, weight, normed, seq_len, hidden_size,
                                     eps, vv::as_stream(stream));
}

vv_status_t vv_embedding_rmsnorm_dev(const void* table, const int32_t* ids, const void* weight,
                                     void* hidden, void* normed, int seq_len, int hidden_size,
                                     float eps, void* stream) {
    if (!table || !ids || !weight || !hidden || !normed) return VV_ERR_NULL_PTR;
    return vv::launch_rows<vv::kGather>(table, hidden, ids, weight, normed, seq_len, hidden_size,
                                        eps, vv::as_stream(stream));
}

vv_status_t vv_embedding_dev(const void* table, const int32_t* ids, void* output, int seq_len,
                             int hidden_size, void* stream) {
    if (!table || !ids || !output) return VV_ERR_NULL_PTR;
    // weight/normed are unused in this mode; aligned placeholders keep the vector path.
    return vv::launch_rows<vv::kGatherOnly>(table, output, ids, output, output, seq_len,
                                            hidden_size, 0.0f, vv::as_stream(stream));
}

}  // extern "C"
