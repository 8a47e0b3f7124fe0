// Row kernels: RMSNorm, residual-add + RMSNorm, embedding gather (+ RMSNorm).
//
// All of them stream [rows, hidden] FP16 once and are bound by HBM bandwidth.
// Layout of the fast path: ONE WORKGROUP OWNS ONE ROW (or two), ONE 16-BYTE
// CHUNK PER THREAD, the chunk kept in registers between the sum-of-squares pass
// and the scaling pass, so a row is read from memory exactly once. hidden =
// 3584 is 448 chunks = a 448-thread workgroup of 7 waves. The sum of squares
// is reduced inside each wave with DPP permutes, across the waves through 7
// floats of LDS and one barrier. Rows wider than 1024 chunks use 2 or 3 chunks
// per thread; widths that are not a multiple of 8, rows wider than 3072
// chunks, or unaligned pointers take a two-pass workgroup-per-row kernel.
//
// Why light threads: on MI355X a copy with this structure moves 6.4 TB/s for
// the add+norm traffic pattern, one with a whole row per wave (7 chunks per
// lane, 14 loads in flight per lane, no LDS) 5.8 TB/s; the measured kernels
// follow (add+norm 66.6 vs 71.0 us at 14449 rows).
#include "row_math.hpp"

namespace vv {
namespace {

enum RowMode : int {
    kPlain = 0,    // normed = rmsnorm(src)
    kAdd = 1,      // state = half(state + src); normed = rmsnorm(state)
    kGather = 2,   // state = src[ids[row]];      normed = rmsnorm(state)
    kGatherOnly = 3  // state = src[ids[row]]
};

// ── one workgroup per row, one chunk per thread ──────────────────────────
// blockDim = the row's chunk count rounded up to whole waves (448 threads = 7
// waves for hidden 3584), kCpt chunks per thread for rows wider than 1024
// chunks. Every wave is light (one or two 16-byte loads per lane), which is the
// shape the memory system rewards: a pure copy with this structure moves
// 6.4 TB/s for the add+norm traffic pattern against 5.8 TB/s with one wave per
// row. Sum of squares: DPP reduction inside each wave, then one float per wave
// through LDS and a single barrier.
template <int kCpt, int kRows, int kMode, bool kStream, bool kFull>   // kFull: nchunks == kCpt * blockDim.x
__global__ __launch_bounds__(kMaxWgThreads) void norm_rows_wg(
    const Chunk* src, Chunk* state, const int32_t* __restrict__ ids,
    const Chunk* __restrict__ weight, Chunk* normed, int rows, int nchunks, float inv_n,
    float eps) {
    __shared__ float partial[kRows][kMaxWgThreads / kWave];
    const int t = (int)threadIdx.x;
    const int nthreads = (int)blockDim.x;
    const int row0 = (int)blockIdx.x * kRows;
    constexpr bool kGathers = kMode == kGather || kMode == kGatherOnly;
    constexpr bool kStreamSrc = kStream && !kGathers;

    // kRows consecutive rows share the workgroup: one weight load serves them
    // all, and their loads are all in flight before the first use. A row past
    // the end (odd row count) re-reads the last row and is not stored.
    Chunk a[kRows][kCpt], b[kRows][kCpt], w[kCpt];
    bool live[kRows];
    size_t out_base[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        live[r] = kRows == 1 || row0 + r < rows;
        const int row = live[r] ? row0 + r : rows - 1;
        const size_t src_row = kGathers ? (size_t)ids[row] : (size_t)row;
        const Chunk* s = src + src_row * (size_t)nchunks;
        out_base[r] = (size_t)row * (size_t)nchunks;
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            if (kFull || c < nchunks) {
                a[r][j] = load_chunk_as<kStreamSrc>(s + c);
                if (kMode == kAdd) b[r][j] = load_chunk_as<kStream>(state + out_base[r] + c);
            }
        }
    }
    if (kMode == kGatherOnly) {
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int j = 0; j < kCpt; ++j) {
                const int c = j * nthreads + t;
                if ((kFull || c < nchunks) && live[r])
                    store_chunk_as<kStream>(state + out_base[r] + c, a[r][j]);
            }
        return;
    }
#pragma unroll
    for (int j = 0; j < kCpt; ++j) {
        const int c = j * nthreads + t;
        if (kFull || c < nchunks) w[j] = load_chunk(weight + c);
    }

#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            if (kFull || c < nchunks) {
                f32x8 x = unpack(a[r][j]);
                if (kMode == kAdd) {
                    const f32x8 res = unpack(b[r][j]);
#pragma unroll
                    for (int i = 0; i < 8; ++i) x[i] = res[i] + x[i];
                    // stored residual = FP16 rounding of the sum; the norm reads that value
                    a[r][j] = pack(x);
                    x = unpack(a[r][j]);
                }
                acc = chunk_sumsq(x, acc);
            }
        }
        acc = wave_sum(acc);
        if (lane_id() == 0) partial[r][t >> 6] = acc;
    }
    __syncthreads();
    const int nwaves = nthreads >> 6;

    // The stores come last, a row's normed chunk before its updated residual / gathered chunk. Measured on the
    // gather (14449 random 7 KB rows): storing the gathered row before the barrier, where it is first known,
    // 55.0 us; after the barrier, ahead of the normed row, 53.4 us; behind it, 52.9 us - stores issued early
    // queue ahead of other workgroups' loads. (Ordinary instead of streaming stores for either output: 58.3 us.
    // All normed rows first, then all residual rows: no different. add+norm does not care: 66.2 us either way.)
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        float total = 0.0f;
        for (int i = 0; i < nwaves; ++i) total += partial[r][i];
        const float inv = inv_rms(total, inv_n, eps);
#pragma unroll
        for (int j = 0; j < kCpt; ++j) {
            const int c = j * nthreads + t;
            if ((kFull || c < nchunks) && live[r]) {
                store_chunk_as<kStream>(normed + out_base[r] + c, scale_chunk(a[r][j], inv, w[j]));
                if (kMode == kAdd || kMode == kGather) store_chunk_as<kStream>(state + out_base[r] + c, a[r][j]);
            }
        }
    }
}

// ── one wave per row, kCpl chunks per lane ──────────────────────────────
// For launches of a few thousand rows. With a workgroup per row the chip holds
// about 1024 rows at a time (four 7-wave workgroups per compute unit), so a
// 2048-row prefill chunk runs as two dependent rounds of load -> reduce -> store
// and never has more than half of its reads in flight. Here a row is one wave
// with all of its loads (kCpl per tensor) issued back to back: 2048 rows are
// 2048 waves, two per SIMD, every byte of the launch requested in the first
// microsecond; the only barrier publishes the weight row, which the four waves
// of a workgroup share through LDS. The sum of squares keeps the workgroup
// kernel's order bit for bit: group j of 64 chunks is reduced like wave j of
// that kernel (same DPP tree), and the groups are added in order from zero.
template <int kCpl, int kMode, bool kStream, bool kFull>      // kFull: nchunks == 64 * kCpl
__global__ __launch_bounds__(kBlock) void norm_rows_wave(
    const Chunk* src, Chunk* state, const int32_t* __restrict__ ids,
    const Chunk* __restrict__ weight, Chunk* normed, int rows, int nchunks, float inv_n,
    float eps) {
    // The weight row goes through LDS once per workgroup instead of once per wave: measured
    // cold against each wave loading its own copy, gather+norm 8.1 / 8.4 us at 2048 rows and
    // 16.8 / 17.3 us at 4096, norm 6.0 / 6.6 us at 2048.
    __shared__ Chunk wsh[kCpl * kWave];
    constexpr bool kGathers = kMode == kGather || kMode == kGatherOnly;
    constexpr bool kStreamSrc = kStream && !kGathers;
    constexpr int kWeightLoads = (kCpl * kWave + kBlock - 1) / kBlock;
    const int lane = lane_id();
    const int want = (int)blockIdx.x * kWavesPerBlock + wave_in_block();
    const bool live = want < rows;               // a wave past the end re-reads the last row, stores nothing
    const int row = live ? want : rows - 1;

    // All loads are unconditional (an index past the end is clamped and its value unused), so
    // the code up to the stores is one straight line and the waits count loads exactly. The
    // weight chunks are requested first: loads are counted in order, so waiting for them does
    // not wait for the row.
    Chunk wmine[kWeightLoads];
    if (kMode != kGatherOnly) {
#pragma unroll
        for (int i = 0; i < kWeightLoads; ++i)
            wmine[i] = load_chunk(weight + min(i * kBlock + (int)threadIdx.x, nchunks - 1));
    }
    const size_t src_row = kGathers ? (size_t)ids[row] : (size_t)row;
    const Chunk* s = src + src_row * (size_t)nchunks;
    const size_t out_base = (size_t)row * (size_t)nchunks;

    Chunk a[kCpl], b[kCpl];
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = kFull ? j * kWave + lane : min(j * kWave + lane, nchunks - 1);
        a[j] = load_chunk_as<kStreamSrc>(s + c);
        if (kMode == kAdd) b[j] = load_chunk_as<kStream>(state + out_base + c);
    }
    if (kMode == kGatherOnly) {
        if (!live) return;
#pragma unroll
        for (int j = 0; j < kCpl; ++j) {
            const int c = j * kWave + lane;
            if (kFull || c < nchunks) store_chunk_as<kStream>(state + out_base + c, a[j]);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < kWeightLoads; ++i)      // clamped duplicates write the same bytes to the same slot
        wsh[min(i * kBlock + (int)threadIdx.x, nchunks - 1)] = wmine[i];
    __syncthreads();
    if (!live) return;                           // no barrier below

    float total = 0.0f;
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        f32x8 x = unpack(a[j]);
        if (kMode == kAdd) {
            const f32x8 res = unpack(b[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = res[i] + x[i];
            a[j] = pack(x);                       // the stored residual; the norm reads that value
            x = unpack(a[j]);
        }
        // The updated residual goes out as soon as it is known; the gathered row waits until the normed row
        // is out (cold at 2048 / 4096 rows: add+norm 10.4 / 20.7 us storing here against 10.6 / 21.2 us
        // storing last; gather+norm 8.6 us storing here against 8.3 us storing last).
        if (kMode == kAdd && (kFull || c < nchunks)) store_chunk_as<kStream>(state + out_base + c, a[j]);
        const float acc = chunk_sumsq(x, 0.0f);
        total += wave_sum((kFull || c < nchunks) ? acc : 0.0f);
    }
    const float inv = inv_rms(total, inv_n, eps);
#pragma unroll
    for (int j = 0; j < kCpl; ++j) {
        const int c = j * kWave + lane;
        if (kFull || c < nchunks) {
            store_chunk_as<kStream>(normed + out_base + c,
                                    scale_chunk(a[j], inv, wsh[kFull ? c : min(c, nchunks - 1)]));
            if (kMode == kGather) store_chunk_as<kStream>(state + out_base + c, a[j]);
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
    if (vec && nchunks <= 3 * kMaxWgThreads) {
        const int cpt = (nchunks + kMaxWgThreads - 1) / kMaxWgThreads;
        int threads = ((nchunks + cpt - 1) / cpt + kWave - 1) / kWave * kWave;
        const size_t tensors = kMode == kAdd ? 4 : (kMode == kGather ? 3 : 2);
        const bool stream = use_streaming(tensors * (size_t)rows * (size_t)hidden * 2u);
        const Chunk* s = static_cast<const Chunk*>(src);
        Chunk* stt = static_cast<Chunk*>(state);
        const Chunk* w = static_cast<const Chunk*>(weight);
        Chunk* o = static_cast<Chunk*>(normed);
        const bool full = nchunks == cpt * threads;
        // Which kernel: measured cold on MI355X at hidden 3584 with streaming accesses, a
        // launch of R rows (us; workgroup per row / two rows per workgroup / wave per row):
        //             R = 1024            2048             4096             8192            14449
        //   add+norm    6.8  6.9  6.3   11.7 12.0 10.5   20.9 21.6 20.7   38.6 39.4 40.2   66.9 67.1 69.6
        //   gather+norm 7.2  5.9  5.1   11.5  9.8  8.1   19.4 18.1 16.8   34.8 32.7 32.7   58.4 54.3 55.4
        //   norm        4.1  4.4  3.9    7.7  6.3  6.0   12.7 12.3 11.2   22.0 20.9 20.8   37.2 34.4 34.7
        // A workgroup per row keeps ~1024 rows on the chip at once, so a few thousand rows
        // run as two or three dependent rounds; a wave per row has them all resident with
        // every load issued at the start. Long launches hide that and prefer light waves.
        // Row counts are scaled to hidden 3584 (448 chunks) for other widths.
        // VV_HIP_ROWS_PER_WG=1|2 forces a workgroup kernel, VV_HIP_NORM_WAVE=0|1 the wave kernel.
        static const int forced_rows = [] {
            const char* e = getenv("VV_HIP_ROWS_PER_WG");
            return (e && (e[0] == '1' || e[0] == '2' || e[0] == '4')) ? e[0] - '0' : 0;
        }();
        static const int forced_wave = [] {
            const char* e = getenv("VV_HIP_NORM_WAVE");
            return (e && (e[0] == '0' || e[0] == '1')) ? e[0] - '0' : -1;
        }();
        const long eq_rows = (long)rows * nchunks / 448;       // rows of 448 chunks with the same bytes
        bool wave = false;
        int rpw = 1;
        if (cpt == 1) {
            if (kMode == kAdd) {
                wave = eq_rows >= 896 && eq_rows <= 4608;
            } else if (kMode == kPlain) {
                wave = eq_rows >= 1024 && eq_rows < 10240;
                rpw = eq_rows >= 1536 ? 2 : 1;
            } else if (kMode == kGather) {
                wave = eq_rows >= 768 && eq_rows < 10240;
                rpw = eq_rows >= 256 ? 2 : 1;
            } else {
                rpw = eq_rows >= 4096 ? 2 : 1;      // gather only: 32.4 us at 14449 rows (80 % of peak)
            }
        }
        if (forced_rows) { rpw = forced_rows; wave = false; }
        if (forced_wave >= 0 && !forced_rows) wave = forced_wave == 1;
        if (wave && cpt == 1 && nchunks <= 8 * kWave) {
            const dim3 wgrid((unsigned)((rows + kWavesPerBlock - 1) / kWavesPerBlock));
#define VV_WAVE_LAUNCH(C, S, F)                                                               \
    norm_rows_wave<C, kMode, S, F><<<wgrid, kBlock, 0, st>>>(s, stt, ids, w, o, rows, nchunks, \
                                                            inv_n, eps)
#define VV_WAVE_CASE(C)                                                  \
    case C: {                                                           \
        const bool wfull = nchunks == C * kWave;                        \
        if (stream && wfull)  VV_WAVE_LAUNCH(C, true, true);            \
        else if (stream)      VV_WAVE_LAUNCH(C, true, false);           \
        else if (wfull)       VV_WAVE_LAUNCH(C, false, true);           \
        else                  VV_WAVE_LAUNCH(C, false, false);          \
    } break;
            switch ((nchunks + kWave - 1) / kWave) {
                VV_WAVE_CASE(1) VV_WAVE_CASE(2) VV_WAVE_CASE(3) VV_WAVE_CASE(4)
                VV_WAVE_CASE(5) VV_WAVE_CASE(6) VV_WAVE_CASE(7) VV_WAVE_CASE(8)
            }
#undef VV_WAVE_LAUNCH
#undef VV_WAVE_CASE
            return launch_status();
        }
        const bool two = rpw == 2 && cpt == 1, four = rpw == 4 && cpt == 1;
        const dim3 grid((unsigned)(four ? (rows + 3) / 4 : two ? (rows + 1) / 2 : rows));
#define VV_WG_LAUNCH(C, R, S, F)                                                          \
    norm_rows_wg<C, R, kMode, S, F><<<grid, threads, 0, st>>>(s, stt, ids, w, o, rows, nchunks, \
                                                              inv_n, eps)
#define VV_WG_PICK(C, R)                                     \
        if (stream && full)  VV_WG_LAUNCH(C, R, true, true);    \
        else if (stream)     VV_WG_LAUNCH(C, R, true, false);   \
        else if (full)       VV_WG_LAUNCH(C, R, false, true);   \
        else                 VV_WG_LAUNCH(C, R, false, false);
        if (four) { VV_WG_PICK(1, 4) }
        else if (two) { VV_WG_PICK(1, 2) }
        else if (cpt == 1) { VV_WG_PICK(1, 1) }
        else if (cpt == 2) { VV_WG_PICK(2, 1) }
        else { VV_WG_PICK(3, 1) }
#undef VV_WG_PICK
#undef VV_WG_LAUNCH
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
