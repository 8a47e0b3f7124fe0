// The greedy head of the token loop: logits[V] = W[V,K] x[K] in FP32, then an
// on-device argmax so only the token id crosses the bus.
//
// The product is bound by the table bytes (152064 x 3584 FP16 = 1.09 GB): one
// wave per vocabulary row streams it once with non-temporal 16-byte loads,
// FP32 FMAs, a DPP wave sum. The argmax is two launches (256 partial winners in
// the caller's scratch, then one workgroup); among equal maxima the LOWEST
// index wins, as in the CPU sampler's in-order scan, and a NaN never wins.
#include <float.h>

#include "vv_common.hpp"

namespace vv {
namespace {

constexpr int kArgmaxPartials = 256;      // what callers size scratch_v / scratch_i for

__global__ __launch_bounds__(kBlock) void lm_head_rows(const h16* __restrict__ x,
                                                       const h16* __restrict__ W,
                                                       float* __restrict__ logits, int V, int K) {
    const int row = (int)blockIdx.x * kWavesPerBlock + wave_in_block();
    if (row >= V) return;
    const int lane = lane_id();
    const int kchunks = K / 8;
    const Chunk* w = reinterpret_cast<const Chunk*>(W + (size_t)row * K);
    const Chunk* xv = reinterpret_cast<const Chunk*>(x);
    float acc = 0.0f;
#pragma unroll 4
    for (int c = lane; c < kchunks; c += kWave) {
        const f32x8 wf = unpack(load_chunk_stream(w + c));
        const f32x8 xf = unpack(load_chunk(xv + c));
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(xf[i], wf[i], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) logits[row] = acc;
}

// K % 8 != 0 or operands off 16 bytes.
__global__ __launch_bounds__(kBlock) void lm_head_rows_scalar(const h16* x, const h16* W,
                                                              float* logits, int V, int K) {
    const int row = (int)blockIdx.x * kWavesPerBlock + wave_in_block();
    if (row >= V) return;
    const int lane = lane_id();
    const h16* w = W + (size_t)row * K;
    float acc = 0.0f;
    for (int k = lane; k < K; k += kWave) acc = fmaf((float)x[k], (float)w[k], acc);
    acc = wave_sum(acc);
    if (lane == 0) logits[row] = acc;
}

struct Best {
    float v;
    int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

// The workgroup's winner, valid in thread 0.
__device__ __forceinline__ Best block_best(Best mine) {
    __shared__ float sv[kWavesPerBlock];
    __shared__ int si[kWavesPerBlock];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Best other;
        other.v = __shfl_xor(mine.v, off);
        other.i = __shfl_xor(mine.i, off);
        mine = better(mine, other);
    }
    if (lane_id() == 0) { sv[wave_in_block()] = mine.v; si[wave_in_block()] = mine.i; }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kWavesPerBlock; ++w) mine = better(mine, Best{sv[w], si[w]});
    }
    return mine;
}

__global__ __launch_bounds__(kBlock) void argmax_partial(const float* __restrict__ logits, int V,
                                                         float* __restrict__ pmax,
                                                         int* __restrict__ pidx) {
    Best mine{-FLT_MAX, 0};
    for (int i = (int)blockIdx.x * kBlock + (int)threadIdx.x; i < V; i += (int)gridDim.x * kBlock) {
        const float v = logits[i];
        if (v > mine.v) mine = Best{v, i};            // ascending i: the first maximum stays
    }
    mine = block_best(mine);
    if (threadIdx.x == 0) { pmax[blockIdx.x] = mine.v; pidx[blockIdx.x] = mine.i; }
}

__global__ __launch_bounds__(kBlock) void argmax_final(const float* __restrict__ pmax,
                                                       const int* __restrict__ pidx, int n,
                                                       int* __restrict__ out_token,
                                                       float* __restrict__ out_value) {
    Best mine{-FLT_MAX, 0x7fffffff};
    for (int i = (int)threadIdx.x; i < n; i += kBlock) mine = better(mine, Best{pmax[i], pidx[i]});
    mine = block_best(mine);
    if (threadIdx.x == 0) {
        *out_token = mine.i == 0x7fffffff ? 0 : mine.i;
        if (out_value) *out_value = mine.v;
    }
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_lm_head_gemv_dev(const void* x, const void* W, void* logits, int V, int K,
                                void* stream) {
    if (!x || !W || !logits) return VV_ERR_NULL_PTR;
    if (V <= 0) return VV_OK;
    if (K < 0) return VV_ERR_INVALID_ARG;
    const dim3 grid((unsigned)((V + vv::kWavesPerBlock - 1) / vv::kWavesPerBlock));
    if (K % 8 == 0 && vv::aligned16(x) && vv::aligned16(W))
        vv::lm_head_rows<<<grid, vv::kBlock, 0, vv::as_stream(stream)>>>(
            static_cast<const vv::h16*>(x), static_cast<const vv::h16*>(W),
            static_cast<float*>(logits), V, K);
    else
        vv::lm_head_rows_scalar<<<grid, vv::kBlock, 0, vv::as_stream(stream)>>>(
            static_cast<const vv::h16*>(x), static_cast<const vv::h16*>(W),
            static_cast<float*>(logits), V, K);
    return vv::launch_status();
}

vv_status_t vv_argmax_dev(const void* logits, int V, void* scratch_v, void* scratch_i,
                          void* out_token, void* out_value, void* stream) {
    if (!logits || !scratch_v || !scratch_i || !out_token) return VV_ERR_NULL_PTR;
    if (V <= 0) return VV_ERR_INVALID_ARG;
    hipStream_t st = vv::as_stream(stream);
    vv::argmax_partial<<<vv::kArgmaxPartials, vv::kBlock, 0, st>>>(
        static_cast<const float*>(logits), V, static_cast<float*>(scratch_v),
        static_cast<int*>(scratch_i));
    if (hipGetLastError() != hipSuccess) return VV_ERR_CUDA_LAUNCH;
    vv::argmax_final<<<1, vv::kBlock, 0, st>>>(static_cast<const float*>(scratch_v),
                                               static_cast<const int*>(scratch_i),
                                               vv::kArgmaxPartials, static_cast<int*>(out_token),
                                               static_cast<float*>(out_value));
    return vv::launch_status();
}

}  // extern "C"
