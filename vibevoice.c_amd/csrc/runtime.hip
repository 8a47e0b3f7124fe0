// The runtime half of the accelerator seam: allocation, copies, fills, streams,
// events, graph capture, and the two tiny kernels a captured decode step needs
// (a device-side position add and a row copy to a device-side index).
//
// Backend choices that differ from a CUDA build, all deliberate:
//   - every stream, "background" included, has the default priority;
//   - existing host memory is never page-locked after the fact
//     (vv_dev_host_register declines); pinned memory is allocated as such;
//   - the stream-ordered fill is a kernel, not a memset node, so it can sit in
//     a captured graph and replay correctly.
#include <stdio.h>

#include <algorithm>
#include <vector>

#include "vv_common.hpp"

namespace vv {
namespace {

__global__ void pos_add_kernel(int* dst, const int* src, int delta) { *dst = *src + delta; }

__global__ __launch_bounds__(kBlock) void copy_at_chunks(Chunk* dst_base, const Chunk* src,
                                                         const int* d_index, int chunks) {
    const int i = (int)blockIdx.x * kBlock + (int)threadIdx.x;
    if (i < chunks) dst_base[(size_t)(*d_index) * (size_t)chunks + (size_t)i] = src[i];
}

__global__ __launch_bounds__(kBlock) void copy_at_bytes(unsigned char* dst_base,
                                                        const unsigned char* src,
                                                        const int* d_index, size_t bytes) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < bytes) dst_base[(size_t)(*d_index) * bytes + i] = src[i];
}

// A stream-ordered device-to-device copy of whole 16-byte chunks, kPer chunks per thread (all loads, then all
// stores), workgroups of ONE wave - the shape this device's memory system rewards (a 256 MiB copy: 6.7 TB/s read +
// written, against 6.1 with 256-thread workgroups and 5.4 for the runtime's own copy) - with streaming accesses
// from 2 MiB on.
template <bool kStream, int kThreads, int kPer>
__global__ __launch_bounds__(kThreads) void copy_chunks(Chunk* __restrict__ dst, const Chunk* __restrict__ src,
                                                        size_t chunks) {
    const size_t i0 = (size_t)blockIdx.x * (kThreads * kPer) + threadIdx.x;
    Chunk c[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const size_t i = i0 + (size_t)j * kThreads;
        if (i < chunks) c[j] = load_chunk_as<kStream>(src + i);
    }
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const size_t i = i0 + (size_t)j * kThreads;
        if (i < chunks) store_chunk_as<kStream>(dst + i, c[j]);
    }
}

// Fill [ptr, ptr+size) with one byte value: unaligned head and tail bytes by
// single-byte stores, the 16-byte aligned middle by chunk stores.
__global__ __launch_bounds__(kBlock) void fill_kernel(unsigned char* ptr, unsigned value,
                                                      size_t head, size_t chunks, size_t tail) {
    const size_t gid = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kBlock;
    const unsigned char b = (unsigned char)value;
    if (gid < head) ptr[gid] = b;
    if (gid < tail) ptr[head + chunks * 16 + gid] = b;
    const uint32_t word = 0x01010101u * (uint32_t)b;
    Chunk c;
    c.w[0] = c.w[1] = c.w[2] = c.w[3] = word;
    Chunk* mid = reinterpret_cast<Chunk*>(ptr + head);
    for (size_t i = gid; i < chunks; i += stride) mid[i] = c;
}

// ── captures in flight on this host thread ───────────────────────────────
// An uncapturable call (a synchronisation, an allocation, a synchronous copy)
// made while this thread is capturing must fail the capture rather than run.
// The HIP runtime does mark such a capture invalid, but it then leaves the
// stream in that state for good: hipStreamEndCapture reports the error without
// ending the capture, and every later launch on the stream fails. The caller
// of a broken capture reissues its work on the same stream, so this backend
// ends the capture itself, cleanly, BEFORE the offending runtime call would
// wedge it: the recorded graph is discarded, the stream is remembered as
// "broken", and vv_dev_graph_end on it reports the failure. Capture is
// thread-local (hipStreamCaptureModeThreadLocal), so thread-local lists suffice
// and other threads' streams are never touched.
thread_local std::vector<hipStream_t> tl_capturing;
thread_local std::vector<hipStream_t> tl_broken;

bool break_captures_of_this_thread() {
    if (tl_capturing.empty()) return false;
    for (hipStream_t s : tl_capturing) {
        hipGraph_t g = nullptr;
        if (hipStreamEndCapture(s, &g) == hipSuccess && g) (void)hipGraphDestroy(g);
        tl_broken.push_back(s);
    }
    tl_capturing.clear();
    (void)hipGetLastError();
    return true;
}

bool forget(std::vector<hipStream_t>& v, hipStream_t s) {
    auto it = std::find(v.begin(), v.end(), s);
    if (it == v.end()) return false;
    v.erase(it);
    return true;
}

vv_status_t rt(hipError_t e) {
    if (e == hipSuccess) return VV_OK;
    (void)hipGetLastError();          // do not let the failure leak into the next call
    return VV_ERR_CUDA;
}

vv_status_t copy(void* dst, const void* src, size_t size, hipMemcpyKind kind, void* stream) {
    if (size == 0) return VV_OK;
    if (!dst || !src) return VV_ERR_NULL_PTR;
    if (stream) return rt(hipMemcpyAsync(dst, src, size, kind, as_stream(stream)));
    if (break_captures_of_this_thread()) return VV_ERR_CUDA;   // synchronous copy
    return rt(hipMemcpy(dst, src, size, kind));
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_dev_alloc(void** ptr, size_t size) {
    if (!ptr) return VV_ERR_NULL_PTR;
    if (vv::break_captures_of_this_thread()) { *ptr = nullptr; return VV_ERR_CUDA; }
    const hipError_t e = hipMalloc(ptr, size);
    if (e == hipErrorOutOfMemory) { (void)hipGetLastError(); *ptr = nullptr; return VV_ERR_CUDA_OOM; }
    if (e != hipSuccess) { *ptr = nullptr; return vv::rt(e); }
    return VV_OK;
}

vv_status_t vv_dev_alloc_pinned(void** ptr, size_t size) {
    if (!ptr) return VV_ERR_NULL_PTR;
    if (vv::break_captures_of_this_thread()) { *ptr = nullptr; return VV_ERR_CUDA; }
    const hipError_t e = hipHostMalloc(ptr, size, hipHostMallocDefault);
    if (e != hipSuccess) { *ptr = nullptr; return vv::rt(e); }
    return VV_OK;
}

vv_status_t vv_dev_free(void* ptr) {
    if (!ptr) return VV_OK;
    vv::break_captures_of_this_thread();      // hipFree synchronises the device
    return vv::rt(hipFree(ptr));
}

vv_status_t vv_dev_free_pinned(void* ptr) {
    if (!ptr) return VV_OK;
    vv::break_captures_of_this_thread();
    return vv::rt(hipHostFree(ptr));
}

vv_status_t vv_dev_memcpy_h2d(void* dst, const void* src, size_t size, void* stream) {
    return vv::copy(dst, src, size, hipMemcpyHostToDevice, stream);
}

vv_status_t vv_dev_memcpy_d2h(void* dst, const void* src, size_t size, void* stream) {
    return vv::copy(dst, src, size, hipMemcpyDeviceToHost, stream);
}

vv_status_t vv_dev_memcpy_d2d(void* dst, const void* src, size_t size, void* stream) {
    // On a stream, whole chunks at aligned addresses go through this library's own copy kernel (the KV
    // append of a contiguous cache, kv_cache.c:238-245, is two such copies per layer and chunk).
    // Without a stream the copy is ordered on the legacy default stream like any kernel launched there (a
    // device-to-device copy need not block the host); a thread that is capturing keeps the runtime's own path.
    if ((stream || vv::tl_capturing.empty()) && dst && src && size && size % 16 == 0 && vv::aligned16(dst) &&
        vv::aligned16(src) &&
        size / 16 / vv::kWave < 0x7fffffffu) {
        const size_t chunks = size / 16;
        vv::Chunk* d = static_cast<vv::Chunk*>(dst);
        const vv::Chunk* sp = static_cast<const vv::Chunk*>(src);
        hipStream_t st = vv::as_stream(stream);
        // One-wave workgroups either way. Long copies: one chunk per thread (256 MiB: 6.7 TB/s read + written).
        // Short ones are over before that many waves have been handed out: four chunks per thread there
        // (cold, 7 / 17 / 29 MB copied: 3.5 / 5.9 / 9.8 us against 4.4 / 6.6 / 10.2 us; 58 MB: 19.9 against 18.7).
        if (2 * size < (96u << 20)) {
            const dim3 grid((unsigned)((chunks + 4 * vv::kWave - 1) / (4 * vv::kWave)));
            if (vv::use_streaming(2 * size)) vv::copy_chunks<true, vv::kWave, 4><<<grid, vv::kWave, 0, st>>>(d, sp, chunks);
            else vv::copy_chunks<false, vv::kWave, 4><<<grid, vv::kWave, 0, st>>>(d, sp, chunks);
        } else {
            const dim3 grid((unsigned)((chunks + vv::kWave - 1) / vv::kWave));
            vv::copy_chunks<true, vv::kWave, 1><<<grid, vv::kWave, 0, st>>>(d, sp, chunks);
        }
        return vv::launch_status();
    }
    return vv::copy(dst, src, size, hipMemcpyDeviceToDevice, stream);
}

vv_status_t vv_pos_add_dev(int* dst, const int* src, int delta, void* stream) {
    if (!dst || !src) return VV_ERR_NULL_PTR;
    vv::pos_add_kernel<<<1, 1, 0, vv::as_stream(stream)>>>(dst, src, delta);
    return vv::launch_status();
}

vv_status_t vv_dev_memcpy_d2d_at(void* dst_base, const void* src, size_t size,
                                 const int* d_index, void* stream) {
    if (!dst_base || !src || !d_index) return VV_ERR_NULL_PTR;
    if (size == 0) return VV_OK;
    hipStream_t st = vv::as_stream(stream);
    if (size % 16 == 0 && size / 16 <= 0x7FFFFFFFu && vv::aligned16(dst_base) &&
        vv::aligned16(src)) {
        const int chunks = (int)(size / 16);
        vv::copy_at_chunks<<<dim3((unsigned)((chunks + vv::kBlock - 1) / vv::kBlock)), vv::kBlock,
                             0, st>>>(static_cast<vv::Chunk*>(dst_base),
                                      static_cast<const vv::Chunk*>(src), d_index, chunks);
    } else {
        const size_t blocks = (size + vv::kBlock - 1) / vv::kBlock;
        vv::copy_at_bytes<<<dim3((unsigned)blocks), vv::kBlock, 0, st>>>(
            static_cast<unsigned char*>(dst_base), static_cast<const unsigned char*>(src),
            d_index, size);
    }
    return vv::launch_status();
}

vv_status_t vv_dev_memset_async(void* ptr, int value, size_t size, void* stream) {
    if (!ptr) return VV_ERR_NULL_PTR;
    if (size == 0) return VV_OK;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(ptr);
    size_t head = (16 - (addr & 15u)) & 15u;
    if (head > size) head = size;
    const size_t chunks = (size - head) / 16;
    const size_t tail = size - head - chunks * 16;
    size_t blocks = (chunks + vv::kBlock - 1) / vv::kBlock;
    if (blocks == 0) blocks = 1;
    if (blocks > 8192) blocks = 8192;       // grid-stride beyond 32 MiB
    vv::fill_kernel<<<dim3((unsigned)blocks), vv::kBlock, 0, vv::as_stream(stream)>>>(
        static_cast<unsigned char*>(ptr), (unsigned)value & 0xFFu, head, chunks, tail);
    return vv::launch_status();
}

vv_status_t vv_dev_memset(void* ptr, int value, size_t size) {
    if (!ptr) return VV_ERR_NULL_PTR;
    if (vv::break_captures_of_this_thread()) return VV_ERR_CUDA;
    return vv::rt(hipMemset(ptr, value, size));
}

vv_status_t vv_dev_stream_create(void** stream) {
    if (!stream) return VV_ERR_NULL_PTR;
    hipStream_t s = nullptr;
    const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamDefault);
    if (e != hipSuccess) { *stream = nullptr; return vv::rt(e); }
    *stream = s;
    return VV_OK;
}

vv_status_t vv_dev_stream_create_background(void** stream) {
    return vv_dev_stream_create(stream);
}

vv_status_t vv_dev_stream_destroy(void* stream) {
    if (!stream) return VV_OK;
    if (vv::forget(vv::tl_capturing, vv::as_stream(stream))) {
        hipGraph_t g = nullptr;
        if (hipStreamEndCapture(vv::as_stream(stream), &g) == hipSuccess && g)
            (void)hipGraphDestroy(g);
        (void)hipGetLastError();
    }
    vv::forget(vv::tl_broken, vv::as_stream(stream));
    return vv::rt(hipStreamDestroy(vv::as_stream(stream)));
}

vv_status_t vv_dev_stream_sync(void* stream) {
    if (stream) {
        hipStream_t s = vv::as_stream(stream);
        if (std::find(vv::tl_capturing.begin(), vv::tl_capturing.end(), s) !=
            vv::tl_capturing.end()) {
            vv::break_captures_of_this_thread();
            return VV_ERR_CUDA;               // a capturing stream cannot be waited on
        }
        return vv::rt(hipStreamSynchronize(s));
    }
    if (vv::break_captures_of_this_thread()) return VV_ERR_CUDA;
    return vv::rt(hipDeviceSynchronize());
}

vv_status_t vv_dev_set_device(int device_id) { return vv::rt(hipSetDevice(device_id)); }

vv_status_t vv_dev_get_device_info(int device_id, size_t* total_mem, size_t* free_mem,
                                   int* sm_count) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_id) != hipSuccess) return vv::rt(hipErrorInvalidDevice);
    if (total_mem) *total_mem = prop.totalGlobalMem;
    if (sm_count) *sm_count = prop.multiProcessorCount;
    if (free_mem) {
        size_t f = 0, t = 0;
        if (hipSetDevice(device_id) != hipSuccess || hipMemGetInfo(&f, &t) != hipSuccess)
            return vv::rt(hipErrorInvalidDevice);
        *free_mem = f;
    }
    return VV_OK;
}

int vv_dev_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}

vv_status_t vv_dev_get_device_name(int device_id, char* buf, size_t buf_size) {
    if (!buf || buf_size == 0) return VV_ERR_NULL_PTR;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_id) != hipSuccess) {
        buf[0] = '\0';
        return vv::rt(hipErrorInvalidDevice);
    }
    snprintf(buf, buf_size, "%s", prop.name);
    return VV_OK;
}

bool vv_dev_host_shares_memory(int device_id) {
    (void)device_id;
    return false;        // discrete HBM: host copies are separate bytes
}

vv_status_t vv_dev_memcpy_peer(void* dst, int dst_device, const void* src, int src_device,
                               size_t size, void* stream) {
    if (!dst || !src) return VV_ERR_NULL_PTR;
    if (size == 0) return VV_OK;
    return vv::rt(hipMemcpyPeerAsync(dst, dst_device, src, src_device, size,
                                     vv::as_stream(stream)));
}

vv_status_t vv_dev_enable_peer(int device, int peer) {
    if (device == peer) return VV_OK;
    int can = 0;
    if (hipDeviceCanAccessPeer(&can, device, peer) != hipSuccess || !can) {
        (void)hipGetLastError();
        return VV_ERR_UNSUPPORTED;
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    if (hipSetDevice(device) != hipSuccess) return vv::rt(hipErrorInvalidDevice);
    const hipError_t e = hipDeviceEnablePeerAccess(peer, 0);
    (void)hipSetDevice(prev);
    if (e == hipErrorPeerAccessAlreadyEnabled) { (void)hipGetLastError(); return VV_OK; }
    if (e != hipSuccess) { (void)hipGetLastError(); return VV_ERR_UNSUPPORTED; }
    return VV_OK;
}

vv_status_t vv_dev_event_create(void** ev) {
    if (!ev) return VV_ERR_NULL_PTR;
    hipEvent_t e = nullptr;
    // ordering only: no timestamps are taken
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) {
        *ev = nullptr;
        return vv::rt(hipErrorUnknown);
    }
    *ev = e;
    return VV_OK;
}

vv_status_t vv_dev_event_destroy(void* ev) {
    if (!ev) return VV_OK;
    return vv::rt(hipEventDestroy(static_cast<hipEvent_t>(ev)));
}

vv_status_t vv_dev_event_record(void* ev, void* stream) {
    if (!ev) return VV_ERR_NULL_PTR;
    return vv::rt(hipEventRecord(static_cast<hipEvent_t>(ev), vv::as_stream(stream)));
}

vv_status_t vv_dev_event_sync(void* ev) {
    if (!ev) return VV_ERR_NULL_PTR;
    return vv::rt(hipEventSynchronize(static_cast<hipEvent_t>(ev)));
}

vv_status_t vv_dev_stream_wait_event(void* stream, void* ev) {
    if (!ev) return VV_ERR_NULL_PTR;
    return vv::rt(hipStreamWaitEvent(vv::as_stream(stream), static_cast<hipEvent_t>(ev), 0));
}

vv_status_t vv_dev_host_register(void* p, size_t n) {
    if (!p || n == 0) return VV_ERR_NULL_PTR;
    return VV_ERR_UNSUPPORTED;
}

vv_status_t vv_dev_host_unregister(void* p) {
    (void)p;
    return VV_OK;
}

const char* vv_dev_backend_name(void) { return "HIP"; }

vv_status_t vv_dev_graph_begin(void* stream) {
    if (!stream) return VV_ERR_INVALID_ARG;      // the default stream cannot be captured
    hipStream_t s = vv::as_stream(stream);
    vv::forget(vv::tl_broken, s);
    const vv_status_t st = vv::rt(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    if (st == VV_OK) vv::tl_capturing.push_back(s);
    return st;
}

vv_status_t vv_dev_graph_end(void* stream, void** graph_exec) {
    if (!stream || !graph_exec) return VV_ERR_NULL_PTR;
    *graph_exec = nullptr;
    // Ended early by an uncapturable call: nothing was kept, the stream is usable.
    if (vv::forget(vv::tl_broken, vv::as_stream(stream))) return VV_ERR_CUDA;
    vv::forget(vv::tl_capturing, vv::as_stream(stream));
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(vv::as_stream(stream), &graph);
    if (e != hipSuccess || !graph) {
        // A capture broken from outside discards what was recorded; the caller
        // reissues the work directly, so the error must not linger.
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        return VV_ERR_CUDA;
    }
    hipGraphExec_t exec = nullptr;
    const hipError_t ie = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (ie != hipSuccess) { (void)hipGetLastError(); return VV_ERR_CUDA; }
    *graph_exec = exec;
    return VV_OK;
}

vv_status_t vv_dev_graph_launch(void* graph_exec, void* stream) {
    if (!graph_exec) return VV_ERR_NULL_PTR;
    const hipError_t e = hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec),
                                        vv::as_stream(stream));
    if (e != hipSuccess) { (void)hipGetLastError(); return VV_ERR_CUDA_LAUNCH; }
    return VV_OK;
}

void vv_dev_graph_destroy(void* graph_exec) {
    if (graph_exec) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec));
}

}  // extern "C"
