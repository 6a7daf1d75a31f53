// extern "C" surface of libpmetal_hip.so (declared in include/pmetal_hip.h).
//
// Host-side argument validation mirrors the reference's dispatchers
// (crates/pmetal-gguf/src/quantize.rs:17-87, crates/pmetal-gguf/src/dequant.rs:92-132 and :184-216)
// so that a Rust caller sees the same error classes; failures are reported through a return code
// plus a thread-local message slot, the pattern of crates/pmetal-bridge/cpp/bridge/common.h:41-58.
// There is no CPU fallback anywhere in this file: without a HIP device every compute call fails.
#include "../../include/pmetal_hip.h"

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "internal.hpp"

namespace {

thread_local int32_t g_err_code = 0;
thread_local char g_err_msg[512] = {0};

int32_t fail(int32_t code, const char *fmt, ...) {
    g_err_code = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err_msg, sizeof g_err_msg, fmt, ap);
    va_end(ap);
    return code;
}

int32_t ok() {
    g_err_code = 0;
    g_err_msg[0] = 0;
    return PMETAL_HIP_OK;
}

int32_t hip_fail(hipError_t e, const char *what) {
    (void)hipGetLastError();  // do not let a sticky error leak into the next call
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice || e == hipErrorInsufficientDriver)
        return fail(PMETAL_HIP_ERR_NO_DEVICE, "%s: %s", what, hipGetErrorString(e));
    return fail(PMETAL_HIP_ERR_HIP_RUNTIME, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                      \
    do {                                                   \
        hipError_t _e = (expr);                            \
        if (_e != hipSuccess) return hip_fail(_e, #expr);  \
    } while (0)

// types with quantized-linear kernels
bool path_type(uint32_t t) {
    return t == PMETAL_GGML_TYPE_Q8_0 || t == PMETAL_GGML_TYPE_Q4K || t == PMETAL_GGML_TYPE_Q6K;
}
// types with quantize / dequantize kernels: the above, Q5_K (the Q4_K_M recipe gives it to fused attn_qkv tensors) and
// Q8_K (the activation format of the integer dot products, and the first candidate of the KL calibration)
// the 32-element formats beside Q8_0: quantize / dequantize only
bool legacy32_type(uint32_t t) {
    return t == PMETAL_GGML_TYPE_Q4_0 || t == PMETAL_GGML_TYPE_Q4_1 || t == PMETAL_GGML_TYPE_Q5_0 || t == PMETAL_GGML_TYPE_Q5_1 ||
           t == PMETAL_GGML_TYPE_Q8_1;
}
bool codec_type(uint32_t t) {
    return path_type(t) || legacy32_type(t) || t == PMETAL_GGML_TYPE_Q2K || t == PMETAL_GGML_TYPE_Q3K || t == PMETAL_GGML_TYPE_Q5K ||
           t == PMETAL_GGML_TYPE_Q8K;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// One-time check that a usable device exists; compute entry points call it first.
int32_t require_device() {
    static std::once_flag once;
    static hipError_t status = hipSuccess;
    static int count = 0;
    std::call_once(once, [] {
        status = hipGetDeviceCount(&count);
        if (status != hipSuccess) (void)hipGetLastError();
    });
    if (status != hipSuccess) return hip_fail(status, "hipGetDeviceCount");
    if (count <= 0) return fail(PMETAL_HIP_ERR_NO_DEVICE, "no HIP device is visible");
    return PMETAL_HIP_OK;
}

// dequant.rs:193-206 shape_n_elements
int32_t shape_elements(const int32_t *shape, size_t ndim, size_t *out) {
    if (ndim > 0 && !shape) return fail(PMETAL_HIP_ERR_INVALID_ARG, "shape is NULL");
    for (size_t i = 0; i < ndim; i++)
        if (shape[i] < 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "dimensions must be non-negative");
    size_t n = 1;
    for (size_t i = 0; i < ndim; i++) {
        const size_t dim = (size_t)shape[i];
        if (dim != 0 && n > SIZE_MAX / dim) return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "shape is too large");
        n *= dim;
    }
    *out = n;
    return PMETAL_HIP_OK;
}

struct DevBuf {
    void *p = nullptr;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
};

// Library-owned scratch, grown on demand: one buffer per (thread, device, stream), so that neither concurrent callers nor
// one caller's launches on different streams share it.  Launches on one stream run in order and may.
//  * The buffers live in one process-wide list behind a mutex; an entry carries the thread that asked for it.
//  * A buffer that was handed out while its stream was being recorded is pinned: the recording holds its address, so it is
//    neither freed nor replaced while the stream lives -- not when a larger request comes (that one gets a new buffer, the
//    pinned one is kept aside), and not when the thread that recorded ends (a recording may be replayed from any thread).
//  * While a stream is being recorded nothing may be allocated or synchronised on it: a request that the current buffer
//    cannot serve fails with a clear error instead (run the same or a larger shape once before recording).
//  * pmetal_hip_stream_destroy releases every buffer of that stream, whichever thread asked for it, pinned ones included
//    (the recordings made on a destroyed stream must not be replayed any more), so a later stream that happens to get the
//    same handle value starts without entries.
//  * A thread that ends releases its unpinned buffers.
struct Workspace {
    void *p = nullptr;
    size_t bytes = 0;
    int device = -1;
    hipStream_t stream = nullptr;
    bool pinned = false;
    bool retired = false;  // a pinned buffer that a larger one replaced: kept for the recordings that name it
    uint64_t owner = 0;    // token of the thread that asked for it
};
std::mutex g_ws_mu;
std::vector<Workspace> g_ws_all;  // guarded by g_ws_mu
std::atomic<uint64_t> g_ws_next_owner{1};

struct WorkspaceOwner {
    const uint64_t token = g_ws_next_owner.fetch_add(1);
    ~WorkspaceOwner() {  // at thread exit; hipFree fails harmlessly once the runtime is gone
        std::lock_guard<std::mutex> lock(g_ws_mu);
        for (size_t i = 0; i < g_ws_all.size();) {
            Workspace &w = g_ws_all[i];
            if (w.owner == token && !w.pinned) {
                if (w.p) (void)hipFree(w.p);
                g_ws_all.erase(g_ws_all.begin() + (long)i);
            } else {
                i++;
            }
        }
    }
};
thread_local WorkspaceOwner g_ws_owner;

int32_t workspace(size_t bytes, hipStream_t stream, void **out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (stream) HIP_TRY(hipStreamIsCapturing(stream, &cap));
    const bool recording = cap != hipStreamCaptureStatusNone;
    const uint64_t me = g_ws_owner.token;
    std::lock_guard<std::mutex> lock(g_ws_mu);
    size_t at = g_ws_all.size();
    for (size_t i = 0; i < g_ws_all.size(); i++) {
        const Workspace &c = g_ws_all[i];
        if (c.owner == me && c.device == dev && c.stream == stream && !c.retired) at = i;
    }
    if (at == g_ws_all.size()) {
        Workspace fresh;
        fresh.device = dev, fresh.stream = stream, fresh.owner = me;
        g_ws_all.push_back(fresh);
    }
    if (g_ws_all[at].bytes < bytes) {
        if (recording)
            return fail(PMETAL_HIP_ERR_INVALID_ARG,
                        "this call needs %zu bytes of scratch and the stream's buffer holds %zu: nothing can be allocated while the "
                        "stream is being recorded (run a call of this or a larger shape on the stream first)", bytes, g_ws_all[at].bytes);
        if (g_ws_all[at].p) {
            if (g_ws_all[at].pinned) {
                Workspace old = g_ws_all[at];  // a recording still names it
                old.retired = true;
                g_ws_all.push_back(old);
            } else {
                HIP_TRY(hipStreamSynchronize(stream));  // earlier launches on this stream may still use the smaller buffer
                HIP_TRY(hipFree(g_ws_all[at].p));
            }
            g_ws_all[at].p = nullptr, g_ws_all[at].bytes = 0, g_ws_all[at].pinned = false;
        }
        if (bytes) {
            HIP_TRY(hipMalloc(&g_ws_all[at].p, bytes));
            g_ws_all[at].bytes = bytes;
        }
    }
    if (recording) g_ws_all[at].pinned = true;
    *out = g_ws_all[at].p;
    return PMETAL_HIP_OK;
}

// Releases what workspace() holds for `stream`, for every thread.
void drop_workspaces_of(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    for (size_t i = 0; i < g_ws_all.size();) {
        if (g_ws_all[i].stream == stream) {
            if (g_ws_all[i].p) (void)hipFree(g_ws_all[i].p);
            g_ws_all.erase(g_ws_all.begin() + (long)i);
        } else {
            i++;
        }
    }
}

// ---- scratch memory of the entry point that allocates nothing (pmetal_hip_qgemm_noalloc) ----
// A fixed array in the code object: every device that loads the library holds its own copy, at its own address, until the
// process ends.  In host code the name `scratch` is only a handle for hipGetSymbolAddress; kernels and copies get the
// device address looked up below, once per device.
constexpr size_t kNoAllocScratchBytes = PMETAL_HIP_NOALLOC_SCRATCH_BYTES;  // 32 MiB
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
constexpr int kMaxScratchDevices = 64;
// Per device: the array's address, and what tells a second user of the array from the first.  Launches on one stream run
// in order and may follow one another; a call on another stream while the previous call's kernels have not finished (the
// event recorded behind them is not reached), or from another thread while a call is being issued, would overwrite
// scratch that is still being read: such a call is refused.  Calls made while a stream is being recorded cannot be told
// apart this way (an event recorded there belongs to the recording) and stay the caller's to keep apart.
struct NoAllocScratch {
    void *ptr = nullptr;
    hipEvent_t done = nullptr;      // recorded behind the kernels of the last call that was not being recorded
    hipStream_t last = nullptr;     // the stream of that call
    bool pending = false;           // `done` has been recorded and not yet been seen reached
    std::atomic<bool> busy{false};  // a thread is inside the entry point for this device
};
NoAllocScratch g_scratch[kMaxScratchDevices];
std::mutex g_scratch_mu;

// Looks the array's device address up for the calling thread's current device and makes that device's event: set-up, once
// per device (from pmetal_hip_init, else on the first call for that device).
int32_t scratch_of_current_device(NoAllocScratch **out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxScratchDevices) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device %d is beyond the %d devices the library keeps scratch for", dev, kMaxScratchDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    NoAllocScratch &sc = g_scratch[dev];
    if (!sc.ptr) {
        void *p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(PMETAL_HIP_ERR_HIP_RUNTIME, "hipGetSymbolAddress returned no address for the scratch array");
        HIP_TRY(hipEventCreateWithFlags(&sc.done, hipEventDisableTiming));
        sc.ptr = p;
    }
    *out = &sc;
    return PMETAL_HIP_OK;
}

// ---- host-to-host codec calls on large tensors ----
// A tensor of at least kPipeMinElems elements in pageable host memory goes through chunks (a quarter of the tensor, at
// most kPipeElems elements; smaller tensors take one allocate-copy-run-copy round): a few host threads copy a chunk into a
// pinned staging buffer, a copy engine moves it, the kernel runs, and the result comes back the same way, each chunk on
// the stream of its slot, so that the host copies, both transfer directions and the kernels of neighbouring chunks
// overlap.  The slots (pinned and device buffers, streams, events) are made on first use, per device, and kept until
// the process ends; calls take turns (one mutex).
constexpr size_t kPipeElems = (size_t)4 << 20;  // 16 MiB of f32; a multiple of every block size
constexpr size_t kPipeQBytes = kPipeElems / 256 * 292;  // the largest encoded chunk (Q8_K)
constexpr size_t kPipeGrain = 8192, kPipeMinElems = (size_t)256 << 10;  // chunks are multiples of the grain, at least 1 MiB of f32
constexpr int kPipeSlots = 3, kCopyThreads = 4;  // measured: 26 / 38 / 41 / 41 GB/s with 1 / 2 / 4 / 8 copy threads

struct PipeSlot {
    float *h_f32 = nullptr, *d_f32 = nullptr;
    uint8_t *h_q = nullptr, *d_q = nullptr;
    hipStream_t st = nullptr;
    hipEvent_t done = nullptr;
};
struct HostPipe {
    bool ready = false;
    PipeSlot slot[kPipeSlots];
};
std::mutex g_pipe_mutex;
std::map<int, HostPipe> g_pipes;

int32_t host_pipe(HostPipe **out) {  // caller holds g_pipe_mutex
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    HostPipe &p = g_pipes[dev];
    if (!p.ready) {
        for (PipeSlot &sl : p.slot) {  // (a call that failed half way left what it had: only the missing pieces are made)
            if (!sl.h_f32) HIP_TRY(hipHostMalloc((void **)&sl.h_f32, kPipeElems * sizeof(float), hipHostMallocDefault));
            if (!sl.h_q) HIP_TRY(hipHostMalloc((void **)&sl.h_q, kPipeQBytes, hipHostMallocDefault));
            if (!sl.d_f32) HIP_TRY(hipMalloc((void **)&sl.d_f32, kPipeElems * sizeof(float)));
            if (!sl.d_q) HIP_TRY(hipMalloc((void **)&sl.d_q, kPipeQBytes));
            if (!sl.st) HIP_TRY(hipStreamCreateWithFlags(&sl.st, hipStreamNonBlocking));
            if (!sl.done) HIP_TRY(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
        }
        p.ready = true;
    }
    *out = &p;
    return PMETAL_HIP_OK;
}

void par_copy(void *dst, const void *src, size_t bytes) {
    if (bytes < ((size_t)1 << 20)) {
        memcpy(dst, src, bytes);
        return;
    }
    const size_t piece = (bytes / kCopyThreads + 4095) & ~(size_t)4095;
    std::thread helpers[kCopyThreads - 1];
    for (int i = 1; i < kCopyThreads; i++) {
        const size_t off = piece * (size_t)i, len = off < bytes ? (bytes - off < piece ? bytes - off : piece) : 0;
        helpers[i - 1] = std::thread([=] {
            if (len) memcpy((uint8_t *)dst + off, (const uint8_t *)src + off, len);
        });
    }
    memcpy(dst, src, piece < bytes ? piece : bytes);
    for (std::thread &h : helpers) h.join();
}

// quantize == true: f32 at `plain` -> blocks at `packed`; false: the other way (n elements, element order `order`).
int32_t codec_pipelined(bool quantize, uint32_t t, float *plain, uint8_t *packed, size_t n, uint32_t order);

}  // namespace

extern "C" {

int32_t pmetal_hip_device_count(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        hip_fail(e, "hipGetDeviceCount");
        return 0;
    }
    ok();
    return n;
}

int32_t pmetal_hip_init(int32_t device) {
    if (int32_t rc = require_device()) return rc;
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device %d out of range [0, %d)", device, n);
    HIP_TRY(hipSetDevice(device));
    HIP_TRY(hipFree(nullptr));  // forces context creation and code-object load
    NoAllocScratch *sp = nullptr;
    if (int32_t rc = scratch_of_current_device(&sp)) return rc;  // so that pmetal_hip_qgemm_noalloc has nothing left to set up
    return ok();
}

int32_t pmetal_hip_last_error_code(void) { return g_err_code; }
const char *pmetal_hip_last_error_message(void) { return g_err_msg; }
void pmetal_hip_clear_error(void) { ok(); }

// ---- sizes: types.rs:102-187 ----
size_t pmetal_hip_type_size(uint32_t t) {
    switch (t) {
    case PMETAL_GGML_TYPE_Q4_0: return 18;
    case PMETAL_GGML_TYPE_Q4_1: return 20;
    case PMETAL_GGML_TYPE_Q5_0: return 22;
    case PMETAL_GGML_TYPE_Q5_1: return 24;
    case PMETAL_GGML_TYPE_Q8_1: return 36;
    case PMETAL_GGML_TYPE_Q8_0: return 34;
    case PMETAL_GGML_TYPE_Q4K: return 144;
    case PMETAL_GGML_TYPE_Q2K: return 84;
    case PMETAL_GGML_TYPE_Q3K: return 110;
    case PMETAL_GGML_TYPE_Q5K: return 176;
    case PMETAL_GGML_TYPE_Q6K: return 210;
    case PMETAL_GGML_TYPE_Q8K: return 292;
    default: return 0;
    }
}

size_t pmetal_hip_block_size(uint32_t t) {
    switch (t) {
    case PMETAL_GGML_TYPE_Q4_0:
    case PMETAL_GGML_TYPE_Q4_1:
    case PMETAL_GGML_TYPE_Q5_0:
    case PMETAL_GGML_TYPE_Q5_1:
    case PMETAL_GGML_TYPE_Q8_1:
    case PMETAL_GGML_TYPE_Q8_0: return 32;
    case PMETAL_GGML_TYPE_Q4K:
    case PMETAL_GGML_TYPE_Q2K:
    case PMETAL_GGML_TYPE_Q3K:
    case PMETAL_GGML_TYPE_Q5K:
    case PMETAL_GGML_TYPE_Q6K:
    case PMETAL_GGML_TYPE_Q8K: return 256;
    default: return 0;
    }
}

size_t pmetal_hip_tensor_size(uint32_t t, size_t n) {
    const size_t bs = pmetal_hip_block_size(t);
    if (!bs) return 0;
    return (n / bs + (n % bs != 0)) * pmetal_hip_type_size(t);
}

int32_t pmetal_hip_is_supported(uint32_t t) { return codec_type(t) ? 1 : 0; }

int32_t pmetal_hip_expected_byte_size(uint32_t t, const int32_t *shape, size_t ndim, size_t *out_bytes,
                                      size_t *out_elements) {
    if (!codec_type(t)) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "unsupported GGML type %u", t);
    size_t n = 0;
    if (int32_t rc = shape_elements(shape, ndim, &n)) return rc;
    const size_t bs = pmetal_hip_block_size(t), ts = pmetal_hip_type_size(t);
    const size_t blocks = n / bs + (n % bs != 0);
    if (blocks > SIZE_MAX / ts) return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "shape is too large");
    if (out_bytes) *out_bytes = blocks * ts;
    if (out_elements) *out_elements = n;
    return ok();
}

// ---- memory ----
void *pmetal_hip_alloc(size_t bytes) {
    if (require_device()) return nullptr;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        hip_fail(e, "hipMalloc");
        return nullptr;
    }
    ok();
    return p;
}

int32_t pmetal_hip_free(void *p) {
    if (!p) return ok();
    HIP_TRY(hipFree(p));
    return ok();
}

int32_t pmetal_hip_h2d(void *dst, const void *src, size_t bytes) {
    if (bytes && (!dst || !src)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (bytes) HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return ok();
}

int32_t pmetal_hip_d2h(void *dst, const void *src, size_t bytes) {
    if (bytes && (!dst || !src)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (bytes) HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return ok();
}

int32_t pmetal_hip_memset(void *dst, int value, size_t bytes, void *stream) {
    if (bytes && !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (stream) {  // a memset node in a recording has replayed wrongly on this hardware: keep it out
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing((hipStream_t)stream, &st));
        if (st != hipStreamCaptureStatusNone)
            return fail(PMETAL_HIP_ERR_INVALID_ARG, "pmetal_hip_memset cannot be recorded");
    }
    if (bytes) HIP_TRY(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
    return ok();
}

int32_t pmetal_hip_sync(void *stream) {
    if (int32_t rc = require_device()) return rc;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return ok();
}

// ---- streams and recordings ----
void *pmetal_hip_stream_create(void) {
    if (require_device()) return nullptr;
    hipStream_t st = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);  // default priority
    if (e != hipSuccess) {
        hip_fail(e, "hipStreamCreateWithFlags");
        return nullptr;
    }
    ok();
    return st;
}

int32_t pmetal_hip_stream_destroy(void *stream) {
    if (!stream) return ok();
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    drop_workspaces_of((hipStream_t)stream);  // every thread's scratch for this stream, pinned buffers included
    HIP_TRY(hipStreamDestroy((hipStream_t)stream));
    return ok();
}

int32_t pmetal_hip_record_begin(void *stream) {
    if (!stream) return fail(PMETAL_HIP_ERR_INVALID_ARG, "recording needs a stream from pmetal_hip_stream_create");
    if (int32_t rc = require_device()) return rc;
    HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return ok();
}

void *pmetal_hip_record_end(void *stream) {
    if (!stream) {
        fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL stream");
        return nullptr;
    }
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture((hipStream_t)stream, &graph);
    if (e != hipSuccess || !graph) {
        hip_fail(e != hipSuccess ? e : hipErrorUnknown, "hipStreamEndCapture");
        return nullptr;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        hip_fail(e, "hipGraphInstantiate");
        return nullptr;
    }
    ok();
    return exec;
}

int32_t pmetal_hip_replay(void *recording, void *stream) {
    if (!recording) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL recording");
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)recording, (hipStream_t)stream));
    return ok();
}

int32_t pmetal_hip_recording_destroy(void *recording) {
    if (!recording) return ok();
    HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)recording));
    return ok();
}

// ---- events ----
void *pmetal_hip_event_create(void) {
    if (require_device()) return nullptr;
    hipEvent_t ev = nullptr;
    hipError_t e = hipEventCreate(&ev);
    if (e != hipSuccess) {
        hip_fail(e, "hipEventCreate");
        return nullptr;
    }
    ok();
    return ev;
}

int32_t pmetal_hip_event_record(void *event, void *stream) {
    if (!event) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL event");
    HIP_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return ok();
}

int32_t pmetal_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!start || !stop || !ms) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL argument");
    HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
    HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return ok();
}

int32_t pmetal_hip_event_destroy(void *event) {
    if (!event) return ok();
    HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return ok();
}

// ---- quantize ----
int32_t pmetal_hip_quantize_dev(uint32_t t, const float *src, size_t n, uint8_t *dst, size_t dst_len, void *stream) {
    if (!codec_type(t))
        return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Quantization to GGML type %u not yet implemented", t);
    const size_t expected = pmetal_hip_tensor_size(t, n);
    if (dst_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, dst_len);
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(src) || !aligned16(dst)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (legacy32_type(t)) e = pmh::launch_quantize_legacy32(t, src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q8_0) e = pmh::launch_quantize_q8_0(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q4K) e = pmh::launch_quantize_q4k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q5K) e = pmh::launch_quantize_q5k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q8K) e = pmh::launch_quantize_q8k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q2K) e = pmh::launch_quantize_q2k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q3K) e = pmh::launch_quantize_q3k(src, n, dst, s);
    else e = pmh::launch_quantize_q6k(src, n, dst, s);
    if (e != hipSuccess) return hip_fail(e, "quantize kernel launch");
    return ok();
}

// ---- several tensors in one call ----
// A second stream of the library, per calling thread, that takes every other tensor of a batch: a quantizer kernel's last
// workgroups and the next kernel's first then overlap instead of leaving the machine half empty between the launches.
struct SideStream {
    int device = -1;
    hipStream_t s = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    void release() {
        if (fork) (void)hipEventDestroy(fork);
        if (join) (void)hipEventDestroy(join);
        if (s) (void)hipStreamDestroy(s);
        s = nullptr, fork = nullptr, join = nullptr, device = -1;
    }
    ~SideStream() { release(); }  // at thread exit; the calls fail harmlessly once the runtime is gone
};
thread_local SideStream g_side;

// The side stream of the current device for a batch on `s`, or NULL (no error) while `s` is being recorded: a stream that
// joins a recording belongs to it until the recording ends, and this one serves every stream of the thread, so it never
// joins one -- a recorded batch runs on the caller's stream alone.
int32_t side_stream(hipStream_t s, SideStream **out) {
    *out = nullptr;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) HIP_TRY(hipStreamIsCapturing(s, &cap));
    if (cap != hipStreamCaptureStatusNone) return PMETAL_HIP_OK;
    if (g_side.s && g_side.device != dev) {
        (void)hipStreamSynchronize(g_side.s);
        g_side.release();
    }
    if (!g_side.s) {
        HIP_TRY(hipStreamCreateWithFlags(&g_side.s, hipStreamNonBlocking));  // default priority
        HIP_TRY(hipEventCreateWithFlags(&g_side.fork, hipEventDisableTiming));
        HIP_TRY(hipEventCreateWithFlags(&g_side.join, hipEventDisableTiming));
        g_side.device = dev;
    }
    *out = &g_side;
    return PMETAL_HIP_OK;
}

int32_t pmetal_hip_quantize_batch_dev(const pmetal_hip_quantize_desc *descs, size_t count, void *stream) {
    if (count && !descs) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL descriptor array");
    size_t work = 0, only = 0;  // tensors with elements; the last of them
    for (size_t i = 0; i < count; i++) {  // every descriptor is checked before anything is launched
        const pmetal_hip_quantize_desc &d = descs[i];
        if (!codec_type(d.ggml_type))
            return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Quantization to GGML type %u not yet implemented (tensor %zu)", d.ggml_type, i);
        const size_t expected = pmetal_hip_tensor_size(d.ggml_type, d.n);
        if (d.dst_len != expected)
            return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu (tensor %zu)", expected, d.dst_len, i);
        if (d.n == 0) continue;
        if (!d.src_dev || !d.dst_dev) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer (tensor %zu)", i);
        if (!aligned16(d.src_dev) || !aligned16(d.dst_dev))
            return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned (tensor %zu)", i);
        work++, only = i;
    }
    if (work == 0) return ok();
    if (int32_t rc = require_device()) return rc;
    hipStream_t s = (hipStream_t)stream;
    // a single large tensor of a k-quant type is cut in two for the same reason (its super-blocks are independent; Q4_K at
    // 14336 x 4096: 122 -> 114 us, Q6_K 171 -> 149)
    constexpr size_t kSplitMin = (size_t)1 << 24;
    const bool split = work == 1 && descs[only].n >= kSplitMin && pmetal_hip_block_size(descs[only].ggml_type) == 256;
    SideStream *side = nullptr;
    if (work >= 2 || split)
        if (int32_t rc = side_stream(s, &side)) return rc;
    if (side) {
        HIP_TRY(hipEventRecord(side->fork, s));
        HIP_TRY(hipStreamWaitEvent(side->s, side->fork, 0));
    }
    // The tensors take turns between the two streams.  (Giving each to the stream with less work so far keeps the streams in
    // step, so that their kernels end together and the overlap is lost: 15.6 against 15.0 ms for a Llama-3-8B-shaped model.)
    int32_t rc = PMETAL_HIP_OK;
    bool to_side = false;
    for (size_t i = 0; i < count && rc == PMETAL_HIP_OK; i++) {
        const pmetal_hip_quantize_desc &d = descs[i];
        if (d.n == 0) continue;
        if (split && side) {
            const size_t head = (d.n / 2 + 2047) / 2048 * 2048, head_bytes = pmetal_hip_tensor_size(d.ggml_type, head);
            rc = pmetal_hip_quantize_dev(d.ggml_type, d.src_dev, head, d.dst_dev, head_bytes, stream);
            if (rc == PMETAL_HIP_OK)
                rc = pmetal_hip_quantize_dev(d.ggml_type, d.src_dev + head, d.n - head, d.dst_dev + head_bytes, d.dst_len - head_bytes, side->s);
            continue;
        }
        rc = pmetal_hip_quantize_dev(d.ggml_type, d.src_dev, d.n, d.dst_dev, d.dst_len, to_side ? (void *)side->s : stream);
        to_side = side && !to_side;
    }
    if (side) {  // the caller's stream continues behind both, also after a failed launch
        const hipError_t e1 = hipEventRecord(side->join, side->s);
        const hipError_t e2 = e1 == hipSuccess ? hipStreamWaitEvent(s, side->join, 0) : e1;
        if (rc == PMETAL_HIP_OK && e2 != hipSuccess) return hip_fail(e2, "joining the side stream");
    }
    return rc == PMETAL_HIP_OK ? ok() : rc;
}

int32_t pmetal_hip_quantize(uint32_t t, const float *src, size_t n, uint8_t *dst, size_t dst_len) {
    if (!codec_type(t))
        return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Quantization to GGML type %u not yet implemented", t);
    const size_t expected = pmetal_hip_tensor_size(t, n);
    if (dst_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, dst_len);
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (int32_t rc = require_device()) return rc;
    if (n >= kPipeMinElems) return codec_pipelined(true, t, const_cast<float *>(src), dst, n, 0);
    DevBuf din, dout;
    HIP_TRY(hipMalloc(&din.p, n * sizeof(float)));
    HIP_TRY(hipMalloc(&dout.p, expected));
    HIP_TRY(hipMemcpy(din.p, src, n * sizeof(float), hipMemcpyHostToDevice));
    if (int32_t rc = pmetal_hip_quantize_dev(t, (const float *)din.p, n, (uint8_t *)dout.p, expected, nullptr)) return rc;
    HIP_TRY(hipMemcpy(dst, dout.p, expected, hipMemcpyDeviceToHost));  // synchronises the null stream
    return ok();
}

// ---- dequantize ----
int32_t pmetal_hip_dequantize_dev(uint32_t t, const uint8_t *src, size_t src_len, float *dst, size_t n, uint32_t order,
                                  void *stream) {
    if (!codec_type(t)) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Unsupported quantization type: %u", t);
    if (order > PMETAL_HIP_ORDER_GGML) return fail(PMETAL_HIP_ERR_INVALID_ARG, "order must be 0 (REF) or 1 (GGML)");
    const size_t expected = pmetal_hip_tensor_size(t, n);
    if (src_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, src_len);
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(src) || !aligned16(dst)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (legacy32_type(t)) e = pmh::launch_dequantize_legacy32(t, src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q8_0) e = pmh::launch_dequantize_q8_0(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q4K) e = pmh::launch_dequantize_q4k(src, n, dst, order, s);
    else if (t == PMETAL_GGML_TYPE_Q5K) e = pmh::launch_dequantize_q5k(src, n, dst, order, s);
    else if (t == PMETAL_GGML_TYPE_Q8K) e = pmh::launch_dequantize_q8k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q2K) e = pmh::launch_dequantize_q2k(src, n, dst, s);
    else if (t == PMETAL_GGML_TYPE_Q3K) e = pmh::launch_dequantize_q3k(src, n, dst, s);
    else e = pmh::launch_dequantize_q6k(src, n, dst, s);
    if (e != hipSuccess) return hip_fail(e, "dequantize kernel launch");
    return ok();
}

int32_t pmetal_hip_dequantize(uint32_t t, const uint8_t *src, size_t src_len, const int32_t *shape, size_t ndim,
                              float *dst, size_t dst_len, uint32_t order) {
    if (!codec_type(t)) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Unsupported quantization type: %u", t);
    if (order > PMETAL_HIP_ORDER_GGML) return fail(PMETAL_HIP_ERR_INVALID_ARG, "order must be 0 (REF) or 1 (GGML)");
    size_t n = 0;
    if (int32_t rc = shape_elements(shape, ndim, &n)) return rc;
    const size_t bs = pmetal_hip_block_size(t), ts = pmetal_hip_type_size(t);
    const size_t blocks = n / bs + (n % bs != 0);
    if (blocks > SIZE_MAX / ts) return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "shape is too large");
    const size_t expected = blocks * ts;
    if (src_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, src_len);
    if (dst_len < n) return fail(PMETAL_HIP_ERR_INVALID_SIZE, "output holds %zu floats, need %zu", dst_len, n);
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (int32_t rc = require_device()) return rc;
    if (n >= kPipeMinElems) return codec_pipelined(false, t, dst, const_cast<uint8_t *>(src), n, order);
    DevBuf din, dout;
    HIP_TRY(hipMalloc(&din.p, expected));
    HIP_TRY(hipMalloc(&dout.p, n * sizeof(float)));
    HIP_TRY(hipMemcpy(din.p, src, expected, hipMemcpyHostToDevice));
    if (int32_t rc = pmetal_hip_dequantize_dev(t, (const uint8_t *)din.p, expected, (float *)dout.p, n, order, nullptr))
        return rc;
    HIP_TRY(hipMemcpy(dst, dout.p, n * sizeof(float), hipMemcpyDeviceToHost));
    return ok();
}

}  // extern "C"

namespace {
int32_t codec_pipelined(bool quantize, uint32_t t, float *plain, uint8_t *packed, size_t n, uint32_t order) {
    std::lock_guard<std::mutex> lock(g_pipe_mutex);
    HostPipe *p = nullptr;
    if (int32_t rc = host_pipe(&p)) return rc;
    // chunk: a quarter of the tensor (so that the stages of neighbouring chunks overlap), at most what a slot holds
    size_t chunk = ((n / 4 + kPipeGrain - 1) / kPipeGrain) * kPipeGrain;
    chunk = chunk < kPipeMinElems ? kPipeMinElems : (chunk > kPipeElems ? kPipeElems : chunk);
    const size_t chunks = (n + chunk - 1) / chunk, q_chunk = pmetal_hip_tensor_size(t, chunk);
    auto elems_of = [&](size_t i) { return i + 1 < chunks ? chunk : n - i * chunk; };
    int32_t rc = PMETAL_HIP_OK;
    auto retire = [&](size_t i) -> int32_t {  // chunk i's result: staging buffer -> caller's memory
        PipeSlot &sl = p->slot[i % kPipeSlots];
        HIP_TRY(hipEventSynchronize(sl.done));
        if (quantize) par_copy(packed + i * q_chunk, sl.h_q, pmetal_hip_tensor_size(t, elems_of(i)));
        else par_copy(plain + i * chunk, sl.h_f32, elems_of(i) * sizeof(float));
        return PMETAL_HIP_OK;
    };
    auto submit = [&](size_t i) -> int32_t {
        PipeSlot &sl = p->slot[i % kPipeSlots];
        const size_t elems = elems_of(i), qb = pmetal_hip_tensor_size(t, elems);
        if (quantize) {
            par_copy(sl.h_f32, plain + i * chunk, elems * sizeof(float));
            HIP_TRY(hipMemcpyAsync(sl.d_f32, sl.h_f32, elems * sizeof(float), hipMemcpyHostToDevice, sl.st));
            if (int32_t r = pmetal_hip_quantize_dev(t, sl.d_f32, elems, sl.d_q, qb, sl.st)) return r;
            HIP_TRY(hipMemcpyAsync(sl.h_q, sl.d_q, qb, hipMemcpyDeviceToHost, sl.st));
        } else {
            par_copy(sl.h_q, packed + i * q_chunk, qb);
            HIP_TRY(hipMemcpyAsync(sl.d_q, sl.h_q, qb, hipMemcpyHostToDevice, sl.st));
            if (int32_t r = pmetal_hip_dequantize_dev(t, sl.d_q, qb, sl.d_f32, elems, order, sl.st)) return r;
            HIP_TRY(hipMemcpyAsync(sl.h_f32, sl.d_f32, elems * sizeof(float), hipMemcpyDeviceToHost, sl.st));
        }
        HIP_TRY(hipEventRecord(sl.done, sl.st));
        return PMETAL_HIP_OK;
    };
    size_t retired = 0;
    for (size_t i = 0; i < chunks && rc == PMETAL_HIP_OK; i++) {
        if (i >= (size_t)kPipeSlots) {
            rc = retire(retired);
            if (rc == PMETAL_HIP_OK) retired++;
        }
        if (rc == PMETAL_HIP_OK) rc = submit(i);
    }
    for (; retired < chunks && rc == PMETAL_HIP_OK; retired++) rc = retire(retired);
    if (rc != PMETAL_HIP_OK) {  // leave nothing in flight on the staging buffers; keep the first error
        const int32_t code = g_err_code;
        char msg[sizeof g_err_msg];
        memcpy(msg, g_err_msg, sizeof msg);
        for (PipeSlot &sl : p->slot) (void)hipStreamSynchronize(sl.st);
        (void)hipGetLastError();
        g_err_code = code;
        memcpy(g_err_msg, msg, sizeof msg);
        return rc;
    }
    return ok();
}
}  // namespace

extern "C" {

// ---- quantized linear ----
constexpr int64_t kRowLoopMax = 2;  // activation rows up to which qlinear sends a small Q5_K / Q3_K / Q2_K weight through the GEMV, row by row
// types with a fused GEMV but no GEMM kernel of their own (their GEMM goes through Q6_K, see qgemm_reblocked)
static bool gemv_only_type(uint32_t t) { return t == PMETAL_GGML_TYPE_Q5K || t == PMETAL_GGML_TYPE_Q3K || t == PMETAL_GGML_TYPE_Q2K; }
// (These got their GEMV kernels first and reached the matrix cores through re-blocking into Q6_K; each has a matrix kernel of
// its own now, and the re-blocked form is kept for callers that prepared one.)
// check_linear for a GEMM entry point: they are accepted beside the path types, and y must take 16-byte stores
static int32_t check_gemm(uint32_t t, const void *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, const void *y, uint32_t order);

static int32_t check_linear(uint32_t t, const void *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype,
                            const void *y, uint32_t order, bool gemv_only = false) {
    if (!path_type(t) && !(gemv_only && gemv_only_type(t)))
        return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "Unsupported quantization type: %u", t);
    if (order > PMETAL_HIP_ORDER_GGML) return fail(PMETAL_HIP_ERR_INVALID_ARG, "order must be 0 (REF) or 1 (GGML)");
    if (x_dtype > PMETAL_HIP_DTYPE_BF16) return fail(PMETAL_HIP_ERR_INVALID_ARG, "x_dtype must be 0 (f32) or 1 (bf16)");
    if (n <= 0 || k <= 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "n and k must be positive (n=%lld, k=%lld)", (long long)n, (long long)k);
    const int64_t bs = (int64_t)pmetal_hip_block_size(t);
    if (k % bs != 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "k=%lld is not a multiple of the block size %lld", (long long)k, (long long)bs);
    if (n > 0x7FFFFFFF || k / bs > 0x7FFFFFF) return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "n or k too large");
    if (!w || !x || !y) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    // the GEMV kernels store y one float at a time (so that the rows of an [m, n] output can be written one GEMV each);
    // the GEMM stores 16-byte vectors
    if (!aligned16(w) || !aligned16(x) || (gemv_only ? (reinterpret_cast<uintptr_t>(y) & 3u) != 0 : !aligned16(y)))
        return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    return require_device();
}

static int32_t check_gemm(uint32_t t, const void *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, const void *y, uint32_t order) {
    if (int32_t rc = check_linear(t, w, n, k, x, x_dtype, y, order, gemv_only_type(t))) return rc;
    if (!aligned16(y)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    return PMETAL_HIP_OK;
}

int32_t pmetal_hip_qgemv(uint32_t t, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, float *y,
                         uint32_t order, void *stream) {
    if (int32_t rc = check_linear(t, w, n, k, x, x_dtype, y, order, true)) return rc;
    hipError_t e = pmh::launch_qgemv(t, w, n, k, x, x_dtype, y, order, (hipStream_t)stream);
    if (e == hipErrorInvalidValue)  // refused by the launcher before anything ran
        return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE,
                    "qgemv: n=%lld, k=%lld does not fit the kernel of GGML type %u (the activations of a row must fit in LDS: k <= 32768 "
                    "for Q5_K / Q3_K / Q2_K; a tensor must stay below 4 GiB)", (long long)n, (long long)k, t);
    if (e != hipSuccess) return hip_fail(e, "qgemv kernel launch");
    return ok();
}

int32_t pmetal_hip_qgemv_batch(const pmetal_hip_linear_desc *descs, size_t count, void *stream) {
    if (count && !descs) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL descriptor array");
    size_t i = 0;
    while (i < count) {
        const pmetal_hip_linear_desc &d = descs[i];
        // Consecutive small Q4_K projections of the same activation vector (q / k / v, gate / up) share a launch.
        size_t j = i + 1;
        if (d.ggml_type == PMETAL_GGML_TYPE_Q4K && d.k > 0 && d.k % 256 == 0 && d.n > 0 && pmh::qgemv_q4k_groupable(d.n, d.k)) {
            while (j < count && j - i < (size_t)pmh::kMaxGemvGroup) {
                const pmetal_hip_linear_desc &e = descs[j];
                if (e.ggml_type != d.ggml_type || e.k != d.k || e.x_dev != d.x_dev || e.x_dtype != d.x_dtype ||
                    e.order != d.order || e.n <= 0 || !pmh::qgemv_q4k_groupable(e.n, e.k))
                    break;
                j++;
            }
        }
        // A Q6_K projection of the same activations right after such a group (the v of a Q4_K_M layer whose q and k are
        // Q4_K) joins its launch when the shapes suit it.
        if (j > i && j < count && j - i < (size_t)pmh::kMaxGemvGroup && d.ggml_type == PMETAL_GGML_TYPE_Q4K && d.k > 0 && d.k % 256 == 0 &&
            d.n > 0 && pmh::qgemv_q4k_groupable(d.n, d.k)) {
            const pmetal_hip_linear_desc &v = descs[j];
            if (v.ggml_type == PMETAL_GGML_TYPE_Q6K && v.k == d.k && v.x_dev == d.x_dev && v.x_dtype == d.x_dtype && v.order == d.order &&
                v.n > 0) {
                const uint8_t *w[pmh::kMaxGemvGroup];
                float *y[pmh::kMaxGemvGroup];
                int64_t n[pmh::kMaxGemvGroup];
                for (size_t g = i; g < j; g++) {
                    const pmetal_hip_linear_desc &e = descs[g];
                    if (int32_t rc = check_linear(e.ggml_type, e.w_dev, e.n, e.k, e.x_dev, e.x_dtype, e.y_dev, e.order, true)) return rc;
                    w[g - i] = e.w_dev, y[g - i] = e.y_dev, n[g - i] = e.n;
                }
                if (int32_t rc = check_linear(v.ggml_type, v.w_dev, v.n, v.k, v.x_dev, v.x_dtype, v.y_dev, v.order, true)) return rc;
                const hipError_t err = pmh::launch_qgemv_q4k_q6k_group(w, n, y, (int)(j - i), v.w_dev, v.n, v.y_dev, d.k, d.x_dev, d.x_dtype,
                                                                       d.order, (hipStream_t)stream);
                if (err == hipSuccess) {
                    i = j + 1;
                    continue;
                }
                if (err != hipErrorNotSupported) return hip_fail(err, "mixed grouped qgemv kernel launch");
            }
        }
        if (j - i < 2) {
            // Two consecutive large Q4_K projections of the same activation vector (gate / up of a large model) share a
            // launch of the large-matrix kernel.
            if (i + 1 < count && d.ggml_type == PMETAL_GGML_TYPE_Q4K && d.k > 0 && d.k % 256 == 0 && d.n > 0 &&
                !pmh::qgemv_q4k_groupable(d.n, d.k)) {
                const pmetal_hip_linear_desc &e = descs[i + 1];
                if (e.ggml_type == d.ggml_type && e.k == d.k && e.x_dev == d.x_dev && e.x_dtype == d.x_dtype && e.order == d.order &&
                    e.n > 0 && !pmh::qgemv_q4k_groupable(e.n, e.k)) {
                    if (int32_t rc = check_linear(d.ggml_type, d.w_dev, d.n, d.k, d.x_dev, d.x_dtype, d.y_dev, d.order, true)) return rc;
                    if (int32_t rc = check_linear(e.ggml_type, e.w_dev, e.n, e.k, e.x_dev, e.x_dtype, e.y_dev, e.order, true)) return rc;
                    const hipError_t err = pmh::launch_qgemv_q4k_pair(d.w_dev, d.n, d.y_dev, e.w_dev, e.n, e.y_dev, d.k, d.x_dev, d.x_dtype,
                                                                      d.order, (hipStream_t)stream);
                    if (err == hipSuccess) {
                        i += 2;
                        continue;
                    }
                    if (err != hipErrorNotSupported) return hip_fail(err, "paired qgemv kernel launch");
                }
            }
            if (int32_t rc = pmetal_hip_qgemv(d.ggml_type, d.w_dev, d.n, d.k, d.x_dev, d.x_dtype, d.y_dev, d.order, stream))
                return rc;
            i++;
            continue;
        }
        const uint8_t *w[pmh::kMaxGemvGroup];
        float *y[pmh::kMaxGemvGroup];
        int64_t n[pmh::kMaxGemvGroup];
        for (size_t g = i; g < j; g++) {
            const pmetal_hip_linear_desc &e = descs[g];
            if (int32_t rc = check_linear(e.ggml_type, e.w_dev, e.n, e.k, e.x_dev, e.x_dtype, e.y_dev, e.order, true)) return rc;
            w[g - i] = e.w_dev, y[g - i] = e.y_dev, n[g - i] = e.n;
        }
        hipError_t err = pmh::launch_qgemv_q4k_group(w, n, y, (int)(j - i), d.k, d.x_dev, d.x_dtype, d.order, (hipStream_t)stream);
        if (err != hipSuccess) return hip_fail(err, "grouped qgemv kernel launch");
        i = j;
    }
    return ok();
}

// Q3_K and Q2_K have no GEMM kernel of their own (Q5_K got one later and keeps this path for weights re-blocked at load
// time): their super-blocks are re-blocked, exactly, into one or two Q6_K
// tensors (W = A + B), which go through the Q6_K GEMM; two partial results are added in f32.  The re-blocked tensors are
// [A][B], each n * (k / 256) * 210 bytes rounded up to 16.
static size_t up16(size_t v) { return (v + 15) & ~(size_t)15; }

static size_t reblocked_part_bytes(int64_t n, int64_t k) { return up16((size_t)n * (size_t)(k / 256) * 210); }

// The GEMM over re-blocked weights.  scratch: [GEMM scratch][partial result of B][partial result of A when y is not f32].
static int32_t qgemm_over_reblocked(uint32_t t, const uint8_t *wa, int64_t n, int64_t k, const void *x, uint32_t x_dtype, int64_t m,
                                    void *y, uint32_t y_dtype, uint8_t *scratch, size_t gemm_bytes, hipStream_t s) {
    const int parts = pmh::reblock_q6k_parts(t);
    const size_t y_elems = (size_t)m * (size_t)n, y_bytes = up16(y_elems * 4);
    const bool y_f32 = y_dtype == PMETAL_HIP_DTYPE_F32;
    const uint8_t *wb = wa + reblocked_part_bytes(n, k);
    float *yb = (float *)(scratch + gemm_bytes), *ya = y_f32 ? (float *)y : (float *)((uint8_t *)yb + y_bytes);
    hipError_t e;
    if (parts == 1) {
        e = pmh::launch_qgemm(PMETAL_GGML_TYPE_Q6K, wa, n, k, x, x_dtype, m, y, y_dtype, 0, scratch, s);
    } else {  // the second product reuses the first one's converted activations
        e = pmh::launch_qgemm(PMETAL_GGML_TYPE_Q6K, wa, n, k, x, x_dtype, m, ya, PMETAL_HIP_DTYPE_F32, 0, scratch, s);
        if (e == hipSuccess) e = pmh::launch_qgemm(PMETAL_GGML_TYPE_Q6K, wb, n, k, x, x_dtype, m, yb, PMETAL_HIP_DTYPE_F32, 0, scratch, s, true);
        if (e == hipSuccess) e = pmh::launch_add_store(ya, yb, y_elems, y, !y_f32, s);
    }
    if (e == hipErrorNotSupported) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: configuration not supported");
    if (e != hipSuccess) return hip_fail(e, "qgemm kernel launch");
    return ok();
}

static size_t reblocked_scratch_bytes(uint32_t t, int64_t m, int64_t n, int64_t k, uint32_t y_dtype, size_t *gemm_bytes) {
    *gemm_bytes = up16(pmh::qgemm_workspace_bytes(PMETAL_GGML_TYPE_Q6K, m, n, k));
    const size_t y_bytes = up16((size_t)m * (size_t)n * 4);
    return *gemm_bytes + (pmh::reblock_q6k_parts(t) == 2 ? y_bytes * (y_dtype == PMETAL_HIP_DTYPE_F32 ? 1 : 2) : 0);
}

static int32_t check_reblocked_shape(int64_t n, int64_t k, int64_t m) {
    const size_t n_blocks = (size_t)n * (size_t)(k / 256);
    if (n_blocks > SIZE_MAX / 512 || (m > 0 && (size_t)m > SIZE_MAX / 16 / (size_t)n))
        return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "qgemm: shape is too large");
    return PMETAL_HIP_OK;
}

size_t pmetal_hip_reblock_size(uint32_t t, int64_t n, int64_t k) {
    if (!gemv_only_type(t) || n <= 0 || k <= 0 || k % 256 != 0) return 0;
    return (size_t)pmh::reblock_q6k_parts(t) * reblocked_part_bytes(n, k);
}

int32_t pmetal_hip_reblock_dev(uint32_t t, const uint8_t *w, int64_t n, int64_t k, uint32_t order, uint8_t *dst, size_t dst_len,
                               void *stream) {
    if (!gemv_only_type(t)) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "GGML type %u is not re-blocked (Q5_K, Q3_K and Q2_K are)", t);
    if (int32_t rc = check_linear(t, w, n, k, w, 0, dst, order, true)) return rc;
    if (!aligned16(dst)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = check_reblocked_shape(n, k, 0)) return rc;
    const size_t expected = pmetal_hip_reblock_size(t, n, k);
    if (dst_len != expected) return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, dst_len);
    const size_t w_bytes = reblocked_part_bytes(n, k);
    hipError_t e = pmh::launch_reblock_q6k(t, w, (size_t)n * (size_t)(k / 256), order, dst, dst + w_bytes, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "re-blocking kernel launch");
    return ok();
}

int32_t pmetal_hip_qgemm_reblocked(uint32_t t, const uint8_t *reblocked, size_t reblocked_len, int64_t n, int64_t k, const void *x,
                                   uint32_t x_dtype, int64_t m, void *y, uint32_t y_dtype, void *stream) {
    if (!gemv_only_type(t)) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "GGML type %u is not re-blocked (Q5_K, Q3_K and Q2_K are)", t);
    if (int32_t rc = check_linear(t, reblocked, n, k, x, x_dtype, y, 0, true)) return rc;
    if (!aligned16(y)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (y_dtype > PMETAL_HIP_DTYPE_BF16) return fail(PMETAL_HIP_ERR_INVALID_ARG, "y_dtype must be 0 (f32) or 1 (bf16)");
    if (m <= 0 || m > 0x7FFFFFFF) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "m must be in [1, 2^31)");
    if (!pmh::qgemm_fits(PMETAL_GGML_TYPE_Q6K, m, n, k))
        return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: m and k must be at most 2^22 (m = %lld, k = %lld)", (long long)m, (long long)k);
    if (int32_t rc = check_reblocked_shape(n, k, m)) return rc;
    const size_t expected = pmetal_hip_reblock_size(t, n, k);
    if (reblocked_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes of re-blocked weights, got %zu", expected, reblocked_len);
    size_t gemm_bytes = 0;
    const size_t mul_bytes = reblocked_scratch_bytes(t, m, n, k, y_dtype, &gemm_bytes);
    void *ws = nullptr;
    if (int32_t rc = workspace(mul_bytes, (hipStream_t)stream, &ws)) return rc;
    return qgemm_over_reblocked(t, reblocked, n, k, x, x_dtype, m, y, y_dtype, (uint8_t *)ws, gemm_bytes, (hipStream_t)stream);
}

int32_t pmetal_hip_qgemm(uint32_t t, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, int64_t m,
                         void *y, uint32_t y_dtype, uint32_t order, void *stream) {
    if (int32_t rc = check_gemm(t, w, n, k, x, x_dtype, y, order)) return rc;
    if (y_dtype > PMETAL_HIP_DTYPE_BF16) return fail(PMETAL_HIP_ERR_INVALID_ARG, "y_dtype must be 0 (f32) or 1 (bf16)");
    if (m <= 0 || m > 0x7FFFFFFF) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "m must be in [1, 2^31)");
    if (k % 256 != 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: k=%lld is not a multiple of 256", (long long)k);
    if (!pmh::qgemm_fits(t, m, n, k))
        return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: m and k must be at most 2^22 (m = %lld, k = %lld)", (long long)m, (long long)k);
    void *ws = nullptr;
    if (int32_t rc = workspace(pmh::qgemm_workspace_bytes(t, m, n, k), (hipStream_t)stream, &ws)) return rc;
    hipError_t e = pmh::launch_qgemm(t, w, n, k, x, x_dtype, m, y, y_dtype, order, ws, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: configuration not supported");
    if (e != hipSuccess) return hip_fail(e, "qgemm kernel launch");
    return ok();
}

// Several weights against the same activations (gate / up, q / k / v of a prefill): the activation pre-pass runs once per
// element order instead of once per weight.
int32_t pmetal_hip_qgemm_batch(const pmetal_hip_gemm_desc *descs, size_t count, int64_t k, const void *x, uint32_t x_dtype, int64_t m,
                               void *stream) {
    if (count && !descs) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL descriptor array");
    size_t need = 0;
    for (size_t i = 0; i < count; i++) {
        const pmetal_hip_gemm_desc &d = descs[i];
        if (int32_t rc = check_gemm(d.ggml_type, d.w_dev, d.n, k, x, x_dtype, d.y_dev, d.order)) return rc;
        if (d.y_dtype > PMETAL_HIP_DTYPE_BF16) return fail(PMETAL_HIP_ERR_INVALID_ARG, "y_dtype must be 0 (f32) or 1 (bf16)");
        if (m <= 0 || m > 0x7FFFFFFF) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "m must be in [1, 2^31)");
        if (k % 256 != 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: k=%lld is not a multiple of 256", (long long)k);
        if (!pmh::qgemm_fits(d.ggml_type, m, d.n, k))
            return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: m and k must be at most 2^22 (m = %lld, k = %lld)", (long long)m, (long long)k);
        const size_t b = pmh::qgemm_workspace_bytes(d.ggml_type, m, d.n, k);
        need = b > need ? b : need;
    }
    if (count == 0) return ok();
    void *ws = nullptr;
    if (int32_t rc = workspace(need, (hipStream_t)stream, &ws)) return rc;
    // the converted activations depend on the weight type and element order only through the order they are laid out in
    auto layout = [](const pmetal_hip_gemm_desc &d) {
        if (d.ggml_type == PMETAL_GGML_TYPE_Q8_0) return 3;
        if (d.ggml_type == PMETAL_GGML_TYPE_Q6K) return 2;
        if (d.ggml_type == PMETAL_GGML_TYPE_Q3K || d.ggml_type == PMETAL_GGML_TYPE_Q2K) return 5;  // (one element order)
        if (d.order != PMETAL_HIP_ORDER_REF) return 1;  // Q4_K and Q5_K agree in the GGML order
        return d.ggml_type == PMETAL_GGML_TYPE_Q5K ? 4 : 0;
    };
    // ... and through the padded row count of the launch plan, which follows n: the item stride and the place of the row
    // scales behind the items change with it, so a narrow weight behind a wide one gets a pre-pass of its own
    int have = -1, have_mp = -1;
    for (size_t i = 0; i < count; i++) {
        const pmetal_hip_gemm_desc &d = descs[i];
        const int want = layout(d), want_mp = pmh::qgemm_plan(m, d.n, k, d.ggml_type).mp;
        hipError_t e = pmh::launch_qgemm(d.ggml_type, d.w_dev, d.n, k, x, x_dtype, m, d.y_dev, d.y_dtype, d.order, ws, (hipStream_t)stream,
                                         want == have && want_mp == have_mp);
        if (e == hipErrorNotSupported) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: configuration not supported");
        if (e != hipSuccess) return hip_fail(e, "qgemm kernel launch");
        have = want, have_mp = want_mp;
    }
    return ok();
}

// pmetal_hip_qgemm for callers that cannot allocate: the scratch is the fixed `scratch` array of the current device.
// Calls no hipMalloc / hipFree and nothing else that allocates.  Every call on a device uses the same array, so calls that
// overlap on one device race; nothing in it has to start at zero (the pre-pass writes every activation item and row scale
// the main kernel reads, padding rows included, and a K split writes every partial tile before the reduction reads it).
int32_t pmetal_hip_qgemm_noalloc(uint32_t t, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, int64_t m,
                                 void *y, uint32_t y_dtype, uint32_t order, void *stream) {
    if (int32_t rc = check_gemm(t, w, n, k, x, x_dtype, y, order)) return rc;
    if (y_dtype > PMETAL_HIP_DTYPE_BF16) return fail(PMETAL_HIP_ERR_INVALID_ARG, "y_dtype must be 0 (f32) or 1 (bf16)");
    if (m <= 0 || m > 0x7FFFFFFF) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "m must be in [1, 2^31)");
    if (k % 256 != 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: k=%lld is not a multiple of 256", (long long)k);
    if (!pmh::qgemm_fits(t, m, n, k))
        return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemm: m and k must be at most 2^22 (m = %lld, k = %lld)", (long long)m, (long long)k);
    const size_t need = pmh::qgemm_workspace_bytes(t, m, n, k);
    if (need > kNoAllocScratchBytes)
        return fail(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "qgemm_noalloc: m=%lld, n=%lld, k=%lld needs %zu bytes of scratch, the fixed array holds %zu",
                    (long long)m, (long long)n, (long long)k, need, kNoAllocScratchBytes);
    NoAllocScratch *sc = nullptr;
    if (int32_t rc = scratch_of_current_device(&sc)) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) HIP_TRY(hipStreamIsCapturing(s, &cap));
    const bool recording = cap != hipStreamCaptureStatusNone;
    if (sc->busy.exchange(true))
        return fail(PMETAL_HIP_ERR_BUSY, "qgemm_noalloc: another thread is issuing a call on this device, and all calls share one scratch array");
    struct Release {
        std::atomic<bool> &flag;
        ~Release() { flag.store(false); }
    } release{sc->busy};
    if (!recording && sc->pending) {
        if (sc->last == s) {
            // same stream: this call's kernels run behind the previous call's
        } else {
            const hipError_t q = hipEventQuery(sc->done);
            if (q == hipErrorNotReady)
                return fail(PMETAL_HIP_ERR_BUSY, "qgemm_noalloc: the previous call on this device, on another stream, has not finished and "
                                                 "all calls share one scratch array (wait for that stream, or use one stream)");
            if (q != hipSuccess) return hip_fail(q, "hipEventQuery");
            sc->pending = false;
        }
    }
    hipError_t e = pmh::launch_qgemm(t, w, n, k, x, x_dtype, m, y, y_dtype, order, sc->ptr, s);
    if (e == hipErrorNotSupported) return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: configuration not supported");
    if (e != hipSuccess) return hip_fail(e, "qgemm kernel launch");
    if (!recording) {
        HIP_TRY(hipEventRecord(sc->done, s));
        sc->last = s, sc->pending = true;
    }
    return ok();
}

int32_t pmetal_hip_qlinear(uint32_t t, const uint8_t *w, int64_t n, int64_t k, const void *x, uint32_t x_dtype, int64_t m,
                           void *y, uint32_t y_dtype, uint32_t order, void *stream) {
    if (m == 1 && y_dtype == PMETAL_HIP_DTYPE_F32) {
        const int32_t rc = pmetal_hip_qgemv(t, w, n, k, x, x_dtype, (float *)y, order, stream);
        // a shape the GEMV kernels refuse (a row too long for LDS) still has the GEMM, which takes one activation row
        if (rc != PMETAL_HIP_ERR_SHAPE_TOO_LARGE || k % 256 != 0) return rc;
        return pmetal_hip_qgemm(t, w, n, k, x, x_dtype, m, y, y_dtype, order, stream);
    }
    const bool q8_ragged = t == PMETAL_GGML_TYPE_Q8_0 && k % 256 != 0;
    if (q8_ragged && y_dtype != PMETAL_HIP_DTYPE_F32)
        return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qlinear: a Q8_0 row of k=%lld (not a multiple of 256) runs through the GEMV, whose output is f32 only",
                    (long long)k);
    const bool q4k_pair = t == PMETAL_GGML_TYPE_Q4K && m == 2;
    // Two rows of Q5_K, Q3_K or Q2_K through the short-batch GEMM beat two GEMVs (Q5_K: 17.3 against 23.1 us at 14336 x 4096,
    // 11.6 against 12.9 at 6144 x 4096; Q2_K 14.6 against 19.2, Q3_K 17.1 against 22) except on a small weight, where the
    // GEMM's two launches cost more than they save (Q5_K: 10.7 against 7.5 us at 1024 x 4096).
    const bool row_loop_type = gemv_only_type(t) && m <= kRowLoopMax && n * k <= (int64_t(1) << 23);
    if ((q8_ragged || q4k_pair || row_loop_type) && y_dtype == PMETAL_HIP_DTYPE_F32 && m > 1 && n > 0 && k > 0 && x && y) {
        // The fused GEMM walks k in steps of 256, and a Q8_0 row may be any multiple of 32: one fused GEMV per activation row
        // then, back to back on the stream.  Two Q4_K rows are two GEMVs: 13.7 against 16.1 us at 14336 x 4096
        // (three rows: 19.6 against 16.4).
        const size_t x_row = (size_t)k * (x_dtype == PMETAL_HIP_DTYPE_F32 ? 4 : 2);
        for (int64_t r = 0; r < m; r++) {
            const int32_t rc = pmetal_hip_qgemv(t, w, n, k, (const uint8_t *)x + (size_t)r * x_row, x_dtype,
                                                (float *)y + (size_t)r * (size_t)n, order, stream);
            if (rc == PMETAL_HIP_ERR_SHAPE_TOO_LARGE && r == 0 && !q8_ragged) break;  // the GEMM below takes every shape
            if (rc != PMETAL_HIP_OK) return rc;
            if (r == m - 1) return ok();
        }
    }
    return pmetal_hip_qgemm(t, w, n, k, x, x_dtype, m, y, y_dtype, order, stream);
}

// ---- Q4_K_M recipe: crates/pmetal/src/commands/quantize.rs ----
int32_t pmetal_hip_use_more_bits(size_t layer, size_t n_layers) {  // :988-993
    if (n_layers == 0) return 0;
    const size_t eighth = n_layers / 8;
    const size_t rel = layer >= eighth ? layer - eighth : 0;
    return (layer < eighth || layer >= 7 * n_layers / 8 || rel % 3 == 2) ? 1 : 0;
}

int32_t pmetal_hip_is_quantizable_gguf_tensor(const char *name, size_t ndim) {  // :955-980
    if (!name) return 0;
    const size_t len = strlen(name);
    if (!(ndim == 2 || ndim == 3) || len < 7 || strcmp(name + len - 7, ".weight") != 0) return 0;
    std::string lower(name);
    for (char &c : lower)
        if (c >= 'A' && c <= 'Z') c = (char)(c - 'A' + 'a');
    static const char *const kDense[] = {"_norm.weight", "norm.weight", "ffn_gate_inp.weight", "router", "altup",
                                         "laurel", "per_layer_model_proj", "pos_embd", "token_types", "ssm_conv1d",
                                         "shortconv.conv.weight", "attn_rel_b.weight", ".position_embd", ".rel_pos",
                                         ".patch_embd", ".patch_merger"};
    for (const char *pat : kDense)
        if (lower.find(pat) != std::string::npos) return 0;
    return 1;
}

uint32_t pmetal_hip_q4km_tensor_type(const char *name, size_t ndim, size_t n_layers) {  // :999-1137, method q4_k_m
    if (!name || !pmetal_hip_is_quantizable_gguf_tensor(name, ndim)) return PMETAL_GGML_TYPE_F16;
    const std::string s(name);
    if (s == "output.weight" || s == "token_embd.weight") return PMETAL_GGML_TYPE_Q6K;
    size_t layer = 0;  // parse_layer_from_gguf_name :982-986, default 0
    if (s.rfind("blk.", 0) == 0) {
        const size_t dot = s.find('.', 4);
        if (dot != std::string::npos && dot > 4) {
            size_t i = 4, v = 0;
            if (s[i] == '+' && dot > 5) i++;
            bool digits = true;
            for (size_t q = i; q < dot; q++) {
                if (s[q] < '0' || s[q] > '9') {
                    digits = false;
                    break;
                }
                v = v * 10 + (size_t)(s[q] - '0');
            }
            if (digits) layer = v;
        }
    }
    const bool more = pmetal_hip_use_more_bits(layer, n_layers) != 0;
    if (s.find("attn_v.weight") != std::string::npos) return more ? PMETAL_GGML_TYPE_Q6K : PMETAL_GGML_TYPE_Q4K;
    if (s.find("ffn_down.weight") != std::string::npos || s.find("ffn_down_exps.weight") != std::string::npos)
        return more ? PMETAL_GGML_TYPE_Q6K : PMETAL_GGML_TYPE_Q4K;
    if (s.find("attn_output.weight") != std::string::npos) return PMETAL_GGML_TYPE_Q4K;
    if (s.find("attn_qkv.weight") != std::string::npos) return PMETAL_GGML_TYPE_Q5K;
    return PMETAL_GGML_TYPE_Q4K;
}

// ---- synthetic tensors ----
int32_t pmetal_hip_fill_normal_f32(float *dst, size_t n, uint64_t seed, float std, float outlier_rate, float outlier_mag,
                                   void *stream) {
    if (n == 0) return ok();
    if (!dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (int32_t rc = require_device()) return rc;
    hipError_t e = pmh::launch_fill_normal(dst, n, seed, std, outlier_rate, outlier_mag, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "fill kernel launch");
    return ok();
}

int32_t pmetal_hip_f32_to_bf16_dev(const float *src, uint16_t *dst, size_t n, void *stream) {
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (int32_t rc = require_device()) return rc;
    hipError_t e = pmh::launch_f32_to_bf16(src, dst, n, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "convert kernel launch");
    return ok();
}

// ---- Q8_K activations ----
size_t pmetal_hip_q8k_size(size_t n) { return (n / 256 + (n % 256 != 0)) * 292; }

int32_t pmetal_hip_quantize_q8k_dev(const float *src, size_t n, uint8_t *dst, size_t dst_len, void *stream) {
    const size_t expected = pmetal_hip_q8k_size(n);
    if (dst_len != expected)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected %zu bytes, got %zu", expected, dst_len);
    if (n == 0) return ok();
    if (!src || !dst) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(src) || !aligned16(dst)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    hipError_t e = pmh::launch_quantize_q8k(src, n, dst, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "quantize_q8k kernel launch");
    return ok();
}

int32_t pmetal_hip_qgemv_q8k(uint32_t t, const uint8_t *w, int64_t n, int64_t k, const uint8_t *xq, float *y, void *stream) {
    if (t != PMETAL_GGML_TYPE_Q4K && t != PMETAL_GGML_TYPE_Q6K && t != PMETAL_GGML_TYPE_Q5K && t != PMETAL_GGML_TYPE_Q3K &&
        t != PMETAL_GGML_TYPE_Q2K)
        return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "qgemv_q8k: GGML type %u has no Q8_K dot product here", t);
    if (n < 0 || k < 0 || n > 0x7FFFFFFF) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "n and k must be non-negative, n below 2^31");
    if (k % 256 != 0) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemv_q8k: k=%lld is not a multiple of 256", (long long)k);
    if (k > 32768) return fail(PMETAL_HIP_ERR_INVALID_SHAPE, "qgemv_q8k: k=%lld exceeds 32768", (long long)k);
    if (n == 0) return ok();
    if (!w || !xq || !y) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(w) || !aligned16(xq) || !aligned16(y)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    if (k == 0) {  // an empty sum
        hipError_t z = pmh::launch_zero_bytes(reinterpret_cast<uint8_t *>(y), (size_t)n * 4, (hipStream_t)stream);
        if (z != hipSuccess) return hip_fail(z, "fill kernel launch");
        return ok();
    }
    hipError_t e = pmh::launch_qgemv_q8k(t, w, n, k, xq, y, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "qgemv_q8k kernel launch");
    return ok();
}

// ---- KL calibration metric ----
namespace {
// compute_kl_divergence (dynamic.rs:155-178) from the per-workgroup partial sums, added in workgroup order
int32_t kl_score_from_partials(const void *part, int groups, size_t n, double *score, hipStream_t stream) {
    std::vector<double> host((size_t)groups * 4);
    HIP_TRY(hipMemcpyAsync(host.data(), part, host.size() * sizeof(double), hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipStreamSynchronize(stream));
    double sq_err = 0.0, aa = 0.0, ab = 0.0, bb = 0.0;
    for (int g = 0; g < groups; g++) sq_err += host[4 * g], aa += host[4 * g + 1], ab += host[4 * g + 2], bb += host[4 * g + 3];
    const double dn = (double)n;
    const double nrmse = aa > 0.0 ? std::sqrt(sq_err / dn) / std::sqrt(aa / dn) : 0.0;
    const double cos_sim = (aa > 0.0 && bb > 0.0) ? ab / (std::sqrt(aa) * std::sqrt(bb)) : 1.0;
    *score = nrmse + (1.0 - cos_sim);
    return ok();
}
}  // namespace

int32_t pmetal_hip_kl_divergence_dev(const float *original, const float *dequantized, size_t n, double *score, void *stream) {
    if (!score) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (n == 0) {  // dynamic.rs:143-145
        *score = 0.0;
        return ok();
    }
    if (!original || !dequantized) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(original) || !aligned16(dequantized)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    const int groups = pmh::kl_sums_workgroups(n);
    void *part = nullptr;  // the stream's scratch (shared with qgemm: calls on one stream run in order, and this one synchronises)
    if (int32_t rc = workspace((size_t)groups * 4 * sizeof(double), (hipStream_t)stream, &part)) return rc;
    hipError_t e = pmh::launch_kl_sums(original, dequantized, n, (double *)part, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "kl sums kernel launch");
    return kl_score_from_partials(part, groups, n, score, (hipStream_t)stream);
}

int32_t pmetal_hip_kl_divergence_quantized_dev(uint32_t t, const uint8_t *quantized, size_t quantized_len, const float *original, size_t n,
                                               uint32_t order, double *score, void *stream) {
    if (!codec_type(t) || pmetal_hip_block_size(t) != 256)
        return fail(PMETAL_HIP_ERR_UNSUPPORTED_TYPE, "the fused comparison takes the k-quant types only, not GGML type %u", t);
    if (order > PMETAL_HIP_ORDER_GGML) return fail(PMETAL_HIP_ERR_INVALID_ARG, "invalid element order %u", order);
    if (!score) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (quantized_len % pmetal_hip_type_size(t) || n > quantized_len / pmetal_hip_type_size(t) * 256)
        return fail(PMETAL_HIP_ERR_INVALID_SIZE, "%zu bytes of GGML type %u do not hold %zu elements", quantized_len, t, n);
    if (n == 0) {  // dynamic.rs:143-145
        *score = 0.0;
        return ok();
    }
    if (!original || !quantized) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(original) || !aligned16(quantized)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    const int groups = pmh::kl_sums_quantized_workgroups(n);
    void *part = nullptr;
    if (int32_t rc = workspace((size_t)groups * 4 * sizeof(double), (hipStream_t)stream, &part)) return rc;
    hipError_t e = pmh::launch_kl_sums_quantized(t, quantized, original, n, order, (double *)part, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "fused kl sums kernel launch");
    return kl_score_from_partials(part, groups, n, score, (hipStream_t)stream);
}

// ---- measurement aid ----
int32_t pmetal_hip_mfma_probe_f16(int32_t iters, int32_t vary, int32_t workgroups, float *sink, void *stream) {
    if (iters < 0 || workgroups < 1 || workgroups > 65536) return fail(PMETAL_HIP_ERR_INVALID_ARG, "iters >= 0, 1 <= workgroups <= 65536");
    if (!sink) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (int32_t rc = require_device()) return rc;
    hipError_t e = pmh::launch_mfma_probe(iters, vary != 0, workgroups, sink, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "probe kernel launch");
    return ok();
}

int32_t pmetal_hip_read_probe(const void *src, size_t bytes, uint32_t *sink, void *stream) {
    if (!src || !sink) return fail(PMETAL_HIP_ERR_INVALID_ARG, "NULL pointer");
    if (!aligned16(src)) return fail(PMETAL_HIP_ERR_INVALID_ARG, "device pointers must be 16-byte aligned");
    if (int32_t rc = require_device()) return rc;
    hipError_t e = pmh::launch_read_probe(src, bytes, sink, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "probe kernel launch");
    return ok();
}

}  // extern "C"
