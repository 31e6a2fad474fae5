// C ABI of libskainet_hip.so (declared in include/skainet_hip.h): device selection, allocation, one-time
// packed-weight upload, stream and launch. No arithmetic lives here.
//
// Contract mirrored from the reference's native provider: a missing device or library is an answer
// ("unavailable"), never a crash
//   /root/reference/skainet-backends/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/NativeLibraryLoader.kt:24-29
// and the C functions return void, ignore non-positive dimensions and leave the output untouched on a
// resource failure
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/q4k_matmul.c:326-333.
#include "common.h"
#include "gemv_q4k.h"
#include "../../include/skainet_hip.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <mutex>
#include <thread>

namespace skh {

// kernels (one translation unit each)
int launch_dequant(int enc, const uint8_t* w, int64_t nblocks, float* out, const int32_t* row_ids, int bpr, int rows);
int launch_gemv(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y);
int launch_gemm(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y);
int launch_gemm_fused(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y, const float* gain, float eps,
                      const float* residual, int epilogue, float* tmp, bool x_pairs);
int set_tuning(const char* key, int value);
int launch_rms_norm(const float* in, const float* gamma, float* out, int rows, int cols, float eps);
int launch_layer_norm(const float* in, const float* gamma, const float* beta, float* out, int rows, int cols, float eps);
int launch_softmax_rows(const float* in, float* out, int rows, int cols, int log_form);
int launch_silu_mul(const float* gate, const float* up, float* out, int64_t n);
int launch_add(const float* a, const float* b, float* out, int64_t n);
int launch_argmax_rows(const float* in, int rows, int cols, int32_t* out);
int launch_rope_scatter(const float* in, int64_t in_row_pitch, float* out, int tokens, int heads, int head_dim, int pos_start,
                        const int32_t* pos_dev, float theta, int rotate, int64_t out_head_stride, int out_row_is_pos);
int launch_swiglu_pairs(const float* gate_up, float* out, int64_t n);
int launch_q4k_gemv_rows_fused(const uint8_t* w, const float* x, float* y, int k, int n, int batch, const float* gain, float eps,
                               const float* residual, int epilogue, const RopeQkvEpilogue* rope);
int launch_rope_qkv(const float* qkv, float* q_out, float* k_cache, float* v_cache, int tokens, int heads, int kv_heads,
                    int head_dim, int kv_capacity, int pos_start, const int32_t* pos_dev, float theta);
int launch_i32_store_at(int32_t* dst, const int32_t* index, int32_t offset, const int32_t* src);
int launch_rope_table(const int32_t* pos, float theta, int head_dim, float* table);
int launch_narrow_matmul(const float* a, int64_t a_stride, const uint8_t* b, int64_t b_byte_stride, float* c, int64_t c_stride,
                         int m, int n, int k, int fp16);
int launch_decode_advance(int32_t* pos, int32_t* kv_len, const int32_t* token, int32_t* log, int32_t capacity);
int launch_heads_to_rows(const float* in, float* out, int heads, int tokens, int head_dim);
int launch_sdpa_prefill(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads, int seq_q,
                        int seq_kv, int kv_capacity, int head_dim, float scale, int causal, int window, int right_context,
                        const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q, int mask_k, int out_rows);
int launch_i32_increment(int32_t* v, int32_t delta);
int launch_stream_read(const void* p, int64_t bytes, int grid, uint32_t* sink);
int launch_relayout_to_row_major(const uint8_t* src, uint8_t* dst, int rows, int bpr, int block_bytes);
int launch_fp32_matmul(const float* a, int64_t a_stride, const float* b, int64_t b_stride, float* c, int64_t c_stride,
                       int m, int n, int k, bool b_transposed);
int launch_f32_binary(int op, const float* a, int a_mode, const float* b, int b_mode, float* out, int64_t n, int inner);   // elementwise.hip
int launch_f32_unary(int op, const float* in, float* out, int64_t n);
int launch_f32_reduce_all(const float* in, int64_t n, int mean, float* out);
int launch_f32_reduce_axis(const float* in, int outer, int red, int inner, int mean, float* out);
int launch_attn_out_proj_q4k(const uint8_t* wo, int n, int k, const float* q, const float* k_cache, const float* v_cache, int heads,
                             int kv_heads, int head_dim, int seq_kv, int kv_capacity, float scale, int window,
                             const int32_t* lengths, const float* residual, float* out);
int launch_sdpa(const float* q, const float* k, const float* v, float* out, int batch, int heads, int kv_heads,
                int seq_q, int seq_kv, int kv_capacity, int head_dim, float scale, int causal, int window, int right_context,
                const int32_t* lengths, const float* mask, int mask_b, int mask_h, int mask_q, int mask_k);

// ------------------------------------------------------------------------------------------ state
static thread_local char t_error[512] = "";
static thread_local hipStream_t t_stream = nullptr;
static thread_local hipEvent_t t_ev0 = nullptr, t_ev1 = nullptr;

struct Scratch { void* ptr = nullptr; size_t cap = 0; };
static thread_local Scratch t_workspace;          // kernel scratch (attention split-K partials, GEMM staging)
static thread_local Scratch t_stage[6];           // device staging of the host-pointer entries
static thread_local Scratch t_fuse[3];            // normalised input / raw product of the unfused route of matmul_fused / (gate, up) product of the MLP entry
static thread_local Scratch t_pinned[2];          // page-locked host staging of skainet_hip_matmul_host (activations in, product out)
static std::atomic<int> g_upload_chunk_mib{8};    // skainet_hip_weight_upload's page-locked chunks; 0: one blocking copy straight from the caller's memory
static std::atomic<int> g_upload_lanes{4};        // host threads that fill them

static std::mutex g_mutex;
static int g_state = 0;        // 0 = not probed, 1 = usable, -1 = unusable
static int g_device = 0;
static int g_cus = 0;
static char g_name[256] = "";

int set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error, sizeof(t_error), fmt, ap);
    va_end(ap);
    return -1;
}
int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    (void)hipGetLastError();   // clear the sticky error so later calls report their own
    return set_error("%s failed: %s", what, hipGetErrorString(e));
}
static thread_local const char* t_last_kernel = "";
void note_kernel(const char* family) { t_last_kernel = family; }
hipStream_t current_stream() { return t_stream; }
int num_cus() { return g_cus > 0 ? g_cus : 256; }

static int probe_locked(int device) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        g_state = -1;
        return set_error("no HIP device visible");
    }
    if (device < 0 || device >= count) { g_state = -1; return set_error("device %d out of range (%d visible)", device, count); }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) { (void)hipGetLastError(); g_state = -1; return set_error("cannot query device %d", device); }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        g_state = -1;
        return set_error("device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    }
    if (hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); g_state = -1; return set_error("cannot select device %d", device); }
    g_device = device;
    g_cus = prop.multiProcessorCount;
    snprintf(g_name, sizeof(g_name), "%s (%s)", prop.name, prop.gcnArchName);
    g_state = 1;
    return 0;
}

int ensure_device() {
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (g_state == 0) probe_locked(0);
        if (g_state != 1) return t_error[0] ? -1 : set_error("HIP backend unavailable");
    }
    // hipSetDevice is per thread
    static thread_local bool bound = false;
    if (!bound) { if (check_hip(hipSetDevice(g_device), "hipSetDevice") != 0) return -1; bound = true; }
    return 0;
}

// Recorded graphs hold the scratch addresses of the moment they were recorded. Every time a buffer of this thread is
// given back to the device (it grew, or the thread released its scratch) the thread's scratch generation moves on;
// a graph remembers the generation it was recorded under and is refused afterwards (skainet_hip_graph_launch). While a
// capture is open nothing may grow: the call that would need it fails instead of freeing memory under the capture.
static thread_local uint64_t t_scratch_generation = 1;
static thread_local hipStream_t t_capture_stream = nullptr;
static void* scratch_get(Scratch& s, size_t bytes) {
    if (bytes <= s.cap) return s.ptr;
    if (t_capture_stream) {
        set_error("scratch of %zu bytes is needed while a graph capture is open (held: %zu): run the sequence once outside the capture first",
                  bytes, s.cap);
        return nullptr;
    }
    // the old buffer may still be read by queued kernels of this thread's stream
    if (s.ptr) {
        (void)hipStreamSynchronize(t_stream); (void)hipFree(s.ptr); s.ptr = nullptr; s.cap = 0;
        ++t_scratch_generation;
    }
    const size_t cap = (bytes + (1u << 20) - 1) & ~((size_t)(1u << 20) - 1);
    void* p = nullptr;
    if (check_hip(hipMalloc(&p, cap), "hipMalloc(scratch)") != 0) return nullptr;
    s.ptr = p; s.cap = cap;
    return p;
}
// Page-locked host memory, grown on demand (allocated, never registered: existing host memory cannot be pinned here).
static void* pinned_get(Scratch& s, size_t bytes) {
    if (bytes <= s.cap) return s.ptr;
    if (s.ptr) { (void)hipStreamSynchronize(t_stream); (void)hipHostFree(s.ptr); s.ptr = nullptr; s.cap = 0; }
    const size_t cap = (bytes + (1u << 16) - 1) & ~((size_t)(1u << 16) - 1);
    void* p = nullptr;
    if (check_hip(hipHostMalloc(&p, cap, hipHostMallocDefault), "hipHostMalloc(staging)") != 0) return nullptr;
    s.ptr = p; s.cap = cap;
    return p;
}
// Persistent, zero-initialised device memory for cross-workgroup counters (a kernel that uses one leaves it at zero).
// One allocation per host thread, made on first use and never moved, so recorded graphs keep a valid address.
constexpr size_t SYNC_SCRATCH_BYTES = 1u << 20;
static thread_local void* t_sync = nullptr;
void* sync_scratch(size_t bytes) {
    if (bytes > SYNC_SCRATCH_BYTES) { set_error("sync scratch request of %zu bytes exceeds %zu", bytes, SYNC_SCRATCH_BYTES); return nullptr; }
    if (!t_sync) {
        if (t_capture_stream) {
            set_error("the cross-workgroup counters would be allocated while a graph capture is open: run the sequence once outside the capture first");
            return nullptr;
        }
        void* p = nullptr;
        if (check_hip(hipMalloc(&p, SYNC_SCRATCH_BYTES), "hipMalloc(sync scratch)") != 0) return nullptr;
        if (check_hip(hipMemset(p, 0, SYNC_SCRATCH_BYTES), "hipMemset(sync scratch)") != 0) { (void)hipFree(p); return nullptr; }
        t_sync = p;
    }
    return t_sync;
}
// Host -> device copy of `bytes` bytes that returns when the data is on the device. Page-locked sources (the caller
// read the file into memory from skainet_hip_host_alloc) go as ONE asynchronous copy at bus rate. Pageable sources go
// through page-locked chunks: a lane owns two of them and a stream, and copies chunk j + 1 into one buffer while the
// DMA engine moves chunk j out of the other. One host core fills a chunk at about half the bus rate, so large uploads
// run several lanes on threads of their own, lane t taking chunks t, t + lanes, ...
struct UploadLane {
    void* pin[2] = {nullptr, nullptr};
    size_t cap = 0;
    hipEvent_t ev[2] = {nullptr, nullptr};
    hipStream_t stream = nullptr;
};
constexpr int UPLOAD_MAX_LANES = 8;
static UploadLane g_lanes[UPLOAD_MAX_LANES];     // made on first use, kept until the process ends
static std::mutex g_upload_mutex;                // one staged upload at a time: they would share the bus anyway

static hipError_t lane_prepare(UploadLane& l, size_t chunk) {
    hipError_t e;
    if (!l.stream && (e = hipStreamCreateWithFlags(&l.stream, hipStreamNonBlocking)) != hipSuccess) return e;
    for (int b = 0; b < 2; ++b)
        if (!l.ev[b] && (e = hipEventCreateWithFlags(&l.ev[b], hipEventDisableTiming)) != hipSuccess) return e;
    if (l.cap < chunk) {
        for (int b = 0; b < 2; ++b) {
            if (l.pin[b]) { (void)hipHostFree(l.pin[b]); l.pin[b] = nullptr; }
            l.cap = 0;
            if ((e = hipHostMalloc(&l.pin[b], chunk, hipHostMallocDefault)) != hipSuccess) return e;
        }
        l.cap = chunk;
    }
    return hipSuccess;
}
static hipError_t lane_run(UploadLane& l, int lane, int lanes, uint8_t* dst, const uint8_t* src, size_t bytes, size_t chunk) {
    hipError_t e;
    int j = 0;
    for (size_t off = (size_t)lane * chunk; off < bytes; off += (size_t)lanes * chunk, ++j) {
        const int b = j & 1;
        const size_t len = bytes - off < chunk ? bytes - off : chunk;
        // the copy that last left this buffer (two of this lane's chunks ago) must be off the bus before it is overwritten
        if (j >= 2 && (e = hipEventSynchronize(l.ev[b])) != hipSuccess) return e;
        memcpy(l.pin[b], src + off, len);
        if ((e = hipMemcpyAsync(dst + off, l.pin[b], len, hipMemcpyHostToDevice, l.stream)) != hipSuccess) return e;
        if ((e = hipEventRecord(l.ev[b], l.stream)) != hipSuccess) return e;
    }
    return hipStreamSynchronize(l.stream);
}
static int staged_h2d(void* dst, const uint8_t* src, size_t bytes) {
    if (bytes == 0) return 0;
    const size_t chunk = (size_t)g_upload_chunk_mib.load() << 20;
    bool pinned_src = false;
    {
        hipPointerAttribute_t attr;
        const hipError_t e = hipPointerGetAttributes(&attr, src);
        if (e == hipSuccess) pinned_src = attr.type == hipMemoryTypeHost;
        else (void)hipGetLastError();                  // plain malloc memory: not known to the runtime
    }
    // `dst` is fresh memory that no queued work touches, so the lanes' own streams need not wait for the caller's; the
    // call returns only when every lane's stream has drained, which orders the data before anything launched later
    if (pinned_src) {
        if (check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, t_stream), "hipMemcpy(weight)") != 0) return -1;
        return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
    }
    if (chunk == 0 || bytes <= chunk) return check_hip(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy(weight)");
    const size_t chunks = (bytes + chunk - 1) / chunk;
    int lanes = g_upload_lanes.load();
    if ((size_t)lanes > chunks / 2) lanes = (int)(chunks / 2);      // a lane without two chunks of its own overlaps nothing
    if (lanes < 1) lanes = 1;
    std::lock_guard<std::mutex> lock(g_upload_mutex);
    for (int t = 0; t < lanes; ++t)
        if (check_hip(lane_prepare(g_lanes[t], chunk), "upload lane set-up") != 0) return -1;
    hipError_t result[UPLOAD_MAX_LANES];
    std::thread workers[UPLOAD_MAX_LANES];
    const int device = g_device;
    bool started[UPLOAD_MAX_LANES] = {};
    for (int t = 1; t < lanes; ++t) {
        try {
            workers[t] = std::thread([&, t] {
                hipError_t e = hipSetDevice(device);
                result[t] = e != hipSuccess ? e : lane_run(g_lanes[t], t, lanes, static_cast<uint8_t*>(dst), src, bytes, chunk);
            });
            started[t] = true;
        } catch (...) {}                                // no thread to be had: the caller runs that lane below
    }
    result[0] = lane_run(g_lanes[0], 0, lanes, static_cast<uint8_t*>(dst), src, bytes, chunk);
    for (int t = 1; t < lanes; ++t) {
        if (started[t]) workers[t].join();
        else result[t] = lane_run(g_lanes[t], t, lanes, static_cast<uint8_t*>(dst), src, bytes, chunk);
    }
    for (int t = 0; t < lanes; ++t)
        if (check_hip(result[t], "hipMemcpy(weight, staged)") != 0) return -1;
    return 0;
}
float* sdpa_workspace(size_t bytes) { return static_cast<float*>(scratch_get(t_workspace, bytes)); }
void* kernel_workspace(size_t bytes) { return scratch_get(t_workspace, bytes); }

}  // namespace skh

using namespace skh;

struct skainet_hip_weight {
    uint8_t* data;
    int64_t nbytes;
    int32_t encoding, rows, cols;
    bool owned;
};

extern "C" {

// ------------------------------------------------------------------------------------------ runtime
int32_t skainet_hip_available(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_state == 0) probe_locked(0);
    return g_state == 1 ? 1 : 0;
}
int32_t skainet_hip_init(int32_t device) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_state == 1 && device == g_device) return 0;
    // threads bind to the selected device once and their scratch lives there: a process keeps the device it started on
    if (g_state == 1) return set_error("init: this process already runs on device %d; device %d refused", g_device, device);
    return probe_locked(device);          // first probe, or a new attempt after a failed one
}
const char* skainet_hip_last_error(void) { return t_error; }
const char* skainet_hip_device_name(void) { return g_name; }
int32_t skainet_hip_compute_units(void) { return g_cus; }
const char* skainet_hip_last_kernel(void) { return t_last_kernel; }
int32_t skainet_hip_set_stream(void* stream) { t_stream = static_cast<hipStream_t>(stream); return 0; }
// A non-blocking stream of the calling thread's own, made on first use and kept until skainet_hip_thread_release: with
// it the thread's device entries no longer queue behind every other thread's on the null stream.
static thread_local hipStream_t t_own_stream = nullptr;
int32_t skainet_hip_thread_stream(void) {
    if (ensure_device() != 0) return -1;
    if (t_capture_stream) return set_error("thread_stream: a graph capture is open on this thread");
    if (!t_own_stream && check_hip(hipStreamCreateWithFlags(&t_own_stream, hipStreamNonBlocking), "hipStreamCreate") != 0) return -1;
    t_stream = t_own_stream;
    return 0;
}
int32_t skainet_hip_sync(void) {
    if (ensure_device() != 0) return -1;
    return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}
// The calling thread's scratch (kernel workspace, staging of the host-pointer entries, counters, timer events) goes back
// to the device: for worker threads that end while the process lives on. Recorded graphs of this thread hold the old
// addresses and must be freed first; the next call on this thread allocates afresh.
int32_t skainet_hip_thread_release(void) {
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (g_state != 1) return 0;   // nothing was ever allocated
    }
    if (ensure_device() != 0) return -1;
    int rc = check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
    auto drop = [&](Scratch& sc) {
        if (sc.ptr && check_hip(hipFree(sc.ptr), "hipFree(scratch)") != 0) rc = -1;
        sc.ptr = nullptr; sc.cap = 0;
    };
    if (t_own_stream) {
        if (t_stream == t_own_stream) t_stream = nullptr;
        if (check_hip(hipStreamDestroy(t_own_stream), "hipStreamDestroy") != 0) rc = -1;
        t_own_stream = nullptr;
    }
    ++t_scratch_generation;                       // graphs recorded on this thread are stale from here on
    drop(t_workspace);
    for (Scratch& sc : t_stage) drop(sc);
    for (Scratch& sc : t_fuse) drop(sc);
    auto drop_pinned = [&](Scratch& sc) {
        if (sc.ptr && check_hip(hipHostFree(sc.ptr), "hipHostFree(staging)") != 0) rc = -1;
        sc.ptr = nullptr; sc.cap = 0;
    };
    for (Scratch& sc : t_pinned) drop_pinned(sc);
    if (t_sync && check_hip(hipFree(t_sync), "hipFree(sync scratch)") != 0) rc = -1;
    t_sync = nullptr;
    if (t_ev0 && check_hip(hipEventDestroy(t_ev0), "hipEventDestroy") != 0) rc = -1;
    if (t_ev1 && check_hip(hipEventDestroy(t_ev1), "hipEventDestroy") != 0) rc = -1;
    t_ev0 = t_ev1 = nullptr;
    return rc;
}
void* skainet_hip_malloc(size_t bytes) {
    if (ensure_device() != 0) return nullptr;
    void* p = nullptr;
    if (check_hip(hipMalloc(&p, bytes ? bytes : 1), "hipMalloc") != 0) return nullptr;
    return p;
}
int32_t skainet_hip_free(void* p) {
    if (!p) return 0;
    if (ensure_device() != 0) return -1;
    return check_hip(hipFree(p), "hipFree");
}
// Page-locked host memory for a loader to read packed weights into: an upload from it is one DMA transfer with no
// staging copy on the host. Allocated, never registered (existing host memory cannot be pinned here).
void* skainet_hip_host_alloc(size_t bytes) {
    if (ensure_device() != 0) return nullptr;
    void* p = nullptr;
    if (check_hip(hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault), "hipHostMalloc") != 0) return nullptr;
    return p;
}
int32_t skainet_hip_host_free(void* p) {
    if (!p) return 0;
    if (ensure_device() != 0) return -1;
    return check_hip(hipHostFree(p), "hipHostFree");
}
int32_t skainet_hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    if (ensure_device() != 0) return -1;
    if (bytes == 0) return 0;
    if (check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, t_stream), "hipMemcpy h2d") != 0) return -1;
    return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}
int32_t skainet_hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    if (ensure_device() != 0) return -1;
    if (bytes == 0) return 0;
    if (check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, t_stream), "hipMemcpy d2h") != 0) return -1;
    return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}
int32_t skainet_hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    if (ensure_device() != 0) return -1;
    if (bytes == 0) return 0;
    return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, t_stream), "hipMemcpy d2d");
}
int32_t skainet_hip_timer_begin(void) {
    if (ensure_device() != 0) return -1;
    if (!t_ev0) {
        if (check_hip(hipEventCreate(&t_ev0), "hipEventCreate") != 0) return -1;
        if (check_hip(hipEventCreate(&t_ev1), "hipEventCreate") != 0) return -1;
    }
    return check_hip(hipEventRecord(t_ev0, t_stream), "hipEventRecord");
}
float skainet_hip_timer_end_ms(void) {
    if (!t_ev0) { set_error("timer_end without timer_begin"); return -1.f; }
    if (check_hip(hipEventRecord(t_ev1, t_stream), "hipEventRecord") != 0) return -1.f;
    if (check_hip(hipEventSynchronize(t_ev1), "hipEventSynchronize") != 0) return -1.f;
    float ms = -1.f;
    if (check_hip(hipEventElapsedTime(&ms, t_ev0, t_ev1), "hipEventElapsedTime") != 0) return -1.f;
    return ms;
}
int32_t skainet_hip_set_tuning(const char* key, int32_t value) {
    if (!key) return set_error("set_tuning: null key");
    if (!strcmp(key, "upload_chunk_mib")) {
        if (value < 0 || value > 256) return set_error("set_tuning: upload_chunk_mib must be 0 .. 256; got %d", value);
        g_upload_chunk_mib = value;
        return 0;
    }
    if (!strcmp(key, "upload_lanes")) {
        if (value < 1 || value > UPLOAD_MAX_LANES) return set_error("set_tuning: upload_lanes must be 1 .. %d; got %d", UPLOAD_MAX_LANES, value);
        g_upload_lanes = value;
        return 0;
    }
    if (set_tuning(key, value) != 0) return set_error("set_tuning: unknown key '%s'", key);
    return 0;
}

// ------------------------------------------------------------------------------------------ weights
static int check_weight_shape(const char* who, int32_t encoding, int32_t rows, int32_t cols, int64_t* nbytes) {
    if (!is_packed(encoding)) return set_error("%s: unsupported encoding %d", who, encoding);
    if (rows <= 0 || cols <= 0) return set_error("%s: rows and cols must be positive; got %d x %d", who, rows, cols);
    if (cols % block_elems(encoding) != 0)
        return set_error("%s: inputDim must be a multiple of %d; got %d", who, block_elems(encoding), cols);
    *nbytes = (int64_t)rows * (cols / block_elems(encoding)) * block_bytes(encoding);
    return 0;
}

skainet_hip_weight* skainet_hip_weight_upload(const uint8_t* bytes, int64_t nbytes, int32_t encoding, int32_t order,
                                              int32_t rows, int32_t cols) {
    if (ensure_device() != 0) return nullptr;
    int64_t need = 0;
    if (check_weight_shape("weight_upload", encoding, rows, cols, &need) != 0) return nullptr;
    if (!bytes || nbytes < need) { set_error("weight_upload: %lld bytes given, %lld needed", (long long)nbytes, (long long)need); return nullptr; }
    if (order != SKAINET_HIP_ORDER_ROW_MAJOR && order != SKAINET_HIP_ORDER_INPUT_BLOCK_MAJOR) { set_error("weight_upload: unknown block order %d", order); return nullptr; }
    void* dev = nullptr;
    if (check_hip(hipMalloc(&dev, (size_t)need), "hipMalloc(weight)") != 0) return nullptr;
    bool ok;
    if (order == SKAINET_HIP_ORDER_ROW_MAJOR) {
        ok = staged_h2d(dev, bytes, (size_t)need) == 0;
    } else {
        void* tmp = nullptr;
        ok = check_hip(hipMalloc(&tmp, (size_t)need), "hipMalloc(weight staging)") == 0;
        ok = ok && staged_h2d(tmp, bytes, (size_t)need) == 0;
        ok = ok && launch_relayout_to_row_major(static_cast<uint8_t*>(tmp), static_cast<uint8_t*>(dev), rows,
                                                cols / block_elems(encoding), block_bytes(encoding)) == 0;
        ok = ok && check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize") == 0;
        if (tmp) (void)hipFree(tmp);
    }
    if (!ok) { (void)hipFree(dev); return nullptr; }
    return new skainet_hip_weight{static_cast<uint8_t*>(dev), need, encoding, rows, cols, true};
}

skainet_hip_weight* skainet_hip_weight_wrap(const void* device_bytes, int32_t encoding, int32_t rows, int32_t cols) {
    int64_t need = 0;
    if (check_weight_shape("weight_wrap", encoding, rows, cols, &need) != 0) return nullptr;
    if (!device_bytes) { set_error("weight_wrap: null device pointer"); return nullptr; }
    if (reinterpret_cast<uintptr_t>(device_bytes) & 15) { set_error("weight_wrap: device bytes must be 16-byte aligned"); return nullptr; }
    return new skainet_hip_weight{static_cast<uint8_t*>(const_cast<void*>(device_bytes)), need, encoding, rows, cols, false};
}
void skainet_hip_weight_free(skainet_hip_weight* w) {
    if (!w) return;
    if (w->owned && w->data) (void)hipFree(w->data);
    delete w;
}
const void* skainet_hip_weight_data(const skainet_hip_weight* w) { return w ? w->data : nullptr; }
int64_t skainet_hip_weight_nbytes(const skainet_hip_weight* w) { return w ? w->nbytes : 0; }

int32_t skainet_hip_matmul_kind_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out, int32_t kind) {
    if (ensure_device() != 0) return -1;
    if (!w) return set_error("matmul: null weight handle");
    if (m <= 0) return 0;
    if (!x || !out) return set_error("matmul: null activation or output pointer");
    if (kind == 0) return launch_gemv(w->encoding, w->data, x, m, w->cols, w->rows, out);
    if (kind == 1) return launch_gemm(w->encoding, w->data, x, m, w->cols, w->rows, out);
    return set_error("matmul: unknown kernel kind %d", kind);
}
int32_t skainet_hip_matmul_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out) {
    return skainet_hip_matmul_kind_dev(w, x, m, out, m <= 8 ? 0 : 1);
}
// The view-kernel route of the SPI on a resident weight: activations and result live in host memory, the weight stays
// on the device. One call = copy the rows into page-locked staging, one asynchronous upload, the product, one
// asynchronous download, one wait; every buffer belongs to the calling thread and is reused, so a call allocates
// nothing once the thread has seen its largest shape.
int32_t skainet_hip_matmul_host(const skainet_hip_weight* w, const float* x_host, int32_t m, float* out_host) {
    if (ensure_device() != 0) return -1;
    if (!w) return set_error("matmul_host: null weight handle");
    if (m <= 0) return 0;
    if (!x_host || !out_host) return set_error("matmul_host: null activation or output pointer");
    const size_t in_bytes = sizeof(float) * (size_t)m * w->cols, out_bytes = sizeof(float) * (size_t)m * w->rows;
    void* pin_in = pinned_get(t_pinned[0], in_bytes);
    void* pin_out = pinned_get(t_pinned[1], out_bytes);
    float* xd = static_cast<float*>(scratch_get(t_stage[1], in_bytes));
    float* yd = static_cast<float*>(scratch_get(t_stage[2], out_bytes));
    if (!pin_in || !pin_out || !xd || !yd) return -1;
    memcpy(pin_in, x_host, in_bytes);
    if (check_hip(hipMemcpyAsync(xd, pin_in, in_bytes, hipMemcpyHostToDevice, t_stream), "hipMemcpy h2d") != 0) return -1;
    if (skainet_hip_matmul_dev(w, xd, m, yd) != 0) return -1;
    if (check_hip(hipMemcpyAsync(pin_out, yd, out_bytes, hipMemcpyDeviceToHost, t_stream), "hipMemcpy d2h") != 0) return -1;
    if (check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize") != 0) return -1;
    memcpy(out_host, pin_out, out_bytes);
    return 0;
}
// out = epilogue(W . prologue(x)), the products of a decoder block with their neighbouring row ops folded in:
//   gain != NULL: x is RMS-normalised first (x / sqrt(mean(x^2) + eps) * gain, per activation row);
//   epilogue 0: out [m, rows] = product; 1: out = residual + product (residual [m, rows], may be `out`);
//   2: out [m, rows / 2], out[j] = silu(p[2j]) * p[2j + 1] (the weight's rows alternate gate row, up row).
// Decode shapes of Q4_K weights run as ONE kernel, prompt shapes (m > 8) as the tile GEMM with the norm in its bf16 pass and
// the epilogue in the launch that sums its K splits; everything else runs the same arithmetic as separate launches.
int32_t skainet_hip_matmul_fused_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out, const float* gain,
                                     float eps, const float* residual, int32_t epilogue) {
    if (ensure_device() != 0) return -1;
    if (!w) return set_error("matmul_fused: null weight handle");
    if (m <= 0) return 0;
    if (!x || !out) return set_error("matmul_fused: null activation or output pointer");
    if (epilogue < 0 || epilogue > 2) return set_error("matmul_fused: unknown epilogue %d", epilogue);
    if (epilogue == 1 && !residual) return set_error("matmul_fused: the residual epilogue needs a residual pointer");
    if (epilogue == 2 && (w->rows & 1)) return set_error("matmul_fused: the SwiGLU epilogue needs an even row count; got %d", w->rows);
    if (w->encoding == ENC_Q4_K && m <= 2) {
        const int r = launch_q4k_gemv_rows_fused(w->data, x, out, w->cols, w->rows, m, gain, eps, residual, epilogue, nullptr);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    if (m > 8 && is_packed(w->encoding)) {
        // prompt shapes: the norm rides in the pass that rounds the activations to bf16, the epilogue in the launch that
        // sums K splits (no split: a row kernel over the plain product, parked in tmp)
        float* tmp = epilogue != 0 ? static_cast<float*>(scratch_get(t_fuse[1], sizeof(float) * (size_t)m * w->rows)) : nullptr;
        if (epilogue != 0 && !tmp) return -1;
        const int r = launch_gemm_fused(w->encoding, w->data, x, m, w->cols, w->rows, out, gain, eps, residual, epilogue, tmp, false);
        if (r <= 0) return r;
    }
    const float* xin = x;
    if (gain) {
        float* xn = static_cast<float*>(scratch_get(t_fuse[0], sizeof(float) * (size_t)m * w->cols));
        if (!xn || launch_rms_norm(x, gain, xn, m, w->cols, eps) != 0) return -1;
        xin = xn;
    }
    float* y = out;
    if (epilogue != 0) {
        y = static_cast<float*>(scratch_get(t_fuse[1], sizeof(float) * (size_t)m * w->rows));
        if (!y) return -1;
    }
    if (skainet_hip_matmul_dev(w, xin, m, y) != 0) return -1;
    if (epilogue == 1) return launch_add(residual, y, out, (int64_t)m * w->rows);
    if (epilogue == 2) return launch_swiglu_pairs(y, out, (int64_t)m * (w->rows / 2));
    return 0;
}
// A gated MLP block: out = (residual ? residual : 0) + Wdown . swiglu(Wgate_up . rmsnorm(x)), Wgate_up's rows interleaved
// (gate_0, up_0, gate_1, up_1, ...). Prompt shapes (m > 8) of packed weights: the (gate, up) product is parked once, as
// fp32 pairs, and the pass that rounds the down projection's activations to bf16 takes the SwiGLU on the way -- the
// activation itself is never stored as fp32 -- and the residual is added where the down projection stores its tiles.
// Everything else is the two fused products in a row.
int32_t skainet_hip_mlp_swiglu_dev(const skainet_hip_weight* w_gate_up, const skainet_hip_weight* w_down, const float* x, int32_t m,
                                   const float* gain, float eps, const float* residual, float* out) {
    if (ensure_device() != 0) return -1;
    if (!w_gate_up || !w_down) return set_error("mlp_swiglu: null weight handle");
    if (m <= 0) return 0;
    if (!x || !out) return set_error("mlp_swiglu: null activation or output pointer");
    if (w_gate_up->rows & 1) return set_error("mlp_swiglu: the gate/up weight needs an even row count; got %d", w_gate_up->rows);
    if (w_down->cols != w_gate_up->rows / 2)
        return set_error("mlp_swiglu: the down projection takes %d inputs, the gate/up product gives %d", w_down->cols, w_gate_up->rows / 2);
    const int ffn = w_down->cols;
    if (m > 8 && is_packed(w_gate_up->encoding) && is_packed(w_down->encoding)) {
        float* pairs = static_cast<float*>(scratch_get(t_fuse[2], sizeof(float) * (size_t)m * w_gate_up->rows));
        float* tmp = residual ? static_cast<float*>(scratch_get(t_fuse[1], sizeof(float) * (size_t)m * w_down->rows)) : nullptr;
        if (!pairs || (residual && !tmp)) return -1;
        int r = launch_gemm_fused(w_gate_up->encoding, w_gate_up->data, x, m, w_gate_up->cols, w_gate_up->rows, pairs, gain, eps, nullptr, 0,
                                  nullptr, false);
        if (r < 0) return -1;
        if (r == 0) {
            r = launch_gemm_fused(w_down->encoding, w_down->data, pairs, m, ffn, w_down->rows, out, nullptr, 0.f, residual, residual ? 1 : 0,
                                  tmp, true);
            if (r < 0) return -1;
            if (r == 0) return 0;
            // the down projection's shape is outside the tile kernels: finish from the parked pairs
            float* act = static_cast<float*>(scratch_get(t_fuse[0], sizeof(float) * (size_t)m * ffn));
            if (!act || launch_swiglu_pairs(pairs, act, (int64_t)m * ffn) != 0) return -1;
            return skainet_hip_matmul_fused_dev(w_down, act, m, out, nullptr, 0.f, residual, residual ? 1 : 0);
        }
    }
    float* act = static_cast<float*>(scratch_get(t_fuse[2], sizeof(float) * (size_t)m * ffn));
    if (!act) return -1;
    if (skainet_hip_matmul_fused_dev(w_gate_up, x, m, act, gain, eps, nullptr, 2) != 0) return -1;
    return skainet_hip_matmul_fused_dev(w_down, act, m, out, nullptr, 0.f, residual, residual ? 1 : 0);
}
// One decode token's q/k/v projection with everything around it: out row = W . rmsnorm(x) (gain == NULL: no norm),
// W's rows being [q | k | v] heads of head_dim; adjacent pairs of the q and k heads are rotated (RoPE, angle
// pos * theta^(-2i / head_dim), pos read from the device), q goes to q_out [heads, head_dim], k and v to row pos of
// caches laid out [kv_heads, kv_capacity, head_dim]. Q4_K weights: one kernel; otherwise product + rope_qkv.
int32_t skainet_hip_matmul_qkv_rope_dev(const skainet_hip_weight* w, const float* x, const float* gain, float eps, float* q_out,
                                        float* k_cache, float* v_cache, int32_t heads, int32_t kv_heads, int32_t head_dim,
                                        int32_t kv_capacity, const int32_t* pos_dev, float theta, const float* rope_table) {
    if (ensure_device() != 0) return -1;
    if (!w || !x || !q_out || !k_cache || !v_cache || !pos_dev) return set_error("matmul_qkv_rope: null argument");
    if (rope_table && (reinterpret_cast<uintptr_t>(rope_table) & 7)) return set_error("matmul_qkv_rope: the rotation table must be 8-byte aligned");
    if (heads <= 0 || kv_heads <= 0 || head_dim <= 0 || (head_dim & 1))
        return set_error("matmul_qkv_rope: bad head shape %d / %d x %d", heads, kv_heads, head_dim);
    if ((int64_t)w->rows != (int64_t)(heads + 2 * kv_heads) * head_dim)
        return set_error("matmul_qkv_rope: weight has %d rows, the head shape needs %lld", w->rows,
                         (long long)(heads + 2 * kv_heads) * head_dim);
    if (w->encoding == ENC_Q4_K) {
        const RopeQkvEpilogue rope{k_cache, v_cache, pos_dev, reinterpret_cast<const float2*>(rope_table), theta, heads, kv_heads,
                                   head_dim, kv_capacity};
        const int r = launch_q4k_gemv_rows_fused(w->data, x, q_out, w->cols, w->rows, 1, gain, eps, nullptr, EPI_ROPE_QKV, &rope);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    float* qkv = static_cast<float*>(scratch_get(t_fuse[1], sizeof(float) * (size_t)w->rows));
    if (!qkv) return -1;
    if (skainet_hip_matmul_fused_dev(w, x, 1, qkv, gain, eps, nullptr, 0) != 0) return -1;
    return launch_rope_qkv(qkv, q_out, k_cache, v_cache, 1, heads, kv_heads, head_dim, kv_capacity, 0, pos_dev, theta);
}
// `iters` products back to back on this thread's stream, weight i % nweights each time (several copies of one
// weight defeat the memory-side cache), bracketed by HIP events. With use_graph the launches are captured once
// into a HIP graph (kernel nodes only) and replayed, which removes the host's per-launch cost from the GPU timeline.
// The pass is timed `replays` times (each replay is exactly `iters` steps) and the median is returned.
float skainet_hip_matmul_repeat_dev(const skainet_hip_weight* const* weights, int32_t nweights, const float* x, int32_t m,
                                    float* out, int32_t iters, int32_t kind, int32_t use_graph, int32_t replays) {
    if (ensure_device() != 0) return -1.f;
    if (!weights || nweights <= 0 || iters <= 0 || m <= 0) { set_error("matmul_repeat: bad arguments"); return -1.f; }
    if (replays < 1) replays = 1;
    if (replays > 64) replays = 64;
    hipStream_t prev = t_stream, cap = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    float ms = -1.f;
    bool ok = true;
    float samples[64];
    auto median = [&](int count) {
        for (int i = 1; i < count; ++i) for (int j = i; j > 0 && samples[j] < samples[j - 1]; --j) { const float t = samples[j]; samples[j] = samples[j - 1]; samples[j - 1] = t; }
        return samples[count / 2];
    };
    if (use_graph) {
        // capture needs a real (non-null) stream; the graph is then launched on it as well
        ok = check_hip(hipStreamCreateWithFlags(&cap, hipStreamNonBlocking), "hipStreamCreate") == 0;
        if (ok) {
            t_stream = cap;
            // One graph holds about 400 untimed launches (the upload of the graph, clocks and address translations settle
            // on those whatever the step count) and behind them `replays` passes of exactly `iters` launches, with an
            // event-record node between consecutive passes: every timed pass runs in the steady state of one long chain
            // of launches, so a short pass reads the same time per step as a long one (a graph launch of its own per
            // pass costs about 9 us of idle device per pass, 7 % of a 20-step pass). A pass's time is the span
            // between its two events.
            hipEvent_t ev[65] = {};
            for (int r = 0; ok && r <= replays; ++r) ok = check_hip(hipEventCreate(&ev[r]), "hipEventCreate") == 0;
            // every scratch buffer the products need is sized before the capture opens (one eager product per distinct
            // weight shape is enough: the first weight stands for all, they share a shape in every caller); inside the
            // capture a call that would still grow scratch fails instead of freeing memory under it
            ok = ok && skainet_hip_matmul_kind_dev(weights[0], x, m, out, kind) == 0;
            ok = ok && check_hip(hipStreamSynchronize(cap), "hipStreamSynchronize") == 0;
            ok = ok && check_hip(hipStreamBeginCapture(cap, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture") == 0;
            hipStream_t outer_capture = t_capture_stream;
            if (ok) t_capture_stream = cap;
            int step = 0;
            for (int i = 0; ok && i < 400; ++i, ++step) ok = skainet_hip_matmul_kind_dev(weights[step % nweights], x, m, out, kind) == 0;
            bool inner = ok && hipEventRecord(ev[0], cap) == hipSuccess;
            for (int r = 0; ok && r < replays; ++r) {
                for (int i = 0; ok && i < iters; ++i, ++step) ok = skainet_hip_matmul_kind_dev(weights[step % nweights], x, m, out, kind) == 0;
                if (inner && hipEventRecord(ev[r + 1], cap) != hipSuccess) inner = false;
            }
            if (!inner) (void)hipGetLastError();
            t_capture_stream = outer_capture;
            hipError_t e = hipStreamEndCapture(cap, &graph);
            ok = ok && check_hip(e, "hipStreamEndCapture") == 0;
            ok = ok && check_hip(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate") == 0;
            ok = ok && check_hip(hipGraphLaunch(exec, cap), "hipGraphLaunch") == 0;          // uploads the graph
            ok = ok && check_hip(hipStreamSynchronize(cap), "hipStreamSynchronize") == 0;
            ok = ok && skainet_hip_timer_begin() == 0;
            ok = ok && check_hip(hipGraphLaunch(exec, cap), "hipGraphLaunch") == 0;
            float whole = ok ? skainet_hip_timer_end_ms() : -1.f;
            ok = ok && whole >= 0.f;
            for (int r = 0; ok && inner && r < replays; ++r)
                if (hipEventElapsedTime(&samples[r], ev[r], ev[r + 1]) != hipSuccess || samples[r] <= 0.f) { (void)hipGetLastError(); inner = false; }
            if (ok) ms = inner ? median(replays) : whole * (float)iters / (float)(400 + replays * iters);   // no event nodes: the whole chain's mean
            for (int r = 0; r <= replays; ++r) if (ev[r]) (void)hipEventDestroy(ev[r]);
        }
    } else {
        for (int r = 0; ok && r < replays; ++r) {
            ok = skainet_hip_timer_begin() == 0;
            for (int i = 0; ok && i < iters; ++i) ok = skainet_hip_matmul_kind_dev(weights[i % nweights], x, m, out, kind) == 0;
            if (ok) { samples[r] = skainet_hip_timer_end_ms(); ok = samples[r] >= 0.f; }
        }
        if (ok) ms = median(replays);
    }
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    t_stream = prev;
    if (cap) { (void)hipStreamSynchronize(cap); (void)hipStreamDestroy(cap); }
    return ok ? ms : -1.f;
}

// Read-rate calibration: `iters` launches of a pure streaming-read kernel over buffers[i % nbuffers] (each `bytes`
// long), timed with HIP events on this thread's stream. Returns milliseconds, < 0 on failure.
float skainet_hip_read_probe_dev(const void* const* buffers, int32_t nbuffers, int64_t bytes, int32_t iters, int32_t grid) {
    if (ensure_device() != 0) return -1.f;
    if (!buffers || nbuffers <= 0 || iters <= 0 || bytes < 16) { set_error("read_probe: bad arguments"); return -1.f; }
    uint32_t* sink = static_cast<uint32_t*>(scratch_get(t_workspace, 256));
    if (!sink) return -1.f;
    for (int i = 0; i < 3; ++i) if (launch_stream_read(buffers[i % nbuffers], bytes, grid, sink) != 0) return -1.f;
    if (skainet_hip_timer_begin() != 0) return -1.f;
    for (int i = 0; i < iters; ++i) if (launch_stream_read(buffers[i % nbuffers], bytes, grid, sink) != 0) return -1.f;
    return skainet_hip_timer_end_ms();
}

int32_t skainet_hip_dequantize_dev(const skainet_hip_weight* w, float* out) {
    if (ensure_device() != 0) return -1;
    if (!w || !out) return set_error("dequantize: null argument");
    return launch_dequant(w->encoding, w->data, (int64_t)w->rows * (w->cols / block_elems(w->encoding)), out, nullptr, 1, w->rows);
}
int32_t skainet_hip_dequantize_rows_dev(const skainet_hip_weight* w, const int32_t* row_ids, int32_t count, float* out) {
    if (ensure_device() != 0) return -1;
    if (!w || !out || !row_ids) return set_error("dequantize_rows: null argument");
    if (count <= 0) return 0;
    const int bpr = w->cols / block_elems(w->encoding);
    return launch_dequant(w->encoding, w->data, (int64_t)count * bpr, out, row_ids, bpr, w->rows);
}

// ------------------------------------------------------------------------------------------ device entries
int32_t skainet_hip_fp32_matmul_dev(const float* a, int32_t a_offset, int32_t a_stride, const float* b, int32_t b_offset,
                                    int32_t b_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    if (ensure_device() != 0) return -1;
    if (m <= 0 || n <= 0) return 0;
    return launch_fp32_matmul(a + a_offset, a_stride, b + b_offset, b_stride, c + c_offset, c_stride, m, n, k, false);
}
int32_t skainet_hip_fp32_matmul_wt_dev(const float* in, int32_t in_offset, const float* w, int32_t w_offset, float* out,
                                       int32_t out_offset, int32_t m, int32_t n, int32_t k) {
    if (ensure_device() != 0) return -1;
    if (m <= 0 || n <= 0 || k < 0) return 0;
    return launch_fp32_matmul(in + in_offset, k, w + w_offset, k, out + out_offset, n, m, n, k, true);
}
int32_t skainet_hip_f32_rms_norm_dev(const float* in, const float* gamma, float* out, int32_t rows, int32_t cols, float eps) {
    if (ensure_device() != 0) return -1;
    return launch_rms_norm(in, gamma, out, rows, cols, eps);
}
int32_t skainet_hip_f32_layer_norm_dev(const float* in, const float* gamma, const float* beta, float* out, int32_t rows,
                                      int32_t cols, float eps) {
    if (ensure_device() != 0) return -1;
    return launch_layer_norm(in, gamma, beta, out, rows, cols, eps);
}
int32_t skainet_hip_f32_softmax_rows_dev(const float* in, float* out, int32_t rows, int32_t cols, int32_t log_form) {
    if (ensure_device() != 0) return -1;
    return launch_softmax_rows(in, out, rows, cols, log_form);
}
int32_t skainet_hip_f32_sdpa_dev(const float* q, const float* k, const float* v, float* out, int32_t batch, int32_t heads,
                                 int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t head_dim, float scale,
                                 int32_t causal, int32_t window, int32_t right_context, const int32_t* lengths,
                                 const float* mask, int32_t mask_b, int32_t mask_h, int32_t mask_q, int32_t mask_k) {
    if (ensure_device() != 0) return -1;
    return launch_sdpa(q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, seq_kv, head_dim, scale, causal, window, right_context,
                       lengths, mask, mask_b, mask_h, mask_q, mask_k);
}
int32_t skainet_hip_f32_sdpa_cache_dev(const float* q, const float* k_cache, const float* v_cache, float* out, int32_t batch,
                                       int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t kv_capacity,
                                       int32_t head_dim, float scale, int32_t causal, int32_t window, int32_t right_context,
                                       const int32_t* lengths) {
    if (ensure_device() != 0) return -1;
    return launch_sdpa(q, k_cache, v_cache, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale, causal,
                       window, right_context, lengths, nullptr, 0, 0, 0, 0);
}
// skainet_hip_f32_sdpa_cache_dev with the output laid out [batch, seq_q, heads, head_dim]: token rows, the input of the
// output projection as it is. Prompt shapes that the matrix-core kernel carries are stored that way by the kernel; every
// other shape runs the head-major attention into scratch and one transposing pass per sequence.
int32_t skainet_hip_f32_sdpa_cache_rows_dev(const float* q, const float* k_cache, const float* v_cache, float* out, int32_t batch,
                                            int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t kv_capacity,
                                            int32_t head_dim, float scale, int32_t causal, int32_t window, int32_t right_context,
                                            const int32_t* lengths) {
    if (ensure_device() != 0) return -1;
    if (batch <= 0 || heads <= 0 || kv_heads <= 0 || seq_q <= 0 || head_dim <= 0) return 0;
    const bool plain = heads % kv_heads == 0 && window >= 0 && right_context >= 0 && (right_context == 0 || window != 0) &&
                       kv_capacity >= seq_kv && seq_kv > 0;
    if (plain && seq_q > 1) {
        const int r = launch_sdpa_prefill(q, k_cache, v_cache, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale,
                                          causal, window, right_context, lengths, nullptr, 0, 0, 0, 0, 1);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    const size_t per_seq = (size_t)heads * seq_q * head_dim;
    float* tmp = static_cast<float*>(scratch_get(t_fuse[0], sizeof(float) * per_seq * batch));
    if (!tmp) return -1;
    if (launch_sdpa(q, k_cache, v_cache, tmp, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale, causal, window,
                    right_context, lengths, nullptr, 0, 0, 0, 0) != 0) return -1;     // the argument rules and their messages are its own
    for (int b = 0; b < batch; ++b)
        if (launch_heads_to_rows(tmp + b * per_seq, out + b * per_seq, heads, seq_q, head_dim) != 0) return -1;
    return 0;
}
// One decode token: out = (residual ? residual : 0) + Wo . sdpa(q, cache). Q4_K projections whose input is at most 4096
// wide run as two launches (attention leaving its key splits unmerged, the projection merging them as it loads its
// activations); everything else as attention into `attn_tmp` followed by the fused product.
int32_t skainet_hip_attn_out_proj_dev(const skainet_hip_weight* wo, const float* q, const float* k_cache, const float* v_cache,
                                      int32_t heads, int32_t kv_heads, int32_t head_dim, int32_t seq_kv, int32_t kv_capacity,
                                      float scale, int32_t window, const int32_t* lengths, const float* residual, float* out,
                                      float* attn_tmp) {
    if (ensure_device() != 0) return -1;
    if (!wo) return set_error("attn_out_proj: null weight handle");
    if (!q || !k_cache || !v_cache || !out || !attn_tmp) return set_error("attn_out_proj: null pointer");
    if (heads <= 0 || kv_heads <= 0 || head_dim <= 0) return set_error("attn_out_proj: heads, kv_heads and head_dim must be positive");
    if (wo->cols != heads * head_dim) return set_error("attn_out_proj: the weight takes %d inputs, the attention gives %d", wo->cols, heads * head_dim);
    if (wo->encoding == ENC_Q4_K) {
        const int r = launch_attn_out_proj_q4k(wo->data, wo->rows, wo->cols, q, k_cache, v_cache, heads, kv_heads, head_dim, seq_kv,
                                               kv_capacity, scale, window, lengths, residual, out);
        if (r != 0) return r < 0 ? -1 : 0;
    }
    if (launch_sdpa(q, k_cache, v_cache, attn_tmp, 1, heads, kv_heads, 1, seq_kv, kv_capacity, head_dim, scale, 1, window, 0, lengths,
                    nullptr, 0, 0, 0, 0) != 0) return -1;
    return skainet_hip_matmul_fused_dev(wo, attn_tmp, 1, out, nullptr, 0.f, residual, residual ? 1 : 0);
}
int32_t skainet_hip_f32_silu_mul_dev(const float* gate, const float* up, float* out, int64_t n) {
    if (ensure_device() != 0) return -1;
    return launch_silu_mul(gate, up, out, n);
}
int32_t skainet_hip_f32_add_dev(const float* a, const float* b, float* out, int64_t n) {
    if (ensure_device() != 0) return -1;
    return launch_add(a, b, out, n);
}
int32_t skainet_hip_f32_binary_dev(int32_t op, const float* a, int32_t a_mode, const float* b, int32_t b_mode, float* out,
                                   int64_t n, int32_t inner) {
    if (ensure_device() != 0) return -1;
    return launch_f32_binary(op, a, a_mode, b, b_mode, out, n, inner);
}
int32_t skainet_hip_f32_unary_dev(int32_t op, const float* in, float* out, int64_t n) {
    if (ensure_device() != 0) return -1;
    return launch_f32_unary(op, in, out, n);
}
int32_t skainet_hip_f32_reduce_all_dev(const float* in, int64_t n, int32_t mean, float* out) {
    if (ensure_device() != 0) return -1;
    return launch_f32_reduce_all(in, n, mean, out);
}
int32_t skainet_hip_f32_reduce_axis_dev(const float* in, int32_t outer, int32_t red, int32_t inner, int32_t mean, float* out) {
    if (ensure_device() != 0) return -1;
    return launch_f32_reduce_axis(in, outer, red, inner, mean, out);
}
int32_t skainet_hip_f32_argmax_rows_dev(const float* in, int32_t rows, int32_t cols, int32_t* out) {
    if (ensure_device() != 0) return -1;
    return launch_argmax_rows(in, rows, cols, out);
}

int32_t skainet_hip_f32_rope_scatter_dev(const float* in, int64_t in_row_pitch, float* out, int32_t tokens, int32_t heads,
                                         int32_t head_dim, int32_t pos_start, const int32_t* pos_dev, float theta,
                                         int32_t rotate, int64_t out_head_stride, int32_t out_row_is_pos) {
    if (ensure_device() != 0) return -1;
    return launch_rope_scatter(in, in_row_pitch, out, tokens, heads, head_dim, pos_start, pos_dev, theta, rotate, out_head_stride,
                               out_row_is_pos);
}
int32_t skainet_hip_f32_rope_table_dev(const int32_t* pos_dev, float theta, int32_t head_dim, float* table) {
    if (ensure_device() != 0) return -1;
    if (!pos_dev || !table) return set_error("rope_table: null argument");
    return launch_rope_table(pos_dev, theta, head_dim, table);
}
int32_t skainet_hip_decode_advance_dev(int32_t* pos, int32_t* kv_len, const int32_t* token, int32_t* log, int32_t capacity) {
    if (ensure_device() != 0) return -1;
    if (!pos || !kv_len || !token || !log) return set_error("decode_advance: null argument");
    return launch_decode_advance(pos, kv_len, token, log, capacity);
}
int32_t skainet_hip_i32_store_at_dev(int32_t* dst, const int32_t* index_dev, int32_t offset, const int32_t* src) {
    if (ensure_device() != 0) return -1;
    return launch_i32_store_at(dst, index_dev, offset, src);
}
int32_t skainet_hip_f32_swiglu_pairs_dev(const float* gate_up, float* out, int64_t n) {
    if (ensure_device() != 0) return -1;
    return launch_swiglu_pairs(gate_up, out, n);
}
int32_t skainet_hip_f32_rope_qkv_dev(const float* qkv, float* q_out, float* k_cache, float* v_cache, int32_t tokens, int32_t heads,
                                     int32_t kv_heads, int32_t head_dim, int32_t kv_capacity, int32_t pos_start,
                                     const int32_t* pos_dev, float theta) {
    if (ensure_device() != 0) return -1;
    return launch_rope_qkv(qkv, q_out, k_cache, v_cache, tokens, heads, kv_heads, head_dim, kv_capacity, pos_start, pos_dev, theta);
}
int32_t skainet_hip_f32_heads_to_rows_dev(const float* in, float* out, int32_t heads, int32_t tokens, int32_t head_dim) {
    if (ensure_device() != 0) return -1;
    return launch_heads_to_rows(in, out, heads, tokens, head_dim);
}
int32_t skainet_hip_i32_increment_dev(int32_t* value, int32_t delta) {
    if (ensure_device() != 0) return -1;
    return launch_i32_increment(value, delta);
}

// ---- HIP graphs: record this thread's device entries once, replay them with one launch ----
// A graph belongs to the thread that recorded it: the scratch addresses in it are that thread's, and so is the
// generation counter they are checked against (`owner` points at the recording thread's counter; another thread's
// launch is refused).
struct skainet_hip_graph { hipGraph_t graph; hipGraphExec_t exec; uint64_t scratch_generation; const uint64_t* owner; };
static thread_local hipStream_t t_capture_prev = nullptr;

int32_t skainet_hip_graph_begin(void) {
    if (ensure_device() != 0) return -1;
    if (t_capture_stream) return set_error("graph_begin: a capture is already open on this thread");
    hipStream_t cap = nullptr;
    if (check_hip(hipStreamCreateWithFlags(&cap, hipStreamNonBlocking), "hipStreamCreate") != 0) return -1;
    if (check_hip(hipStreamBeginCapture(cap, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture") != 0) {
        (void)hipStreamDestroy(cap);
        return -1;
    }
    t_capture_prev = t_stream;
    t_capture_stream = cap;
    t_stream = cap;
    return 0;
}
skainet_hip_graph* skainet_hip_graph_end(void) {
    if (!t_capture_stream) { set_error("graph_end without graph_begin"); return nullptr; }
    hipStream_t cap = t_capture_stream;
    t_stream = t_capture_prev;
    t_capture_stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    if (check_hip(hipStreamEndCapture(cap, &graph), "hipStreamEndCapture") != 0 ||
        check_hip(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate") != 0) {
        if (graph) (void)hipGraphDestroy(graph);
        (void)hipStreamDestroy(cap);
        return nullptr;
    }
    (void)hipStreamDestroy(cap);   // replays run on the calling thread's stream, in order with its eager work
    return new skainet_hip_graph{graph, exec, t_scratch_generation, &t_scratch_generation};
}
int32_t skainet_hip_graph_valid(const skainet_hip_graph* g) {
    return g && g->owner == &t_scratch_generation && g->scratch_generation == t_scratch_generation ? 1 : 0;
}
int32_t skainet_hip_graph_launch(skainet_hip_graph* g) {
    if (!g) return set_error("graph_launch: null graph");
    if (g->owner != &t_scratch_generation)
        return set_error("graph_launch: refused, a graph is launched by the thread that recorded it (its scratch buffers are that thread's)");
    if (g->scratch_generation != t_scratch_generation)
        return set_error("graph_launch: refused, the library's scratch was reallocated after this graph was recorded "
                         "(generation %llu, now %llu); record it again",
                         (unsigned long long)g->scratch_generation, (unsigned long long)t_scratch_generation);
    return check_hip(hipGraphLaunch(g->exec, t_stream), "hipGraphLaunch");
}
int32_t skainet_hip_graph_sync(skainet_hip_graph* g) {
    if (!g) return set_error("graph_sync: null graph");
    return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}
void skainet_hip_graph_free(skainet_hip_graph* g) {
    if (!g) return;
    (void)hipStreamSynchronize(t_stream);
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
}

// ------------------------------------------------------------------------------------------ host-pointer entries
// Each stages its operands into per-thread device buffers, runs on this thread's stream and copies the
// result back before returning. Each clears the thread's error text first; a failure leaves `output`
// untouched and the reason in last_error().

static void* stage_in(int slot, const void* host, size_t bytes) {
    void* d = scratch_get(t_stage[slot], bytes ? bytes : 1);
    if (!d) return nullptr;
    if (bytes && check_hip(hipMemcpyAsync(d, host, bytes, hipMemcpyHostToDevice, t_stream), "hipMemcpy h2d") != 0) return nullptr;
    return d;
}
static int stage_out(void* host, const void* dev, size_t bytes) {
    if (check_hip(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, t_stream), "hipMemcpy d2h") != 0) return -1;
    return check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}

static void packed_matmul_host(int enc, int order, const float* input, int32_t input_offset, const uint8_t* weight,
                               int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output,
                               int32_t output_offset) {
    t_error[0] = 0;
    if (output_dim <= 0) return;
    if (ensure_device() != 0) return;
    if (input_dim % block_elems(enc) != 0) { set_error("matmul: inputDim must be a multiple of %d; got %d", block_elems(enc), input_dim); return; }
    if (input_dim <= 0) {
        // an empty contraction: the reference's K-quant entries return with the output untouched (q4k_matmul.c:326), its
        // 32-element formats write a row of zeros (q8_0_matmul.c:176)
        if (block_elems(enc) == Q80_ELEMS)
            for (int32_t o = 0; o < output_dim; ++o) output[output_offset + o] = 0.f;
        return;
    }
    const int bpr = input_dim / block_elems(enc);
    const size_t wbytes = (size_t)output_dim * bpr * block_bytes(enc);
    uint8_t* wd = static_cast<uint8_t*>(stage_in(0, weight + weight_byte_offset, wbytes));
    float* xd = static_cast<float*>(stage_in(1, input + input_offset, sizeof(float) * (size_t)input_dim));
    float* yd = static_cast<float*>(scratch_get(t_stage[2], sizeof(float) * (size_t)output_dim));
    if (!wd || !xd || !yd) return;
    if (order == SKAINET_HIP_ORDER_INPUT_BLOCK_MAJOR) {
        uint8_t* rm = static_cast<uint8_t*>(scratch_get(t_stage[3], wbytes));
        if (!rm || launch_relayout_to_row_major(wd, rm, output_dim, bpr, block_bytes(enc)) != 0) return;
        wd = rm;
    }
    if (launch_gemv(enc, wd, xd, 1, input_dim, output_dim, yd) != 0) return;
    stage_out(output + output_offset, yd, sizeof(float) * (size_t)output_dim);
}

#define SKH_PACKED_ENTRY(name, enc)                                                                                        \
    void skainet_hip_##name##_matmul(const float* input, int32_t input_offset, const uint8_t* weight,                        \
                                     int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output,       \
                                     int32_t output_offset) {                                                               \
        packed_matmul_host(enc, SKAINET_HIP_ORDER_INPUT_BLOCK_MAJOR, input, input_offset, weight, weight_byte_offset,      \
                           input_dim, output_dim, output, output_offset);                                                  \
    }                                                                                                                      \
    void skainet_hip_##name##_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,                     \
                                        int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output,    \
                                        int32_t output_offset) {                                                            \
        packed_matmul_host(enc, SKAINET_HIP_ORDER_ROW_MAJOR, input, input_offset, weight, weight_byte_offset, input_dim,   \
                           output_dim, output, output_offset);                                                             \
    }
SKH_PACKED_ENTRY(q4k, ENC_Q4_K)
SKH_PACKED_ENTRY(q6k, ENC_Q6_K)
SKH_PACKED_ENTRY(q8_0, ENC_Q8_0)
SKH_PACKED_ENTRY(q4_0, ENC_Q4_0)
SKH_PACKED_ENTRY(q5_0, ENC_Q5_0)
SKH_PACKED_ENTRY(q5_1, ENC_Q5_1)
SKH_PACKED_ENTRY(q5k, ENC_Q5_K)

void skainet_hip_fp32_matmul(const float* a, int32_t a_offset, int32_t a_stride, const float* b, int32_t b_offset,
                             int32_t b_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    t_error[0] = 0;
    if (m <= 0 || n <= 0) return;
    if (ensure_device() != 0) return;
    if (k < 0) k = 0;
    // Strided operands are staged as their bounding spans: (rows - 1) * stride + cols floats.
    const size_t a_span = k > 0 ? (size_t)(m - 1) * a_stride + k : 0, b_span = k > 0 ? (size_t)(k - 1) * b_stride + n : 0;
    float* ad = static_cast<float*>(stage_in(0, a + a_offset, sizeof(float) * a_span));
    float* bd = static_cast<float*>(stage_in(1, b + b_offset, sizeof(float) * b_span));
    float* cd = static_cast<float*>(scratch_get(t_stage[2], sizeof(float) * (size_t)m * n));
    if (!ad || !bd || !cd) return;
    if (launch_fp32_matmul(ad, a_stride, bd, b_stride, cd, n, m, n, k, false) != 0) return;
    if (c_stride == n) { stage_out(c + c_offset, cd, sizeof(float) * (size_t)m * n); return; }
    if (check_hip(hipMemcpy2DAsync(c + c_offset, sizeof(float) * (size_t)c_stride, cd, sizeof(float) * (size_t)n,
                                   sizeof(float) * (size_t)n, (size_t)m, hipMemcpyDeviceToHost, t_stream), "hipMemcpy2D d2h") != 0) return;
    check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}

static void narrow_matmul_host(int fp16, const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                               int32_t b_byte_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    t_error[0] = 0;
    if (m <= 0 || n <= 0) return;
    if (ensure_device() != 0) return;
    if (k < 0) { set_error("narrow matmul: k must be non-negative; got %d", k); return; }
    const size_t a_span = k > 0 ? (size_t)(m - 1) * a_stride + k : 0, b_span = k > 0 ? (size_t)(k - 1) * b_byte_stride + 2 * (size_t)n : 0;
    float* ad = static_cast<float*>(stage_in(0, a + a_offset, sizeof(float) * a_span));
    uint8_t* bd = static_cast<uint8_t*>(stage_in(1, b + b_byte_offset, b_span));
    float* cd = static_cast<float*>(scratch_get(t_stage[2], sizeof(float) * (size_t)m * n));
    if ((k > 0 && (!ad || !bd)) || !cd) return;
    if (launch_narrow_matmul(ad, a_stride, bd, b_byte_stride, cd, n, m, n, k, fp16) != 0) return;
    if (c_stride == n) { stage_out(c + c_offset, cd, sizeof(float) * (size_t)m * n); return; }
    if (check_hip(hipMemcpy2DAsync(c + c_offset, sizeof(float) * (size_t)c_stride, cd, sizeof(float) * (size_t)n,
                                   sizeof(float) * (size_t)n, (size_t)m, hipMemcpyDeviceToHost, t_stream), "hipMemcpy2D d2h") != 0) return;
    check_hip(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}
void skainet_hip_bf16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                             int32_t b_byte_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    narrow_matmul_host(0, a, a_offset, a_stride, b, b_byte_offset, b_byte_stride, c, c_offset, c_stride, m, n, k);
}
void skainet_hip_fp16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b, int32_t b_byte_offset,
                             int32_t b_byte_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k) {
    narrow_matmul_host(1, a, a_offset, a_stride, b, b_byte_offset, b_byte_stride, c, c_offset, c_stride, m, n, k);
}

void skainet_hip_fp32_matmul_wt(const float* in, int32_t in_offset, const float* w, int32_t w_offset, float* out,
                                int32_t out_offset, int32_t m, int32_t n, int32_t k) {
    t_error[0] = 0;
    if (m <= 0 || n <= 0 || k < 0) return;
    if (ensure_device() != 0) return;
    float* xd = static_cast<float*>(stage_in(0, in + in_offset, sizeof(float) * (size_t)m * k));
    float* wd = static_cast<float*>(stage_in(1, w + w_offset, sizeof(float) * (size_t)n * k));
    float* od = static_cast<float*>(scratch_get(t_stage[2], sizeof(float) * (size_t)m * n));
    if (!xd || !wd || !od) return;
    if (launch_fp32_matmul(xd, k, wd, k, od, n, m, n, k, true) != 0) return;
    stage_out(out + out_offset, od, sizeof(float) * (size_t)m * n);
}

void skainet_hip_f32_rms_norm(const float* in, const float* gamma, float* out, int32_t rows, int32_t cols, float eps) {
    t_error[0] = 0;
    if (rows <= 0 || cols <= 0) return;
    if (ensure_device() != 0) return;
    const size_t bytes = sizeof(float) * (size_t)rows * cols;
    float* xd = static_cast<float*>(stage_in(0, in, bytes));
    float* gd = gamma ? static_cast<float*>(stage_in(1, gamma, sizeof(float) * (size_t)cols)) : nullptr;
    float* od = static_cast<float*>(scratch_get(t_stage[2], bytes));
    if (!xd || (gamma && !gd) || !od) return;
    if (launch_rms_norm(xd, gd, od, rows, cols, eps) != 0) return;
    stage_out(out, od, bytes);
}

void skainet_hip_f32_layer_norm(const float* in, const float* gamma, const float* beta, float* out, int32_t rows, int32_t cols,
                                float eps) {
    t_error[0] = 0;
    if (rows <= 0 || cols <= 0) return;
    if (ensure_device() != 0) return;
    const size_t bytes = sizeof(float) * (size_t)rows * cols;
    float* xd = static_cast<float*>(stage_in(0, in, bytes));
    float* gd = gamma ? static_cast<float*>(stage_in(1, gamma, sizeof(float) * (size_t)cols)) : nullptr;
    float* bd = beta ? static_cast<float*>(stage_in(3, beta, sizeof(float) * (size_t)cols)) : nullptr;
    float* od = static_cast<float*>(scratch_get(t_stage[2], bytes));
    if (!xd || (gamma && !gd) || (beta && !bd) || !od) return;
    if (launch_layer_norm(xd, gd, bd, od, rows, cols, eps) != 0) return;
    stage_out(out, od, bytes);
}

void skainet_hip_f32_softmax_rows(const float* in, float* out, int32_t rows, int32_t cols, int32_t log_form) {
    t_error[0] = 0;
    if (rows <= 0 || cols <= 0) return;
    if (ensure_device() != 0) return;
    const size_t bytes = sizeof(float) * (size_t)rows * cols;
    float* xd = static_cast<float*>(stage_in(0, in, bytes));
    float* od = static_cast<float*>(scratch_get(t_stage[2], bytes));
    if (!xd || !od) return;
    if (launch_softmax_rows(xd, od, rows, cols, log_form) != 0) return;
    stage_out(out, od, bytes);
}

void skainet_hip_f32_sdpa(const float* q, const float* k, const float* v, float* out, int32_t batch, int32_t heads,
                          int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t head_dim, float scale, int32_t causal,
                          int32_t window, int32_t right_context, const int32_t* lengths, const float* mask, int32_t mask_b,
                          int32_t mask_h, int32_t mask_q, int32_t mask_k) {
    t_error[0] = 0;
    if (batch <= 0 || heads <= 0 || kv_heads <= 0 || seq_q <= 0 || head_dim <= 0) return;
    const size_t qn = (size_t)batch * heads * seq_q * head_dim;
    if (seq_kv <= 0) { for (size_t i = 0; i < qn; ++i) out[i] = 0.f; return; }
    if (ensure_device() != 0) return;
    const size_t kn = (size_t)batch * kv_heads * seq_kv * head_dim;
    float* qd = static_cast<float*>(stage_in(0, q, sizeof(float) * qn));
    float* kd = static_cast<float*>(stage_in(1, k, sizeof(float) * kn));
    float* vd = static_cast<float*>(stage_in(3, v, sizeof(float) * kn));
    float* od = static_cast<float*>(scratch_get(t_stage[2], sizeof(float) * qn));
    int32_t* ld = lengths ? static_cast<int32_t*>(stage_in(4, lengths, sizeof(int32_t) * (size_t)batch)) : nullptr;
    float* md = mask ? static_cast<float*>(stage_in(5, mask, sizeof(float) * (size_t)mask_b * mask_h * mask_q * mask_k)) : nullptr;
    if (!qd || !kd || !vd || !od || (lengths && !ld) || (mask && !md)) return;
    if (launch_sdpa(qd, kd, vd, od, batch, heads, kv_heads, seq_q, seq_kv, seq_kv, head_dim, scale, causal, window, right_context, ld,
                    md, mask_b, mask_h, mask_q, mask_k) != 0) return;
    stage_out(out, od, sizeof(float) * qn);
}

}  // extern "C"
