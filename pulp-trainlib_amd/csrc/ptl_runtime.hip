// Library state, error reporting, workspace and host-pointer staging.
#include "ptl_common.hpp"
#include "ptl_host.hpp"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <vector>

namespace ptl {

static thread_local char g_err[512] = "";
static thread_local int g_status = 0;

State &state() {
    static State s;
    return s;
}

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

const char *last_error() { return g_err; }
int last_status() { return g_status; }
void set_status(int s) {
    g_status = s;
    if (s != 0) fflush(stdout);  // make the rejection message visible right away
}

bool hip_ok(hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    set_error("%s: %s", what, hipGetErrorString(e));
    return false;
}

int init_device(int device) {
    State &st = state();
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) {
        (void)hipGetLastError();
        set_error("libptl_hip: no HIP device available (%s); there is no CPU fallback",
                  e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        return 2;
    }
    if (device < 0 || device >= count) {
        set_error("libptl_hip: device %d out of range (0..%d)", device, count - 1);
        return 1;
    }
    if (!hip_ok(hipSetDevice(device), "hipSetDevice")) return 2;
    if (st.ready && st.device == device) return 0;
    hipDeviceProp_t prop;
    if (!hip_ok(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties")) return 2;
    st.num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (!st.ev0) {
        if (!hip_ok(hipEventCreate(&st.ev0), "hipEventCreate")) return 2;
        if (!hip_ok(hipEventCreate(&st.ev1), "hipEventCreate")) return 2;
    }
    if (!st.zeros) {
        if (!hip_ok(hipMalloc(&st.zeros, 256), "hipMalloc(zeros)")) return 2;
        if (!hip_ok(hipMemset(st.zeros, 0, 256), "hipMemset(zeros)")) return 2;
    }
    if (int rc = dw_noalloc_setup(device)) return rc;
    st.device = device;
    st.ready = true;
    return 0;
}

bool ensure_init() {
    State &st = state();
    if (st.ready) return true;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        dev = 0;
    }
    return init_device(dev) == 0;
}

// True while the library's stream records into a HIP graph: synchronising, freeing and allocating are illegal then
// (each of them would invalidate the capture).
static bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &status) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return status != hipStreamCaptureStatusNone;
}

static void *grow(void *&buf, size_t &have, size_t want, const char *what) {
    if (want <= have) return buf;
    State &st = state();
    if (stream_is_capturing(st.stream)) {
        set_error("%s: %zu bytes are needed and %zu are there, and the stream is being captured into a graph; call "
                  "ptl_reserve() or run this shape once before the capture begins", what, want, have);
        return nullptr;
    }
    if (buf) {
        // kernels enqueued earlier - on this stream or on one the caller selected before - may still read the
        // old buffer
        if (!hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize")) return nullptr;
        (void)hipFree(buf);
        buf = nullptr;
        have = 0;
    }
    size_t sz = want < (size_t)(8u << 20) ? (size_t)(8u << 20) : want + want / 4;
    if (!hip_ok(hipMalloc(&buf, sz), what)) {
        buf = nullptr;
        return nullptr;
    }
    have = sz;
    return buf;
}

float *workspace(size_t bytes) {
    State &st = state();
    void *p = st.ws;
    p = grow(p, st.ws_bytes, bytes, "hipMalloc(workspace)");
    st.ws = static_cast<float *>(p);
    return st.ws;
}

void *scratch(size_t bytes) {
    State &st = state();
    return grow(st.scratch, st.scratch_bytes, bytes, "hipMalloc(scratch)");
}

// ---------------------------------------------------------------------------
// Staging of host pointers
// ---------------------------------------------------------------------------
static bool is_device_ptr(const void *p) {
    hipPointerAttribute_t attr;
    memset(&attr, 0, sizeof(attr));
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // plain host memory is reported as an error on some runtimes
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// Device buffers for staged host tensors are kept between calls: a call that stages the same sizes again (a
// training loop on host arrays) allocates nothing.  A buffer is handed out again only after the call that used
// it has synchronised its stream (finish(), or the destructor of a Stager that never got there).
struct StagePool {
    struct Buf {
        void *dev;
        size_t bytes;
        bool busy;
    };
    std::vector<Buf> bufs;
    size_t total = 0;
};
static const size_t STAGE_POOL_LIMIT = (size_t)1 << 30;  // idle buffers beyond this are freed on release

static StagePool &stage_pool() {
    static StagePool p;
    return p;
}

static void *stage_acquire(size_t bytes) {
    StagePool &p = stage_pool();
    int best = -1;
    for (size_t i = 0; i < p.bufs.size(); ++i) {
        const StagePool::Buf &b = p.bufs[i];
        if (b.busy || b.bytes < bytes || b.bytes > 2 * bytes + (1u << 20)) continue;
        if (best < 0 || b.bytes < p.bufs[best].bytes) best = (int)i;
    }
    if (best >= 0) {
        p.bufs[best].busy = true;
        return p.bufs[best].dev;
    }
    void *dev = nullptr;
    if (!hip_ok(hipMalloc(&dev, bytes), "hipMalloc(staging)")) return nullptr;
    p.bufs.push_back({dev, bytes, true});
    p.total += bytes;
    return dev;
}

static void stage_release(void *dev) {
    StagePool &p = stage_pool();
    for (auto &b : p.bufs)
        if (b.dev == dev) b.busy = false;
    // keep the pool bounded: drop idle buffers, largest first
    while (p.total > STAGE_POOL_LIMIT) {
        int big = -1;
        for (size_t i = 0; i < p.bufs.size(); ++i)
            if (!p.bufs[i].busy && (big < 0 || p.bufs[i].bytes > p.bufs[big].bytes)) big = (int)i;
        if (big < 0) break;
        (void)hipFree(p.bufs[big].dev);
        p.total -= p.bufs[big].bytes;
        p.bufs.erase(p.bufs.begin() + big);
    }
}

Stager::~Stager() {
    if (items_.empty()) return;
    // copies or kernels of a call that bailed out early may still be in flight on the buffers
    if (!finished_) (void)hipStreamSynchronize(state().stream);
    for (auto &t : items_)
        if (t.dev) stage_release(t.dev);
}

void *Stager::map(const void *host_or_dev, size_t bytes, bool copy_in, bool copy_out) {
    if (failed_) return nullptr;
    if (!host_or_dev) {
        set_error("null tensor pointer");
        failed_ = rejected_ = true;
        return nullptr;
    }
    if (bytes == 0) return const_cast<void *>(host_or_dev);
    if (is_device_ptr(host_or_dev)) return const_cast<void *>(host_or_dev);
    if (device_only_) {
        set_error("host pointer passed to an entry point that may not allocate (staging needs device buffers)");
        failed_ = rejected_ = true;
        return nullptr;
    }
    Item *hit = nullptr;
    for (auto &t : items_)
        if (t.host == host_or_dev && t.bytes >= bytes) hit = &t;
    if (!hit) {
        Item it;
        it.host = const_cast<void *>(host_or_dev);
        it.bytes = bytes;
        it.copy_out = false;
        it.copied_in = false;
        it.dev = stage_acquire(bytes);
        if (!it.dev) {
            failed_ = true;
            return nullptr;
        }
        items_.push_back(it);
        hit = &items_.back();
    }
    hit->copy_out = hit->copy_out || copy_out;
    // a tensor first mapped as an output and later as an input still gets its contents
    if (copy_in && !hit->copied_in) {
        if (!hip_ok(hipMemcpyAsync(hit->dev, host_or_dev, hit->bytes, hipMemcpyHostToDevice, state().stream),
                    "hipMemcpy(H2D)")) {
            failed_ = true;
            return nullptr;
        }
        hit->copied_in = true;
    }
    return hit->dev;
}

void Stager::discard() {
    if (items_.empty()) return;
    // copies into the buffers may still be in flight
    (void)hipStreamSynchronize(state().stream);
    for (auto &t : items_)
        if (t.dev) stage_release(t.dev);
    items_.clear();
}

int Stager::finish(int rc) {
    if (items_.empty()) return failed_ ? 2 : rc;
    State &st = state();
    if (!failed_ && rc == 0) {
        for (auto &t : items_)
            if (t.copy_out) {
                if (!hip_ok(hipMemcpyAsync(t.host, t.dev, t.bytes, hipMemcpyDeviceToHost, st.stream),
                            "hipMemcpy(D2H)"))
                    failed_ = true;
            }
    }
    if (!hip_ok(hipStreamSynchronize(st.stream), "hipStreamSynchronize")) failed_ = true;
    else finished_ = true;
    return failed_ ? 2 : rc;
}

}  // namespace ptl

extern "C" {

int ptl_init(int device) { return ptl::init_device(device); }
const char *ptl_last_error(void) { return ptl::last_error(); }
int ptl_last_status(void) { return ptl::last_status(); }
// Work already enqueued on the stream being left may still use the library's workspace; the next call would
// write it from the new stream, so the old stream is drained first (a no-op when it is idle).  A stream that is
// being captured cannot be drained: the switch is refused then (status 1, the stream stays), and a drain that
// fails (a destroyed handle) is reported the same way after the switch.
void ptl_set_stream(void *s) {
    ptl::State &st = ptl::state();
    hipStream_t next = static_cast<hipStream_t>(s);
    ptl::set_status(0);
    if (st.ready && next != st.stream) {
        if (ptl::stream_is_capturing(st.stream)) {
            ptl::set_error("ptl_set_stream: the current stream is being captured into a graph; switch streams "
                           "before the capture begins or after it ends");
            ptl::set_status(1);
            return;
        }
        hipError_t e = hipStreamSynchronize(st.stream);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            ptl::set_error("ptl_set_stream: draining the previous stream failed (%s)", hipGetErrorString(e));
            ptl::set_status(2);
        }
    }
    st.stream = next;
}

// Grows the two internal buffers (partial sums; blocked / padded copies) to at least the given sizes now, so that
// no later call has to: callers that capture the library's launches into a graph, or that may not allocate in
// their steady state, reserve once after ptl_init.  ptl_reserved reports the present sizes (after a warm-up pass
// over the caller's shapes they are the sizes those shapes need).
int ptl_reserve(size_t workspace_bytes, size_t scratch_bytes) {
    if (!ptl::ensure_init()) return 2;
    if (workspace_bytes && !ptl::workspace(workspace_bytes)) return 2;
    if (scratch_bytes && !ptl::scratch(scratch_bytes)) return 2;
    return 0;
}

void ptl_reserved(size_t *workspace_bytes, size_t *scratch_bytes) {
    ptl::State &st = ptl::state();
    if (workspace_bytes) *workspace_bytes = st.ws_bytes;
    if (scratch_bytes) *scratch_bytes = st.scratch_bytes;
}

void ptl_set_gemm_path(int path) { ptl::state().gemm_path = path; }
int ptl_last_conv_direct(void) { return ptl::state().last_conv_direct; }
int ptl_last_gemm_streamed(void) { return ptl::state().last_gemm_streamed; }
int ptl_last_conv_resident(void) { return ptl::state().last_conv_resident; }
int ptl_last_gemm_tile(void) { return ptl::state().last_gemm_tile; }

int ptl_sync(void) {
    if (!ptl::ensure_init()) return 2;
    return ptl::hip_ok(hipStreamSynchronize(ptl::state().stream), "hipStreamSynchronize") ? 0 : 2;
}

int ptl_timer_begin(void) {
    if (!ptl::ensure_init()) return 2;
    return ptl::hip_ok(hipEventRecord(ptl::state().ev0, ptl::state().stream), "hipEventRecord") ? 0 : 2;
}

float ptl_timer_end_ms(void) {
    if (!ptl::ensure_init()) return -1.f;
    ptl::State &st = ptl::state();
    if (!ptl::hip_ok(hipEventRecord(st.ev1, st.stream), "hipEventRecord")) return -1.f;
    if (!ptl::hip_ok(hipEventSynchronize(st.ev1), "hipEventSynchronize")) return -1.f;
    float ms = -1.f;
    if (!ptl::hip_ok(hipEventElapsedTime(&ms, st.ev0, st.ev1), "hipEventElapsedTime")) return -1.f;
    return ms;
}

}  // extern "C"
