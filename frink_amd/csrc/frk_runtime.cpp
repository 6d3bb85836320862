// Host runtime of libfrink_hip: error strings, device probe, the env switch, the resident
// weight cache, the per-device workspace and the extern "C" entry points.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "frk_internal.hpp"

namespace frk {

static thread_local char g_err[512] = {0};

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
void clear_error() { g_err[0] = 0; }

// ---- device state ----
struct DeviceState {
    std::mutex mu;
    bool probed = false;
    int device_count = 0;
    hipStream_t stream = nullptr;  // for host-buffer entry points
    // host staging for the host-buffer entry points
    void *x_dev = nullptr, *y_dev = nullptr;
    size_t x_bytes = 0, y_bytes = 0;
    std::map<std::pair<const void *, size_t>, frk_weights *> cache;
};
static DeviceState g_dev;

static int ensure_device_locked() {
    if (!g_dev.probed) {
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        g_dev.probed = true;
        g_dev.device_count = (e == hipSuccess) ? n : 0;
        if (e != hipSuccess) (void)hipGetLastError();
    }
    if (g_dev.device_count <= 0) return set_error(FRK_ERR_NO_DEVICE, "no HIP device is visible");
    if (!g_dev.stream) {
        // default priority on purpose
        hipError_t e = hipStreamCreateWithFlags(&g_dev.stream, hipStreamNonBlocking);
        if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipStreamCreateWithFlags: %s", hipGetErrorString(e));
    }
    return FRK_OK;
}

hipStream_t own_stream() { return g_dev.stream; }

struct StreamWorkspace {
    std::recursive_mutex mu;  // held by the thread whose entry point is enqueueing on the stream
    void *ptr = nullptr;
    size_t bytes = 0;
    bool in_a_graph = false;  // a call was enqueued on it while the stream was being captured: a graph holds its address
    int depth = 0;                 // nested leases of the holder
    std::vector<std::pair<void *, size_t>> outgrown;  // replaced under a lease; retired when the outermost ends
};
struct RetiredBuffer {
    void *ptr;
    size_t bytes;
    hipEvent_t passed;  // recorded on the stream that used the buffer last
};
static std::map<hipStream_t, StreamWorkspace *> g_ws;  // under g_dev.mu; entries live until the process ends
static std::vector<RetiredBuffer> g_retired;           // under g_dev.mu

// A retired buffer of at least `bytes` whose last use has passed, or a fresh allocation.  Nothing is
// given back to the driver here: hipFree waits for the whole device, which would stall every other
// stream's calls from inside this one.  Idle retired buffers stay in the pool (a stream's buffer is
// replaced only when a larger shape first runs on it, so the pool holds a handful of them).
static int take_buffer_locked(size_t bytes, void **ptr, size_t *got) {
    size_t best = g_retired.size();
    for (size_t i = 0; i < g_retired.size(); i++) {
        if (hipEventQuery(g_retired[i].passed) != hipSuccess) {
            (void)hipGetLastError();  // not ready is not an error
            continue;
        }
        if (g_retired[i].bytes >= bytes && (best == g_retired.size() || g_retired[i].bytes < g_retired[best].bytes)) best = i;
    }
    if (best < g_retired.size()) {
        *ptr = g_retired[best].ptr;
        *got = g_retired[best].bytes;
        (void)hipEventDestroy(g_retired[best].passed);
        g_retired.erase(g_retired.begin() + (long)best);
        return FRK_OK;
    }
    const size_t want = std::max<size_t>(round_up(bytes, 1 << 20), 4u << 20);
    FRK_HIP_TRY(hipMalloc(ptr, want));
    *got = want;
    return FRK_OK;
}

int workspace(size_t bytes, hipStream_t stream, WorkspaceLease &lease) {
    StreamWorkspace *w = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_dev.mu);
        auto it = g_ws.find(stream);
        if (it == g_ws.end()) it = g_ws.emplace(stream, new StreamWorkspace()).first;
        w = it->second;
    }
    if (lease.held_ != w) {  // (a lease asked again, by a later step of the same call, keeps its one hold)
        w->mu.lock();
        w->depth++;
        lease.held_ = w;
        lease.stream_ = stream;
    }
    // A graph captured from this stream replays the buffer's address for as long as the graph lives, which
    // the library cannot see: a buffer that was current during a capture is never handed to another stream
    // nor reused after a growth -- it stays allocated, untouched by later calls, until the process ends.
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess) (void)hipGetLastError();
    if (cs != hipStreamCaptureStatusNone && bytes <= w->bytes) w->in_a_graph = true;
    if (bytes > w->bytes) {
        if (cs != hipStreamCaptureStatusNone)
            return set_error(FRK_ERR_HIP,
                             "the stream's scratch buffer holds %zu bytes and this call needs %zu: it cannot grow while the "
                             "stream is being captured (run the shape once before capturing)", w->bytes, bytes);
        void *fresh = nullptr;
        size_t got = 0;
        {
            std::lock_guard<std::mutex> lk(g_dev.mu);
            int rc = take_buffer_locked(bytes, &fresh, &got);
            if (rc) return rc;
        }
        if (w->ptr && !w->in_a_graph) w->outgrown.emplace_back(w->ptr, w->bytes);  // (one a graph holds: kept, see above)
        w->ptr = fresh;
        w->bytes = got;
        w->in_a_graph = false;
    }
    lease.ptr = w->ptr;
    return FRK_OK;
}

WorkspaceLease::~WorkspaceLease() {
    StreamWorkspace *w = held_;
    if (!w) return;
    if (--w->depth == 0 && !w->outgrown.empty()) {
        // kernels enqueued under this lease may still read a replaced buffer: it is free once the
        // stream has passed this point
        std::lock_guard<std::mutex> lk(g_dev.mu);
        for (auto &b : w->outgrown) {
            hipEvent_t ev = nullptr;
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess && hipEventRecord(ev, stream_) == hipSuccess) {
                g_retired.push_back({b.first, b.second, ev});
            } else {
                (void)hipGetLastError();
                if (ev) (void)hipEventDestroy(ev);
                // without an event the buffer cannot be shown idle: it is kept until the process ends
            }
        }
        w->outgrown.clear();
    }
    w->mu.unlock();
}

static void fingerprint_of(const uint8_t *bytes, size_t len, uint8_t out[192]) {
    // first, middle and last 64 bytes (crates/frink-quant/src/fingerprint.rs:17-40)
    auto take = [&](size_t at, uint8_t *dst) {
        memset(dst, 0, 64);
        at = std::min(at, len);
        size_t n = std::min<size_t>(len - at, 64);
        memcpy(dst, bytes + at, n);
    };
    take(0, out);
    take(len / 2, out + 64);
    take(len >= 64 ? len - 64 : 0, out + 128);
}

static int check_matrix_shape(int kind, size_t len, size_t rows, size_t cols) {
    int be = block_elems(kind), bb = block_bytes(kind);
    if (!be) return set_error(FRK_ERR_UNSUPPORTED, "no kernel for quant kind %d", kind);
    if (rows == 0 || cols == 0) return set_error(FRK_ERR_SHAPE, "empty shape: rows=%zu cols=%zu", rows, cols);
    if (cols % (size_t)be) return set_error(FRK_ERR_SHAPE, "cols %zu is not a multiple of the %d-element block", cols, be);
    size_t want = rows * (cols / (size_t)be) * (size_t)bb;
    if (len != want) return set_error(FRK_ERR_SHAPE, "weights are %zu bytes, shape %zux%zu needs %zu", len, rows, cols, want);
    if (rows > 0x7fffffffu || cols > 0x7fffffffu) return set_error(FRK_ERR_SHAPE, "shape too large");
    return FRK_OK;
}

// Creates the resident copy from GGUF bytes already on the device.
static int make_resident(int kind, const uint8_t *src_dev, size_t rows, size_t cols, hipStream_t s,
                         frk_weights **out) {
    auto *w = new frk_weights();
    w->kind = kind;
    w->rows = rows;
    w->cols = cols;
    w->src_row_bytes = cols / (size_t)block_elems(kind) * (size_t)block_bytes(kind);
    w->layout = layout_for(kind, cols);
    // 256 bytes of slack: kernels may issue (masked-out or clamped) 16-byte loads near the end
    w->dev_bytes = w->layout.row_stride * rows + 256;
    (void)hipGetDevice(&w->device);
    hipError_t e = hipMalloc((void **)&w->dev, w->dev_bytes);
    if (e != hipSuccess) {
        const size_t wanted = w->dev_bytes;
        delete w;
        return set_error(FRK_ERR_OOM, "hipMalloc(%zu) for resident weights: %s", wanted, hipGetErrorString(e));
    }
    int rc = launch_repack(kind, src_dev, w->dev, rows, cols, w->layout, s);
    if (rc == FRK_OK) {
        e = hipMemsetAsync(w->dev + w->layout.row_stride * rows, 0, 256, s);
        if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemsetAsync: %s", hipGetErrorString(e));
    }
    // (MXFP4: whether the scales are f16 values decides the batched path; one pass over the scale bytes, once)
    if (rc == FRK_OK && kind == FRK_KIND_MXFP4) rc = mxfp4_scale_range(w, &w->e8m0_min, &w->e8m0_max, s);
    if (rc != FRK_OK) {
        (void)hipFree(w->dev);
        delete w;
        return rc;
    }
    *out = w;
    return FRK_OK;
}

}  // namespace frk

using namespace frk;

extern "C" {

const char *frk_hip_last_error(void) { return g_err; }

int frk_hip_probe(frk_device_info *out) {
    clear_error();
    if (!out) return set_error(FRK_ERR_ARG, "frk_hip_probe: out is null");
    memset(out, 0, sizeof *out);
    std::lock_guard<std::mutex> lk(g_dev.mu);
    int rc = ensure_device_locked();
    if (rc) return rc;
    out->device_count = g_dev.device_count;
    hipDeviceProp_t p;
    FRK_HIP_TRY(hipGetDeviceProperties(&p, 0));
    snprintf(out->name, sizeof out->name, "%s", p.name);
    snprintf(out->gcn_arch, sizeof out->gcn_arch, "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    size_t fr = 0, tot = 0;
    FRK_HIP_TRY(hipMemGetInfo(&fr, &tot));
    out->free_vram_bytes = fr;
    out->total_vram_bytes = tot;
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return set_error(FRK_ERR_NO_DEVICE, "device 0 is %s; this library holds gfx950 code only", p.gcnArchName);
    return FRK_OK;
}

int frk_hip_dense_enabled(void) {
    static std::once_flag once;
    static int enabled = 0;
    std::call_once(once, [] {
        const char *v = getenv("FRINK_HIP");
        std::string s = v ? v : "";
        std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return (char)tolower(c); });
        if (s == "0" || s == "false" || s == "off" || s == "cpu") {
            enabled = 0;  // forced off: no device is opened
            return;
        }
        frk_device_info info;
        int rc = frk_hip_probe(&info);
        enabled = (rc == FRK_OK);
        clear_error();
    });
    return enabled;
}

const char *frk_hip_matvec_kernel(int kind) {
    switch (kind) {
    case FRK_KIND_Q4_0: return "Q4_0";
    case FRK_KIND_Q5_0: return "Q5_0";
    case FRK_KIND_IQ4_XS: return "IQ4_XS";
    case FRK_KIND_MXFP4: return "MXFP4";
    case FRK_KIND_Q8_0: return "Q8_0";
    case FRK_KIND_Q4_K: return "Q4_K";
    case FRK_KIND_Q5_K: return "Q5_K";
    case FRK_KIND_Q6_K: return "Q6_K";
    }
    return nullptr;
}
int frk_hip_has_launch(int kind) { return frk_hip_matvec_kernel(kind) != nullptr; }
int frk_hip_gemm_supported(int kind) {
    // (Q5_0 and MXFP4 through the Q8_0 matrix-core kernel, IQ4_XS through its form with integer block scales)
    return kind == FRK_KIND_Q4_K || kind == FRK_KIND_Q5_K || kind == FRK_KIND_Q6_K || kind == FRK_KIND_Q8_0 ||
           kind == FRK_KIND_Q4_0 || kind == FRK_KIND_Q5_0 || kind == FRK_KIND_MXFP4 || kind == FRK_KIND_IQ4_XS;
}
int frk_hip_block_bytes(int kind) { return block_bytes(kind); }
int frk_hip_block_elems(int kind) { return block_elems(kind); }
int frk_hip_worth_a_gemm(size_t batch) { return batch >= 2; }

int frk_hip_weights_register(int kind, const void *host_bytes, size_t len, size_t rows, size_t cols,
                             frk_weights **out) {
    clear_error();
    if (!host_bytes || !out) return set_error(FRK_ERR_ARG, "frk_hip_weights_register: null argument");
    int rc = check_matrix_shape(kind, len, rows, cols);
    if (rc) return rc;
    std::lock_guard<std::mutex> lk(g_dev.mu);
    rc = ensure_device_locked();
    if (rc) return rc;
    uint8_t fp[192];
    fingerprint_of((const uint8_t *)host_bytes, len, fp);
    auto key = std::make_pair(host_bytes, len);
    auto it = g_dev.cache.find(key);
    if (it != g_dev.cache.end()) {
        frk_weights *c = it->second;
        if (c->kind == kind && c->rows == rows && c->cols == cols && memcmp(c->fingerprint, fp, 192) == 0) {
            c->refcount++;
            *out = c;
            return FRK_OK;
        }
        // same address and length, different bytes: the buffer that entry came from is gone
        g_dev.cache.erase(it);
        c->cached = false;
        if (--c->refcount == 0) {
            (void)hipFree(c->dev);
            delete c;
        }
    }
    uint8_t *staging = nullptr;
    FRK_HIP_TRY(hipMalloc((void **)&staging, len));
    hipError_t e = hipMemcpyAsync(staging, host_bytes, len, hipMemcpyHostToDevice, g_dev.stream);
    frk_weights *w = nullptr;
    if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(weights): %s", hipGetErrorString(e));
    if (!rc) rc = make_resident(kind, staging, rows, cols, g_dev.stream, &w);
    hipError_t e2 = hipStreamSynchronize(g_dev.stream);
    (void)hipFree(staging);
    if (!rc && e2 != hipSuccess) {
        rc = set_error(FRK_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e2));
        (void)hipFree(w->dev);
        delete w;
    }
    if (rc) return rc;
    w->host_key = host_bytes;
    w->host_len = len;
    memcpy(w->fingerprint, fp, 192);
    w->cached = true;
    w->refcount = 2;  // one for the cache, one for the caller
    g_dev.cache[key] = w;
    *out = w;
    return FRK_OK;
}

int frk_hip_weights_from_device(int kind, const void *dev_bytes, size_t len, size_t rows, size_t cols,
                                void *stream, frk_weights **out) {
    clear_error();
    if (!dev_bytes || !out) return set_error(FRK_ERR_ARG, "frk_hip_weights_from_device: null argument");
    int rc = check_matrix_shape(kind, len, rows, cols);
    if (rc) return rc;
    {
        std::lock_guard<std::mutex> lk(g_dev.mu);
        rc = ensure_device_locked();
        if (rc) return rc;
    }
    return make_resident(kind, (const uint8_t *)dev_bytes, rows, cols, (hipStream_t)stream, out);
}

int frk_hip_weights_release(frk_weights *w) {
    clear_error();
    if (!w) return FRK_OK;
    std::lock_guard<std::mutex> lk(g_dev.mu);
    if (--w->refcount > 0) {
        // the cache keeps its own reference until the process ends or the bytes change
        return FRK_OK;
    }
    if (w->cached) g_dev.cache.erase(std::make_pair(w->host_key, w->host_len));
    hipError_t e = hipFree(w->dev);
    if (uint8_t *kept = w->decoded.load(std::memory_order_acquire)) {
        const hipError_t e2 = hipFree(kept);
        if (e == hipSuccess) e = e2;
    }
    delete w;
    if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFree: %s", hipGetErrorString(e));
    return FRK_OK;
}

int frk_hip_weights_keep_decoded(frk_weights *w, void *stream) {
    clear_error();
    if (!w) return set_error(FRK_ERR_ARG, "frk_hip_weights_keep_decoded: null argument");
    if (!is_unit_kind(w->kind) || !units_have_planar_form(w))
        return set_error(FRK_ERR_UNSUPPORTED, "quant kind %d has no decoded form to keep (Q5_0, IQ4_XS, MXFP4 with scale bytes within 104..143)",
                         w->kind);
    std::lock_guard<std::mutex> lk(g_dev.mu);
    if (w->decoded.load(std::memory_order_acquire)) return FRK_OK;
    uint8_t *room = nullptr;
    FRK_HIP_TRY(hipMalloc((void **)&room, units_planar_bytes(w->rows, w->cols)));
    int rc = launch_units_decode(w, room, (hipStream_t)stream);
    hipError_t e = rc ? hipSuccess : hipStreamSynchronize((hipStream_t)stream);
    if (rc || e != hipSuccess) {
        (void)hipFree(room);
        return rc ? rc : set_error(FRK_ERR_HIP, "frk_hip_weights_keep_decoded: %s", hipGetErrorString(e));
    }
    w->decoded.store(room, std::memory_order_release);  // (behind the synchronization: any stream may read it from here on)
    return FRK_OK;
}

size_t frk_hip_weights_rows(const frk_weights *w) { return w ? w->rows : 0; }
size_t frk_hip_weights_cols(const frk_weights *w) { return w ? w->cols : 0; }
int frk_hip_weights_kind(const frk_weights *w) { return w ? w->kind : 0; }

// ---- device-pointer entry points ----

int frk_hip_quantize_q8_k_dev(const float *x, size_t n, int8_t *q, float *d, int16_t *bsums, void *stream) {
    clear_error();
    if (!x || !q || !d || !bsums) return set_error(FRK_ERR_ARG, "frk_hip_quantize_q8_k_dev: null argument");
    if (n % QK_K) return set_error(FRK_ERR_SHAPE, "length %zu is not a multiple of 256", n);
    if (n == 0) return FRK_OK;
    return launch_quantize_q8_k(x, n, q, d, bsums, (hipStream_t)stream);
}

int frk_hip_quantize_q8_0_dev(const float *x, size_t n, int8_t *q, float *d, void *stream) {
    clear_error();
    if (!x || !q || !d) return set_error(FRK_ERR_ARG, "frk_hip_quantize_q8_0_dev: null argument");
    if (n % Q8_0_ELEMS) return set_error(FRK_ERR_SHAPE, "length %zu is not a multiple of 32", n);
    if (n == 0) return FRK_OK;
    return launch_quantize_q8_0(x, n, q, d, (hipStream_t)stream);
}

int frk_hip_dequant_dev(const frk_weights *w, float *out, void *stream) {
    clear_error();
    if (!w || !out) return set_error(FRK_ERR_ARG, "frk_hip_dequant_dev: null argument");
    return launch_dequant(w, out, (hipStream_t)stream);
}

int frk_hip_get_rows_dev(const frk_weights *w, const int32_t *ids, size_t n_ids, float *out, void *stream) {
    clear_error();
    if (!w || (n_ids && (!ids || !out))) return set_error(FRK_ERR_ARG, "frk_hip_get_rows_dev: null argument");
    return launch_dequant_rows(w, ids, n_ids, out, (hipStream_t)stream);
}

int frk_hip_copy_dev(const void *src, void *dst, size_t bytes, void *stream) {
    clear_error();
    if (!src || !dst) return set_error(FRK_ERR_ARG, "frk_hip_copy_dev: null argument");
    if (bytes % 16) return set_error(FRK_ERR_SHAPE, "bytes %zu is not a multiple of 16", bytes);
    return launch_copy(src, dst, bytes, (hipStream_t)stream);
}

int frk_hip_issue_probe(float *out16_host) {
    clear_error();
    if (!out16_host) return set_error(FRK_ERR_ARG, "frk_hip_issue_probe: null argument");
    {
        std::lock_guard<std::mutex> lk(g_dev.mu);
        int rc = ensure_device_locked();
        if (rc) return rc;
    }
    return launch_issue_probe(out16_host, nullptr);
}

int frk_hip_read_dev(const void *src, size_t bytes, void *sink, void *stream) {
    clear_error();
    if (!src || !sink) return set_error(FRK_ERR_ARG, "frk_hip_read_dev: null argument");
    if (bytes % 16) return set_error(FRK_ERR_SHAPE, "bytes %zu is not a multiple of 16", bytes);
    return launch_read(src, bytes, sink, (hipStream_t)stream);
}

int frk_hip_read_shape_dev(const void *src, size_t bytes, void *sink, int span_kb, int waves, int to_lds, int policy,
                           void *stream) {
    clear_error();
    if (!src || !sink) return set_error(FRK_ERR_ARG, "frk_hip_read_shape_dev: null argument");
    return launch_read_shape(src, bytes, sink, span_kb, waves, to_lds, policy, (hipStream_t)stream);
}

// Where one call's scratch memory comes from: the stream's leased buffer (grown on demand), or a fixed
// region that has to suffice (the entry point that allocates nothing).  It must outlive the launches that
// use the memory; nested requests of one call get the same start address, as with the lease.
struct Scratch {
    WorkspaceLease lease;
    void *fixed = nullptr;
    size_t fixed_bytes = 0;
    Scratch() = default;
    Scratch(void *region, size_t bytes) : fixed(region), fixed_bytes(bytes) {}
    int get(size_t bytes, hipStream_t s, void **out) {
        if (fixed) {
            if (bytes > fixed_bytes)
                return set_error(FRK_ERR_SHAPE, "this shape needs %zu bytes of scratch memory, the entry point that allocates nothing has %zu",
                                 bytes, fixed_bytes);
            *out = fixed;
            return FRK_OK;
        }
        int rc = workspace(bytes, s, lease);
        *out = lease.ptr;
        return rc;
    }
};

// Quantizes `batch` activation rows of w->cols values to Q8_K in the call's scratch memory.
static int quantize_acts_q8_k(const frk_weights *w, const float *x, size_t batch, hipStream_t s, Scratch &scratch,
                              Q8KActs *a) {
    size_t n = batch * w->cols;
    size_t q_bytes = round_up(n, 256), d_bytes = round_up(n / QK_K * 4, 256), b_bytes = round_up(n / 16 * 2, 256);
    void *ws = nullptr;
    int rc = scratch.get(q_bytes + d_bytes + b_bytes, s, &ws);
    if (rc) return rc;
    int8_t *q = (int8_t *)ws;
    float *d = (float *)((char *)ws + q_bytes);
    int16_t *b = (int16_t *)((char *)ws + q_bytes + d_bytes);
    rc = launch_quantize_q8_k(x, n, q, d, b, s);
    if (rc) return rc;
    a->q = q;
    a->d = d;
    a->bsums = b;
    return FRK_OK;
}

// The integer tier of Q5_0 / MXFP4 (the activation as Q8_0 blocks: q8_row_dot, crates/frink-core/src/weight_matrix.rs:
// 392-407) and of IQ4_XS (as Q8_K: q8k_row_dot, :415-420): one activation row quantized into the call's scratch
// memory, then the integer GEMV.
static int gemv_units_int(const frk_weights *w, const float *x, float *y, hipStream_t s, Scratch &scratch) {
    if (!gemv_units_int_fits(w))
        return set_error(FRK_ERR_UNSUPPORTED, "the integer GEMV of quant kind %d does not take rows of %zu columns", w->kind, w->cols);
    if (w->kind == FRK_KIND_IQ4_XS) {
        Q8KActs a;
        int rc = quantize_acts_q8_k(w, x, 1, s, scratch, &a);
        if (rc) return rc;
        return launch_gemv_units_int(w, a.q, a.d, y, s);
    }
    const size_t n = w->cols;
    void *ws = nullptr;
    int rc = scratch.get(round_up(n, 256) + n / 32 * 4, s, &ws);
    if (rc) return rc;
    int8_t *q = (int8_t *)ws;
    float *d = (float *)((char *)ws + round_up(n, 256));
    rc = launch_quantize_q8_0(x, n, q, d, s);
    if (rc) return rc;
    return launch_gemv_units_int(w, q, d, y, s);
}

static int gemv_impl(const frk_weights *w, const float *x, float *y, int act_mode, hipStream_t s, Scratch &scratch) {
    if (act_mode == FRK_ACT_F32_DOT && (w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K || w->kind == FRK_KIND_Q6_K)) {
        if (!kquant_f32_gemv_fits(w))
            return set_error(FRK_ERR_UNSUPPORTED, "the f32-dot GEMV of the K-quants takes rows of at most 16384 columns (%zu)", w->cols);
        return launch_gemv_kquant_f32(w, x, y, s);
    }
    if (act_mode == FRK_ACT_F32_DOT) act_mode = FRK_ACT_F32;  // (Q8_0 and Q4_0: their FRK_ACT_F32 is the f32 dot)
    if (is_unit_kind(w->kind)) {
        if (act_mode == FRK_ACT_F32) return launch_gemv_units_f32(w, x, y, s);
        return gemv_units_int(w, x, y, s, scratch);
    }
    switch (w->kind) {
    case FRK_KIND_Q4_K:
    case FRK_KIND_Q5_K: {
        const int form = rows_gemv_form(w);  // rows of 17..31 and of 33..64 blocks: whole rows to a wavefront
        if (form == ROWS_FORM_COLUMNS) return launch_gemv_q4_k_cols(w, x, y, s);
        if (form == ROWS_FORM_ONE_LAUNCH) return launch_gemv_rows_fused(w, x, y, s);
        if (form == ROWS_FORM_QUANTIZED) {
            Q8KActs a;
            int rc = quantize_acts_q8_k(w, x, 1, s, scratch, &a);
            if (rc) return rc;
            return launch_gemv_rows_preq(w, a, y, s);
        }
        if (w->kind == FRK_KIND_Q4_K && fused_gemv_fits(w)) return launch_gemv_q4_k_fused(w, x, y, s);
        if (q5_k_lines_gemv_fits(w)) return launch_gemv_q5_k_fused(w, x, y, s);
    }
        [[fallthrough]];
    case FRK_KIND_Q6_K: {
        if (w->kind == FRK_KIND_Q6_K && (direct_gemv_fits(w) || q6_k_cols_form(w))) return launch_gemv_q6_k_fused(w, x, y, s);
        Q8KActs a;
        int rc = quantize_acts_q8_k(w, x, 1, s, scratch, &a);
        if (rc) return rc;
        if (w->kind == FRK_KIND_Q4_K) return launch_gemv_q4_k(w, a, y, s);
        if (w->kind == FRK_KIND_Q5_K) return launch_gemv_q5_k(w, a, y, s);
        return direct_gemv_fits(w) ? launch_gemv_q6_k_direct(w, a, y, s) : launch_gemv_q6_k(w, a, y, s);
    }
    case FRK_KIND_Q4_0:
    case FRK_KIND_Q8_0: {
        if (act_mode == FRK_ACT_F32) {
            if (w->kind == FRK_KIND_Q4_0) return q4_0_cols_form(w) ? launch_gemv_q4_0_f32_cols(w, x, y, s) : launch_gemv_q4_0_f32(w, x, y, s);
            return direct_gemv_fits(w) ? launch_gemv_q8_0_f32_direct(w, x, y, s) : launch_gemv_q8_0_f32(w, x, y, s);
        }
        size_t n = w->cols;
        void *ws = nullptr;
        int rc = scratch.get(round_up(n, 256) + n / 32 * 4, s, &ws);
        if (rc) return rc;
        int8_t *q = (int8_t *)ws;
        float *d = (float *)((char *)ws + round_up(n, 256));
        rc = launch_quantize_q8_0(x, n, q, d, s);
        if (rc) return rc;
        return w->kind == FRK_KIND_Q4_0 ? launch_gemv_q4_0_q8(w, q, d, y, s) : launch_gemv_q8_0_q8(w, q, d, y, s);
    }
    }
    return set_error(FRK_ERR_UNSUPPORTED, "no matvec kernel for quant kind %d", w->kind);
}

int frk_hip_gemv_dev(const frk_weights *w, const float *x, float *y, int act_mode, void *stream) {
    clear_error();
    if (!w || !x || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemv_dev: null argument");
    Scratch scratch;
    return gemv_impl(w, x, y, act_mode, (hipStream_t)stream, scratch);
}

int frk_hip_gemv_q8k_dev(const frk_weights *w, const int8_t *q, const float *d, const int16_t *bsums, float *y,
                         void *stream) {
    clear_error();
    if (!w || !q || !d || !bsums || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemv_q8k_dev: null argument");
    Q8KActs a{q, d, bsums};
    if ((w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K) && rows_gemv_takes_quantized(w))
        return launch_gemv_rows_preq(w, a, y, (hipStream_t)stream);
    if (w->kind == FRK_KIND_Q4_K)
        return fused_gemv_fits(w) ? launch_gemv_q4_k_preq(w, a, y, (hipStream_t)stream)
                                  : launch_gemv_q4_k(w, a, y, (hipStream_t)stream);
    if (w->kind == FRK_KIND_Q5_K)
        return q5_k_lines_gemv_fits(w) ? launch_gemv_q5_k_preq(w, a, y, (hipStream_t)stream)
                                       : launch_gemv_q5_k(w, a, y, (hipStream_t)stream);
    if (w->kind == FRK_KIND_Q6_K)
        return direct_gemv_fits(w) ? launch_gemv_q6_k_direct(w, a, y, (hipStream_t)stream)
                                   : launch_gemv_q6_k(w, a, y, (hipStream_t)stream);
    return set_error(FRK_ERR_UNSUPPORTED, "Q8_K activations feed Q4_K, Q5_K and Q6_K weights only (kind %d)", w->kind);
}

// Q4_K: the thin kernel takes 16 rows a launch.  Measured (us; thin launches / the matrix-core GEMM, whose cost
// is flat up to 64 rows): 4096x4096 8.8 at 16 rows, 14.5 at 32 / 17.6; 1024x4096 7.5, 12.9 / 15.0 -- two thin
// launches are ahead for small matrices; 14336x4096 23.9, 44.9 / 24.9; 5120x5120 15.1, 26.8 / 20.4; 4096x11008
// 25.3 at 16 rows / 23.7 -- from 20 M weights on a second thin launch is not.
static bool q4_k_takes_the_matrix_cores(const frk_weights *w, size_t batch) {
    const size_t q4k_thin_rows = w->rows * w->cols > (size_t)20 << 20 ? 16 : 32;
    return w->kind == FRK_KIND_Q4_K && batch > 16 && (batch > q4k_thin_rows || thin_gemm_max_batch(w) < 16);
}
// Q5_K: the same kernel with a third plane for the fifth bits, from the batch on where it is ahead of the
// thin kernel's 16-row groups
static bool q5_k_takes_the_matrix_cores(const frk_weights *w, size_t batch) {
    const size_t q5k_thin_rows = 32;
    return w->kind == FRK_KIND_Q5_K && batch > q5k_thin_rows;
}

// Q6_K: the matrix-core GEMM (with its blocks split between workgroups for small batches: 53 us at
// 4096x14336 and 31 us at 4096x4096 up to 64 rows) is ahead of the thin kernel's 8-row groups (15 us
// and 6 us each) from four groups on for large matrices and from six on for small ones
static bool q6_k_takes_the_matrix_cores(const frk_weights *w, size_t batch) {
    const size_t q6k_gemm_from = w->rows * w->cols > (size_t)2 * 4096 * 4096 ? 25 : 41;
    return w->kind == FRK_KIND_Q6_K && batch >= q6k_gemm_from;
}
// whether a batch of this matrix multiplies on the thin kernels (over plain Q8_K rows)
static bool batch_takes_the_thin_kernels(const frk_weights *w, size_t batch) {
    const bool k_quant = w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K || w->kind == FRK_KIND_Q6_K;
    if (!k_quant || batch < 2) return false;
    if (q4_k_takes_the_matrix_cores(w, batch) || q5_k_takes_the_matrix_cores(w, batch) || q6_k_takes_the_matrix_cores(w, batch))
        return false;
    return thin_gemm_max_batch(w) >= 2;
}

// a thin batch over activations already in Q8_K: `thin` rows a launch (thin_gemm_max_batch), or one launch over a
// grid of such groups where the kernel has that form
static int thin_gemm_acts(const frk_weights *w, const Q8KActs &a, size_t batch, int thin, float *y, hipStream_t s) {
    const size_t nb = w->cols / QK_K;
    if (batch > (size_t)thin && batch <= (size_t)thin_gemm_wide_rows(w)) return launch_thin_gemm_wide(w, (int)batch, a, y, s);
    for (size_t b0 = 0; b0 < batch; b0 += (size_t)thin) {
        const int n = (int)std::min<size_t>((size_t)thin, batch - b0);
        Q8KActs c = {a.q + b0 * w->cols, a.d + b0 * nb, a.bsums + b0 * nb * 16};
        int rc = launch_thin_gemm(w, n, c, y + b0 * w->rows, s);
        if (rc) return rc;
    }
    return FRK_OK;
}

// Whether a Q5_0 / MXFP4 batch goes through the matrix cores: the weights decoded into the Q8_0 planar form (signed
// bytes, f16 scales) in scratch memory, then the Q8_0 GEMM.  From four rows on (below that the decode kernel per row
// reads less than the decoded copy costs); MXFP4 only when every scale 2^(e - 128) is an f16 value.
static bool units_batch_takes_the_matrix_cores(const frk_weights *w, size_t batch) {
    if (batch < 4) return false;
    if (w->kind == FRK_KIND_Q5_0) return true;
    return w->kind == FRK_KIND_MXFP4 && w->e8m0_min >= 104 && w->e8m0_max <= 143;
}
static int gemm_units_int(const frk_weights *w, const float *x, size_t batch, float *y, hipStream_t s, Scratch &scratch) {
    if (units_batch_takes_the_matrix_cores(w, batch)) {
        const Layout planar = layout_for(FRK_KIND_Q8_0, w->cols);
        // (no room for the decoded rows where a copy of them is kept)
        const size_t planar_bytes = w->decoded.load(std::memory_order_acquire) ? 0 : round_up(planar.row_stride * w->rows + 256, 256);
        void *ws = nullptr;
        int rc = scratch.get(planar_bytes + gemm_q8_0_workspace_bytes(batch, w->cols, w->rows), s, &ws);
        if (rc) return rc;
        const uint8_t *decoded = nullptr;
        rc = units_decoded(w, (uint8_t *)ws, s, &decoded);
        if (rc) return rc;
        return launch_gemm_q8_0_planar(decoded, planar.row_stride, planar.off_a, w->rows, w->cols, false, x, batch, y,
                                       (char *)ws + planar_bytes, s);
    }
    if (!gemv_units_int_fits(w))
        return set_error(FRK_ERR_UNSUPPORTED, "the integer tier of quant kind %d does not take rows of %zu columns", w->kind, w->cols);
    if (w->kind == FRK_KIND_IQ4_XS && batch >= 4) {
        // the matrix cores: the rows decoded to signed bytes with their block scales, the batch quantized to Q8_K
        const Layout planar = layout_for(FRK_KIND_Q8_0, w->cols);
        // (no room for the decoded rows where a copy of them is kept)
        const size_t planar_bytes = w->decoded.load(std::memory_order_acquire) ? 0 : round_up(planar.row_stride * w->rows + 256, 256);
        const size_t n = batch * w->cols;
        const size_t q_bytes = round_up(n, 256), d_bytes = round_up(n / QK_K * 4, 256), b_bytes = round_up(n / 16 * 2, 256);
        void *ws = nullptr;
        int rc = scratch.get(planar_bytes + q_bytes + d_bytes + b_bytes + gemm_sub_partial_bytes(batch, w->cols, w->rows), s, &ws);
        if (rc) return rc;
        const uint8_t *decoded = nullptr;
        int8_t *q = (int8_t *)((char *)ws + planar_bytes);
        float *d = (float *)((char *)q + q_bytes);
        int16_t *bs = (int16_t *)((char *)d + d_bytes);
        rc = units_decoded(w, (uint8_t *)ws, s, &decoded);
        if (rc) return rc;
        rc = launch_quantize_q8_k(x, n, q, d, bs, s);
        if (rc) return rc;
        return launch_gemm_sub_planar(decoded, planar.row_stride, planar.off_a, w->rows, w->cols, q, d, batch, y, (char *)bs + b_bytes, s);
    }
    if (w->kind == FRK_KIND_IQ4_XS) {  // one Q8_K quantization of the batch, the decode kernel per row
        Q8KActs a;
        int rc = quantize_acts_q8_k(w, x, batch, s, scratch, &a);
        if (rc) return rc;
        const size_t nb = w->cols / QK_K;
        for (size_t b = 0; b < batch; b++) {
            rc = launch_gemv_units_int(w, a.q + b * w->cols, a.d + b * nb, y + b * w->rows, s);
            if (rc) return rc;
        }
        return FRK_OK;
    }
    // one Q8_0 quantization of the batch (the decode path's kernel, block by block), the decode kernel per row
    const size_t n = batch * w->cols;
    void *ws = nullptr;
    int rc = scratch.get(round_up(n, 256) + n / 32 * 4, s, &ws);
    if (rc) return rc;
    int8_t *q = (int8_t *)ws;
    float *d = (float *)((char *)ws + round_up(n, 256));
    rc = launch_quantize_q8_0(x, n, q, d, s);
    if (rc) return rc;
    for (size_t b = 0; b < batch; b++) {
        rc = launch_gemv_units_int(w, q + b * w->cols, d + b * (w->cols / 32), y + b * w->rows, s);
        if (rc) return rc;
    }
    return FRK_OK;
}

static int gemm_impl(const frk_weights *w, const float *x, size_t batch, float *y, void *stream, Scratch &scratch) {
    // one row is the decode path, whatever the kind
    if (batch == 1) return gemv_impl(w, x, y, FRK_ACT_F32, (hipStream_t)stream, scratch);
    if (q4_k_takes_the_matrix_cores(w, batch) || q5_k_takes_the_matrix_cores(w, batch)) {  // (frk_hip_gemm_pair_dev: the same test)
        void *ws = nullptr;
        int rc = scratch.get(gemm_q4_k_workspace_bytes(batch, w->cols, w->rows, w->kind == FRK_KIND_Q5_K),
                             (hipStream_t)stream, &ws);
        if (rc) return rc;
        return launch_gemm_q4_k(w, x, batch, y, ws, (hipStream_t)stream);
    }
    if (q6_k_takes_the_matrix_cores(w, batch)) {
        void *ws = nullptr;
        int rc = scratch.get(gemm_q6_k_workspace_bytes(batch, w->cols, w->rows), (hipStream_t)stream, &ws);
        if (rc) return rc;
        return launch_gemm_q6_k(w, x, batch, y, ws, (hipStream_t)stream);
    }
    // Q8_0: a batch is the integer path, as in the reference (Q8_0 activation blocks and dot_q8_0_q8,
    // crates/frink-core/src/weight_matrix.rs:2701-2829); a single row keeps the f32 dot of its decode path
    if ((w->kind == FRK_KIND_Q8_0 || w->kind == FRK_KIND_Q4_0) && batch >= 2) {  // (Q4_0: the same kernel, dot_q4_0_q8)
        void *ws = nullptr;
        int rc = scratch.get(gemm_q8_0_workspace_bytes(batch, w->cols, w->rows), (hipStream_t)stream, &ws);
        if (rc) return rc;
        return launch_gemm_q8_0(w, x, batch, y, ws, (hipStream_t)stream);
    }
    // Q5_0 / IQ4_XS / MXFP4: a batch is the integer tier too, as in the reference (q8_row_dot / q8k_row_dot per
    // (row, activation) over activations quantized once, crates/frink-core/src/weight_matrix.rs:392-420)
    if (is_unit_kind(w->kind) && batch >= 2) return gemm_units_int(w, x, batch, y, (hipStream_t)stream, scratch);
    // thin batches of the K-quants: the weights are read once per 8 (Q6_K) or 16 (Q4_K) activation rows
    if (batch_takes_the_thin_kernels(w, batch)) {
        const int thin = thin_gemm_max_batch(w);
        Q8KActs a;
        int rc = quantize_acts_q8_k(w, x, batch, (hipStream_t)stream, scratch, &a);
        if (rc) return rc;
        return thin_gemm_acts(w, a, batch, thin, y, (hipStream_t)stream);
    }
    // Q5_K rows too long for the thin kernel's LDS: the batch is quantized once and every row takes the
    // decode kernel
    if (w->kind == FRK_KIND_Q5_K) {
        Q8KActs a;
        int rc = quantize_acts_q8_k(w, x, batch, (hipStream_t)stream, scratch, &a);
        if (rc) return rc;
        const size_t nb = w->cols / QK_K;
        for (size_t b = 0; b < batch; b++) {
            Q8KActs c = {a.q + b * w->cols, a.d + b * nb, a.bsums + b * nb * 16};
            rc = launch_gemv_q5_k(w, c, y + b * w->rows, (hipStream_t)stream);
            if (rc) return rc;
        }
        return FRK_OK;
    }
    // otherwise one matvec per activation row (the reference's own path below its GEMM threshold,
    // crates/frink-core/src/weight_matrix.rs:2636-2652)
    for (size_t b = 0; b < batch; b++) {
        int rc = gemv_impl(w, x + b * w->cols, y + b * w->rows, FRK_ACT_F32, (hipStream_t)stream, scratch);
        if (rc) return rc;
    }
    return FRK_OK;
}

int frk_hip_gemm_dev(const frk_weights *w, const float *x, size_t batch, float *y, void *stream) {
    clear_error();
    if (!w || !x || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemm_dev: null argument");
    if (batch == 0) return set_error(FRK_ERR_SHAPE, "empty shape: batch=0");
    Scratch scratch;
    return gemm_impl(w, x, batch, y, stream, scratch);
}

int frk_hip_gemm_q8k_dev(const frk_weights *w, const int8_t *q, const float *d, const int16_t *bsums, size_t batch, float *y,
                         void *stream) {
    clear_error();
    if (!w || !q || !d || !bsums || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemm_q8k_dev: null argument");
    if (batch == 0) return set_error(FRK_ERR_SHAPE, "empty shape: batch=0");
    if (batch == 1) return frk_hip_gemv_q8k_dev(w, q, d, bsums, y, stream);
    const bool k_quant = w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K || w->kind == FRK_KIND_Q6_K;
    if (!k_quant) return set_error(FRK_ERR_UNSUPPORTED, "Q8_K activations feed Q4_K, Q5_K and Q6_K weights only (kind %d)", w->kind);
    if (!batch_takes_the_thin_kernels(w, batch))
        return set_error(FRK_ERR_UNSUPPORTED,
                         "a batch of %zu rows of this matrix does not multiply on the thin kernels (the matrix-core GEMM "
                         "quantizes into a tiled form of its own): frk_hip_gemm_dev / frk_hip_gemm_pair_dev", batch);
    Q8KActs a{q, d, bsums};
    return thin_gemm_acts(w, a, batch, thin_gemm_max_batch(w), y, (hipStream_t)stream);
}

int frk_hip_gemm_pair_dev(const frk_weights *w0, const frk_weights *w1, const float *x, size_t batch, float *y0, float *y1,
                          void *stream) {
    clear_error();
    if (!w0 || !w1 || !x || !y0 || !y1) return set_error(FRK_ERR_ARG, "frk_hip_gemm_pair_dev: null argument");
    if (batch == 0) return set_error(FRK_ERR_SHAPE, "empty shape: batch=0");
    if (w0->cols != w1->cols)
        return set_error(FRK_ERR_SHAPE, "the matrices have %zu and %zu columns: they share one batch of activations", w0->cols, w1->cols);
    hipStream_t s = (hipStream_t)stream;
    Scratch scratch;
    auto tiled = [&](const frk_weights *w) { return q4_k_takes_the_matrix_cores(w, batch) || q5_k_takes_the_matrix_cores(w, batch); };
    if (tiled(w0) && tiled(w1)) {
        // one quantization into the tiled form, then the two GEMMs (each with its own room for a split's parts)
        const size_t acts_bytes = round_up(q8k_tiled_bytes(batch, w0->cols), 256);
        const size_t part0 = gemm_q4_k_workspace_bytes(batch, w0->cols, w0->rows, w0->kind == FRK_KIND_Q5_K) - acts_bytes;
        const size_t part1 = gemm_q4_k_workspace_bytes(batch, w1->cols, w1->rows, w1->kind == FRK_KIND_Q5_K) - acts_bytes;
        void *ws = nullptr;
        int rc = scratch.get(acts_bytes + round_up(part0, 256) + part1, s, &ws);
        if (rc) return rc;
        const Q8KTiled acts = q8k_tiled_carve(ws, batch, w0->cols);
        rc = launch_quantize_q8_k_tiled(x, batch, w0->cols, acts, s);
        if (rc) return rc;
        rc = launch_gemm_q4_k_acts(w0, acts, batch, y0, reinterpret_cast<float *>((char *)ws + acts_bytes), s);
        if (rc) return rc;
        return launch_gemm_q4_k_acts(w1, acts, batch, y1, reinterpret_cast<float *>((char *)ws + acts_bytes + round_up(part0, 256)), s);
    }
    // otherwise each matrix takes the path frk_hip_gemm_dev gives it (the same results, two quantizations)
    int rc = gemm_impl(w0, x, batch, y0, stream, scratch);
    if (rc) return rc;
    return gemm_impl(w1, x, batch, y1, stream, scratch);
}

// ---- a batch's activations quantized once, for any number of matrices (BatchActs::Q8K) ----
// The object owns room for both forms the K-quant kernels read: plain Q8_K rows (the decode and thin kernels)
// and the tiled form (the matrix-core GEMMs).  Which of them a batch gets depends on its size alone, so that
// the quantization does not need to know the matrices: plain rows up to ACTS_PLAIN_MAX_BATCH rows (the thin
// kernels take at most 40), tiles from ACTS_TILED_MIN_BATCH rows on (no matrix-core GEMM starts below 17).
constexpr size_t ACTS_PLAIN_MAX_BATCH = 64, ACTS_TILED_MIN_BATCH = 17;
}  // extern "C"
struct frk_batch_acts {
    size_t max_batch = 0, cols = 0;
    void *base = nullptr;       // one allocation: plain rows, then the tiled form
    size_t tiled_off = 0;
    size_t batch = 0;           // rows of the last quantization (0: none yet)
    frk::Q8KActs plain{nullptr, nullptr, nullptr};
};
namespace {
size_t acts_plain_bytes(size_t batch, size_t cols) {
    const size_t n = batch * cols;
    return frk::round_up(n, 256) + frk::round_up(n / frk::QK_K * 4, 256) + frk::round_up(n / 16 * 2, 256);
}
}  // namespace
extern "C" {

int frk_hip_batch_acts_create(size_t max_batch, size_t cols, frk_batch_acts **out) {
    clear_error();
    if (!out) return set_error(FRK_ERR_ARG, "frk_hip_batch_acts_create: null argument");
    *out = nullptr;
    if (max_batch == 0 || cols == 0 || cols % QK_K != 0)
        return set_error(FRK_ERR_SHAPE, "batch activations: %zu rows of %zu columns (whole 256-column blocks, at least one row)", max_batch, cols);
    {
        std::lock_guard<std::mutex> lk(g_dev.mu);
        int rc = ensure_device_locked();
        if (rc) return rc;
    }
    frk_batch_acts *a = new frk_batch_acts();
    a->max_batch = max_batch;
    a->cols = cols;
    a->tiled_off = round_up(acts_plain_bytes(std::min(max_batch, ACTS_PLAIN_MAX_BATCH), cols), 256);
    const size_t bytes = a->tiled_off + (max_batch >= ACTS_TILED_MIN_BATCH ? round_up(q8k_tiled_bytes(max_batch, cols), 256) : 0);
    hipError_t e = hipMalloc(&a->base, bytes);
    if (e != hipSuccess) {
        delete a;
        return set_error(FRK_ERR_HIP, "hipMalloc(%zu) for batch activations: %s", bytes, hipGetErrorString(e));
    }
    *out = a;
    return FRK_OK;
}

int frk_hip_batch_acts_release(frk_batch_acts *a) {
    clear_error();
    if (!a) return FRK_OK;
    hipError_t e = hipFree(a->base);
    delete a;
    if (e != hipSuccess) return set_error(FRK_ERR_HIP, "hipFree: %s", hipGetErrorString(e));
    return FRK_OK;
}

int frk_hip_quantize_batch_acts_dev(frk_batch_acts *a, const float *x, size_t batch, void *stream) {
    clear_error();
    if (!a || !x) return set_error(FRK_ERR_ARG, "frk_hip_quantize_batch_acts_dev: null argument");
    if (batch == 0 || batch > a->max_batch)
        return set_error(FRK_ERR_SHAPE, "a batch of %zu rows in an object made for at most %zu", batch, a->max_batch);
    hipStream_t s = (hipStream_t)stream;
    a->batch = 0;
    if (batch <= ACTS_PLAIN_MAX_BATCH) {
        const size_t n = batch * a->cols;
        int8_t *q = (int8_t *)a->base;
        float *d = (float *)((char *)a->base + round_up(n, 256));
        int16_t *b = (int16_t *)((char *)a->base + round_up(n, 256) + round_up(n / QK_K * 4, 256));
        int rc = launch_quantize_q8_k(x, n, q, d, b, s);
        if (rc) return rc;
        a->plain = Q8KActs{q, d, b};
    }
    if (batch >= ACTS_TILED_MIN_BATCH) {
        int rc = launch_quantize_q8_k_tiled(x, batch, a->cols, q8k_tiled_carve((char *)a->base + a->tiled_off, batch, a->cols), s);
        if (rc) return rc;
    }
    a->batch = batch;
    return FRK_OK;
}

int frk_hip_gemm_acts_dev(const frk_weights *w, const frk_batch_acts *a, float *y, void *stream) {
    clear_error();
    if (!w || !a || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemm_acts_dev: null argument");
    if (a->batch == 0) return set_error(FRK_ERR_ARG, "frk_hip_gemm_acts_dev: the activations hold no quantized batch");
    if (w->cols != a->cols)
        return set_error(FRK_ERR_SHAPE, "the matrix has %zu columns, the quantized activations %zu", w->cols, a->cols);
    const bool k_quant = w->kind == FRK_KIND_Q4_K || w->kind == FRK_KIND_Q5_K || w->kind == FRK_KIND_Q6_K;
    if (!k_quant)
        return set_error(FRK_ERR_UNSUPPORTED, "Q8_K activations feed Q4_K, Q5_K and Q6_K weights only (kind %d): frk_hip_gemm_dev", w->kind);
    const size_t batch = a->batch;
    hipStream_t s = (hipStream_t)stream;
    const bool q45 = q4_k_takes_the_matrix_cores(w, batch) || q5_k_takes_the_matrix_cores(w, batch);
    if (q45 || q6_k_takes_the_matrix_cores(w, batch)) {
        const Q8KTiled acts = q8k_tiled_carve((char *)a->base + a->tiled_off, batch, a->cols);
        const size_t acts_bytes = round_up(q8k_tiled_bytes(batch, w->cols), 256);
        const size_t need = q45 ? gemm_q4_k_workspace_bytes(batch, w->cols, w->rows, w->kind == FRK_KIND_Q5_K)
                                : gemm_q6_k_workspace_bytes(batch, w->cols, w->rows);
        float *partial = nullptr;
        Scratch scratch;
        if (need > acts_bytes) {  // a split of the blocks between workgroups: room for the parts' sums
            void *ws = nullptr;
            int rc = scratch.get(need - acts_bytes, s, &ws);
            if (rc) return rc;
            partial = (float *)ws;
        }
        return q45 ? launch_gemm_q4_k_acts(w, acts, batch, y, partial, s) : launch_gemm_q6_k_acts(w, acts, batch, y, partial, s);
    }
    // (below the matrix-core GEMMs' batches the plain rows are there: ACTS_PLAIN_MAX_BATCH covers every such batch)
    if (batch > ACTS_PLAIN_MAX_BATCH)
        return set_error(FRK_ERR_UNSUPPORTED, "a batch of %zu rows of this matrix has no kernel over quantized activations", batch);
    if (batch == 1) return frk_hip_gemv_q8k_dev(w, a->plain.q, a->plain.d, a->plain.bsums, y, stream);
    if (batch_takes_the_thin_kernels(w, batch)) return thin_gemm_acts(w, a->plain, batch, thin_gemm_max_batch(w), y, s);
    const size_t nb = w->cols / QK_K;  // rows too long for the thin kernels: a decode launch per row
    for (size_t b = 0; b < batch; b++) {
        int rc = frk_hip_gemv_q8k_dev(w, a->plain.q + b * w->cols, a->plain.d + b * nb, a->plain.bsums + b * nb * 16, y + b * w->rows, stream);
        if (rc) return rc;
    }
    return FRK_OK;
}

// ---- the entry point that allocates nothing ----
// Its scratch memory is this array in the library's device image: every GPU the library runs on holds
// its own copy, at its own address, until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress; what the kernels get is the address looked up once per device.
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)FRK_NOALLOC_SCRATCH_MIB << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
constexpr int NOALLOC_MAX_DEVICES = 64;
static void *g_scratch_addr[NOALLOC_MAX_DEVICES] = {nullptr};  // under g_dev.mu

static int noalloc_scratch(void **out) {
    int dev = -1;
    FRK_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return set_error(FRK_ERR_NO_DEVICE, "device %d: at most %d devices", dev, NOALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> lk(g_dev.mu);
    if (!g_scratch_addr[dev]) {  // first call on this device, which is the current one
        void *ptr = nullptr;
        FRK_HIP_TRY(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return set_error(FRK_ERR_HIP, "hipGetSymbolAddress gave no address for the scratch array");
        g_scratch_addr[dev] = ptr;
    }
    *out = g_scratch_addr[dev];
    return FRK_OK;
}

int frk_hip_gemm_noalloc_dev(const frk_weights *w, const float *x, size_t batch, float *y, void *stream) {
    clear_error();
    if (!w || !x || !y) return set_error(FRK_ERR_ARG, "frk_hip_gemm_noalloc_dev: null argument");
    if (batch == 0) return set_error(FRK_ERR_SHAPE, "empty shape: batch=0");
    void *region = nullptr;
    int rc = noalloc_scratch(&region);
    if (rc) return rc;
    Scratch fixed(region, NOALLOC_SCRATCH_BYTES);
    return gemm_impl(w, x, batch, y, stream, fixed);
}

int frk_hip_gemv_multi_dev(const frk_weights *const *ws, size_t n, const float *x, float *const *ys, void *stream) {
    clear_error();
    if (n == 0) return FRK_OK;
    if (!ws || !x || !ys) return set_error(FRK_ERR_ARG, "frk_hip_gemv_multi_dev: null argument");
    hipStream_t s = (hipStream_t)stream;
    bool any_k = false;
    for (size_t i = 0; i < n; i++) {
        if (!ws[i] || !ys[i]) return set_error(FRK_ERR_ARG, "frk_hip_gemv_multi_dev: null matrix or output %zu", i);
        if (ws[i]->cols != ws[0]->cols)
            return set_error(FRK_ERR_SHAPE, "matrix %zu has %zu columns, matrix 0 has %zu: they share one activation", i,
                             ws[i]->cols, ws[0]->cols);
        any_k = any_k || ws[i]->kind == FRK_KIND_Q4_K || ws[i]->kind == FRK_KIND_Q5_K || ws[i]->kind == FRK_KIND_Q6_K;
    }
    // Where every matrix has a one-launch GEMV that quantizes the activation inside the kernel (in
    // the shadow of its first weight loads), sharing a quantization launch is slower than not having
    // one: measured 8.5 us per fused launch against 4.7 + 8.2 per matrix with the shared pass.
    bool all_fused = true;
    for (size_t i = 0; i < n; i++) {
        const frk_weights *w = ws[i];
        all_fused = all_fused && ((w->kind == FRK_KIND_Q4_K && fused_gemv_fits(w)) ||
                                  (w->kind == FRK_KIND_Q6_K && (direct_gemv_fits(w) || q6_k_cols_form(w))) || w->kind == FRK_KIND_Q8_0 ||
                                  w->kind == FRK_KIND_Q4_0);
    }
    if (all_fused) {
        // Q4_K neighbours go out in one launch, four at most: the kernel walks their rows as one list
        size_t i = 0;
        while (i < n) {
            size_t m = 1;
            size_t rows = ws[i]->rows;
            if (ws[i]->kind == FRK_KIND_Q4_K)
                while (i + m < n && m < 4 && ws[i + m]->kind == FRK_KIND_Q4_K && rows + ws[i + m]->rows < (1u << 30)) {
                    rows += ws[i + m]->rows;
                    m++;
                }
            int rc = m > 1 ? launch_gemv_q4_k_group(ws + i, m, x, ys + i, s)
                           : frk_hip_gemv_dev(ws[i], x, ys[i], FRK_ACT_F32, stream);
            if (rc) return rc;
            i += m;
        }
        return FRK_OK;
    }
    // otherwise one Q8_K quantization for every K-quant matrix of the group
    Q8KActs a = {nullptr, nullptr, nullptr};
    Scratch scratch;
    if (any_k) {
        int rc = quantize_acts_q8_k(ws[0], x, 1, s, scratch, &a);
        if (rc) return rc;
    }
    for (size_t i = 0; i < n; i++) {
        int rc;
        if (ws[i]->kind == FRK_KIND_Q8_0 || ws[i]->kind == FRK_KIND_Q4_0 || is_unit_kind(ws[i]->kind))
            rc = frk_hip_gemv_dev(ws[i], x, ys[i], FRK_ACT_F32, stream);  // (these kinds multiply the f32 activation itself)
        else rc = frk_hip_gemv_q8k_dev(ws[i], a.q, a.d, a.bsums, ys[i], stream);
        if (rc) return rc;
    }
    return FRK_OK;
}

int frk_hip_ffn_swiglu_dev(const frk_weights *gate, const frk_weights *up, const frk_weights *down, const float *x,
                           float *y, void *stream) {
    clear_error();
    if (!gate || !up || !down || !x || !y) return set_error(FRK_ERR_ARG, "frk_hip_ffn_swiglu_dev: null argument");
    if (gate->rows != up->rows || gate->cols != up->cols || down->cols != gate->rows)
        return set_error(FRK_ERR_SHAPE, "FFN shapes disagree: gate %zux%zu up %zux%zu down %zux%zu", gate->rows, gate->cols,
                         up->rows, up->cols, down->rows, down->cols);
    hipStream_t s = (hipStream_t)stream;
    const size_t ffn = gate->rows;
    // scratch for gate(x), up(x) and silu(gate)*up behind the quantized activation
    const size_t q_cols = std::max(gate->cols, down->cols);  // either projection may quantize its input here
    const size_t q_area = round_up(q_cols, 256) + round_up(q_cols / 32 * 4, 256) + round_up(q_cols / 8, 256);
    WorkspaceLease lease;
    int rc = workspace(q_area + 3 * round_up(ffn * 4, 256), s, lease);
    if (rc) return rc;
    void *ws = lease.ptr;
    float *g_out = (float *)((char *)ws + q_area), *u_out = g_out + round_up(ffn * 4, 256) / 4,
          *act = u_out + round_up(ffn * 4, 256) / 4;
    if (gate->kind == FRK_KIND_Q4_K && up->kind == FRK_KIND_Q4_K && fused_gemv_fits(gate) &&
        gate->layout.row_stride == up->layout.row_stride) {
        // gate, up and SwiGLU in one launch: row r of both matrices is computed by the same lanes
        rc = launch_gemv_q4_k_glu(gate, up, x, act, s);
        if (rc) return rc;
    } else {
        const frk_weights *pair[2] = {gate, up};
        float *outs[2] = {g_out, u_out};
        rc = frk_hip_gemv_multi_dev(pair, 2, x, outs, stream);
        if (rc) return rc;
        rc = launch_swiglu(g_out, u_out, ffn, act, s);
        if (rc) return rc;
    }
    return frk_hip_gemv_dev(down, act, y, FRK_ACT_F32, stream);
}

int frk_hip_route_top_k_softmax_dev(const float *logits, size_t batch, size_t n_experts, size_t k, int norm,
                                    int32_t *ids, float *weights, void *stream) {
    clear_error();
    if (!logits || !ids || !weights) return set_error(FRK_ERR_ARG, "frk_hip_route_top_k_softmax_dev: null argument");
    if (batch == 0 || n_experts == 0) return set_error(FRK_ERR_SHAPE, "empty shape: batch=%zu experts=%zu", batch, n_experts);
    if (k == 0 || k > n_experts)
        return set_error(FRK_ERR_SHAPE, "top-k %zu must be between 1 and the %zu experts", k, n_experts);
    if (n_experts > 1024 || k > 64)
        return set_error(FRK_ERR_SHAPE, "experts=%zu (max 1024), k=%zu (max 64)", n_experts, k);
    return launch_route_top_k_softmax(logits, (int)batch, (int)n_experts, (int)k, norm, ids, weights,
                                      (hipStream_t)stream);
}

int frk_hip_moe_ffn_dev(const frk_weights *gate, const frk_weights *up, const frk_weights *down, size_t n_experts,
                        const float *x, size_t batch, const int32_t *ids, const float *weights, size_t k, float *out,
                        void *stream) {
    clear_error();
    if (!gate || !up || !down || !x || !ids || !weights || !out)
        return set_error(FRK_ERR_ARG, "frk_hip_moe_ffn_dev: null argument");
    if (batch == 0 || n_experts == 0 || k == 0)
        return set_error(FRK_ERR_SHAPE, "empty shape: batch=%zu experts=%zu k=%zu", batch, n_experts, k);
    if (n_experts > 1024 || k > 64 || k > n_experts)
        return set_error(FRK_ERR_SHAPE, "experts=%zu (max 1024), k=%zu (max 64, at most the expert count)", n_experts, k);
    const bool unit_experts = is_unit_kind(gate->kind) && up->kind == gate->kind && is_unit_kind(down->kind);
    if (!unit_experts &&
        (gate->kind != FRK_KIND_Q4_K || up->kind != FRK_KIND_Q4_K || (down->kind != FRK_KIND_Q4_K && down->kind != FRK_KIND_Q6_K)))
        return set_error(FRK_ERR_UNSUPPORTED,
                         "the expert GEMMs take Q4_K gate and up and Q4_K or Q6_K down experts, or Q5_0 / IQ4_XS / MXFP4 experts "
                         "with gate and up of one kind (got kinds %d/%d/%d)",
                         gate->kind, up->kind, down->kind);
    if (gate->rows % n_experts || down->rows % n_experts)
        return set_error(FRK_ERR_SHAPE, "stacked rows %zu/%zu do not divide into %zu experts", gate->rows, down->rows,
                         n_experts);
    const size_t ffn = gate->rows / n_experts, hidden = down->rows / n_experts;
    if (up->rows != gate->rows || up->cols != gate->cols || gate->cols != hidden || down->cols != ffn)
        return set_error(FRK_ERR_SHAPE,
                         "expert shapes disagree: gate %zux%zu up %zux%zu down %zux%zu over %zu experts (hidden %zu, ffn %zu)",
                         gate->rows, gate->cols, up->rows, up->cols, down->rows, down->cols, n_experts, hidden, ffn);
    if (batch * k > (size_t)1 << 30) return set_error(FRK_ERR_SHAPE, "batch*k = %zu pairs is too many", batch * k);
    WorkspaceLease lease;
    if (unit_experts && moe_units_takes_grouped_path(gate, up, down, batch)) {
        int rc = workspace(moe_units_grouped_workspace_bytes(batch, (int)k, (int)n_experts, (int)hidden, (int)ffn), (hipStream_t)stream, lease);
        if (rc) return rc;
        return launch_moe_ffn_units_grouped(gate, up, down, (int)n_experts, x, batch, ids, weights, (int)k, out, lease.ptr,
                                            (hipStream_t)stream);
    }
    if (unit_experts) {
        if (!gemv_units_int_fits(gate) || !gemv_units_int_fits(down))
            return set_error(FRK_ERR_UNSUPPORTED, "experts of kinds %d/%d with rows of %zu / %zu columns", gate->kind, down->kind,
                             gate->cols, down->cols);
        int rc = workspace(moe_units_workspace_bytes(batch, (int)k, (int)hidden, (int)ffn), (hipStream_t)stream, lease);
        if (rc) return rc;
        return launch_moe_ffn_units(gate, up, down, (int)n_experts, x, batch, ids, weights, (int)k, out, lease.ptr, (hipStream_t)stream);
    }
    int rc = workspace(moe_workspace_bytes(batch, (int)k, (int)n_experts, (int)hidden, (int)ffn), (hipStream_t)stream, lease);
    if (rc) return rc;
    return launch_moe_ffn(gate, up, down, (int)n_experts, x, batch, ids, weights, (int)k, out, lease.ptr, (hipStream_t)stream);
}

int frk_hip_gemm_grouped_dev(const frk_weights *stacked, size_t n_groups, const int32_t *group_off, const int32_t *gather,
                             const float *x, size_t x_rows, size_t pairs, float *y, void *stream) {
    clear_error();
    if (!stacked || !group_off || (pairs && (!x || !y))) return set_error(FRK_ERR_ARG, "frk_hip_gemm_grouped_dev: null argument");
    if (n_groups == 0 || n_groups > 1024) return set_error(FRK_ERR_SHAPE, "groups=%zu (1 .. 1024)", n_groups);
    const bool units = is_unit_kind(stacked->kind) && units_have_planar_form(stacked);
    if (stacked->kind != FRK_KIND_Q4_K && stacked->kind != FRK_KIND_Q6_K && !units)
        return set_error(FRK_ERR_UNSUPPORTED,
                         "the grouped GEMM takes Q4_K, Q6_K, Q5_0, IQ4_XS or MXFP4 (scale bytes within 104..143) weights (got kind %d)",
                         stacked->kind);
    if (stacked->rows % n_groups)
        return set_error(FRK_ERR_SHAPE, "stacked rows %zu do not divide into %zu groups", stacked->rows, n_groups);
    if (pairs > (size_t)1 << 30 || x_rows > (size_t)1 << 30)
        return set_error(FRK_ERR_SHAPE, "pairs=%zu, activation rows=%zu: too many", pairs, x_rows);
    if (pairs == 0) return FRK_OK;
    if (x_rows == 0) return set_error(FRK_ERR_SHAPE, "%zu pairs over no activation rows", pairs);
    WorkspaceLease lease;
    if (units) {
        int rc = workspace(grouped_units_workspace_bytes(n_groups, stacked->rows, x_rows, pairs, stacked->cols), (hipStream_t)stream, lease);
        if (rc) return rc;
        return launch_gemm_grouped_units(stacked, n_groups, group_off, gather, x, x_rows, pairs, y, lease.ptr, (hipStream_t)stream);
    }
    int rc = workspace(grouped_gemm_workspace_bytes(n_groups, x_rows, pairs, stacked->cols), (hipStream_t)stream, lease);
    if (rc) return rc;
    return launch_gemm_grouped(stacked, n_groups, group_off, gather, x, x_rows, pairs, y, lease.ptr, (hipStream_t)stream);
}

int frk_hip_moe_intermediates_dev(size_t batch, size_t k, size_t n_experts, size_t hidden, size_t ffn,
                                  float *gate_out, float *up_out, int8_t *act_q, float *act_d, int32_t *pos_of,
                                  void *stream) {
    clear_error();
    if (batch == 0 || k == 0 || n_experts == 0 || hidden == 0 || ffn == 0)
        return set_error(FRK_ERR_SHAPE, "frk_hip_moe_intermediates_dev: empty shape");
    // (the hook does not know the experts' kinds: it refuses what Q4_K experts would have run per token)
    if (moe_takes_per_token_path(batch, hidden, ffn, FRK_KIND_Q4_K))
        return set_error(FRK_ERR_UNSUPPORTED, "a batch of %zu runs per token and keeps no grouped intermediates", batch);
    WorkspaceLease lease;
    int rc = workspace(moe_workspace_bytes(batch, (int)k, (int)n_experts, (int)hidden, (int)ffn), (hipStream_t)stream, lease);
    if (rc) return rc;
    return moe_copy_intermediates(lease.ptr, batch, (int)k, (int)n_experts, (int)hidden, (int)ffn, gate_out, up_out, act_q,
                                  act_d, pos_of, (hipStream_t)stream);
}

// ---- host-buffer entry points ----

static int stage_buffers(size_t x_bytes, size_t y_bytes) {
    if (x_bytes > g_dev.x_bytes) {
        if (g_dev.x_dev) (void)hipFree(g_dev.x_dev);
        g_dev.x_dev = nullptr;
        g_dev.x_bytes = 0;
        FRK_HIP_TRY(hipMalloc(&g_dev.x_dev, round_up(x_bytes, 1 << 16)));
        g_dev.x_bytes = round_up(x_bytes, 1 << 16);
    }
    if (y_bytes > g_dev.y_bytes) {
        if (g_dev.y_dev) (void)hipFree(g_dev.y_dev);
        g_dev.y_dev = nullptr;
        g_dev.y_bytes = 0;
        FRK_HIP_TRY(hipMalloc(&g_dev.y_dev, round_up(y_bytes, 1 << 16)));
        g_dev.y_bytes = round_up(y_bytes, 1 << 16);
    }
    return FRK_OK;
}

// One mutex serialises the host-buffer entry points: they share the staging buffers and the
// library's stream, and the reference calls them from many worker threads at once
// (crates/frink-core/src/weight_matrix/gpu_backend.rs:722-725).
static std::mutex g_launch_mu;

static int host_launch(int kind, const uint8_t *weights, size_t weights_len, const float *x, size_t rows,
                       size_t cols, size_t batch, float *out) {
    frk_weights *w = nullptr;
    int rc = frk_hip_weights_register(kind, weights, weights_len, rows, cols, &w);
    if (rc) return rc;
    std::lock_guard<std::mutex> lk(g_launch_mu);
    size_t xb = batch * cols * sizeof(float), yb = batch * rows * sizeof(float);
    rc = stage_buffers(xb, yb);
    hipStream_t s = g_dev.stream;
    if (!rc) {
        hipError_t e = hipMemcpyAsync(g_dev.x_dev, x, xb, hipMemcpyHostToDevice, s);
        if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(x): %s", hipGetErrorString(e));
    }
    if (!rc)
        rc = batch == 1 ? frk_hip_gemv_dev(w, (const float *)g_dev.x_dev, (float *)g_dev.y_dev, FRK_ACT_F32, s)
                        : frk_hip_gemm_dev(w, (const float *)g_dev.x_dev, batch, (float *)g_dev.y_dev, s);
    if (!rc) {
        hipError_t e = hipMemcpyAsync(out, g_dev.y_dev, yb, hipMemcpyDeviceToHost, s);
        if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(y): %s", hipGetErrorString(e));
    }
    hipError_t e = hipStreamSynchronize(s);
    if (!rc && e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e));
    char keep[sizeof g_err];
    memcpy(keep, g_err, sizeof keep);
    frk_hip_weights_release(w);
    memcpy(g_err, keep, sizeof keep);
    return rc;
}

int frk_hip_get_rows(const frk_weights *w, const int32_t *ids, size_t n_ids, float *out) {
    clear_error();
    if (!w || (n_ids && (!ids || !out))) return set_error(FRK_ERR_ARG, "frk_hip_get_rows: null argument");
    for (size_t i = 0; i < n_ids; i++)
        if (ids[i] < 0 || (size_t)ids[i] >= w->rows)
            return set_error(FRK_ERR_SHAPE, "id %zu is %d, the table has %zu rows", i, ids[i], w->rows);
    if (n_ids == 0) return FRK_OK;
    std::lock_guard<std::mutex> lk(g_launch_mu);
    const size_t ib = n_ids * sizeof(int32_t), ob = n_ids * w->cols * sizeof(float);
    int rc = stage_buffers(ib, ob);
    hipStream_t s = g_dev.stream;
    if (!rc) {
        hipError_t e = hipMemcpyAsync(g_dev.x_dev, ids, ib, hipMemcpyHostToDevice, s);
        if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(ids): %s", hipGetErrorString(e));
    }
    if (!rc) rc = launch_dequant_rows(w, (const int32_t *)g_dev.x_dev, n_ids, (float *)g_dev.y_dev, s);
    if (!rc) {
        hipError_t e = hipMemcpyAsync(out, g_dev.y_dev, ob, hipMemcpyDeviceToHost, s);
        if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(rows): %s", hipGetErrorString(e));
    }
    hipError_t e = hipStreamSynchronize(s);
    if (!rc && e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e));
    return rc;
}

int frk_hip_launch_matvec(int kind, const uint8_t *weights, size_t weights_len, const float *x, size_t x_len,
                          size_t rows, size_t row_bytes, float *out) {
    clear_error();
    if (!frk_hip_has_launch(kind)) return set_error(FRK_ERR_UNSUPPORTED, "no matvec kernel for quant kind %d", kind);
    if (!weights || !x || !out) return set_error(FRK_ERR_ARG, "frk_hip_launch_matvec: null argument");
    size_t bb = (size_t)block_bytes(kind), be = (size_t)block_elems(kind);
    if (rows == 0) return set_error(FRK_ERR_SHAPE, "empty shape: rows=0");
    if (row_bytes == 0 || row_bytes % bb)
        return set_error(FRK_ERR_SHAPE, "row_bytes %zu is not a whole number of %zu-byte %s blocks", row_bytes, bb,
                         frk_hip_matvec_kernel(kind));
    size_t nb = row_bytes / bb;
    if (weights_len != rows * row_bytes)
        return set_error(FRK_ERR_SHAPE, "weights are %zu bytes, %zu rows of %zu bytes need %zu", weights_len, rows,
                         row_bytes, rows * row_bytes);
    if (x_len != nb * be)
        return set_error(FRK_ERR_SHAPE, "activation has %zu values, %zu blocks of %zu need %zu", x_len, nb, be, nb * be);
    return host_launch(kind, weights, weights_len, x, rows, nb * be, 1, out);
}

int frk_hip_launch_mul_mm(int kind, const uint8_t *weights, size_t weights_len, const float *x_batch, size_t x_len,
                          size_t n_rows, size_t n_cols, size_t batch, size_t row_bytes, float *out) {
    clear_error();
    if (!frk_hip_has_launch(kind)) return set_error(FRK_ERR_UNSUPPORTED, "no GEMM kernel for quant kind %d", kind);
    if (!weights || !x_batch || !out) return set_error(FRK_ERR_ARG, "frk_hip_launch_mul_mm: null argument");
    size_t bb = (size_t)block_bytes(kind), be = (size_t)block_elems(kind);
    if (n_rows == 0 || n_cols == 0 || batch == 0)
        return set_error(FRK_ERR_SHAPE, "empty shape: rows=%zu cols=%zu batch=%zu", n_rows, n_cols, batch);
    if (n_cols % be)
        return set_error(FRK_ERR_SHAPE, "cols %zu is not a multiple of the %zu-element %s block", n_cols, be,
                         frk_hip_matvec_kernel(kind));
    size_t expect = n_cols / be * bb;
    if (row_bytes != expect) return set_error(FRK_ERR_SHAPE, "row_bytes %zu, expected %zu", row_bytes, expect);
    if (weights_len < n_rows * row_bytes)
        return set_error(FRK_ERR_SHAPE, "weights too small: got %zu bytes, want %zu", weights_len, n_rows * row_bytes);
    if (x_len < batch * n_cols)
        return set_error(FRK_ERR_SHAPE, "activations too small: got %zu values, want %zu", x_len, batch * n_cols);
    return host_launch(kind, weights, n_rows * row_bytes, x_batch, n_rows, n_cols, batch, out);
}


static int check_launch(const frk_matvec_launch *l, size_t *cols) {
    if (!l || !l->weights) return set_error(FRK_ERR_ARG, "null launch or weights");
    if (!frk_hip_has_launch(l->kind)) return set_error(FRK_ERR_UNSUPPORTED, "no matvec kernel for quant kind %d", l->kind);
    size_t bb = (size_t)block_bytes(l->kind), be = (size_t)block_elems(l->kind);
    if (l->rows == 0) return set_error(FRK_ERR_SHAPE, "empty shape: rows=0");
    if (l->row_bytes == 0 || l->row_bytes % bb)
        return set_error(FRK_ERR_SHAPE, "row_bytes %zu is not a whole number of %zu-byte blocks", l->row_bytes, bb);
    if (l->weights_len != l->rows * l->row_bytes)
        return set_error(FRK_ERR_SHAPE, "weights are %zu bytes, %zu rows of %zu bytes need %zu", l->weights_len, l->rows,
                         l->row_bytes, l->rows * l->row_bytes);
    *cols = l->row_bytes / bb * be;
    return FRK_OK;
}

// Uploads x once, runs `dev_fn` on the library's stream, downloads n outputs; weights stay resident.
int frk_hip_launch_matvec_multi(const float *x, size_t x_len, const frk_matvec_launch *launches, size_t n,
                                float *const *outs) {
    clear_error();
    if (n == 0) return FRK_OK;
    if (!x || !launches || !outs) return set_error(FRK_ERR_ARG, "frk_hip_launch_matvec_multi: null argument");
    std::vector<frk_weights *> ws(n, nullptr);
    size_t total_rows = 0;
    int rc = FRK_OK;
    for (size_t i = 0; i < n && !rc; i++) {
        size_t cols = 0;
        rc = check_launch(&launches[i], &cols);
        if (!rc && cols != x_len)
            rc = set_error(FRK_ERR_SHAPE, "activation has %zu values, matrix %zu needs %zu", x_len, i, cols);
        if (!rc && !outs[i]) rc = set_error(FRK_ERR_ARG, "output %zu is null", i);
        if (!rc)
            rc = frk_hip_weights_register(launches[i].kind, launches[i].weights, launches[i].weights_len, launches[i].rows,
                                          cols, &ws[i]);
        total_rows += launches[i].rows;
    }
    if (!rc) {
        std::lock_guard<std::mutex> lk(g_launch_mu);
        rc = stage_buffers(x_len * sizeof(float), total_rows * sizeof(float));
        hipStream_t s = g_dev.stream;
        if (!rc) {
            hipError_t e = hipMemcpyAsync(g_dev.x_dev, x, x_len * sizeof(float), hipMemcpyHostToDevice, s);
            if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(x): %s", hipGetErrorString(e));
        }
        std::vector<float *> ys(n);
        size_t off = 0;
        for (size_t i = 0; i < n; i++) {
            ys[i] = (float *)g_dev.y_dev + off;
            off += launches[i].rows;
        }
        if (!rc) rc = frk_hip_gemv_multi_dev(ws.data(), n, (const float *)g_dev.x_dev, ys.data(), s);
        for (size_t i = 0; i < n && !rc; i++) {
            hipError_t e = hipMemcpyAsync(outs[i], ys[i], launches[i].rows * sizeof(float), hipMemcpyDeviceToHost, s);
            if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(y): %s", hipGetErrorString(e));
        }
        hipError_t e = hipStreamSynchronize(s);
        if (!rc && e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e));
    }
    char keep[sizeof g_err];
    memcpy(keep, g_err, sizeof keep);
    for (frk_weights *w : ws)
        if (w) frk_hip_weights_release(w);
    memcpy(g_err, keep, sizeof keep);
    return rc;
}

int frk_hip_launch_dense_ffn_swiglu(const frk_matvec_launch *gate, const frk_matvec_launch *up,
                                    const frk_matvec_launch *down, const float *x, size_t x_len, float *out) {
    clear_error();
    if (!x || !out) return set_error(FRK_ERR_ARG, "frk_hip_launch_dense_ffn_swiglu: null argument");
    const frk_matvec_launch *ls[3] = {gate, up, down};
    frk_weights *ws[3] = {nullptr, nullptr, nullptr};
    size_t cols[3] = {0, 0, 0};
    int rc = FRK_OK;
    for (int i = 0; i < 3 && !rc; i++) rc = check_launch(ls[i], &cols[i]);
    if (!rc && (cols[0] != x_len || cols[1] != x_len))
        rc = set_error(FRK_ERR_SHAPE, "activation has %zu values, gate/up need %zu/%zu", x_len, cols[0], cols[1]);
    if (!rc && (gate->rows != up->rows || cols[2] != gate->rows))
        rc = set_error(FRK_ERR_SHAPE, "gate rows %zu, up rows %zu, down columns %zu must agree", gate->rows, up->rows, cols[2]);
    for (int i = 0; i < 3 && !rc; i++)
        rc = frk_hip_weights_register(ls[i]->kind, ls[i]->weights, ls[i]->weights_len, ls[i]->rows, cols[i], &ws[i]);
    if (!rc) {
        std::lock_guard<std::mutex> lk(g_launch_mu);
        rc = stage_buffers(x_len * sizeof(float), down->rows * sizeof(float));
        hipStream_t s = g_dev.stream;
        if (!rc) {
            hipError_t e = hipMemcpyAsync(g_dev.x_dev, x, x_len * sizeof(float), hipMemcpyHostToDevice, s);
            if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(x): %s", hipGetErrorString(e));
        }
        if (!rc) rc = frk_hip_ffn_swiglu_dev(ws[0], ws[1], ws[2], (const float *)g_dev.x_dev, (float *)g_dev.y_dev, s);
        if (!rc) {
            hipError_t e = hipMemcpyAsync(out, g_dev.y_dev, down->rows * sizeof(float), hipMemcpyDeviceToHost, s);
            if (e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipMemcpyAsync(y): %s", hipGetErrorString(e));
        }
        hipError_t e = hipStreamSynchronize(s);
        if (!rc && e != hipSuccess) rc = set_error(FRK_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e));
    }
    char keep[sizeof g_err];
    memcpy(keep, g_err, sizeof keep);
    for (frk_weights *w : ws)
        if (w) frk_hip_weights_release(w);
    memcpy(g_err, keep, sizeof keep);
    return rc;
}

}  // extern "C"
