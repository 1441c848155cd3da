// C ABI of libcamelid_hip (declared in include/camelid_hip.h): lifecycle,
// device-resident weights, and dispatch to the per-format kernels.
//
// The conventions follow the reference's device seam (src/cuda.rs:167-236 for
// gating, :691-699 for the process-global backend, :1044-1218 for the
// "handled / not handled" contract): nothing here throws or aborts; every
// failure becomes a status code plus a thread-local message.
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "cml_host.hpp"

namespace cml {

static thread_local char g_error[512] = "";
static std::atomic<int> g_device{-1};
static std::atomic<uint64_t> g_runs{0};
static std::mutex g_mutex;

// Staging area of cml_matmul_f32_static: the quantized activation rows (int8 values, then f32
// scales) of one call.  Device memory that lives in the code object, one copy per GPU, from the
// moment the library is loaded on that GPU until the process ends.  The name below is a host-side
// stand-in: only the address hipGetSymbolAddress reports for the current device (kept in
// g_static_workspace, filled by cml_init) may be handed to a kernel.
constexpr size_t kStaticWorkspaceBytes = CML_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];
constexpr int kMaxDevices = 64;
static void *g_static_workspace[kMaxDevices] = {};

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_error[0] = '\0'; }

bool ready() { return g_device.load(std::memory_order_acquire) >= 0; }

static std::atomic<LaunchCounter *> g_counters{nullptr};

LaunchCounter::LaunchCounter(const std::string &nm) : LaunchCounter(strdup(nm.c_str())) {}

LaunchCounter::LaunchCounter(const char *nm) : name(nm ? nm : "?") {
    LaunchCounter *head = g_counters.load(std::memory_order_acquire);
    do {
        next = head;
    } while (!g_counters.compare_exchange_weak(head, this, std::memory_order_release, std::memory_order_acquire));
}

// Knobs (CAMELID_HIP_*) are read from the environment ONCE, into a snapshot taken by
// cml_init and again by cml_reload_env (reference: every CAMELID_* knob sits in a OnceLock,
// src/inference.rs:23679-23692).  A launch only walks the snapshot -- normally empty -- and never
// calls getenv, so it neither pays for it nor races with a setenv in another thread.
// Two kinds.  The few knobs that choose WHAT is computed or where (the device, and which of the
// reference's accumulation orders the results follow) are always honoured.  Everything else chooses
// among kernels that give the same bits -- launch shapes, ring depths, thresholds: the switches
// of this library's own tests and measurements -- and is honoured only when CAMELID_HIP_TUNING=1 is set
// with it, so that a stray variable in a production host's environment cannot move a call onto a
// slower kernel.
struct EnvSnapshot {
    std::vector<std::pair<std::string, int>> knobs;  // names without the CAMELID_HIP_ prefix
};
static std::atomic<const EnvSnapshot *> g_env{nullptr};
static std::vector<const EnvSnapshot *> g_env_retired;  // guarded by g_mutex
extern "C" char **environ;

static void load_env_snapshot() {
    auto *snap = new EnvSnapshot();
    static const char prefix[] = "CAMELID_HIP_";
    static const char *const always[] = {"DEVICE", "EXACT_ORDER", "Q4K_LANE_ORDER", "Q6K_LANE_ORDER"};
    const char *tuning_env = getenv("CAMELID_HIP_TUNING");
    const bool tuning = tuning_env && atoi(tuning_env) != 0;
    for (char **e = environ; e && *e; e++) {
        if (strncmp(*e, prefix, sizeof(prefix) - 1) != 0) continue;
        const char *eq = strchr(*e, '=');
        if (!eq || !eq[1]) continue;  // unset or empty: the default applies
        std::string key(static_cast<const char *>(*e) + sizeof(prefix) - 1, eq);
        bool take = tuning;
        for (const char *a : always) take = take || key == a;
        if (take) snap->knobs.emplace_back(std::move(key), atoi(eq + 1));
    }
    // a superseded snapshot is not freed here -- a launch on another thread may still be walking it -- but
    // retired, and freed by cml_shutdown, which by contract runs alone (callers hold g_mutex)
    const EnvSnapshot *old = g_env.exchange(snap, std::memory_order_acq_rel);
    if (old) g_env_retired.push_back(old);
}

int env_int(const char *name, int dflt) {
    const EnvSnapshot *snap = g_env.load(std::memory_order_acquire);
    if (!snap) {  // before cml_init (library gating only)
        const char *v = getenv(name);
        return (!v || !*v) ? dflt : atoi(v);
    }
    if (snap->knobs.empty()) return dflt;
    const char *key = name + 12;  // every knob name starts with CAMELID_HIP_
    for (const auto &kv : snap->knobs)
        if (kv.first == key) return kv.second;
    return dflt;
}

// Environment masking is checked before any driver call (reference
// devices_masked_by_env, src/cuda.rs:206-218).
static bool masked_by_env() {
    const char *off = getenv("CAMELID_HIP");
    if (off && (!strcmp(off, "0") || !strcasecmp(off, "off") || !strcasecmp(off, "false"))) return true;
    const char *names[] = {"HIP_VISIBLE_DEVICES", "ROCR_VISIBLE_DEVICES"};
    for (const char *n : names) {
        const char *v = getenv(n);
        if (v && (!*v || !strcmp(v, "-1"))) return true;
    }
    return false;
}

static int check_ready() {
    if (!ready()) return fail(CML_ERR_UNAVAILABLE, "cml_init has not succeeded");
    return CML_OK;
}

}  // namespace cml

using namespace cml;

// Nothing may unwind through the C boundary: an entry point whose body can allocate host memory
// (containers, std::string) runs it inside this guard and reports an allocation failure as a status.
#define CML_NOTHROW_BEGIN try {
#define CML_NOTHROW_END                                                        \
    }                                                                          \
    catch (const std::bad_alloc &) {                                           \
        return fail(CML_ERR_OOM, "host allocation failed");                    \
    }                                                                          \
    catch (...) {                                                              \
        return fail(CML_ERR_INVALID, "unexpected C++ exception at the C boundary"); \
    }

// Read-only yardstick: every lane keeps `in_flight` 16-byte non-temporal loads out over a grid-stride
// walk of the buffer and stores nothing (what a launch that only reads can reach on this chip).
template <int INFL>
__global__ void __launch_bounds__(256) read_kernel(const uint4 *__restrict__ src, size_t n16, uint32_t *sink) {
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const v4u *p = reinterpret_cast<const v4u *>(src);
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    v4u acc = {0, 0, 0, 0};
    for (; i + (INFL - 1) * stride < n16; i += INFL * stride) {
        v4u v[INFL];
#pragma unroll
        for (int k = 0; k < INFL; k++) v[k] = __builtin_nontemporal_load(p + i + k * stride);
#pragma unroll
        for (int k = 0; k < INFL; k++) acc ^= v[k];
    }
    for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(p + i);
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345679u && sink) sink[0] = 1;  // keeps the loads alive
}

namespace {
struct CacheKey {
    const void *ptr;
    size_t len;
    int fmt;
    bool operator==(const CacheKey &o) const { return ptr == o.ptr && len == o.len && fmt == o.fmt; }
};
struct CacheHash {
    size_t operator()(const CacheKey &k) const {
        return std::hash<const void *>()(k.ptr) ^ (std::hash<size_t>()(k.len) * 1315423911u) ^ static_cast<size_t>(k.fmt);
    }
};
// State of the host-slice seam, all under g_mutex: weights cached on the device by (pointer,
// length, format) and one grow-only device buffer for the activations and outputs of a call.
std::unordered_map<CacheKey, cml_weight *, CacheHash> g_weight_cache;
uint8_t *g_seam_buf = nullptr;
size_t g_seam_bytes = 0;
}  // namespace

extern "C" {

int cml_block_values(int fmt) { return geometry(fmt).block_values; }
int cml_block_bytes(int fmt) { return geometry(fmt).block_bytes; }

int cml_available(void) {
    if (masked_by_env()) return 0;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    for (int i = 0; i < n; i++) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, i) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0) return 1;
    }
    return 0;
}

int cml_init(int device) {
    clear_error();
    if (masked_by_env()) return fail(CML_ERR_UNAVAILABLE, "GPU use is masked by the environment");
    std::lock_guard<std::mutex> lock(g_mutex);
    CML_NOTHROW_BEGIN
    if (!g_env.load(std::memory_order_acquire)) load_env_snapshot();
    CML_NOTHROW_END
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(CML_ERR_UNAVAILABLE, "no HIP device");
    }
    if (device < 0) device = env_int("CAMELID_HIP_DEVICE", 0);
    if (device >= n) return fail(CML_ERR_INVALID, "device %d out of range (%d present)", device, n);
    hipDeviceProp_t prop;
    CML_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(CML_ERR_UNAVAILABLE, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    CML_HIP_TRY(hipSetDevice(device));
    if (device < kMaxDevices && g_static_workspace[device] == nullptr) {
        // with `device` current: every GPU has its own copy of the array at its own address
        void *p = nullptr;
        CML_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_static_workspace[device] = p;
    }
    g_device.store(device, std::memory_order_release);
    return CML_OK;
}

void cml_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (ready()) {
        // what the library itself owns on the device: the seam's cached weights and its staging buffer
        for (auto &kv : g_weight_cache) cml_weight_free(kv.second);
        g_weight_cache.clear();
        if (g_seam_buf) (void)hipFree(g_seam_buf);
        g_seam_buf = nullptr;
        g_seam_bytes = 0;
    }
    for (const EnvSnapshot *e : g_env_retired) delete e;  // snapshots superseded by cml_reload_env
    g_env_retired.clear();
    g_device.store(-1, std::memory_order_release);
}

int cml_reload_env(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    CML_NOTHROW_BEGIN
    load_env_snapshot();
    CML_NOTHROW_END
    return CML_OK;
}

const char *cml_last_error(void) { return g_error; }
uint64_t cml_run_count(void) { return g_runs.load(std::memory_order_relaxed); }

uint64_t cml_kernel_launches(const char *prefix) {
    const size_t len = prefix ? strlen(prefix) : 0;
    uint64_t total = 0;
    for (const LaunchCounter *c = g_counters.load(std::memory_order_acquire); c; c = c->next)
        if (len == 0 || strncmp(c->name, prefix, len) == 0) total += c->n.load(std::memory_order_relaxed);
    return total;
}

size_t cml_kernel_launch_report(char *buf, size_t cap) {
    // "name count\n" per counter; returns the size the whole report needs (with its terminator)
    size_t need = 1, at = 0;
    for (const LaunchCounter *c = g_counters.load(std::memory_order_acquire); c; c = c->next) {
        char line[160];
        const int n = snprintf(line, sizeof(line), "%s %llu\n", c->name, static_cast<unsigned long long>(c->n.load(std::memory_order_relaxed)));
        if (n <= 0) continue;
        need += static_cast<size_t>(n);
        if (buf && at + static_cast<size_t>(n) < cap) {
            memcpy(buf + at, line, static_cast<size_t>(n));
            at += static_cast<size_t>(n);
        }
    }
    if (buf && cap) buf[at] = '\0';
    return need;
}

// ---- device memory plumbing ------------------------------------------------------------------------

int cml_dev_alloc(size_t nbytes, void **out_dev) {
    if (!out_dev) return fail(CML_ERR_INVALID, "null out pointer");
    *out_dev = nullptr;
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) nbytes = 16;
    CML_HIP_TRY(hipMalloc(out_dev, nbytes));
    return CML_OK;
}

int cml_dev_free(void *ptr_dev) {
    if (!ptr_dev) return CML_OK;  // also after cml_shutdown: the caller's buffers outlive it
    CML_HIP_TRY(hipFree(ptr_dev));
    return CML_OK;
}

int cml_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) return CML_OK;
    if (!dst_dev || !src_host) return fail(CML_ERR_INVALID, "null pointer");
    CML_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, as_stream(stream)));
    CML_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return CML_OK;
}

int cml_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) return CML_OK;
    if (!dst_host || !src_dev) return fail(CML_ERR_INVALID, "null pointer");
    CML_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, as_stream(stream)));
    CML_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return CML_OK;
}

int cml_memset_dev(void *dst_dev, int value, size_t nbytes, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) return CML_OK;
    if (!dst_dev) return fail(CML_ERR_INVALID, "null pointer");
    CML_HIP_TRY(hipMemsetAsync(dst_dev, value, nbytes, as_stream(stream)));
    return CML_OK;
}

// Plain streaming copy, 16 bytes per lane per trip: the yardstick the byte counters and the matvec
// kernels are read against (it moves nbytes in and nbytes out and nothing else).
__global__ void __launch_bounds__(256) copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

int cml_copy_dev(void *dst_dev, const void *src_dev, size_t nbytes, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) return CML_OK;
    if (!dst_dev || !src_dev) return fail(CML_ERR_INVALID, "null pointer");
    if ((nbytes | (uintptr_t)dst_dev | (uintptr_t)src_dev) & 15) return fail(CML_ERR_INVALID, "cml_copy_dev needs 16-byte aligned pointers and size");
    const size_t n16 = nbytes / 16;
    const unsigned blocks = (unsigned)std::min<size_t>((n16 + 255) / 256, 256u * 32u);
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), (uint4 *)dst_dev, (const uint4 *)src_dev, n16);
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_calibrate_read(const void *src_dev, size_t nbytes, int in_flight, int workgroups, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (nbytes == 0) return CML_OK;
    if (!src_dev) return fail(CML_ERR_INVALID, "null pointer");
    if ((nbytes | reinterpret_cast<uintptr_t>(src_dev)) & 15) return fail(CML_ERR_INVALID, "cml_calibrate_read needs a 16-byte aligned pointer and size");
    const size_t n16 = nbytes / 16;
    if (workgroups <= 0) workgroups = 2048;
    const dim3 grid(static_cast<unsigned>(std::min<size_t>((n16 + 255) / 256, static_cast<size_t>(workgroups)))), block(256);
    const uint4 *src = static_cast<const uint4 *>(src_dev);
    switch (in_flight) {
        case 1: hipLaunchKernelGGL(read_kernel<1>, grid, block, 0, as_stream(stream), src, n16, nullptr); break;
        case 2: hipLaunchKernelGGL(read_kernel<2>, grid, block, 0, as_stream(stream), src, n16, nullptr); break;
        case 8: hipLaunchKernelGGL(read_kernel<8>, grid, block, 0, as_stream(stream), src, n16, nullptr); break;
        case 4: hipLaunchKernelGGL(read_kernel<4>, grid, block, 0, as_stream(stream), src, n16, nullptr); break;
        default: return fail(CML_ERR_INVALID, "in_flight must be 1, 2, 4 or 8");
    }
    CML_HIP_TRY(hipGetLastError());
    return CML_OK;
}

int cml_calibrate_weight_loads(const cml_weight *w, void *scratch_dev, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (w->fmt != CML_Q4_K) return fail(CML_ERR_UNSUPPORTED, "the loads-only twin exists for the Q4_K matvec");
    return launch_gemv_q4k_loads_only(w, static_cast<float *>(scratch_dev), as_stream(stream));
}

int cml_calibrate_matvec_ablation(const cml_weight *w, const float *x_dev, float *out_dev, int mask, cml_stream_t stream) {
    if (!w || !x_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (int rc = check_ready()) return rc;
    if (w->fmt != CML_Q4_K) return fail(CML_ERR_UNSUPPORTED, "the ablated launches exist for the Q4_K matvec");
    return launch_gemv_q4k_ablated(w, x_dev, out_dev, mask, as_stream(stream));
}

int cml_stream_sync(cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    CML_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return CML_OK;
}

int cml_stream_create(cml_stream_t *out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    if (int rc = check_ready()) return rc;
    hipStream_t s;
    CML_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = s;
    return CML_OK;
}

int cml_stream_destroy(cml_stream_t stream) {
    if (!stream) return CML_OK;
    CML_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return CML_OK;
}

int cml_event_create(cml_event_t *out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    if (int rc = check_ready()) return rc;
    hipEvent_t e;
    CML_HIP_TRY(hipEventCreate(&e));
    *out = e;
    return CML_OK;
}

int cml_event_record(cml_event_t event, cml_stream_t stream) {
    if (!event) return fail(CML_ERR_INVALID, "null event");
    CML_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return CML_OK;
}

int cml_event_elapsed_ms(cml_event_t start, cml_event_t stop, float *ms) {
    if (!start || !stop || !ms) return fail(CML_ERR_INVALID, "null pointer");
    CML_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    CML_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return CML_OK;
}

int cml_event_destroy(cml_event_t event) {
    if (!event) return CML_OK;
    CML_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return CML_OK;
}

int cml_graph_begin_capture(cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (!stream) return fail(CML_ERR_INVALID, "capture needs a stream created with cml_stream_create");
    CML_HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return CML_OK;
}

int cml_graph_end_capture(cml_stream_t stream, cml_graph_t *out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    hipGraph_t graph = nullptr;
    CML_HIP_TRY(hipStreamEndCapture(as_stream(stream), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail(CML_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    *out = exec;
    return CML_OK;
}

int cml_graph_launch(cml_graph_t graph, cml_stream_t stream) {
    if (!graph) return fail(CML_ERR_INVALID, "null graph");
    CML_HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), as_stream(stream)));
    return CML_OK;
}

int cml_graph_destroy(cml_graph_t graph) {
    if (!graph) return CML_OK;
    CML_HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
    return CML_OK;
}

// ---- weights ---------------------------------------------------------------------------------------

static int check_weight_shape(int fmt, int64_t rows, int64_t cols, size_t nbytes, int64_t *nb_out) {
    const Geometry g = geometry(fmt);
    if (g.block_values == 0) return fail(CML_ERR_INVALID, "unknown weight format %d", fmt);
    if (rows < 0 || cols <= 0) return fail(CML_ERR_SHAPE, "bad shape %lld x %lld", (long long)rows, (long long)cols);
    if (cols % g.block_values != 0)
        return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of the %d-value block", (long long)cols, g.block_values);
    if (rows > INT32_MAX / 2 || cols > (int64_t)1 << 24) return fail(CML_ERR_SHAPE, "shape too large");
    const int64_t nb = cols / g.block_values;
    const size_t want = static_cast<size_t>(rows) * static_cast<size_t>(nb) * g.block_bytes;
    if (nbytes != want)
        return fail(CML_ERR_SHAPE, "%zu wire bytes given, %zu expected for %lld x %lld", nbytes, want, (long long)rows, (long long)cols);
    *nb_out = nb;
    return CML_OK;
}

static int make_weight(int fmt, int64_t rows, int64_t cols, int64_t nb, cml_weight **out) {
    cml_weight *w = new (std::nothrow) cml_weight();
    if (!w) return fail(CML_ERR_OOM, "host allocation failed");
    w->fmt = fmt;
    w->rows = rows;
    w->cols = cols;
    w->nb = nb;
    size_t offset[4], total = 0;
    int64_t stride[4];
    plane_layout(fmt, rows, nb, stride, offset, &total);
    void *base = nullptr;
    hipError_t e = hipMalloc(&base, total ? total : 256);
    if (e != hipSuccess) {
        delete w;
        return fail(e == hipErrorOutOfMemory ? CML_ERR_OOM : CML_ERR_HIP, "hipMalloc(%zu) failed: %s", total, hipGetErrorString(e));
    }
    w->allocation = base;
    w->allocation_bytes = total;
    for (int i = 0; i < 4; i++) {
        w->planes.p[i] = static_cast<uint8_t *>(base) + offset[i];
        w->planes.row_stride[i] = stride[i];
    }
    *out = w;
    return CML_OK;
}

int cml_weight_upload_dev(int fmt, int64_t rows, int64_t cols, const void *wire_dev, size_t nbytes,
                          cml_stream_t stream, cml_weight **out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    if (int rc = check_ready()) return rc;
    int64_t nb = 0;
    if (int rc = check_weight_shape(fmt, rows, cols, nbytes, &nb)) return rc;
    if (!wire_dev && nbytes) return fail(CML_ERR_INVALID, "null wire pointer");
    cml_weight *w = nullptr;
    if (int rc = make_weight(fmt, rows, cols, nb, &w)) return rc;
    int rc = launch_wire_to_planes(fmt, static_cast<const uint8_t *>(wire_dev), rows, nb, w->planes, as_stream(stream));
    if (rc != CML_OK) {
        cml_weight_free(w);
        return rc;
    }
    *out = w;
    return CML_OK;
}

int cml_weight_upload(int fmt, int64_t rows, int64_t cols, const void *wire_host, size_t nbytes, cml_weight **out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    if (int rc = check_ready()) return rc;
    int64_t nb = 0;
    if (int rc = check_weight_shape(fmt, rows, cols, nbytes, &nb)) return rc;
    if (!wire_host && nbytes) return fail(CML_ERR_INVALID, "null wire pointer");
    void *staging = nullptr;
    CML_HIP_TRY(hipMalloc(&staging, nbytes ? nbytes : 16));
    hipError_t e = nbytes ? hipMemcpy(staging, wire_host, nbytes, hipMemcpyHostToDevice) : hipSuccess;
    int rc = CML_OK;
    if (e != hipSuccess) rc = fail(CML_ERR_HIP, "hipMemcpy failed: %s", hipGetErrorString(e));
    if (rc == CML_OK) rc = cml_weight_upload_dev(fmt, rows, cols, staging, nbytes, nullptr, out);
    if (rc == CML_OK) {
        e = hipStreamSynchronize(nullptr);
        if (e != hipSuccess) rc = fail(CML_ERR_HIP, "re-layout failed: %s", hipGetErrorString(e));
    }
    (void)hipFree(staging);
    if (rc != CML_OK && *out) {
        cml_weight_free(*out);
        *out = nullptr;
    }
    return rc;
}

int cml_weight_slice(const cml_weight *parent, int64_t row_start, int64_t rows, cml_weight **out) {
    if (!out) return fail(CML_ERR_INVALID, "null out pointer");
    *out = nullptr;
    if (!parent) return fail(CML_ERR_INVALID, "null weight");
    if (row_start < 0 || rows < 0 || row_start + rows > parent->rows)
        return fail(CML_ERR_SHAPE, "rows [%lld, %lld) outside 0..%lld", (long long)row_start, (long long)(row_start + rows), (long long)parent->rows);
    cml_weight *w = new (std::nothrow) cml_weight(*parent);
    if (!w) return fail(CML_ERR_OOM, "host allocation failed");
    w->allocation = nullptr;
    w->allocation_bytes = 0;
    w->rows = rows;
    if (parent->fmt == CML_Q4_K) {
        // tiles are 2304-byte chunks inside each super-block slab; a band that starts inside a
        // tile keeps the tile and skips its leading rows
        const int64_t first = parent->row_skip + row_start;
        w->planes.p[0] += (first / 16) * 2304;
        w->row_skip = static_cast<int>(first % 16);
    } else {
        for (int i = 0; i < 4; i++)
            if (w->planes.p[i]) w->planes.p[i] += row_start * w->planes.row_stride[i];
    }
    *out = w;
    return CML_OK;
}

int cml_weight_info(const cml_weight *w, int *fmt, int64_t *rows, int64_t *cols, size_t *wire_bytes) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (fmt) *fmt = w->fmt;
    if (rows) *rows = w->rows;
    if (cols) *cols = w->cols;
    if (wire_bytes) *wire_bytes = static_cast<size_t>(w->rows) * w->nb * geometry(w->fmt).block_bytes;
    return CML_OK;
}

int cml_weight_download(const cml_weight *w, void *wire_host, size_t nbytes) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    const size_t want = static_cast<size_t>(w->rows) * w->nb * geometry(w->fmt).block_bytes;
    if (nbytes != want) return fail(CML_ERR_SHAPE, "%zu bytes given, %zu expected", nbytes, want);
    if (want == 0) return CML_OK;
    if (!wire_host) return fail(CML_ERR_INVALID, "null pointer");
    void *staging = nullptr;
    CML_HIP_TRY(hipMalloc(&staging, want));
    int rc = launch_planes_to_wire(w->fmt, w->planes, w->rows, w->nb, w->row_skip, static_cast<uint8_t *>(staging), nullptr);
    if (rc == CML_OK) {
        hipError_t e = hipMemcpy(wire_host, staging, want, hipMemcpyDeviceToHost);
        if (e != hipSuccess) rc = fail(CML_ERR_HIP, "hipMemcpy failed: %s", hipGetErrorString(e));
    }
    (void)hipFree(staging);
    return rc;
}

void cml_weight_free(cml_weight *w) {
    if (!w) return;
    if (w->allocation) (void)hipFree(w->allocation);
    delete w;
}

static bool misaligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

// ---- activation quantizers ------------------------------------------------------------------------

int cml_quantize_q8_0(const float *x_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev, float *scales_dev,
                      cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0 || cols < 0 || cols % 32 != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of 32", (long long)cols);
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (!x_dev || !q_dev || !scales_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || (reinterpret_cast<uintptr_t>(q_dev) & 3u)) return fail(CML_ERR_INVALID, "x must be 16-byte and q 4-byte aligned");
    return launch_quantize_q8_0(x_dev, n_tokens, cols, q_dev, scales_dev, as_stream(stream));
}

int cml_quantize_q8_k(const float *x_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev, float *d_dev,
                      cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0 || cols < 0 || cols % 256 != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of 256", (long long)cols);
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (!x_dev || !q_dev || !d_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || (reinterpret_cast<uintptr_t>(q_dev) & 3u)) return fail(CML_ERR_INVALID, "x must be 16-byte and q 4-byte aligned");
    return launch_quantize_q8_k(x_dev, n_tokens, cols, q_dev, d_dev, as_stream(stream));
}

int cml_rms_norm_quantize(int act, const float *x_dev, const float *weight_dev, float eps, int64_t n_tokens, int64_t cols,
                          float *normed_dev, int8_t *q_dev, float *scales_dev, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (act != CML_ACT_F32 && act != CML_ACT_Q8_0 && act != CML_ACT_Q8_K) return fail(CML_ERR_INVALID, "unknown activation format %d", act);
    const int64_t unit = act == CML_ACT_Q8_K ? 256 : (act == CML_ACT_Q8_0 ? 32 : 4);
    if (n_tokens < 0 || cols < 0 || cols % unit != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of %lld", (long long)cols, (long long)unit);
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (!x_dev || !weight_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (act == CML_ACT_F32 ? !normed_dev : (!q_dev || !scales_dev)) return fail(CML_ERR_INVALID, "null output pointer");
    if (misaligned16(x_dev) || misaligned16(weight_dev) || (normed_dev && misaligned16(normed_dev)) ||
        (act != CML_ACT_F32 && (reinterpret_cast<uintptr_t>(q_dev) & 3u)))
        return fail(CML_ERR_INVALID, "x, weight and normed must be 16-byte and q 4-byte aligned");
    return launch_rms_norm_quantize(act, x_dev, weight_dev, eps, n_tokens, cols, normed_dev, q_dev, scales_dev, as_stream(stream));
}

int cml_sum_squares_f32(const float *x_dev, int64_t n_rows, int64_t cols, float *out_dev, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (n_rows < 0 || cols < 0 || cols % 4 != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of 4", (long long)cols);
    if (n_rows == 0) return CML_OK;
    if (!x_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev)) return fail(CML_ERR_INVALID, "x must be 16-byte aligned");
    if (cols == 0) return cml_memset_dev(out_dev, 0, static_cast<size_t>(n_rows) * 4, stream);
    return launch_rms_norm_quantize(3, x_dev, nullptr, 0.0f, n_rows, cols, out_dev, nullptr, nullptr, as_stream(stream));
}

int cml_rms_inv_norm_quantize(int act, const float *x_dev, const float *weight_dev, float rms_inv, int64_t cols, int8_t *q_dev,
                              float *scales_dev, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (act != CML_ACT_Q8_0 && act != CML_ACT_Q8_K) return fail(CML_ERR_INVALID, "activation format %d is not a quantized one", act);
    const int64_t unit = act == CML_ACT_Q8_K ? 256 : 32;
    if (cols < 0 || cols % unit != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of %lld", (long long)cols, (long long)unit);
    if (cols == 0) return CML_OK;
    if (!x_dev || !weight_dev || !q_dev || !scales_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || misaligned16(weight_dev) || (reinterpret_cast<uintptr_t>(q_dev) & 3u))
        return fail(CML_ERR_INVALID, "x and weight must be 16-byte and q 4-byte aligned");
    return launch_rms_inv_norm_quantize(act, x_dev, weight_dev, rms_inv, cols, q_dev, scales_dev, as_stream(stream));
}

int cml_silu_mul_quantize(int act, const float *gate_dev, const float *up_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev,
                          float *scales_dev, cml_stream_t stream) {
    return cml_glu_quantize(CML_GLU_SILU, act, gate_dev, up_dev, n_tokens, cols, q_dev, scales_dev, stream);
}

int cml_glu_quantize(int glu, int act, const float *gate_dev, const float *up_dev, int64_t n_tokens, int64_t cols, int8_t *q_dev,
                     float *scales_dev, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (glu != CML_GLU_SILU && glu != CML_GLU_GELU_TANH) return fail(CML_ERR_INVALID, "unknown activation %d", glu);
    if (act != CML_ACT_Q8_0 && act != CML_ACT_Q8_K) return fail(CML_ERR_INVALID, "activation format %d is not a quantized one", act);
    const int64_t unit = act == CML_ACT_Q8_K ? 256 : 32;
    if (n_tokens < 0 || cols < 0 || cols % unit != 0) return fail(CML_ERR_SHAPE, "cols %lld is not a multiple of %lld", (long long)cols, (long long)unit);
    if (n_tokens == 0 || cols == 0) return CML_OK;
    if (!gate_dev || !up_dev || !q_dev || !scales_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(gate_dev) || misaligned16(up_dev) || (reinterpret_cast<uintptr_t>(q_dev) & 3u))
        return fail(CML_ERR_INVALID, "gate and up must be 16-byte and q 4-byte aligned");
    return launch_glu_quantize(glu, act, gate_dev, up_dev, n_tokens, cols, cols, q_dev, scales_dev, as_stream(stream));
}

int cml_dequantize(const cml_weight *w, float *out_dev, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (w->rows == 0) return CML_OK;
    if (!out_dev) return fail(CML_ERR_INVALID, "null pointer");
    return launch_dequantize(w, out_dev, as_stream(stream));
}

int cml_embed_gather(const cml_weight *table, const uint32_t *token_ids_dev, int64_t n_tokens, float *out_dev, cml_stream_t stream) {
    if (!table) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0) return fail(CML_ERR_SHAPE, "negative token count");
    if (n_tokens == 0 || table->cols == 0) return CML_OK;
    if (!token_ids_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    return launch_embed_gather(table, token_ids_dev, n_tokens, out_dev, as_stream(stream));
}

int cml_argmax_f32(const float *logits_dev, int64_t n_rows, int64_t n, uint32_t *out_idx_dev, cml_stream_t stream) {
    if (int rc = check_ready()) return rc;
    if (n_rows < 0 || n <= 0 || n > INT32_MAX) return fail(CML_ERR_SHAPE, "argmax over %lld rows of %lld values", (long long)n_rows, (long long)n);
    if (n_rows == 0) return CML_OK;
    if (!logits_dev || !out_idx_dev) return fail(CML_ERR_INVALID, "null pointer");
    return launch_argmax_f32(logits_dev, n_rows, n, out_idx_dev, as_stream(stream));
}

// ---- matvec / matmul --------------------------------------------------------------------------------

// The packed-dot kernels serve 8, 4, 2 or 1 tokens per pass over the weight: 3, 5, 6 and 7 tokens
// are two or three passes, and one pass of the matrix-core kernel beats them even below the batch
// size from which it wins pass for pass (measured: Q4_0 128256x3072, 3 tokens 73 -> 55 us; Q4_K
// 14336x4096, 3 tokens 17.0 -> 12.0 us).  A forced threshold (the tuning knobs) is taken as is.
static bool mfma_pays(int64_t n, int min_tokens, const char *knob) {
    if (n >= min_tokens) return true;
    if (env_int(knob, 0) > 0) return false;
    return n == 3 || (n >= 5 && n <= 7);
}

static int dispatch(const MatArgs &a, hipStream_t st) {
    int rc;
    switch (a.w->fmt) {
        case CML_Q4_K:
            // int8 matrix cores for the batched shapes (speculative-verify / prefill); packed dot below.
            // (A residual only comes with single-token calls; the matrix-core kernels do not add one,
            // so such a call stays on the packed-dot kernel whatever the thresholds say.)
            // Measured on MI355X at 14336x4096: the matrix-core kernel takes 12 us for any batch up to
            // 16 tokens, the packed-dot kernel 7.2 / 9.9 us for 1 / 2 tokens and two launches for 3.
            if (!a.group_offsets && !a.ints && !a.residual && !q4k_lane_order() && a.n_tokens >= env_int("CAMELID_HIP_Q4K_MFMA_MIN_TOKENS", 3))
                rc = launch_gemm_q4k_mfma(a, st);
            else
                rc = launch_gemv_q4k(a, st);
            if (rc == CML_ERR_UNSUPPORTED && !a.group_offsets && a.n_tokens > 1) {
                // rows too long for the matrix-core kernel's LDS staging (it refuses before it
                // launches anything): the packed-dot kernel serves them in passes of fewer tokens
                clear_error();
                rc = launch_gemv_q4k(a, st);
            }
            break;
        case CML_Q8_0:
        case CML_Q4_0:
            // the same split for the 32-value-block formats (rows of whole 256-value slabs)
            if (!a.group_offsets && !a.ints && !a.residual && mfma_pays(a.n_tokens, b32_mfma_min_tokens(a.w->rows), "CAMELID_HIP_B32_MFMA_MIN_TOKENS") && b32_mfma_usable(a.w))
                rc = launch_gemm_b32_mfma(a, st);
            else
                rc = a.w->fmt == CML_Q8_0 ? launch_gemv_q8_0(a, st) : launch_gemv_q4_0(a, st);
            if (rc == CML_ERR_UNSUPPORTED && !a.group_offsets && a.n_tokens > 1) {
                clear_error();
                rc = a.w->fmt == CML_Q8_0 ? launch_gemv_q8_0(a, st) : launch_gemv_q4_0(a, st);
            }
            break;
        case CML_Q6_K:
            if (!a.group_offsets && !a.ints && !a.residual && !q6k_lane_order() &&
                mfma_pays(a.n_tokens, q6k_mfma_min_tokens(a.w->rows, a.w->nb), "CAMELID_HIP_Q6K_MFMA_MIN_TOKENS"))
                rc = launch_gemm_q6k_mfma(a, st);
            else
                rc = launch_gemv_q6k(a, st);
            if (rc == CML_ERR_UNSUPPORTED && !a.group_offsets && a.n_tokens > 1) {
                clear_error();
                rc = launch_gemv_q6k(a, st);
            }
            break;
        default: return fail(CML_ERR_INVALID, "unknown weight format %d", a.w->fmt);
    }
    if (rc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
    return rc;
}

static MatArgs plain_args(const cml_weight *w, const int8_t *q, const float *s, int64_t n_tokens, float *out) {
    MatArgs a{};
    a.w = w;
    a.q = q;
    a.scales = s;
    a.n_tokens = n_tokens;
    a.out = out;
    a.residual = nullptr;
    a.ints = nullptr;
    a.group_offsets = nullptr;
    a.group_rows = nullptr;
    a.n_groups = 1;
    a.band_rows = 0;
    return a;
}

int cml_gemv(const cml_weight *w, const int8_t *q_dev, const float *scales_dev, float *out_dev,
             const float *residual_dev, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (w->rows == 0) return CML_OK;
    if (!q_dev || !scales_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(q_dev)) return fail(CML_ERR_INVALID, "activation quants must be 16-byte aligned");
    MatArgs a = plain_args(w, q_dev, scales_dev, 1, out_dev);
    a.residual = residual_dev;
    return dispatch(a, as_stream(stream));
}

int cml_gemm(const cml_weight *w, const int8_t *q_dev, const float *scales_dev, int64_t n_tokens, float *out_dev,
             cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0) return fail(CML_ERR_SHAPE, "negative token count");
    if (w->rows == 0 || n_tokens == 0) return CML_OK;
    if (!q_dev || !scales_dev || !out_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(q_dev)) return fail(CML_ERR_INVALID, "activation quants must be 16-byte aligned");
    return dispatch(plain_args(w, q_dev, scales_dev, n_tokens, out_dev), as_stream(stream));
}

int cml_block_dots(const cml_weight *w, const int8_t *q_dev, int32_t *ints_dev, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (w->rows == 0) return CML_OK;
    if (!q_dev || !ints_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(q_dev)) return fail(CML_ERR_INVALID, "activation quants must be 16-byte aligned");
    // The integers do not depend on the activation scales; run the real gemv
    // kernel with zero scales into a scratch output and keep its integers.
    float *scratch = nullptr;
    const size_t n_scales = static_cast<size_t>(w->nb);
    CML_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&scratch), (n_scales + static_cast<size_t>(w->rows)) * sizeof(float)));
    hipStream_t st = as_stream(stream);
    int rc = CML_OK;
    hipError_t e = hipMemsetAsync(scratch, 0, n_scales * sizeof(float), st);
    if (e != hipSuccess) rc = fail(CML_ERR_HIP, "hipMemsetAsync failed: %s", hipGetErrorString(e));
    if (rc == CML_OK) {
        MatArgs a = plain_args(w, q_dev, scratch, 1, scratch + n_scales);
        a.ints = ints_dev;
        rc = dispatch(a, st);
    }
    if (rc == CML_OK) {
        e = hipStreamSynchronize(st);
        if (e != hipSuccess) rc = fail(CML_ERR_HIP, "block-dot kernel failed: %s", hipGetErrorString(e));
    }
    (void)hipFree(scratch);
    return rc;
}

size_t cml_matmul_workspace_bytes(int fmt, int64_t cols, int64_t n_tokens) {
    const Geometry g = geometry(fmt);
    if (g.block_values == 0 || cols <= 0 || n_tokens <= 0) return 0;
    const int64_t per = is_k_family(fmt) ? 256 : 32;
    const size_t q = (static_cast<size_t>(n_tokens) * cols + 255) & ~size_t(255);
    const size_t s = (static_cast<size_t>(n_tokens) * (cols / per) * 4 + 255) & ~size_t(255);
    return q + s;
}

int cml_matmul_f32(const cml_weight *w, const float *x_dev, int64_t n_tokens, float *out_dev, void *workspace_dev,
                   size_t workspace_bytes, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0) return fail(CML_ERR_SHAPE, "negative token count");
    if (w->rows == 0 || n_tokens == 0) return CML_OK;
    if (!x_dev || !out_dev || !workspace_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || misaligned16(workspace_dev)) return fail(CML_ERR_INVALID, "activations and workspace must be 16-byte aligned");
    const size_t need = cml_matmul_workspace_bytes(w->fmt, w->cols, n_tokens);
    if (workspace_bytes < need) return fail(CML_ERR_SHAPE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    int8_t *q = static_cast<int8_t *>(workspace_dev);
    float *s = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace_dev) +
                                         ((static_cast<size_t>(n_tokens) * w->cols + 255) & ~size_t(255)));
    hipStream_t st = as_stream(stream);
    const int fuse = env_int("CAMELID_HIP_FUSED_QUANT", 1);  // 0 = never, 1 = by shape, 2 = whenever possible
    const bool fuse_two = n_tokens == 2 && env_int("CAMELID_HIP_FUSED_QUANT_TWO", 1) && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0);
    if (w->fmt == CML_Q4_K && !q4k_lane_order() && (n_tokens == 1 || fuse_two) &&
        (fuse == 2 || (fuse == 1 && (w->nb <= 32 || gemv_q4k_long_rows_fuse(w, static_cast<int>(n_tokens)))))) {
        // rows of up to 8192 values (and the longer rows the one-launch K-cut forms serve): one launch quantizes the activation in every workgroup (one or
        // two passes of its four waves; twice that for a pair of tokens) and runs the matvec
        // (4096 x 8192: 7.1 -> 6.6 us, 2048 x 8192: 6.3 -> 4.7); at 14336 values the passes cost
        // what the second launch does (4096 x 14336: 9.6 -> 10.0) and the two launches below stay
        const int frc = launch_gemv_q4k_f32(w, x_dev, out_dev, st, static_cast<int>(n_tokens));
        if (frc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
        return frc;
    }
    // (not on a vocabulary-sized weight: there the matrix-core kernel that walks the weight with one resident
    // workgroup per compute unit takes 55 us for 3 to 8 tokens at 128256 x 4096, quantizing launch included,
    // against 58 / 68 us here for 3 / 4; at 24576 x 4096 this launch is ahead, 11.9 against 17 us for 3)
    const int64_t q4k_sbs = w->rows * w->nb;
    const bool tall_for_tokens = w->nb <= 16 && q4k_sbs >= (n_tokens == 4 ? int64_t(49152) * 16 : int64_t(98304) * 16) &&
                                 env_int("CAMELID_HIP_Q4K_TALL_TOKENS_MFMA", 1);
    if (w->fmt == CML_Q4_K && !q4k_lane_order() && (n_tokens == 3 || n_tokens == 4) && fuse != 0 && !tall_for_tokens &&
        (w->nb <= 32 || gemv_q4k_long_rows_fuse(w, static_cast<int>(n_tokens))) && !env_int("CAMELID_HIP_Q4K_GENERAL_ENTRY", 0)) {
        // three or four tokens on rows of 4096 values with no K cut: the eight-wave packed-dot launch replays each
        // step's unpacked weight against the tokens (one launch, quantizer inside); -1 = not such a shape
        const int frc = launch_gemv_q4k_f32(w, x_dev, out_dev, st, static_cast<int>(n_tokens));
        if (frc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
        if (frc != -1) return frc;
    }
    if (w->fmt == CML_Q4_K && !q4k_lane_order() && n_tokens >= 3 && fuse != 0 && env_int("CAMELID_HIP_FUSED_QUANT_BATCH", 1)) {
        // 3 to 6 tokens on the matrix cores: the workgroups quantize the few rows themselves (14336 x 4096,
        // 4 tokens: 12.4 -> 11.0 us per step); more tokens cost every workgroup more than the launch saves
        const int frc = launch_gemm_q4k_mfma_f32(w, x_dev, n_tokens, out_dev, st);
        if (frc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
        if (frc != -1) return frc;
    }
    if (w->fmt == CML_Q6_K && (n_tokens == 1 || fuse_two) && env_int("CAMELID_HIP_Q6K_FUSED_QUANT", 1) && !q6k_lane_order() &&
        (fuse == 2 || (fuse == 1 && ((w->nb <= 32 && w->rows <= (n_tokens == 1 ? 98304 : 32768)) || (n_tokens == 1 && gemv_q6k_long_rows_fuse(w)))))) {
        // the same for Q6_K: 4096 x 4096 7.0 -> 5.5 us, 14336 x 4096 12.3 -> 10.8, 65536 x 4096 36.1 -> 34.5; not on
        // the largest vocabulary heads, whose 4008 workgroups would each quantize the row (128256 x 3072: 49.5 either
        // way, 128256 x 4096 67.5 / 67.3; two tokens 53.3 -> 57.2).  A launch of about the resident workgroups, each
        // quantizing once and walking every n-th group of row tiles, measured slower there (50.7 - 53.7 us for 512 - 2048).
        const int frc = launch_gemv_q6k_f32(w, x_dev, out_dev, st, static_cast<int>(n_tokens));
        if (frc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
        return frc;
    }
    if ((w->fmt == CML_Q8_0 || w->fmt == CML_Q4_0) && (n_tokens == 1 || fuse_two) &&
        (fuse == 2 || (fuse == 1 && (w->cols <= 8192 || (n_tokens == 1 && gemv_b32_long_rows_fuse(w))) && (n_tokens == 1 || w->rows <= 32768)))) {
        // the same for the 32-value block formats (8192x2048: 7.6 -> 5.9 us per step).  One token: on every row
        // count -- with eight- and sixteen-wave workgroups the quantizer hides on a vocabulary head too (128256 x 3072:
        // Q8_0 62.3 -> 59.7 us, Q4_0 35.7 -> 34.4; 151936 x 3584 Q8_0 83.5 -> 81.4).  Two tokens: up to 32768 rows
        // (128256 x 3072 Q4_0: 42.3 us in two launches, 51.4 in one)
        const int frc = launch_gemv_b32_f32(w, x_dev, out_dev, st, static_cast<int>(n_tokens));
        if (frc == CML_OK) g_runs.fetch_add(1, std::memory_order_relaxed);
        return frc;
    }
    int rc = is_k_family(w->fmt) ? launch_quantize_q8_k(x_dev, n_tokens, w->cols, q, s, st)
                                 : launch_quantize_q8_0(x_dev, n_tokens, w->cols, q, s, st);
    if (rc != CML_OK) return rc;
    return dispatch(plain_args(w, q, s, n_tokens, out_dev), st);
}

// One token against TWO weights of one shape that read the same activation (gate and up of a dense
// FFN): Q4_K rows of up to 8192 values run as one launch that quantizes the token once per
// workgroup and streams both weights (grid.z = 2); every other case is two cml_matmul_f32 calls.
// Same bits as the two calls.
int cml_matmul_f32_pair(const cml_weight *w_a, const cml_weight *w_b, const float *x_dev, float *out_a_dev, float *out_b_dev,
                        void *workspace_dev, size_t workspace_bytes, cml_stream_t stream) {
    if (!w_a || !w_b) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (w_a->cols != w_b->cols) return fail(CML_ERR_SHAPE, "the two weights read activations of %lld and %lld values", (long long)w_a->cols, (long long)w_b->cols);
    if (!x_dev || !out_a_dev || !out_b_dev || !workspace_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || misaligned16(workspace_dev)) return fail(CML_ERR_INVALID, "activations and workspace must be 16-byte aligned");
    const bool same_shape = w_a->fmt == w_b->fmt && w_a->rows == w_b->rows && w_a->nb == w_b->nb && w_a->row_skip == w_b->row_skip &&
                            w_a->planes.row_stride[0] == w_b->planes.row_stride[0];
    const int fuse = env_int("CAMELID_HIP_FUSED_QUANT", 1);
    if (same_shape && w_a->rows > 0 && w_a->fmt == CML_Q4_K && !q4k_lane_order() && (fuse == 2 || (fuse == 1 && w_a->nb <= 32)) &&
        env_int("CAMELID_HIP_PAIR_LAUNCH", 1)) {
        const int frc = launch_gemv_q4k_f32_pair(w_a, w_b, x_dev, out_a_dev, out_b_dev, as_stream(stream));
        if (frc == CML_OK) g_runs.fetch_add(2, std::memory_order_relaxed);
        return frc;
    }
    if (same_shape && w_a->rows > 0 && (w_a->fmt == CML_Q8_0 || w_a->fmt == CML_Q4_0) && w_a->planes.row_stride[1] == w_b->planes.row_stride[1] &&
        (fuse == 2 || (fuse == 1 && w_a->cols <= 8192 && w_a->rows <= 32768)) && env_int("CAMELID_HIP_PAIR_LAUNCH", 1)) {
        int frc = launch_gemv_b32_f32_pair(w_a, w_b, x_dev, out_a_dev, out_b_dev, as_stream(stream));
        if (frc == -1) {
            // a shape the pair launch (16 lanes per row, up to two float4 of the token per thread) does not take: the multi launch
            const cml_weight *const ws[2] = {w_a, w_b};
            float *const outs[2] = {out_a_dev, out_b_dev};
            frc = launch_gemv_b32_f32_multi(ws, 2, x_dev, outs, as_stream(stream));
        }
        if (frc == CML_OK) g_runs.fetch_add(2, std::memory_order_relaxed);
        if (frc != -1) return frc;
    }
    if (same_shape && w_a->rows > 0 && w_a->fmt == CML_Q6_K && !q6k_lane_order() && env_int("CAMELID_HIP_Q6K_FUSED_QUANT", 1) &&
        (fuse == 2 || (fuse == 1 && w_a->nb <= 32)) && env_int("CAMELID_HIP_PAIR_LAUNCH", 1)) {
        // Q6_K: the multi launch of two weights (gate and up of 14336 x 4096: 21.2 -> 19.0 us)
        const cml_weight *const ws[2] = {w_a, w_b};
        float *const outs[2] = {out_a_dev, out_b_dev};
        const int frc = launch_gemv_q6k_f32_multi(ws, 2, x_dev, outs, as_stream(stream));
        if (frc == CML_OK) g_runs.fetch_add(2, std::memory_order_relaxed);
        if (frc != -1) return frc;
    }
    if (int rc = cml_matmul_f32(w_a, x_dev, 1, out_a_dev, workspace_dev, workspace_bytes, stream)) return rc;
    return cml_matmul_f32(w_b, x_dev, 1, out_b_dev, workspace_dev, workspace_bytes, stream);
}

// One token against SEVERAL weights that read the same activation (the q, k and v projections of an attention block,
// gate and up of an FFN: the projections the reference hangs off one SharedActivation, src/gemma4_runtime.rs:1288-1340).
// Groups of up to four Q4_K weights of one row length and one K cut run as one launch; everything else as calls of
// their own.  Same bits as n cml_matmul_f32 calls.
int cml_matmul_f32_multi(const cml_weight *const *weights, int n_weights, const float *x_dev, float *const *outs_dev, void *workspace_dev,
                         size_t workspace_bytes, cml_stream_t stream) {
    if (n_weights < 0) return fail(CML_ERR_SHAPE, "negative weight count");
    if (n_weights == 0) return CML_OK;
    if (!weights || !outs_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (int rc = check_ready()) return rc;
    for (int j = 0; j < n_weights; j++) {
        if (!weights[j] || !outs_dev[j]) return fail(CML_ERR_INVALID, "null weight or output %d", j);
        if (weights[j]->cols != weights[0]->cols)
            return fail(CML_ERR_SHAPE, "weights 0 and %d read activations of %lld and %lld values", j, (long long)weights[0]->cols, (long long)weights[j]->cols);
    }
    if (!x_dev || !workspace_dev) return fail(CML_ERR_INVALID, "null pointer");
    if (misaligned16(x_dev) || misaligned16(workspace_dev)) return fail(CML_ERR_INVALID, "activations and workspace must be 16-byte aligned");
    const int fuse = env_int("CAMELID_HIP_FUSED_QUANT", 1);
    int j = 0;
    while (j < n_weights) {
        // the longest run of up to four weights, starting here, that one launch serves
        int served = 0;
        if (weights[j]->fmt == CML_Q4_K && !q4k_lane_order() && (fuse == 2 || (fuse == 1 && weights[j]->nb <= 32))) {
            for (int take = std::min(4, n_weights - j); take >= 2 && !served; take--) {
                const int frc = launch_gemv_q4k_f32_multi(weights + j, take, x_dev, outs_dev + j, as_stream(stream));
                if (frc == CML_OK) served = take;
                else if (frc != -1) return frc;
            }
        }
        if (!served && (weights[j]->fmt == CML_Q8_0 || weights[j]->fmt == CML_Q4_0) && (fuse == 2 || (fuse == 1 && weights[j]->cols <= 8192))) {
            // the same for the 32-value block formats (q | k | v of one attention block)
            for (int take = std::min(4, n_weights - j); take >= 2 && !served; take--) {
                const int frc = launch_gemv_b32_f32_multi(weights + j, take, x_dev, outs_dev + j, as_stream(stream));
                if (frc == CML_OK) served = take;
                else if (frc != -1) return frc;
            }
        }
        if (!served && weights[j]->fmt == CML_Q6_K && !q6k_lane_order() && env_int("CAMELID_HIP_Q6K_FUSED_QUANT", 1) &&
            (fuse == 2 || (fuse == 1 && weights[j]->nb <= 32))) {
            // and for Q6_K sets whose shapes take one K cut
            for (int take = std::min(4, n_weights - j); take >= 2 && !served; take--) {
                const int frc = launch_gemv_q6k_f32_multi(weights + j, take, x_dev, outs_dev + j, as_stream(stream));
                if (frc == CML_OK) served = take;
                else if (frc != -1) return frc;
            }
        }
        if (served) {
            g_runs.fetch_add(static_cast<uint64_t>(served), std::memory_order_relaxed);
            j += served;
            continue;
        }
        if (int rc = cml_matmul_f32(weights[j], x_dev, 1, outs_dev[j], workspace_dev, workspace_bytes, stream)) return rc;
        j++;
    }
    return CML_OK;
}

// The same call for hosts that may not allocate (a stream under graph capture, a serving loop with
// a fixed memory budget): the quantized activation is staged in the library's own static device
// array instead of a caller workspace.  Nothing here allocates or frees, on the host or the device.
int cml_matmul_f32_static(const cml_weight *w, const float *x_dev, int64_t n_tokens, float *out_dev, cml_stream_t stream) {
    if (!w) return fail(CML_ERR_INVALID, "null weight");
    if (int rc = check_ready()) return rc;
    if (n_tokens < 0) return fail(CML_ERR_SHAPE, "negative token count");
    const int device = g_device.load(std::memory_order_acquire);
    void *ws = device < kMaxDevices ? g_static_workspace[device] : nullptr;
    if (!ws) return fail(CML_ERR_UNAVAILABLE, "device %d has no static workspace", device);
    const size_t need = cml_matmul_workspace_bytes(w->fmt, w->cols, n_tokens);
    if (need > kStaticWorkspaceBytes)
        return fail(CML_ERR_SHAPE, "%lld tokens of %lld values need %zu bytes of staging; the static workspace holds %zu",
                    (long long)n_tokens, (long long)w->cols, need, kStaticWorkspaceBytes);
    return cml_matmul_f32(w, x_dev, n_tokens, out_dev, ws, kStaticWorkspaceBytes, stream);
}

// ---- host-slice seam ----------------------------------------------------------------------------------

// Activations down, one dispatch, outputs up; synchronous.  g_mutex is held by the caller.
static int run_host_seam(const cml_weight *w, const float *input_scales, const int8_t *input_quants, int64_t input_rows, float *output) {
    const int64_t per = is_k_family(w->fmt) ? 256 : 32;
    const size_t qb = static_cast<size_t>(input_rows) * w->cols;
    const size_t sb = static_cast<size_t>(input_rows) * (w->cols / per) * sizeof(float);
    const size_t ob = static_cast<size_t>(input_rows) * w->rows * sizeof(float);
    const size_t q_off = 0, s_off = (qb + 255) & ~size_t(255), o_off = s_off + ((sb + 255) & ~size_t(255));
    if (o_off + ob > g_seam_bytes) {  // grow-only: a decode loop allocates on its first call, then never again
        if (g_seam_buf) (void)hipFree(g_seam_buf);
        g_seam_buf = nullptr;
        g_seam_bytes = 0;
        const size_t want = ((o_off + ob) * 5 / 4 + 4095) & ~size_t(4095);
        CML_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&g_seam_buf), want));
        g_seam_bytes = want;
    }
    uint8_t *buf = g_seam_buf;
    hipError_t e = hipMemcpyAsync(buf + q_off, input_quants, qb, hipMemcpyHostToDevice, nullptr);
    if (e == hipSuccess) e = hipMemcpyAsync(buf + s_off, input_scales, sb, hipMemcpyHostToDevice, nullptr);
    if (e != hipSuccess) return fail(CML_ERR_HIP, "hipMemcpy failed: %s", hipGetErrorString(e));
    if (int rc = dispatch(plain_args(w, reinterpret_cast<int8_t *>(buf + q_off), reinterpret_cast<float *>(buf + s_off),
                                     input_rows, reinterpret_cast<float *>(buf + o_off)),
                          nullptr))
        return rc;
    e = hipMemcpy(output, buf + o_off, ob, hipMemcpyDeviceToHost);  // synchronises the null stream
    if (e != hipSuccess) return fail(CML_ERR_HIP, "device run failed: %s", hipGetErrorString(e));
    return CML_OK;
}

int cml_try_linear_rows(int fmt, const float *input_scales, const int8_t *input_quants, const uint8_t *weight_wire,
                        size_t weight_nbytes, int64_t input_rows, int64_t weight_rows, int64_t cols, float *output) {
    if (!ready()) {
        if (cml_init(-1) != CML_OK) return CML_ERR_UNAVAILABLE;
    }
    if (!input_scales || !input_quants || !weight_wire || !output) return fail(CML_ERR_INVALID, "null pointer");
    if (input_rows <= 0 || weight_rows <= 0) return fail(CML_ERR_SHAPE, "empty shape");
    const Geometry g = geometry(fmt);
    if (g.block_values == 0) return fail(CML_ERR_INVALID, "unknown weight format %d", fmt);
    std::lock_guard<std::mutex> lock(g_mutex);
    cml_weight *w = nullptr;
    const CacheKey key{weight_wire, weight_nbytes, fmt};
    CML_NOTHROW_BEGIN
    auto it = g_weight_cache.find(key);
    if (it != g_weight_cache.end()) {
        w = it->second;
        if (w->rows != weight_rows || w->cols != cols) return fail(CML_ERR_SHAPE, "cached weight has another shape");
    } else {
        if (int rc = cml_weight_upload(fmt, weight_rows, cols, weight_wire, weight_nbytes, &w)) return rc;
        try {
            g_weight_cache.emplace(key, w);
        } catch (...) {
            cml_weight_free(w);
            throw;
        }
    }
    CML_NOTHROW_END
    return run_host_seam(w, input_scales, input_quants, input_rows, output);
}

int cml_try_q8_0_block_linear_row(const float *input_scales, const int8_t *input_quants, const uint8_t *weight_block_bytes,
                                  size_t weight_nbytes, int64_t rows, int64_t blocks_per_row, float *output) {
    if (!ready()) {
        if (cml_init(-1) != CML_OK) return CML_ERR_UNAVAILABLE;
    }
    if (!input_scales || !input_quants || !weight_block_bytes || !output) return fail(CML_ERR_INVALID, "null pointer");
    if (rows <= 0 || blocks_per_row <= 0) return fail(CML_ERR_SHAPE, "empty shape");
    const size_t n_blocks = static_cast<size_t>(rows) * static_cast<size_t>(blocks_per_row);
    if (weight_nbytes != n_blocks * 36) return fail(CML_ERR_SHAPE, "%zu bytes are not %lld x %lld blocks of 36", weight_nbytes, (long long)rows, (long long)blocks_per_row);
    std::lock_guard<std::mutex> lock(g_mutex);
    cml_weight *w = nullptr;
    const CacheKey key{weight_block_bytes, weight_nbytes, -36};  // the in-memory block layout, not a wire format
    CML_NOTHROW_BEGIN
    auto it = g_weight_cache.find(key);
    if (it != g_weight_cache.end()) {
        w = it->second;
        if (w->rows != rows || w->nb != blocks_per_row) return fail(CML_ERR_SHAPE, "cached weight has another shape");
    } else {
        std::vector<uint8_t> wire(n_blocks * 34);
        if (!q8_0_blocks_to_wire(weight_block_bytes, n_blocks, wire.data()))
            return fail(CML_ERR_UNSUPPORTED, "a block scale is not an f16 value: these blocks did not come from Q8_0 wire bytes");
        if (int rc = cml_weight_upload(CML_Q8_0, rows, blocks_per_row * 32, wire.data(), wire.size(), &w)) return rc;
        try {
            g_weight_cache.emplace(key, w);
        } catch (...) {
            cml_weight_free(w);
            throw;
        }
    }
    CML_NOTHROW_END
    return run_host_seam(w, input_scales, input_quants, 1, output);
}

}  // extern "C"
