// Context, memory, copies, events: the part of the C ABI that owns device state.
#include "common.h"
#include "tuning.h"
#include "ws_ledger.h"

#include <stdlib.h>
#include <string.h>
#include <map>
#include <set>
#include <unordered_map>
#include <vector>

namespace aeth {

static thread_local char g_err[512] = "";

Context& ctx() {
    static Context c;
    return c;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

Tuning& tuning() {
    static Tuning t;
    return t;
}

bool tuning_set(const char* name, int value) {
    Tuning& t = tuning();
    if (name == nullptr) {
        t = Tuning();
        return true;
    }
    struct Field { const char* name; int Tuning::*member; };
    static const Field fields[] = {
        {"gather_bm", &Tuning::gather_bm},       {"gather_kc", &Tuning::gather_kc},
        {"gather_nloop", &Tuning::gather_nloop}, {"gather_halo", &Tuning::gather_halo},
        {"gather_split", &Tuning::gather_split}, {"gather_sa", &Tuning::gather_sa},
        {"gather_wide", &Tuning::gather_wide},   {"gather_res", &Tuning::gather_res},
        {"dense_res", &Tuning::dense_res},       {"direct", &Tuning::direct},
        {"wgrad_halo", &Tuning::wgrad_halo},     {"wgrad_cw", &Tuning::wgrad_cw},
        {"wgrad_wide", &Tuning::wgrad_wide},     {"gather_direct_b", &Tuning::gather_direct_b},
        {"gather_clip", &Tuning::gather_clip},       {"gather_merge", &Tuning::gather_merge},
        {"gather_pairs", &Tuning::gather_pairs},
        {"gather_runs", &Tuning::gather_runs},   {"narrow", &Tuning::narrow},   {"gather_bkn", &Tuning::gather_bkn},
        {"wgrad_br", &Tuning::wgrad_br},         {"wgrad_rounds", &Tuning::wgrad_rounds},
        {"wgrad_swap", &Tuning::wgrad_swap},     {"pair_bwd", &Tuning::pair_bwd},     {"gather_border", &Tuning::gather_border},
    };
    for (const Field& f : fields)
        if (strcmp(f.name, name) == 0) {
            t.*(f.member) = value;
            return true;
        }
    return false;
}

void tuning_parse(const char* spec, const char** bad) {
    if (bad) *bad = nullptr;
    if (spec == nullptr) return;
    static thread_local char unknown[64];
    const char* p = spec;
    while (*p) {
        char name[64];
        size_t n = 0;
        while (*p && *p != '=' && *p != ',' && n + 1 < sizeof(name)) name[n++] = *p++;
        name[n] = 0;
        int value = 1;
        if (*p == '=') value = atoi(++p);
        while (*p && *p != ',') ++p;
        if (*p == ',') ++p;
        if (n > 0 && !tuning_set(name, value) && bad && *bad == nullptr) {
            snprintf(unknown, sizeof(unknown), "%s", name);
            *bad = unknown;
        }
    }
}

static WorkspaceLedger g_ws;                            // the scratch workspace and who may still use old ones
static bool recording_open() { return g_ws.recording_open; }

static int64_t g_ws_prefix = 0;
void workspace_prefix(int64_t bytes) { g_ws_prefix = bytes > 0 ? round_up(bytes, 256) : 0; }
void* workspace_base() { return g_ws.cur; }

int workspace(int64_t bytes, void** out) {
    hipError_t err = hipSuccess;
    const WorkspaceLedger::Result r = g_ws.acquire(
        bytes + g_ws_prefix, out,
        [&](int64_t want) -> void* {
            void* p = nullptr;
            err = hipMalloc(&p, (size_t)want);
            if (err != hipSuccess) { (void)hipGetLastError(); return nullptr; }
            return p;
        },
        [](void* p) { (void)hipFree(p); },
        [] { (void)hipStreamSynchronize(ctx().stream); });
    if (r == WorkspaceLedger::kWhileRecording)
        return fail(AETH_E_STATE, "the workspace would have to grow while a step is being recorded: run the step once first");
    if (r == WorkspaceLedger::kAllocFailed)
        return fail(err == hipErrorOutOfMemory ? AETH_E_NOMEM : AETH_E_HIP, "workspace: hipMalloc(%lld bytes) -> %s",
                    (long long)WorkspaceLedger::grown_size(bytes + g_ws_prefix), hipGetErrorString(err));
    *out = static_cast<char*>(*out) + g_ws_prefix;
    return AETH_OK;
}

// Caching allocator.  Every kernel and copy runs on the one library stream, so a
// block handed back by the caller can be reused by a later allocation without a
// synchronisation: anything still reading it was queued earlier on that stream.
struct Pool {
    std::unordered_map<void*, size_t> live;            // pointer -> rounded size
    std::map<size_t, std::vector<void*>> free_blocks;  // rounded size -> idle blocks
    size_t cached_bytes = 0;
    // Blocks handed out while a step is being recorded belong to the recording: its
    // replays write to them, so a block the caller frees stays out of circulation until
    // the recording is destroyed.  pointer -> "the caller has freed it".
    std::unordered_map<void*, bool> reserved;
    std::vector<void*>* recording = nullptr;           // blocks of the recording in progress

    static size_t rounded(int64_t bytes) {
        size_t b = bytes <= 0 ? 256 : (size_t)bytes;
        return (b + 255) & ~(size_t)255;
    }
    // Frees every idle block.  Waits for the stream first, so it must not run while a step
    // is being recorded (a synchronisation invalidates the capture).
    hipError_t release_cached() {
        hipError_t st = hipStreamSynchronize(ctx().stream);
        for (auto& kv : free_blocks)
            for (void* p : kv.second) (void)hipFree(p);
        free_blocks.clear();
        cached_bytes = 0;
        return st;
    }
};
static Pool g_pool;

__global__ void fill_f32_kernel(float* __restrict__ dst, float v, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = v;
}

__global__ void fill_u32_kernel(unsigned int* __restrict__ dst, unsigned int v, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = v;
}

// A recorded step: the instantiated graph and the blocks handed out while it was recorded.
struct Recording {
    hipGraphExec_t exec = nullptr;
    std::vector<void*> blocks;
};
static Recording* g_open_recording = nullptr;          // being captured right now
static std::set<Recording*> g_live_recordings;          // every handle given out and not yet destroyed

}  // namespace aeth

using namespace aeth;

extern "C" {

const char* aeth_last_error(void) { return g_err; }

int aeth_init(int device) {
    Context& c = ctx();
    if (c.ready) {
        if (c.device == device) return AETH_OK;
        return fail(AETH_E_STATE, "aeth_init: already bound to device %d", c.device);
    }
    {   // the one place the library looks at the environment: kernel-choice overrides for measurements
        const char* bad = nullptr;
        tuning_parse(getenv("AETHER_TUNE"), &bad);
        if (bad) return fail(AETH_E_INVALID, "aeth_init: AETHER_TUNE names an unknown switch '%s'", bad);
    }
    int n = 0;
    AETH_HIP(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail(AETH_E_INVALID, "aeth_init: device %d out of range (%d present)", device, n);
    AETH_HIP(hipSetDevice(device));
    AETH_HIP(hipGetDeviceProperties(&c.prop, device));
    if (strncmp(c.prop.gcnArchName, "gfx950", 6) != 0)
        return fail(AETH_E_STATE, "aeth_init: built for gfx950, device is %s", c.prop.gcnArchName);
    AETH_HIP(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
    AETH_HIP(hipMalloc((void**)&c.counters, 256 * sizeof(unsigned int)));
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(256), 0, c.stream, c.counters, 0u, 256);
    AETH_LAUNCH_CHECK();
    AETH_HIP(hipStreamSynchronize(c.stream));
    int rc = conv_scratch_init(device);
    if (rc) return rc;
    c.device = device;
    c.ready = true;
    return AETH_OK;
}

namespace {
void stage_release();                                    // the pinned staging slots of the small host copies (below)
}

int aeth_shutdown(void) {
    Context& c = ctx();
    if (!c.ready) return AETH_OK;
    // a recording left open: end the capture and drop what it collected
    if (g_open_recording) {
        hipGraph_t graph = nullptr;
        if (hipStreamEndCapture(c.stream, &graph) == hipSuccess && graph) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        g_live_recordings.erase(g_open_recording);
        delete g_open_recording;
        g_open_recording = nullptr;
    }
    (void)hipStreamSynchronize(c.stream);
    // graphs the caller never destroyed: their handles become invalid with the context
    for (Recording* r : g_live_recordings) {
        if (r->exec) (void)hipGraphExecDestroy(r->exec);
        delete r;
    }
    g_live_recordings.clear();
    g_pool.recording = nullptr;
    g_pool.reserved.clear();
    g_pool.release_cached();
    for (auto& kv : g_pool.live) (void)hipFree(kv.first);
    g_pool.live.clear();
    g_ws.reset([](void* p) { (void)hipFree(p); });
    if (c.counters) hipFree(c.counters);
    stage_release();
    hipStreamDestroy(c.stream);
    c = Context();
    return AETH_OK;
}

int aeth_debug_set(const char* host_name, int value) {
    if (!tuning_set(host_name, value)) return fail(AETH_E_INVALID, "aeth_debug_set: unknown switch '%s'", host_name);
    return AETH_OK;
}

int aeth_device_info(char* host_buf, int n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(host_buf != nullptr && n > 0);
    Context& c = ctx();
    snprintf(host_buf, (size_t)n, "arch=%s;cus=%d;clock_mhz=%d;mem_clock_mhz=%d;mem_bus_bits=%d;hbm_bytes=%lld;lds_bytes=%lld;l2_bytes=%d",
             c.prop.gcnArchName, c.prop.multiProcessorCount, c.prop.clockRate / 1000,
             c.prop.memoryClockRate / 1000, c.prop.memoryBusWidth,
             (long long)c.prop.totalGlobalMem, (long long)c.prop.sharedMemPerBlock, c.prop.l2CacheSize);
    return AETH_OK;
}

int aeth_malloc(void** host_out_ptr, int64_t bytes) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(host_out_ptr != nullptr);
    AETH_CHECK_ARG(bytes >= 0);
    *host_out_ptr = nullptr;
    size_t sz = Pool::rounded(bytes);
    auto it = g_pool.free_blocks.find(sz);
    if (it != g_pool.free_blocks.end() && !it->second.empty()) {
        void* p = it->second.back();
        it->second.pop_back();
        g_pool.cached_bytes -= sz;
        g_pool.live[p] = sz;
        if (g_pool.recording) { g_pool.recording->push_back(p); g_pool.reserved[p] = false; }
        *host_out_ptr = p;
        return AETH_OK;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, sz);
    if (e == hipErrorOutOfMemory && g_pool.cached_bytes > 0 && !recording_open()) {
        (void)hipGetLastError();
        g_pool.release_cached();                        // waits for the stream: never inside a recording
        e = hipMalloc(&p, sz);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(e == hipErrorOutOfMemory ? AETH_E_NOMEM : AETH_E_HIP,
                    "aeth_malloc: hipMalloc(%lld bytes) -> %s", (long long)bytes, hipGetErrorString(e));
    }
    g_pool.live[p] = sz;
    if (g_pool.recording) { g_pool.recording->push_back(p); g_pool.reserved[p] = false; }
    *host_out_ptr = p;
    return AETH_OK;
}

int aeth_free(void* p) {
    AETH_REQUIRE_INIT();
    if (!p) return AETH_OK;
    auto it = g_pool.live.find(p);
    if (it == g_pool.live.end()) return fail(AETH_E_INVALID, "aeth_free: %p was not returned by aeth_malloc", p);
    auto rs = g_pool.reserved.find(p);
    if (rs != g_pool.reserved.end()) {
        if (rs->second) return fail(AETH_E_INVALID, "aeth_free: %p freed twice", p);
        rs->second = true;                              // returned to the pool by aeth_graph_destroy
        return AETH_OK;
    }
    size_t sz = it->second;
    g_pool.live.erase(it);
    g_pool.free_blocks[sz].push_back(p);
    g_pool.cached_bytes += sz;
    return AETH_OK;
}

// Copies between host and device of up to 2 MB go through pinned staging slots, in pieces of one slot: a pageable source
// makes the driver stage the bytes itself and the call wait for the device (a training step's 512 bytes of labels cost
// 10 us with the device idle; a batch of 128 32x32x3 images is 1.5 MB, a dropout mask of 128 x 256 floats 128 KB).
// A slot is reused once the copy it fed has passed (an event per slot).
namespace {
constexpr int kStageSlots = 16;
constexpr int kStageHeldMax = 8;                        // slots that pending aeth_d2h_begin copies may hold at a time
constexpr int64_t kStageBytes = 256 * 1024;
struct Stage {
    char* host[kStageSlots] = {};
    hipEvent_t done[kStageSlots] = {};
    bool busy[kStageSlots] = {};
    bool held[kStageSlots] = {};                         // holds the bytes of an aeth_d2h_begin until its aeth_d2h_end
    int n_held = 0;
    int next = 0;
    bool ready = false;
    bool failed = false;     // the slots could not be allocated once: copies go the pageable way, no second attempt
} g_stage;

void stage_release() {
    for (int i = 0; i < kStageSlots; ++i) {
        if (g_stage.done[i]) (void)hipEventDestroy(g_stage.done[i]);
        if (g_stage.host[i]) (void)hipHostFree(g_stage.host[i]);
    }
    g_stage = Stage();
}

bool stage_init() {
    if (g_stage.ready) return true;
    if (g_stage.failed) return false;
    for (int i = 0; i < kStageSlots; ++i) {
        if (hipHostMalloc((void**)&g_stage.host[i], (size_t)kStageBytes, hipHostMallocDefault) != hipSuccess ||
            hipEventCreateWithFlags(&g_stage.done[i], hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            stage_release();                 // what was allocated so far
            g_stage.failed = true;
            return false;
        }
    }
    g_stage.ready = true;
    return true;
}

// a free slot (waits for the copy that last used it); slots held by pending two-part copies are passed over
// (at most kStageHeldMax of the kStageSlots are ever held)
int stage_slot() {
    int i = g_stage.next;
    while (g_stage.held[i]) i = (i + 1) % kStageSlots;
    g_stage.next = (i + 1) % kStageSlots;
    if (g_stage.busy[i]) {
        (void)hipEventSynchronize(g_stage.done[i]);
        g_stage.busy[i] = false;
    }
    return i;
}
}  // namespace

int aeth_memcpy_h2d(void* dst, const void* host_src, int64_t bytes) {
    AETH_REQUIRE_INIT();
    if (recording_open()) return fail(AETH_E_STATE, "aeth_memcpy_h2d: waits for the device, not possible while recording");
    AETH_CHECK_ARG(bytes >= 0);
    if (bytes == 0) return AETH_OK;
    AETH_CHECK_ARG(dst != nullptr && host_src != nullptr);
    if (bytes <= 8 * kStageBytes && stage_init()) {
        // through pinned slots: the caller's buffer is free at once and the copies take their turn on the stream
        for (int64_t done = 0; done < bytes; done += kStageBytes) {
            const int64_t piece = bytes - done < kStageBytes ? bytes - done : kStageBytes;
            const int i = stage_slot();
            memcpy(g_stage.host[i], static_cast<const char*>(host_src) + done, (size_t)piece);
            AETH_HIP(hipMemcpyAsync(static_cast<char*>(dst) + done, g_stage.host[i], (size_t)piece, hipMemcpyHostToDevice,
                                    ctx().stream));
            AETH_HIP(hipEventRecord(g_stage.done[i], ctx().stream));
            g_stage.busy[i] = true;
        }
        return AETH_OK;
    }
    // pageable source: the call returns once the source has been staged
    AETH_HIP(hipMemcpyAsync(dst, host_src, (size_t)bytes, hipMemcpyHostToDevice, ctx().stream));
    AETH_HIP(hipStreamSynchronize(ctx().stream));
    return AETH_OK;
}

int aeth_memcpy_d2h(void* host_dst, const void* src, int64_t bytes) {
    AETH_REQUIRE_INIT();
    if (recording_open()) return fail(AETH_E_STATE, "aeth_memcpy_d2h: waits for the device, not possible while recording");
    AETH_CHECK_ARG(bytes >= 0);
    if (bytes == 0) return AETH_OK;
    AETH_CHECK_ARG(host_dst != nullptr && src != nullptr);
    if (bytes <= kStageBytes && stage_init()) {
        const int i = stage_slot();
        AETH_HIP(hipMemcpyAsync(g_stage.host[i], src, (size_t)bytes, hipMemcpyDeviceToHost, ctx().stream));
        AETH_HIP(hipStreamSynchronize(ctx().stream));
        memcpy(host_dst, g_stage.host[i], (size_t)bytes);
        return AETH_OK;
    }
    AETH_HIP(hipMemcpyAsync(host_dst, src, (size_t)bytes, hipMemcpyDeviceToHost, ctx().stream));
    AETH_HIP(hipStreamSynchronize(ctx().stream));
    return AETH_OK;
}

int aeth_d2h_begin(const void* src, int64_t bytes, int* host_out_ticket) {
    AETH_REQUIRE_INIT();
    if (recording_open()) return fail(AETH_E_STATE, "aeth_d2h_begin: a copy to the host cannot be part of a recording");
    AETH_CHECK_ARG(src != nullptr && host_out_ticket != nullptr);
    AETH_CHECK_ARG(bytes > 0 && bytes <= kStageBytes);
    *host_out_ticket = -1;
    if (!stage_init()) return fail(AETH_E_NOMEM, "aeth_d2h_begin: no pinned staging memory");
    if (g_stage.n_held >= kStageHeldMax)
        return fail(AETH_E_STATE, "aeth_d2h_begin: %d copies are pending already (aeth_d2h_end takes them)", kStageHeldMax);
    const int i = stage_slot();
    AETH_HIP(hipMemcpyAsync(g_stage.host[i], src, (size_t)bytes, hipMemcpyDeviceToHost, ctx().stream));
    AETH_HIP(hipEventRecord(g_stage.done[i], ctx().stream));
    g_stage.busy[i] = true;
    g_stage.held[i] = true;
    ++g_stage.n_held;
    *host_out_ticket = i;
    return AETH_OK;
}

int aeth_d2h_end(int ticket, void* host_dst, int64_t bytes) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(ticket >= 0 && ticket < kStageSlots && g_stage.ready && g_stage.held[ticket]);
    AETH_CHECK_ARG(bytes >= 0 && bytes <= kStageBytes && (host_dst != nullptr || bytes == 0));
    const hipError_t e = hipEventSynchronize(g_stage.done[ticket]);     // this copy alone, not what was queued after it
    if (e == hipSuccess && bytes > 0) memcpy(host_dst, g_stage.host[ticket], (size_t)bytes);
    g_stage.busy[ticket] = false;
    g_stage.held[ticket] = false;
    --g_stage.n_held;
    AETH_HIP(e);
    return AETH_OK;
}

int aeth_memcpy_d2d(void* dst, const void* src, int64_t bytes) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(bytes >= 0);
    if (bytes == 0) return AETH_OK;
    AETH_CHECK_ARG(dst != nullptr && src != nullptr);
    AETH_HIP(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, ctx().stream));
    return AETH_OK;
}

int aeth_fill_f32(float* dst, float value, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(dst != nullptr);
    int blocks = (int)((n + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_f32_kernel, dim3(blocks), dim3(256), 0, ctx().stream, dst, value, n);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

// ---- recorded steps (HIP graphs) -----------------------------------------------------
#define AETH_NOT_RECORDING(fn)                                                                    \
    do {                                                                                          \
        if (g_open_recording) return fail(AETH_E_STATE, fn ": waits for the device, not possible while recording"); \
    } while (0)

int aeth_graph_begin(void) {
    AETH_REQUIRE_INIT();
    if (g_open_recording) return fail(AETH_E_STATE, "aeth_graph_begin: a recording is already open");
    Context& c = ctx();
    AETH_HIP(hipStreamSynchronize(c.stream));
    Recording* r = new Recording();
    hipError_t e = hipStreamBeginCapture(c.stream, hipStreamCaptureModeRelaxed);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        delete r;
        return fail(AETH_E_HIP, "aeth_graph_begin: hipStreamBeginCapture -> %s", hipGetErrorString(e));
    }
    g_open_recording = r;
    g_ws.recording_open = true;
    g_pool.recording = &r->blocks;
    return AETH_OK;
}

static void release_recording_blocks(Recording* r) {
    for (void* p : r->blocks) {
        auto rs = g_pool.reserved.find(p);
        if (rs == g_pool.reserved.end()) continue;
        const bool freed = rs->second;
        g_pool.reserved.erase(rs);
        if (freed) {
            auto it = g_pool.live.find(p);
            if (it != g_pool.live.end()) {
                const size_t sz = it->second;
                g_pool.live.erase(it);
                g_pool.free_blocks[sz].push_back(p);
                g_pool.cached_bytes += sz;
            }
        }
    }
    r->blocks.clear();
}

int aeth_graph_end(void** host_out_graph) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(host_out_graph != nullptr);
    *host_out_graph = nullptr;
    if (!g_open_recording) return fail(AETH_E_STATE, "aeth_graph_end: no recording is open");
    Recording* r = g_open_recording;
    g_open_recording = nullptr;
    g_ws.recording_open = false;
    g_pool.recording = nullptr;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx().stream, &graph);
    if (e == hipSuccess) {
        e = hipGraphInstantiate(&r->exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        release_recording_blocks(r);
        delete r;
        return fail(AETH_E_HIP, "aeth_graph_end: %s", hipGetErrorString(e));
    }
    g_ws.recording_ended_ok();
    g_live_recordings.insert(r);
    *host_out_graph = r;
    return AETH_OK;
}

int aeth_graph_launch(void* graph) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(graph != nullptr);
    if (g_open_recording) return fail(AETH_E_STATE, "aeth_graph_launch: a recording is open");
    if (!g_live_recordings.count(static_cast<Recording*>(graph)))
        return fail(AETH_E_INVALID, "aeth_graph_launch: %p is not a live recording", graph);
    AETH_HIP(hipGraphLaunch(static_cast<Recording*>(graph)->exec, ctx().stream));
    return AETH_OK;
}

int aeth_graph_destroy(void* graph) {
    AETH_REQUIRE_INIT();
    if (!graph) return AETH_OK;
    Recording* r = static_cast<Recording*>(graph);
    if (g_open_recording) return fail(AETH_E_STATE, "aeth_graph_destroy: a recording is open");
    if (!g_live_recordings.count(r)) return fail(AETH_E_INVALID, "aeth_graph_destroy: %p is not a live recording", graph);
    AETH_HIP(hipStreamSynchronize(ctx().stream));
    if (r->exec) (void)hipGraphExecDestroy(r->exec);
    release_recording_blocks(r);
    g_live_recordings.erase(r);
    g_ws.recording_destroyed([](void* p) { (void)hipFree(p); });
    delete r;
    return AETH_OK;
}

int aeth_sync(void) {
    AETH_REQUIRE_INIT();
    AETH_NOT_RECORDING("aeth_sync");
    AETH_HIP(hipStreamSynchronize(ctx().stream));
    return AETH_OK;
}

int aeth_event_create(void** host_out_event) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(host_out_event != nullptr);
    hipEvent_t ev;
    AETH_HIP(hipEventCreate(&ev));
    *host_out_event = (void*)ev;
    return AETH_OK;
}

int aeth_event_destroy(void* event) {
    AETH_REQUIRE_INIT();
    if (!event) return AETH_OK;
    AETH_HIP(hipEventDestroy((hipEvent_t)event));
    return AETH_OK;
}

int aeth_event_record(void* event) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(event != nullptr);
    AETH_NOT_RECORDING("aeth_event_record");
    AETH_HIP(hipEventRecord((hipEvent_t)event, ctx().stream));
    return AETH_OK;
}

int aeth_event_elapsed_ms(void* start, void* stop, float* host_out_ms) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(start != nullptr && stop != nullptr && host_out_ms != nullptr);
    AETH_NOT_RECORDING("aeth_event_elapsed_ms");
    AETH_HIP(hipEventSynchronize((hipEvent_t)stop));
    AETH_HIP(hipEventElapsedTime(host_out_ms, (hipEvent_t)start, (hipEvent_t)stop));
    return AETH_OK;
}

}  // extern "C"
