// runtime.hip -- lifecycle, device-resident caches and the extern "C" surface of
// libcwick_hip.so.  Kernels live in the other .hip files; this file only
// validates arguments, moves host operands and enqueues.
#include "common.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <strings.h>
#include <unordered_map>
#include <vector>

namespace cwick {

// ---------------------------------------------------------------------------
// error text, per thread (plays the part of cwick_error.message, src/cwick.h:39-59)
// ---------------------------------------------------------------------------
static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}
void clear_error() { g_err[0] = 0; }

bool hip_ok(hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return false;
}

// ---------------------------------------------------------------------------
// backend state machine: -1 untried, 0 unavailable, 1 ready
// (src/h3_gpu.c:35-40, src/metal.c:22-26)
// ---------------------------------------------------------------------------
static std::mutex g_mu;
static int g_state = -1;
static int g_selected = -1;   // -1 env/auto, 0 explicit CPU, 1 explicit GPU
static int g_cus = 0;
static char g_info[256] = "";

static int env_enabled(const char *name, int dflt) {
    const char *v = getenv(name);
    if (!v || !*v) return dflt;
    return strcmp(v, "1") == 0 || strcasecmp(v, "true") == 0 || strcasecmp(v, "yes") == 0 ||
           strcasecmp(v, "on") == 0;
}

static int bring_up_locked() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        set_error("no HIP device");
        return 0;
    }
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipGetDeviceProperties failed");
        return 0;
    }
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
        set_error("device 0 is %s; this library is built for gfx950 only", p.gcnArchName);
        return 0;
    }
    if (hipSetDevice(0) != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipSetDevice(0) failed");
        return 0;
    }
    g_cus = p.multiProcessorCount;
    snprintf(g_info, sizeof g_info, "%s %s, %d CUs, %.1f GiB, LDS %zu KiB/WG", p.name,
             p.gcnArchName, p.multiProcessorCount,
             (double)p.totalGlobalMem / (1024.0 * 1024.0 * 1024.0),
             (size_t)p.sharedMemPerBlock / 1024);
    return 1;
}

bool backend_ready() {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_state < 0) {
        int enabled = g_selected >= 0 ? g_selected : env_enabled("CWICK_HIP", 1);
        g_state = enabled ? bring_up_locked() : 0;
        if (!enabled) set_error("backend not selected (CWICK_HIP=0 or cwick_hip_force(0))");
    } else if (g_state == 0) {
        set_error("backend unavailable or not selected");
    }
    return g_state == 1;
}

int num_cus() { return g_cus > 0 ? g_cus : 256; }

// ---------------------------------------------------------------------------
// grow-only scratch, WS_SLOTS buffers per stream
// ---------------------------------------------------------------------------
// A buffer that has been handed out is never freed while its stream is known to the library:
// kernels already enqueued and HIP graphs captured earlier carry its address.  When a call
// needs more, a new buffer is allocated and the old one is retired until
// cwick_hip_stream_release() or cwick_hip_shutdown(); nothing waits for the stream.  Capacities at
// least double, so the retired buffers of a stream add up to less than its current one.
struct Scratch {
    void *p = nullptr;
    size_t cap = 0;
    std::vector<void *> retired;
    void free_all() {
        if (p) (void)hipFree(p);
        for (void *r : retired) (void)hipFree(r);
        p = nullptr;
        cap = 0;
        retired.clear();
    }
};
struct StreamScratch {
    Scratch slot[WS_SLOTS];
};
static std::unordered_map<hipStream_t, StreamScratch> g_ws;

// true (and the reason recorded) when `s` is being captured into a graph: nothing may be
// allocated then, and the address of a buffer allocated now would end up in the graph
static bool capturing(hipStream_t s, const char *what) {
    if (!s) return false;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (st == hipStreamCaptureStatusNone) return false;
    set_error("%s would have to allocate while the stream is being captured; run the shape once before the "
              "capture or size the workspace with cwick_hip_reserve_dev", what);
    return true;
}

static void *grow_one(Scratch &b, hipStream_t s, size_t bytes) {
    if (bytes <= b.cap) return b.p;
    if (capturing(s, "the split-K workspace")) return nullptr;
    size_t want = bytes > 2 * b.cap ? bytes : 2 * b.cap;
    want = (want + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    void *np = nullptr;
    if (!hip_ok(hipMalloc(&np, want), "hipMalloc(workspace)")) return nullptr;
    if (b.p) b.retired.push_back(b.p);
    b.p = np;
    b.cap = want;
    return b.p;
}

void *workspace(hipStream_t s, size_t bytes, int slot) {
    std::lock_guard<std::mutex> lk(g_mu);
    return grow_one(g_ws[s].slot[slot], s, bytes);
}

// A few dwords per stream that are zero whenever no kernel of the stream is running: kernels
// that hand out their work by tickets count in them and leave them zero again.
static std::unordered_map<hipStream_t, uint32_t *> g_tickets;
uint32_t *ticket_counters(hipStream_t s) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_tickets.find(s);
    if (it != g_tickets.end()) return it->second;
    if (capturing(s, "the ticket counters")) return nullptr;
    void *p = nullptr;
    if (!hip_ok(hipMalloc(&p, 256), "hipMalloc(tickets)")) return nullptr;
    // cleared on the stream whose kernels will count in them, and the clearing waited for
    if (!hip_ok(hipMemsetAsync(p, 0, 256, s), "hipMemsetAsync(tickets)") ||
        !hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize(tickets)")) {
        (void)hipFree(p);
        return nullptr;
    }
    g_tickets[s] = (uint32_t *)p;
    return (uint32_t *)p;
}

// forget (and free) what the library keeps for a stream that is about to be destroyed
static void drop_workspace(hipStream_t s) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto tk = g_tickets.find(s);
    if (tk != g_tickets.end()) {
        (void)hipFree(tk->second);
        g_tickets.erase(tk);
    }
    auto it = g_ws.find(s);
    if (it == g_ws.end()) return;
    for (Scratch &b : it->second.slot) b.free_all();
    g_ws.erase(it);
}

// What a host-pointer call needs of its own: a stream and a staging buffer for the operands it
// copies in and out.  Every cache handle owns one, so calls on different handles share nothing
// (the split-K workspace is keyed by the stream) and may run on different threads; the calls
// that take no handle share g_free_ctx under g_free_mu.
struct HostCtx {
    hipStream_t stream = nullptr;
    Scratch stage;
    bool init() {
        return hip_ok(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreate(handle)");
    }
    void *staging(size_t bytes) { return grow_one(stage, stream, bytes); }
    void destroy() {
        if (stream) {
            (void)hipStreamSynchronize(stream);
            drop_workspace(stream);
            (void)hipStreamDestroy(stream);
            stream = nullptr;
        }
        stage.free_all();
    }
};
static std::mutex g_free_mu;
static HostCtx g_free_ctx;

// ---------------------------------------------------------------------------
// phase timers: event pairs around kernel launches, summed on read
// ---------------------------------------------------------------------------
struct ProfPair {
    hipEvent_t a, b;
    int which;
};
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<ProfPair> g_prof_pending;       // recorded, not yet summed
static std::vector<ProfPair> g_prof_free;          // reusable event pairs
static double g_prof_ms[CWICK_HIP_PROF_COUNT];
static int64_t g_prof_n[CWICK_HIP_PROF_COUNT];

ProfScope::ProfScope(int w, hipStream_t s) : which(w), stream(s), slot(nullptr) {
    if (!g_prof_on || w < 0) return;                  // w < 0: a launch that must not create events
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfPair *pp = new ProfPair;
    if (!g_prof_free.empty()) {
        *pp = g_prof_free.back();
        g_prof_free.pop_back();
    } else if (hipEventCreate(&pp->a) != hipSuccess || hipEventCreate(&pp->b) != hipSuccess) {
        (void)hipGetLastError();
        delete pp;
        return;
    }
    pp->which = w;
    (void)hipEventRecord(pp->a, s);
    slot = pp;
}

ProfScope::~ProfScope() {
    if (!slot) return;
    ProfPair *pp = (ProfPair *)slot;
    (void)hipEventRecord(pp->b, stream);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_pending.push_back(*pp);
    delete pp;
}

ProfKernel::ProfKernel(int w, hipStream_t s) : which(w), stream(s) {
    if (!g_prof_on || w < 0) return;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfPair pp;
    if (!g_prof_free.empty()) {
        pp = g_prof_free.back();
        g_prof_free.pop_back();
    } else if (hipEventCreate(&pp.a) != hipSuccess || hipEventCreate(&pp.b) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    a = pp.a;
    b = pp.b;
}

ProfKernel::~ProfKernel() {
    if (!a) return;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfPair pp{a, b, which};
    if (bound) g_prof_pending.push_back(pp);
    else g_prof_free.push_back(pp);
}

static void prof_drain_locked() {
    for (ProfPair &pp : g_prof_pending) {
        float ms = 0.0f;
        if (hipEventSynchronize(pp.b) == hipSuccess &&
            hipEventElapsedTime(&ms, pp.a, pp.b) == hipSuccess) {
            g_prof_ms[pp.which] += (double)ms;
            g_prof_n[pp.which] += 1;
        } else {
            (void)hipGetLastError();
        }
        g_prof_free.push_back(pp);
    }
    g_prof_pending.clear();
}

static void free_all_scratch() {
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto &kv : g_ws)
        for (Scratch &b : kv.second.slot) b.free_all();
    g_ws.clear();
    for (auto &kv : g_tickets) (void)hipFree(kv.second);
    g_tickets.clear();
}

}  // namespace cwick

using namespace cwick;

// ---------------------------------------------------------------------------
// cache handles
// ---------------------------------------------------------------------------
struct cwick_hip_kv {
    int64_t capacity;
    int n_kv_heads, head_dim;
    uint16_t *k, *v;
    HostCtx ctx;
};
struct cwick_hip_latent {
    int slots;
    int64_t capacity;
    uint8_t *rows;    // [slots][capacity][576]
    float *scales;    // [slots][capacity][5]
    HostCtx ctx;
};
struct cwick_hip_ikeys {
    int slots;
    int64_t capacity;
    uint8_t *rows;    // [slots][capacity][128]
    float *scales;    // [slots][capacity]
    HostCtx ctx;
};

static size_t pad256(size_t b) { return (b + 255) & ~(size_t)255; }

// The operands of one host-pointer call, laid out in the context's staging buffer: in() copies
// a host operand up on the context's stream, room() reserves space for a result, out() brings
// a result back and waits for everything the call enqueued.
struct Stager {
    HostCtx &ctx;
    char *base;
    size_t off = 0;
    bool ok;
    Stager(HostCtx &c, size_t total) : ctx(c), base((char *)c.staging(total)), ok(base != nullptr) {}
    template <class T>
    T *in(const T *host, size_t bytes) {
        if (!ok) return nullptr;
        T *d = (T *)(base + off);
        off += pad256(bytes);
        if (!hip_ok(hipMemcpyAsync(d, host, bytes, hipMemcpyHostToDevice, ctx.stream), "hipMemcpyAsync(operand)"))
            ok = false;
        return ok ? d : nullptr;
    }
    template <class T>
    T *room(size_t bytes) {
        if (!ok) return nullptr;
        T *d = (T *)(base + off);
        off += pad256(bytes);
        return d;
    }
    bool out(void *host, const void *dev, size_t bytes) {
        return hip_ok(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, ctx.stream), "hipMemcpyAsync(result)");
    }
    bool wait() { return hip_ok(hipStreamSynchronize(ctx.stream), "hipStreamSynchronize(handle)"); }
};

extern "C" {

// ---- lifecycle -------------------------------------------------------------
int cwick_hip_ready(void) {
    clear_error();
    return backend_ready() ? 1 : 0;
}

int cwick_hip_force(int on) {
    clear_error();
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_selected = on ? 1 : 0;
        g_state = on ? -1 : 0;
    }
    if (!on) return 0;
    return backend_ready() ? 0 : -1;
}

void cwick_hip_shutdown(void) {
    bool up;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        up = g_state == 1;
    }
    if (up) (void)hipDeviceSynchronize();
    {
        std::lock_guard<std::mutex> lk(g_free_mu);
        g_free_ctx.destroy();
    }
    free_all_scratch();
}

int cwick_hip_reserve_dev(void *stream, int64_t bytes) {
    clear_error();
    if (!backend_ready()) return 0;
    CWICK_REQUIRE(bytes >= 0 && bytes <= ((int64_t)1 << 40), "reserve: %lld bytes", (long long)bytes);
    hipStream_t s = (hipStream_t)stream;
    // the main slot as asked; the nested one for the largest row the many-workgroup select takes
    // (batch 64); the ticket counters of the prefill
    if (bytes > 0 && !workspace(s, (size_t)bytes, WS_MAIN)) return 0;          // the reason is recorded
    if (!workspace(s, topk_mw_workspace_bytes(64, 131072), WS_NESTED)) return 0;
    if (!ticket_counters(s)) return 0;
    return 1;
}

int64_t cwick_hip_workspace_bytes_dev(void *stream) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_ws.find((hipStream_t)stream);
    return it == g_ws.end() ? 0 : (int64_t)it->second.slot[WS_MAIN].cap;
}

int cwick_hip_stream_release(void *stream) {
    clear_error();
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (g_state != 1) return 1;                  // nothing was ever kept
    }
    hipStream_t s = (hipStream_t)stream;
    if (capturing(s, "cwick_hip_stream_release")) return 0;
    CWICK_HIP_CALL(hipStreamSynchronize(s));
    drop_workspace(s);
    return 1;
}

const char *cwick_hip_last_error(void) { return g_err; }

int cwick_hip_device_info(char *buf, size_t cap) {
    clear_error();
    if (!backend_ready() || !buf || cap == 0) return 0;
    snprintf(buf, cap, "%s", g_info);
    return 1;
}

// ---- GQA cache -------------------------------------------------------------
cwick_hip_kv *cwick_hip_kv_create(int64_t capacity, int n_kv_heads, int head_dim) {
    clear_error();
    if (!backend_ready()) return nullptr;
    if (capacity <= 0 || n_kv_heads <= 0 || (head_dim != 128 && head_dim != 256)) {
        set_error("kv_create: capacity %lld, n_kv_heads %d, head_dim %d unsupported",
                  (long long)capacity, n_kv_heads, head_dim);
        return nullptr;
    }
    cwick_hip_kv *c = new cwick_hip_kv{capacity, n_kv_heads, head_dim, nullptr, nullptr, {}};
    size_t bytes = (size_t)capacity * n_kv_heads * head_dim * sizeof(uint16_t);
    if (!c->ctx.init() || !hip_ok(hipMalloc((void **)&c->k, bytes), "hipMalloc(K cache)") ||
        !hip_ok(hipMalloc((void **)&c->v, bytes), "hipMalloc(V cache)")) {
        if (c->k) (void)hipFree(c->k);
        c->ctx.destroy();
        delete c;
        return nullptr;
    }
    return c;
}

void cwick_hip_kv_free(cwick_hip_kv *c) {
    if (!c) return;
    (void)hipDeviceSynchronize();
    c->ctx.destroy();
    (void)hipFree(c->k);
    (void)hipFree(c->v);
    delete c;
}

#define KV_RANGE_CHECK(what)                                                             \
    if (!backend_ready()) return 0;   /* the reason is recorded */                                  \
    CWICK_REQUIRE(c, what ": null handle");                                               \
    CWICK_REQUIRE(pos0 >= 0 && n > 0 && pos0 + n <= c->capacity,                          \
                  what ": rows %lld..%lld outside capacity %lld", (long long)pos0,       \
                  (long long)(pos0 + n), (long long)c->capacity)

int cwick_hip_kv_write(cwick_hip_kv *c, int64_t pos0, int64_t n, const uint16_t *k_rows,
                       const uint16_t *v_rows) {
    clear_error();
    KV_RANGE_CHECK("kv_write");
    CWICK_REQUIRE(k_rows && v_rows, "kv_write: null argument");
    size_t row = (size_t)c->n_kv_heads * c->head_dim;
    CWICK_HIP_CALL(hipMemcpy(c->k + pos0 * row, k_rows, n * row * 2, hipMemcpyHostToDevice));
    CWICK_HIP_CALL(hipMemcpy(c->v + pos0 * row, v_rows, n * row * 2, hipMemcpyHostToDevice));
    return 1;
}

int cwick_hip_kv_write_f32(cwick_hip_kv *c, int64_t pos0, int64_t n, const float *k_rows,
                           const float *v_rows) {
    clear_error();
    KV_RANGE_CHECK("kv_write_f32");
    CWICK_REQUIRE(k_rows && v_rows, "kv_write_f32: null argument");
    size_t row = (size_t)c->n_kv_heads * c->head_dim;
    size_t bytes = (size_t)n * row * sizeof(float);
    Stager st(c->ctx, 2 * pad256(bytes));
    CWICK_REQUIRE(st.ok, "kv_write_f32: staging allocation failed");
    const float *dk = st.in(k_rows, bytes);
    const float *dv = st.in(v_rows, bytes);
    CWICK_REQUIRE(dk && dv, "kv_write_f32: upload failed");
    if (!launch_narrow_bf16(dk, n * row, c->k + pos0 * row, c->ctx.stream)) return 0;
    if (!launch_narrow_bf16(dv, n * row, c->v + pos0 * row, c->ctx.stream)) return 0;
    return st.wait() ? 1 : 0;
}

int cwick_hip_kv_read(cwick_hip_kv *c, int64_t pos0, int64_t n, uint16_t *k_rows, uint16_t *v_rows) {
    clear_error();
    KV_RANGE_CHECK("kv_read");
    CWICK_REQUIRE(k_rows && v_rows, "kv_read: null argument");
    size_t row = (size_t)c->n_kv_heads * c->head_dim;
    CWICK_HIP_CALL(hipMemcpy(k_rows, c->k + pos0 * row, n * row * 2, hipMemcpyDeviceToHost));
    CWICK_HIP_CALL(hipMemcpy(v_rows, c->v + pos0 * row, n * row * 2, hipMemcpyDeviceToHost));
    return 1;
}

int cwick_hip_kv_read_f32(cwick_hip_kv *c, int64_t pos0, int64_t n, float *k_rows, float *v_rows) {
    clear_error();
    KV_RANGE_CHECK("kv_read_f32");
    CWICK_REQUIRE(k_rows && v_rows, "kv_read_f32: null argument");
    size_t row = (size_t)c->n_kv_heads * c->head_dim;
    size_t bytes = (size_t)n * row * sizeof(float);
    Stager st(c->ctx, 2 * pad256(bytes));
    CWICK_REQUIRE(st.ok, "kv_read_f32: staging allocation failed");
    float *dk = st.room<float>(bytes), *dv = st.room<float>(bytes);
    if (!launch_widen_bf16(c->k + pos0 * row, n * row, dk, c->ctx.stream)) return 0;
    if (!launch_widen_bf16(c->v + pos0 * row, n * row, dv, c->ctx.stream)) return 0;
    if (!st.out(k_rows, dk, bytes) || !st.out(v_rows, dv, bytes)) return 0;
    return st.wait() ? 1 : 0;
}

uint16_t *cwick_hip_kv_k_dev(cwick_hip_kv *c) { return c ? c->k : nullptr; }
uint16_t *cwick_hip_kv_v_dev(cwick_hip_kv *c) { return c ? c->v : nullptr; }

// ---- latent cache ------------------------------------------------------------
cwick_hip_latent *cwick_hip_latent_create(int slots, int64_t capacity) {
    clear_error();
    if (!backend_ready()) return nullptr;
    if (slots <= 0 || capacity <= 0) {
        set_error("latent_create: slots %d capacity %lld", slots, (long long)capacity);
        return nullptr;
    }
    cwick_hip_latent *c = new cwick_hip_latent{slots, capacity, nullptr, nullptr, {}};
    size_t rows = (size_t)slots * capacity;
    // 64 bytes of slack: the kernels read rows in 16-byte pieces
    if (!c->ctx.init() ||
        !hip_ok(hipMalloc((void **)&c->rows, rows * CWICK_HIP_LATENT_KDIM + 64), "hipMalloc(latent)") ||
        !hip_ok(hipMalloc((void **)&c->scales, rows * CWICK_HIP_LATENT_NBLK * sizeof(float) + 64),
                "hipMalloc(latent scales)")) {
        if (c->rows) (void)hipFree(c->rows);
        c->ctx.destroy();
        delete c;
        return nullptr;
    }
    return c;
}

void cwick_hip_latent_free(cwick_hip_latent *c) {
    if (!c) return;
    (void)hipDeviceSynchronize();
    c->ctx.destroy();
    (void)hipFree(c->rows);
    (void)hipFree(c->scales);
    delete c;
}

#define LATENT_RANGE_CHECK(what)                                                          \
    if (!backend_ready()) return 0;   /* the reason is recorded */                                  \
    CWICK_REQUIRE(c, what ": null handle");                                               \
    CWICK_REQUIRE(slot >= 0 && slot < c->slots, what ": slot %d of %d", slot, c->slots);  \
    CWICK_REQUIRE(pos0 >= 0 && n > 0 && pos0 + n <= c->capacity,                          \
                  what ": rows %lld..%lld outside capacity %lld", (long long)pos0,       \
                  (long long)(pos0 + n), (long long)c->capacity)

int cwick_hip_latent_write(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                           const uint8_t *rows, const float *scales) {
    clear_error();
    LATENT_RANGE_CHECK("latent_write");
    CWICK_REQUIRE(rows && scales, "latent_write: null argument");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    CWICK_HIP_CALL(hipMemcpy(c->rows + r0 * CWICK_HIP_LATENT_KDIM, rows,
                             (size_t)n * CWICK_HIP_LATENT_KDIM, hipMemcpyHostToDevice));
    CWICK_HIP_CALL(hipMemcpy(c->scales + r0 * CWICK_HIP_LATENT_NBLK, scales,
                             (size_t)n * CWICK_HIP_LATENT_NBLK * sizeof(float),
                             hipMemcpyHostToDevice));
    return 1;
}

int cwick_hip_latent_write_f32(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                               const float *rows) {
    clear_error();
    LATENT_RANGE_CHECK("latent_write_f32");
    CWICK_REQUIRE(rows, "latent_write_f32: null argument");
    size_t bytes = (size_t)n * CWICK_HIP_LATENT_KDIM * sizeof(float);
    Stager st(c->ctx, pad256(bytes));
    CWICK_REQUIRE(st.ok, "latent_write_f32: staging allocation failed");
    const float *d = st.in(rows, bytes);
    CWICK_REQUIRE(d, "latent_write_f32: upload failed");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    if (!launch_quant_latent(d, n, c->rows + r0 * CWICK_HIP_LATENT_KDIM,
                             c->scales + r0 * CWICK_HIP_LATENT_NBLK, c->ctx.stream))
        return 0;
    return st.wait() ? 1 : 0;
}

int cwick_hip_latent_read(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n, uint8_t *rows,
                          float *scales) {
    clear_error();
    LATENT_RANGE_CHECK("latent_read");
    CWICK_REQUIRE(rows && scales, "latent_read: null argument");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    CWICK_HIP_CALL(hipMemcpy(rows, c->rows + r0 * CWICK_HIP_LATENT_KDIM,
                             (size_t)n * CWICK_HIP_LATENT_KDIM, hipMemcpyDeviceToHost));
    CWICK_HIP_CALL(hipMemcpy(scales, c->scales + r0 * CWICK_HIP_LATENT_NBLK,
                             (size_t)n * CWICK_HIP_LATENT_NBLK * sizeof(float),
                             hipMemcpyDeviceToHost));
    return 1;
}

uint8_t *cwick_hip_latent_rows_dev(cwick_hip_latent *c, int slot) {
    if (!c || slot < 0 || slot >= c->slots) return nullptr;
    return c->rows + (size_t)slot * c->capacity * CWICK_HIP_LATENT_KDIM;
}
float *cwick_hip_latent_scales_dev(cwick_hip_latent *c, int slot) {
    if (!c || slot < 0 || slot >= c->slots) return nullptr;
    return c->scales + (size_t)slot * c->capacity * CWICK_HIP_LATENT_NBLK;
}

// ---- indexer key cache -------------------------------------------------------
cwick_hip_ikeys *cwick_hip_ikeys_create(int slots, int64_t capacity) {
    clear_error();
    if (!backend_ready()) return nullptr;
    if (slots <= 0 || capacity <= 0) {
        set_error("ikeys_create: slots %d capacity %lld", slots, (long long)capacity);
        return nullptr;
    }
    cwick_hip_ikeys *c = new cwick_hip_ikeys{slots, capacity, nullptr, nullptr, {}};
    size_t rows = (size_t)slots * capacity;
    if (!c->ctx.init() ||
        !hip_ok(hipMalloc((void **)&c->rows, rows * CWICK_HIP_INDEX_DIM + 64), "hipMalloc(ikeys)") ||
        !hip_ok(hipMalloc((void **)&c->scales, rows * sizeof(float) + 64), "hipMalloc(ikey scales)")) {
        if (c->rows) (void)hipFree(c->rows);
        c->ctx.destroy();
        delete c;
        return nullptr;
    }
    return c;
}

void cwick_hip_ikeys_free(cwick_hip_ikeys *c) {
    if (!c) return;
    (void)hipDeviceSynchronize();
    c->ctx.destroy();
    (void)hipFree(c->rows);
    (void)hipFree(c->scales);
    delete c;
}

int cwick_hip_ikeys_write(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n,
                          const uint8_t *rows, const float *scales) {
    clear_error();
    LATENT_RANGE_CHECK("ikeys_write");
    CWICK_REQUIRE(rows && scales, "ikeys_write: null argument");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    CWICK_HIP_CALL(hipMemcpy(c->rows + r0 * CWICK_HIP_INDEX_DIM, rows,
                             (size_t)n * CWICK_HIP_INDEX_DIM, hipMemcpyHostToDevice));
    CWICK_HIP_CALL(hipMemcpy(c->scales + r0, scales, (size_t)n * sizeof(float),
                             hipMemcpyHostToDevice));
    return 1;
}

int cwick_hip_ikeys_write_f32(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n,
                              const float *rows) {
    clear_error();
    LATENT_RANGE_CHECK("ikeys_write_f32");
    CWICK_REQUIRE(rows, "ikeys_write_f32: null argument");
    size_t bytes = (size_t)n * CWICK_HIP_INDEX_DIM * sizeof(float);
    Stager st(c->ctx, pad256(bytes));
    CWICK_REQUIRE(st.ok, "ikeys_write_f32: staging allocation failed");
    const float *d = st.in(rows, bytes);
    CWICK_REQUIRE(d, "ikeys_write_f32: upload failed");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    if (!launch_quant_ikeys(d, n, c->rows + r0 * CWICK_HIP_INDEX_DIM, c->scales + r0, c->ctx.stream))
        return 0;
    return st.wait() ? 1 : 0;
}

int cwick_hip_ikeys_read(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n, uint8_t *rows,
                         float *scales) {
    clear_error();
    LATENT_RANGE_CHECK("ikeys_read");
    CWICK_REQUIRE(rows && scales, "ikeys_read: null argument");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    CWICK_HIP_CALL(hipMemcpy(rows, c->rows + r0 * CWICK_HIP_INDEX_DIM, (size_t)n * CWICK_HIP_INDEX_DIM,
                             hipMemcpyDeviceToHost));
    CWICK_HIP_CALL(hipMemcpy(scales, c->scales + r0, (size_t)n * sizeof(float), hipMemcpyDeviceToHost));
    return 1;
}

uint8_t *cwick_hip_ikeys_rows_dev(cwick_hip_ikeys *c, int slot) {
    if (!c || slot < 0 || slot >= c->slots) return nullptr;
    return c->rows + (size_t)slot * c->capacity * CWICK_HIP_INDEX_DIM;
}
float *cwick_hip_ikeys_scales_dev(cwick_hip_ikeys *c, int slot) {
    if (!c || slot < 0 || slot >= c->slots) return nullptr;
    return c->scales + (size_t)slot * c->capacity;
}

// ---- device-pointer entry points ---------------------------------------------
int cwick_hip_gqa_decode_dev(const uint16_t *k, const uint16_t *v, int64_t n_keys, int n_kv_heads,
                             int head_dim, const uint16_t *q, int n_heads, float scale, float *out,
                             void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_gqa_decode(k, v, n_keys, n_kv_heads, head_dim, q, n_heads, scale, out,
                             (hipStream_t)stream);
}

int cwick_hip_gqa_prefill_dev(const uint16_t *k, const uint16_t *v, int64_t pos0, int64_t n,
                              int n_kv_heads, int head_dim, const uint16_t *q, int n_heads,
                              float scale, float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_gqa_prefill(k, v, pos0, n, n_kv_heads, head_dim, q, n_heads, scale, out,
                              (hipStream_t)stream);
}

int cwick_hip_mla_decode_dev(const uint8_t *rows, const float *scales, int64_t row_batch_stride,
                             int64_t scale_batch_stride, int64_t n_rows, int batch, const int32_t *sel,
                             int64_t n_list, const uint16_t *q, int n_heads, float scale,
                             float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_decode(rows, scales, row_batch_stride, scale_batch_stride, n_rows, batch, sel,
                             n_list, q, n_heads, scale, nullptr, out, (hipStream_t)stream);
}

int cwick_hip_mla_decode_static_dev(const uint8_t *rows, const float *scales, int64_t row_batch_stride,
                                    int64_t scale_batch_stride, int64_t n_rows, int batch,
                                    const int32_t *sel, int64_t n_list, const uint16_t *q, int n_heads,
                                    float scale, float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_decode(rows, scales, row_batch_stride, scale_batch_stride, n_rows, batch, sel,
                             n_list, q, n_heads, scale, nullptr, out, (hipStream_t)stream, true);
}

int cwick_hip_mla_decode_sink_dev(const uint8_t *rows, const float *scales, int64_t row_batch_stride,
                                  int64_t scale_batch_stride, int64_t n_rows, int batch,
                                  const int32_t *sel, int64_t n_list, const uint16_t *q, int n_heads,
                                  float scale, const float *sink, float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_decode(rows, scales, row_batch_stride, scale_batch_stride, n_rows, batch, sel,
                             n_list, q, n_heads, scale, sink, out, (hipStream_t)stream);
}

int cwick_hip_mla_prefill_chunk_dev(const uint8_t *rows, const float *scales, int64_t pos0,
                                    int64_t n, const uint16_t *q, int n_heads, float scale,
                                    float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_prefill(rows, scales, pos0, n, q, n_heads, scale, out, (hipStream_t)stream);
}

int cwick_hip_indexer_scores_dev(const uint8_t *keys, const float *kscale, int64_t key_batch_stride,
                                 int64_t kscale_batch_stride, int batch, int64_t n_keys,
                                 const uint16_t *q_idx, const float *w, int n_idx_heads,
                                 float *scores, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_indexer_scores(keys, kscale, key_batch_stride, kscale_batch_stride, batch, n_keys,
                                 q_idx, w, n_idx_heads, CWICK_HIP_INDEXER_GLM, scores, (hipStream_t)stream);
}

int cwick_hip_indexer_scores_mode_dev(const uint8_t *keys, const float *kscale, int64_t key_batch_stride,
                                      int64_t kscale_batch_stride, int batch, int64_t n_keys,
                                      const uint16_t *q_idx, const float *w, int n_idx_heads, int mode,
                                      float *scores, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_indexer_scores(keys, kscale, key_batch_stride, kscale_batch_stride, batch, n_keys,
                                 q_idx, w, n_idx_heads, mode, scores, (hipStream_t)stream);
}

int cwick_hip_topk_dev(const float *scores, int batch, int64_t n, int64_t k, int32_t *out_idx,
                       void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_topk(scores, batch, n, k, out_idx, (hipStream_t)stream);
}

int cwick_hip_dsa_decode_dev(const uint8_t *ikeys, const float *ikscale, int64_t key_batch_stride,
                             int64_t kscale_batch_stride, const uint8_t *rows, const float *scales,
                             int64_t row_batch_stride, int64_t scale_batch_stride, int batch,
                             int64_t n_keys, const uint16_t *q_idx, const float *w, int n_idx_heads,
                             int64_t topk, const uint16_t *q, int n_heads, float scale,
                             float *scores_tmp, int32_t *sel_out, float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(scores_tmp && sel_out, "dsa_decode_dev: scores_tmp and sel_out are required");
    CWICK_REQUIRE(topk > 0 && n_keys > 0, "dsa_decode_dev: topk %lld n_keys %lld",
                  (long long)topk, (long long)n_keys);
    hipStream_t s = (hipStream_t)stream;
    // CWICK_HIP_INDEXER=exact scores every key with the exact kernel; the default scores most
    // keys on the matrix cores and only the ones near the selection threshold exactly (the
    // selected indices are the same)
    static const bool exact_only = [] {
        const char *e = getenv("CWICK_HIP_INDEXER");
        return e && strcmp(e, "exact") == 0;
    }();
    if (!exact_only && indexer_band_applies(n_keys, topk, n_idx_heads)) {
        if (!launch_indexer_banded(ikeys, ikscale, key_batch_stride, kscale_batch_stride, batch, n_keys,
                                   q_idx, w, n_idx_heads, topk, scores_tmp, sel_out, s))
            return 0;
    } else {
        if (!launch_indexer_scores(ikeys, ikscale, key_batch_stride, kscale_batch_stride, batch,
                                   n_keys, q_idx, w, n_idx_heads, CWICK_HIP_INDEXER_GLM, scores_tmp, s))
            return 0;
        if (!launch_topk(scores_tmp, batch, n_keys, topk, sel_out, s)) return 0;
    }
    // rows past min(topk, n_keys) are -1 and are skipped by the attention kernel
    return launch_mla_decode(rows, scales, row_batch_stride, scale_batch_stride, n_keys, batch,
                             sel_out, topk, q, n_heads, scale, nullptr, out, s);
}

// ---- host-pointer entry points -------------------------------------------------
int cwick_hip_gqa_decode(cwick_hip_kv *c, int64_t n_keys, const uint16_t *q, int n_heads,
                         float scale, float *out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q && out, "gqa_decode: null argument");
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= c->capacity, "gqa_decode: n_keys %lld, capacity %lld",
                  (long long)n_keys, (long long)c->capacity);
    CWICK_REQUIRE(n_heads > 0 && n_heads <= 1024, "gqa_decode: n_heads %d", n_heads);
    size_t qb = (size_t)n_heads * c->head_dim * 2, ob = (size_t)n_heads * c->head_dim * 4;
    Stager st(c->ctx, pad256(qb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "gqa_decode: staging allocation failed");
    const uint16_t *dq = st.in(q, qb);
    CWICK_REQUIRE(dq, "gqa_decode: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_gqa_decode(c->k, c->v, n_keys, c->n_kv_heads, c->head_dim, dq, n_heads, scale, dout,
                           c->ctx.stream))
        return 0;
    return st.out(out, dout, ob) && st.wait() ? 1 : 0;
}

int cwick_hip_gqa_decode_sel_dev(const uint16_t *k, const uint16_t *v, int64_t n_rows, int n_kv_heads,
                                 int head_dim, const int32_t *sel, int64_t n_list, const uint16_t *q,
                                 int n_heads, float scale, float *out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(sel && n_rows >= 1 && n_rows <= ((int64_t)1 << 31) - 1, "gqa_decode_sel: list or n_rows %lld",
                  (long long)n_rows);
    return launch_gqa_decode(k, v, n_list, n_kv_heads, head_dim, q, n_heads, scale, out, (hipStream_t)stream, sel,
                             n_rows);
}

int cwick_hip_gqa_decode_sel(cwick_hip_kv *c, const int32_t *sel, int64_t n_list, const uint16_t *q,
                             int n_heads, float scale, float *out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && sel && q && out, "gqa_decode_sel: null argument");
    CWICK_REQUIRE(n_list >= 1 && n_list <= ((int64_t)1 << 24), "gqa_decode_sel: n_list %lld", (long long)n_list);
    CWICK_REQUIRE(n_heads > 0 && n_heads <= 1024, "gqa_decode_sel: n_heads %d", n_heads);
    size_t qb = (size_t)n_heads * c->head_dim * 2, ob = (size_t)n_heads * c->head_dim * 4, sb = (size_t)n_list * 4;
    Stager st(c->ctx, pad256(qb) + pad256(ob) + pad256(sb));
    CWICK_REQUIRE(st.ok, "gqa_decode_sel: staging allocation failed");
    const uint16_t *dq = st.in(q, qb);
    const int32_t *dsel = st.in(sel, sb);
    CWICK_REQUIRE(dq && dsel, "gqa_decode_sel: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_gqa_decode(c->k, c->v, n_list, c->n_kv_heads, c->head_dim, dq, n_heads, scale, dout, c->ctx.stream,
                           dsel, c->capacity))
        return 0;
    return st.out(out, dout, ob) && st.wait() ? 1 : 0;
}

int cwick_hip_mm_select(cwick_hip_kv *idx, int64_t limit, const float *iq, int index_heads, int block,
                        int keep_blocks, int32_t *blk_out, int32_t *sel, int64_t max_sel, int64_t *n_sel) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(idx && iq && sel, "mm_select: null argument");
    CWICK_REQUIRE(idx->n_kv_heads == 1, "mm_select: the index keys are a cache of one head per position, not %d",
                  idx->n_kv_heads);
    CWICK_REQUIRE(limit >= 1 && limit <= idx->capacity, "mm_select: limit %lld, capacity %lld", (long long)limit,
                  (long long)idx->capacity);
    CWICK_REQUIRE(index_heads >= 1 && index_heads <= 8, "mm_select: %d index heads (1..8)", index_heads);
    CWICK_REQUIRE(keep_blocks >= 1 && keep_blocks <= 4096 && max_sel >= 1 && max_sel <= ((int64_t)1 << 24),
                  "mm_select: blocks kept %d, max_sel %lld", keep_blocks, (long long)max_sel);
    size_t qb = (size_t)index_heads * idx->head_dim * 4, scb = (size_t)limit * 4, bb = (size_t)(keep_blocks + 1) * 4;
    size_t sb = (size_t)max_sel * 4;
    Stager st(idx->ctx, pad256(qb) + pad256(scb) + pad256(bb) + pad256(sb) + 256);
    CWICK_REQUIRE(st.ok, "mm_select: staging allocation failed");
    const float *dq = st.in(iq, qb);
    CWICK_REQUIRE(dq, "mm_select: upload failed");
    float *dsc = st.room<float>(scb);
    int32_t *dblk = st.room<int32_t>(bb), *dsel = st.room<int32_t>(sb), *dn = st.room<int32_t>(256);
    if (!launch_mm_select(idx->k, dq, 1, limit, index_heads, idx->head_dim, block, keep_blocks, dsc, limit, dblk, dsel,
                          max_sel, dn, idx->ctx.stream))
        return 0;
    int32_t got = 0;
    if (blk_out && !st.out(blk_out, dblk, bb)) return 0;
    if (!st.out(sel, dsel, sb) || !st.out(&got, dn, 4) || !st.wait()) return 0;
    if (n_sel) *n_sel = got;
    return 1;
}

int cwick_hip_gqa_prefill(cwick_hip_kv *c, int64_t pos0, int64_t n, const uint16_t *q, int n_heads,
                          float scale, float *out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q && out, "gqa_prefill: null argument");
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= c->capacity,
                  "gqa_prefill: positions %lld..%lld outside capacity %lld", (long long)pos0,
                  (long long)(pos0 + n), (long long)c->capacity);
    CWICK_REQUIRE(n_heads > 0 && n_heads <= 1024, "gqa_prefill: n_heads %d", n_heads);
    size_t qb = (size_t)n * n_heads * c->head_dim * 2, ob = (size_t)n * n_heads * c->head_dim * 4;
    Stager st(c->ctx, pad256(qb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "gqa_prefill: staging allocation failed");
    const uint16_t *dq = st.in(q, qb);
    CWICK_REQUIRE(dq, "gqa_prefill: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_gqa_prefill(c->k, c->v, pos0, n, c->n_kv_heads, c->head_dim, dq, n_heads, scale,
                            dout, c->ctx.stream))
        return 0;
    return st.out(out, dout, ob) && st.wait() ? 1 : 0;
}

// sel entries must address rows of the slot; checked on the host because a bad
// index would be an out-of-bounds read on the device.
static int check_sel(const int32_t *sel, int64_t n, int64_t capacity) {
    for (int64_t i = 0; i < n; i++)
        if (sel[i] >= capacity) {
            set_error("sel[%lld] = %d is outside capacity %lld", (long long)i, sel[i],
                      (long long)capacity);
            return 0;
        }
    return 1;
}

int cwick_hip_mla_decode(cwick_hip_latent *c, int slot, const int32_t *sel, int64_t n_list,
                         const uint16_t *q, int n_heads, float scale, float *out) {
    return cwick_hip_mla_decode_sink(c, slot, sel, n_list, q, n_heads, scale, nullptr, out);
}

int cwick_hip_mla_decode_sink(cwick_hip_latent *c, int slot, const int32_t *sel, int64_t n_list,
                              const uint16_t *q, int n_heads, float scale, const float *sink,
                              float *out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q && out, "mla_decode: null argument");
    CWICK_REQUIRE(slot >= 0 && slot < c->slots, "mla_decode: slot %d of %d", slot, c->slots);
    CWICK_REQUIRE(n_list >= 1, "mla_decode: n_list %lld", (long long)n_list);
    CWICK_REQUIRE(sel || n_list <= c->capacity, "mla_decode: n_list %lld > capacity %lld",
                  (long long)n_list, (long long)c->capacity);
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_decode: n_heads %d (1..128)", n_heads);
    if (sel && !check_sel(sel, n_list, c->capacity)) return 0;
    size_t qb = (size_t)n_heads * CWICK_HIP_LATENT_KDIM * 2;
    size_t ob = (size_t)n_heads * CWICK_HIP_LATENT_VDIM * 4;
    size_t sb = sel ? (size_t)n_list * 4 : 0;
    size_t kb = sink ? (size_t)n_heads * 4 : 0;
    Stager st(c->ctx, pad256(qb) + pad256(ob) + pad256(sb) + pad256(kb));
    CWICK_REQUIRE(st.ok, "mla_decode: staging allocation failed");
    const uint16_t *dq = st.in(q, qb);
    const int32_t *dsel = sel ? st.in(sel, sb) : nullptr;
    const float *dsink = sink ? st.in(sink, kb) : nullptr;
    CWICK_REQUIRE(dq && (!sel || dsel) && (!sink || dsink), "mla_decode: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_mla_decode(cwick_hip_latent_rows_dev(c, slot), cwick_hip_latent_scales_dev(c, slot),
                           0, 0, c->capacity, 1, dsel, n_list, dq, n_heads, scale, dsink, dout,
                           c->ctx.stream))
        return 0;
    return st.out(out, dout, ob) && st.wait() ? 1 : 0;
}

int cwick_hip_mla_prefill_chunk(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n,
                                const uint16_t *q, int n_heads, float scale, float *out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q && out, "mla_prefill_chunk: null argument");
    CWICK_REQUIRE(slot >= 0 && slot < c->slots, "mla_prefill_chunk: slot %d of %d", slot, c->slots);
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= c->capacity,
                  "mla_prefill_chunk: positions %lld..%lld outside capacity %lld", (long long)pos0,
                  (long long)(pos0 + n), (long long)c->capacity);
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "mla_prefill_chunk: n_heads %d (1..128)", n_heads);
    size_t qb = (size_t)n * n_heads * CWICK_HIP_LATENT_KDIM * 2;
    size_t ob = (size_t)n * n_heads * CWICK_HIP_LATENT_VDIM * 4;
    Stager st(c->ctx, pad256(qb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "mla_prefill_chunk: staging allocation failed");
    const uint16_t *dq = st.in(q, qb);
    CWICK_REQUIRE(dq, "mla_prefill_chunk: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_mla_prefill(cwick_hip_latent_rows_dev(c, slot), cwick_hip_latent_scales_dev(c, slot),
                            pos0, n, dq, n_heads, scale, dout, c->ctx.stream))
        return 0;
    return st.out(out, dout, ob) && st.wait() ? 1 : 0;
}

int cwick_hip_indexer_scores(cwick_hip_ikeys *c, int slot, int64_t n_keys, const uint16_t *q_idx,
                             const float *w, int n_idx_heads, float *scores) {
    return cwick_hip_indexer_scores_mode(c, slot, n_keys, q_idx, w, n_idx_heads, CWICK_HIP_INDEXER_GLM,
                                         scores);
}

int cwick_hip_indexer_scores_mode(cwick_hip_ikeys *c, int slot, int64_t n_keys, const uint16_t *q_idx,
                                  const float *w, int n_idx_heads, int mode, float *scores) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q_idx && w && scores, "indexer_scores: null argument");
    CWICK_REQUIRE(slot >= 0 && slot < c->slots, "indexer_scores: slot %d of %d", slot, c->slots);
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= c->capacity, "indexer_scores: n_keys %lld, capacity %lld",
                  (long long)n_keys, (long long)c->capacity);
    CWICK_REQUIRE(n_idx_heads >= 1 && n_idx_heads <= 64, "indexer_scores: n_idx_heads %d (1..64)",
                  n_idx_heads);
    size_t qb = (size_t)n_idx_heads * CWICK_HIP_INDEX_DIM * 2, wb = (size_t)n_idx_heads * 4;
    size_t ob = (size_t)n_keys * 4;
    Stager st(c->ctx, pad256(qb) + pad256(wb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "indexer_scores: staging allocation failed");
    const uint16_t *dq = st.in(q_idx, qb);
    const float *dw = st.in(w, wb);
    CWICK_REQUIRE(dq && dw, "indexer_scores: upload failed");
    float *dout = st.room<float>(ob);
    if (!launch_indexer_scores(cwick_hip_ikeys_rows_dev(c, slot), cwick_hip_ikeys_scales_dev(c, slot),
                               0, 0, 1, n_keys, dq, dw, n_idx_heads, mode, dout, c->ctx.stream))
        return 0;
    return st.out(scores, dout, ob) && st.wait() ? 1 : 0;
}

int cwick_hip_indexer_scores_approx(cwick_hip_ikeys *c, int slot, int64_t n_keys,
                                    const uint16_t *q_idx, const float *w, int n_idx_heads,
                                    float *scores, float *bound) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(c && q_idx && w && scores && bound, "indexer_scores_approx: null argument");
    CWICK_REQUIRE(slot >= 0 && slot < c->slots, "indexer_scores_approx: slot %d of %d", slot, c->slots);
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= c->capacity, "indexer_scores_approx: n_keys %lld, capacity %lld",
                  (long long)n_keys, (long long)c->capacity);
    CWICK_REQUIRE(n_idx_heads >= 1 && n_idx_heads <= 64, "indexer_scores_approx: n_idx_heads %d (1..64)",
                  n_idx_heads);
    const int n_slots = indexer_approx_slots(n_keys);
    size_t qb = (size_t)n_idx_heads * CWICK_HIP_INDEX_DIM * 2, wb = (size_t)n_idx_heads * 4;
    size_t ob = (size_t)n_keys * 4, bb = (size_t)n_slots * 4;
    Stager st(c->ctx, pad256(qb) + pad256(wb) + pad256(ob) + pad256(bb) + 256);
    CWICK_REQUIRE(st.ok, "indexer_scores_approx: staging allocation failed");
    const uint16_t *dq = st.in(q_idx, qb);
    const float *dw = st.in(w, wb);
    CWICK_REQUIRE(dq && dw, "indexer_scores_approx: upload failed");
    float *dout = st.room<float>(ob);
    float *dbeta = st.room<float>(bb);
    IndexerBandRow *drow = st.room<IndexerBandRow>(256);
    if (!launch_indexer_approx(cwick_hip_ikeys_rows_dev(c, slot), cwick_hip_ikeys_scales_dev(c, slot), 0, 0,
                               1, n_keys, dq, dw, n_idx_heads, dout, dbeta, drow, nullptr, 0, c->ctx.stream))
        return 0;
    std::vector<float> hb((size_t)n_slots);
    if (!st.out(scores, dout, ob) || !st.out(hb.data(), dbeta, bb) || !st.wait()) return 0;
    float m = hb[0];
    for (int i = 1; i < n_slots; i++) m = (hb[i] <= m) ? m : hb[i];      // NaN sticks
    *bound = m;
    return 1;
}

int cwick_hip_topk(const float *scores, int64_t n, int64_t k, int32_t *out_idx, int64_t *n_out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(scores && out_idx, "topk: null argument");
    CWICK_REQUIRE(n >= 1 && n <= ((int64_t)1 << 24), "topk: n %lld (1..2^24)", (long long)n);
    CWICK_REQUIRE(k >= 1 && k <= 65536, "topk: k %lld (1..65536)", (long long)k);
    // no handle: the calls without one share a context and take turns
    std::lock_guard<std::mutex> lk(g_free_mu);
    if (!g_free_ctx.stream) CWICK_REQUIRE(g_free_ctx.init(), "topk: no stream");
    size_t sb = (size_t)n * 4, ob = (size_t)k * 4;
    Stager st(g_free_ctx, pad256(sb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "topk: staging allocation failed");
    const float *ds = st.in(scores, sb);
    CWICK_REQUIRE(ds, "topk: upload failed");
    int32_t *dout = st.room<int32_t>(ob);
    if (!launch_topk(ds, 1, n, k, dout, g_free_ctx.stream)) return 0;
    int64_t got = k < n ? k : n;
    if (!st.out(out_idx, dout, (size_t)got * 4) || !st.wait()) return 0;
    if (n_out) *n_out = got;
    return 1;
}

int cwick_hip_dsa_decode(cwick_hip_ikeys *ik, cwick_hip_latent *lat, int slot0, int slot_step,
                         int batch, int64_t n_keys, const uint16_t *q_idx, const float *w,
                         int n_idx_heads, int64_t topk, const uint16_t *q, int n_heads, float scale,
                         float *out, int32_t *sel_out) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(ik && lat && q_idx && w && q && out, "dsa_decode: null argument");
    CWICK_REQUIRE(batch >= 1 && batch <= 1024, "dsa_decode: batch %d", batch);
    CWICK_REQUIRE(slot_step == 0 || slot_step == 1, "dsa_decode: slot_step %d (0 or 1)", slot_step);
    int last = slot0 + (batch - 1) * slot_step;
    CWICK_REQUIRE(slot0 >= 0 && last < ik->slots && last < lat->slots,
                  "dsa_decode: slots %d..%d outside the caches", slot0, last);
    CWICK_REQUIRE(n_keys >= 1 && n_keys <= ik->capacity && n_keys <= lat->capacity,
                  "dsa_decode: n_keys %lld exceeds a cache capacity", (long long)n_keys);
    CWICK_REQUIRE(n_idx_heads >= 1 && n_idx_heads <= 64, "dsa_decode: n_idx_heads %d", n_idx_heads);
    CWICK_REQUIRE(n_heads >= 1 && n_heads <= 128, "dsa_decode: n_heads %d", n_heads);
    CWICK_REQUIRE(topk >= 1 && topk <= 65536, "dsa_decode: topk %lld", (long long)topk);
    size_t qib = (size_t)batch * n_idx_heads * CWICK_HIP_INDEX_DIM * 2;
    size_t wb = (size_t)batch * n_idx_heads * 4;
    size_t qb = (size_t)batch * n_heads * CWICK_HIP_LATENT_KDIM * 2;
    size_t scb = (size_t)batch * n_keys * 4, selb = (size_t)batch * topk * 4;
    size_t ob = (size_t)batch * n_heads * CWICK_HIP_LATENT_VDIM * 4;
    // the call runs on the latent cache's context (stream, staging)
    Stager st(lat->ctx, pad256(qib) + pad256(wb) + pad256(qb) + pad256(scb) + pad256(selb) + pad256(ob));
    CWICK_REQUIRE(st.ok, "dsa_decode: staging allocation failed");
    const uint16_t *dqi = st.in(q_idx, qib);
    const float *dw = st.in(w, wb);
    const uint16_t *dq = st.in(q, qb);
    CWICK_REQUIRE(dqi && dw && dq, "dsa_decode: upload failed");
    float *dsc = st.room<float>(scb);
    int32_t *dsel = st.room<int32_t>(selb);
    float *dout = st.room<float>(ob);
    int ok = cwick_hip_dsa_decode_dev(
        cwick_hip_ikeys_rows_dev(ik, slot0), cwick_hip_ikeys_scales_dev(ik, slot0),
        (int64_t)slot_step * ik->capacity * CWICK_HIP_INDEX_DIM, (int64_t)slot_step * ik->capacity,
        cwick_hip_latent_rows_dev(lat, slot0), cwick_hip_latent_scales_dev(lat, slot0),
        (int64_t)slot_step * lat->capacity * CWICK_HIP_LATENT_KDIM,
        (int64_t)slot_step * lat->capacity * CWICK_HIP_LATENT_NBLK, batch, n_keys, dqi, dw,
        n_idx_heads, topk, dq, n_heads, scale, dsc, dsel, dout, lat->ctx.stream);
    if (!ok) return 0;
    if (!st.out(out, dout, ob)) return 0;
    if (sel_out && !st.out(sel_out, dsel, selb)) return 0;
    return st.wait() ? 1 : 0;
}

void cwick_hip_prof_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_on = on != 0;
}

void cwick_hip_prof_reset(void) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    prof_drain_locked();
    for (int i = 0; i < CWICK_HIP_PROF_COUNT; i++) {
        g_prof_ms[i] = 0.0;
        g_prof_n[i] = 0;
    }
}

int cwick_hip_prof_read(int which, double *total_ms, int64_t *launches) {
    clear_error();
    CWICK_REQUIRE(which >= 0 && which < CWICK_HIP_PROF_COUNT, "prof_read: unknown timer %d", which);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    prof_drain_locked();
    if (total_ms) *total_ms = g_prof_ms[which];
    if (launches) *launches = g_prof_n[which];
    return 1;
}

const char *cwick_hip_prof_name(int which) {
    static const char *names[CWICK_HIP_PROF_COUNT] = {
        "gqa_decode_split_kernel", "splitk_merge_wide_kernel<gqa>", "gqa_prefill_kernel",
        "mla_roles_kernel", "mla_merge_frag16_kernel", "indexer kernels", "topk kernels", "mla_prefill64_kernel",
        "mm select kernels", "indexer_approx_kernel"};
    return which >= 0 && which < CWICK_HIP_PROF_COUNT ? names[which] : "";
}

int cwick_hip_mla_absorb_dev(const uint16_t *kv_b_proj, const float *q, int64_t q_batch_stride, int batch,
                             int n_heads, int q_dim, int nope, int rope, int kv_dim, int kv_lora,
                             uint16_t *q_abs, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_absorb(kv_b_proj, q, q_batch_stride, batch, n_heads, q_dim, nope, rope, kv_dim, kv_lora,
                             q_abs, (hipStream_t)stream);
}

int cwick_hip_mla_expand_dev(const uint16_t *kv_b_proj, const float *c_acc, int batch, int n_heads, int nope,
                             int vdim, int kv_dim, int kv_lora, float *attn_out, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mla_expand(kv_b_proj, c_acc, batch, n_heads, nope, vdim, kv_dim, kv_lora, attn_out,
                             (hipStream_t)stream);
}

int cwick_hip_gqa_prepare_dev(const float *q_proj, int64_t q_head_stride, const float *k_proj,
                              const float *v_proj, int64_t n, int64_t pos0, int n_heads, int n_kv_heads,
                              int head_dim, const float *q_norm, const float *k_norm, float eps,
                              const float *rope_cos, const float *rope_sin, int rotary_dim, uint16_t *q_out,
                              cwick_hip_kv *cache, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(cache, "gqa_prepare: null cache");
    CWICK_REQUIRE(n_kv_heads == cache->n_kv_heads && head_dim == cache->head_dim,
                  "gqa_prepare: cache is %d x %d, call says %d x %d", cache->n_kv_heads, cache->head_dim, n_kv_heads,
                  head_dim);
    CWICK_REQUIRE(pos0 >= 0 && n >= 1 && pos0 + n <= cache->capacity, "gqa_prepare: rows %lld..%lld outside capacity %lld",
                  (long long)pos0, (long long)(pos0 + n), (long long)cache->capacity);
    return launch_gqa_prepare(q_proj, q_head_stride, k_proj, v_proj, n, pos0, n_heads, n_kv_heads, head_dim, q_norm,
                              k_norm, eps, rope_cos, rope_sin, rotary_dim, q_out, cache->k, cache->v,
                              (hipStream_t)stream);
}

int cwick_hip_ikeys_pool_append_dev(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n, const float *raw_k,
                                    const float *raw_gate, const uint16_t *ape, const float *k_norm_w,
                                    const float *k_norm_b, float eps, int kpool, float *rows_f32, void *stream) {
    clear_error();
    LATENT_RANGE_CHECK("ikeys_pool_append");
    size_t r0 = (size_t)slot * c->capacity + pos0;
    return launch_ikeys_pool(raw_k, raw_gate, ape, k_norm_w, k_norm_b, eps, kpool, n,
                             c->rows + r0 * CWICK_HIP_INDEX_DIM, c->scales + r0, rows_f32, (hipStream_t)stream);
}

int cwick_hip_candidate_select_dev(const float *scores, int batch, int64_t n, int block, int64_t keep_blocks,
                                   uint8_t *cand, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_candidate_select(scores, batch, n, block, keep_blocks, cand, (hipStream_t)stream);
}

int cwick_hip_candidate_apply_dev(float *scores, const uint8_t *cand, int batch, int64_t n, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_candidate_apply(scores, cand, batch, n, (hipStream_t)stream);
}

int cwick_hip_glm_select_dev(const float *scores, int batch, int64_t n_comp, int64_t npos, int kpool, int64_t topk,
                             int strict, int32_t *sel, int64_t max_sel, int32_t *n_sel, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_glm_select(scores, batch, n_comp, npos, kpool, topk, strict, sel, max_sel, n_sel, (hipStream_t)stream);
}

int cwick_hip_mm_select_dev(const uint16_t *idx_keys, const float *iq, int batch, int64_t limit0, int index_heads,
                            int index_dim, int block, int keep_blocks, float *scores, int64_t score_stride,
                            int32_t *blk_out, int32_t *sel, int64_t max_sel, int32_t *n_sel, void *stream) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return launch_mm_select(idx_keys, iq, batch, limit0, index_heads, index_dim, block, keep_blocks, scores,
                            score_stride, blk_out, sel, max_sel, n_sel, (hipStream_t)stream);
}

int cwick_hip_latent_read_f32(cwick_hip_latent *c, int slot, int64_t pos0, int64_t n, float *rows) {
    clear_error();
    LATENT_RANGE_CHECK("latent_read_f32");
    CWICK_REQUIRE(rows, "latent_read_f32: null argument");
    size_t bytes = (size_t)n * CWICK_HIP_LATENT_KDIM * sizeof(float);
    Stager st(c->ctx, pad256(bytes));
    CWICK_REQUIRE(st.ok, "latent_read_f32: staging allocation failed");
    float *d = st.room<float>(bytes);
    size_t r0 = (size_t)slot * c->capacity + pos0;
    if (!launch_dequant_latent(c->rows + r0 * CWICK_HIP_LATENT_KDIM, c->scales + r0 * CWICK_HIP_LATENT_NBLK, n, d,
                               c->ctx.stream))
        return 0;
    if (!st.out(rows, d, bytes)) return 0;
    return st.wait() ? 1 : 0;
}

int cwick_hip_ikeys_read_f32(cwick_hip_ikeys *c, int slot, int64_t pos0, int64_t n, float *rows) {
    clear_error();
    LATENT_RANGE_CHECK("ikeys_read_f32");
    CWICK_REQUIRE(rows, "ikeys_read_f32: null argument");
    size_t bytes = (size_t)n * CWICK_HIP_INDEX_DIM * sizeof(float);
    Stager st(c->ctx, pad256(bytes));
    CWICK_REQUIRE(st.ok, "ikeys_read_f32: staging allocation failed");
    float *d = st.room<float>(bytes);
    size_t r0 = (size_t)slot * c->capacity + pos0;
    if (!launch_dequant_ikeys(c->rows + r0 * CWICK_HIP_INDEX_DIM, c->scales + r0, n, d, c->ctx.stream)) return 0;
    if (!st.out(rows, d, bytes)) return 0;
    return st.wait() ? 1 : 0;
}

int cwick_hip_probe_hbm_read(size_t bytes, int reps, double *gbps) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return run_probe_hbm_read(bytes, reps, gbps);
}

int cwick_hip_probe_mfma(int kind, int reps, double *tflops) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    return run_probe_mfma(kind, reps, tflops);
}

int cwick_hip_e4m3_table(float *out256) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(out256, "e4m3_table: null argument");
    std::lock_guard<std::mutex> lk(g_free_mu);
    if (!g_free_ctx.stream) CWICK_REQUIRE(g_free_ctx.init(), "e4m3_table: no stream");
    Stager st(g_free_ctx, 1024);
    CWICK_REQUIRE(st.ok, "e4m3_table: staging allocation failed");
    float *d = st.room<float>(1024);
    if (!launch_e4m3_table(d, g_free_ctx.stream)) return 0;
    return st.out(out256, d, 1024) && st.wait() ? 1 : 0;
}

int cwick_hip_lane_ops(const uint32_t *in64, uint32_t *out832) {
    clear_error();
    if (!backend_ready()) return 0;   /* the reason is recorded */
    CWICK_REQUIRE(in64 && out832, "lane_ops: null argument");
    std::lock_guard<std::mutex> lk(g_free_mu);
    if (!g_free_ctx.stream) CWICK_REQUIRE(g_free_ctx.init(), "lane_ops: no stream");
    Stager st(g_free_ctx, 256 + 832 * 4 + 256);
    CWICK_REQUIRE(st.ok, "lane_ops: staging allocation failed");
    const uint32_t *din = st.in(in64, 256);
    uint32_t *dout = st.room<uint32_t>(832 * 4);
    CWICK_REQUIRE(din, "lane_ops: upload failed");
    if (!launch_lane_ops(din, dout, g_free_ctx.stream)) return 0;
    return st.out(out832, dout, 832 * 4) && st.wait() ? 1 : 0;
}

}  // extern "C"
