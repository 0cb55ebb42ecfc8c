// Context, error reporting, per-thread staging, weight upload / fusion.
#include <atomic>
#include <mutex>
#include <thread>
#include <vector>

#include "rmi_internal.h"

namespace {

thread_local char t_error[512] = "";
int g_device = -1;
int g_cus = 0;
size_t g_hbm = 0;
char g_name[128] = "";
std::mutex g_mutex;
// Every context ever made; shutdown empties them (stream and buffers) and leaves the objects, whose owning
// threads may still hold the pointer.  g_generation counts shutdowns: a context of an older generation has no
// stream any more and is rebuilt on its owner's next call.
std::vector<RmiThreadCtx *> g_ctxs;
std::vector<RmiThreadCtx *> g_idle;  // contexts of threads that have exited, handed to the next new thread
std::atomic<uint64_t> g_generation{1};

// The calling thread's context.  When the thread exits its context goes to the idle list, buffers and all, for
// the next thread that needs one: no HIP call runs inside a thread-exit destructor, and a pool that keeps
// starting and ending threads holds as many contexts as it has threads at once, not as many as it ever had.
struct ThreadSlot {
    RmiThreadCtx *c = nullptr;
    ~ThreadSlot() {
        if (!c) return;
        std::lock_guard<std::mutex> lock(g_mutex);
        g_idle.push_back(c);
    }
};
thread_local ThreadSlot t_slot;

}  // namespace

void rmi_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error, sizeof(t_error), fmt, ap);
    va_end(ap);
}

int rmi_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error, sizeof(t_error), fmt, ap);
    va_end(ap);
    return code;
}

bool rmi_ready() { return g_device >= 0; }
int rmi_device_cus() { return g_cus; }
int rmi_device() { return g_device; }

RmiThreadCtx *rmi_thread_ctx() {
    const uint64_t generation = g_generation.load(std::memory_order_acquire);
    RmiThreadCtx *c = t_slot.c;
    if (c && c->generation == generation && c->stream) return c;
    if (hipSetDevice(g_device) != hipSuccess) {
        rmi_set_error("hipSetDevice(%d) failed", g_device);
        return nullptr;
    }
    bool fresh = false;
    if (!c) {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (!g_idle.empty()) {
            c = g_idle.back();
            g_idle.pop_back();
        }
    }
    if (!c) {
        c = new RmiThreadCtx();
        fresh = true;
    }
    if (c->generation != generation || !c->stream) {
        // new, or emptied by a shutdown since its last use: shutdown left no stream and no buffers behind
        c->stream = nullptr;
        // default priority: mixed-priority streams are not used anywhere
        if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess) {
            rmi_set_error("hipStreamCreate failed");
            c->stream = nullptr;
            if (fresh) delete c;
            else {
                std::lock_guard<std::mutex> lock(g_mutex);
                g_idle.push_back(c);
            }
            t_slot.c = nullptr;
            return nullptr;
        }
        c->generation = generation;
    }
    if (fresh) {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_ctxs.push_back(c);
    }
    t_slot.c = c;
    return c;
}

void *rmi_dev_buf(RmiThreadCtx *c, int slot, size_t nbytes) {
    if (nbytes == 0) nbytes = 16;
    if (c->dev_cap[slot] >= nbytes) return c->dev[slot];
    if (c->dev[slot]) {
        // the stream may still read the old buffer
        (void)hipStreamSynchronize(c->stream);
        (void)hipFree(c->dev[slot]);
        c->dev[slot] = nullptr;
        c->dev_cap[slot] = 0;
    }
    size_t cap = (nbytes + 4095) & ~size_t(4095);
    if (hipMalloc(&c->dev[slot], cap) != hipSuccess) {
        rmi_set_error("hipMalloc(%zu) for staging failed", cap);
        return nullptr;
    }
    c->dev_cap[slot] = cap;
    return c->dev[slot];
}

void *rmi_pin_buf(RmiThreadCtx *c, int slot, size_t nbytes) {
    if (nbytes == 0) nbytes = 16;
    if (c->pin_cap[slot] >= nbytes) return c->pin[slot];
    if (c->pin[slot]) {
        (void)hipStreamSynchronize(c->stream);
        (void)hipHostFree(c->pin[slot]);
        c->pin[slot] = nullptr;
        c->pin_cap[slot] = 0;
    }
    size_t cap = (nbytes + 4095) & ~size_t(4095);
    if (hipHostMalloc(&c->pin[slot], cap, hipHostMallocDefault) != hipSuccess) {
        rmi_set_error("hipHostMalloc(%zu) for staging failed", cap);
        return nullptr;
    }
    c->pin_cap[slot] = cap;
    return c->pin[slot];
}

// How the forward_batched entry points of the Kernel trait multiply more than one token; process-wide, read at each call.
static std::atomic<int> g_batched_mode{RMI_HIP_BATCHED_X86_ORDER};
int rmi_batched_mode() { return g_batched_mode.load(std::memory_order_relaxed); }

extern "C" {

const char *rmi_hip_last_error(void) { return t_error; }

int rmi_hip_init(int device) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_device >= 0) {
        if (g_device == device) return RMI_HIP_OK;
        return rmi_fail(RMI_HIP_E_INVALID, "already initialised on device %d", g_device);
    }
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return rmi_fail(RMI_HIP_E_NO_DEVICE, "no HIP device visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count) return rmi_fail(RMI_HIP_E_INVALID, "device %d out of range (have %d)", device, count);
    hipDeviceProp_t prop;
    RMI_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return rmi_fail(RMI_HIP_E_NO_DEVICE, "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
    RMI_HIP_CHECK(hipSetDevice(device));
    int rc = rmi_noalloc_setup(device);
    if (rc != RMI_HIP_OK) return rc;
    g_cus = prop.multiProcessorCount;
    g_hbm = prop.totalGlobalMem;
    snprintf(g_name, sizeof(g_name), "%s (%s)", prop.name, prop.gcnArchName);
    g_device = device;
    return RMI_HIP_OK;
}

void rmi_hip_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_device < 0) return;
    (void)hipDeviceSynchronize();
    for (RmiThreadCtx *c : g_ctxs) {
        for (int i = 0; i < 6; i++) {
            if (c->dev[i]) (void)hipFree(c->dev[i]);
            if (c->pin[i]) (void)hipHostFree(c->pin[i]);
            c->dev[i] = nullptr;
            c->pin[i] = nullptr;
            c->dev_cap[i] = c->pin_cap[i] = 0;
        }
        for (int i = 0; i < 2; i++) {
            if (c->up_pin[i]) (void)hipHostFree(c->up_pin[i]);
            if (c->up_dev[i]) (void)hipFree(c->up_dev[i]);
            if (c->up_done[i]) (void)hipEventDestroy(c->up_done[i]);
            c->up_pin[i] = c->up_dev[i] = nullptr;
            c->up_done[i] = nullptr;
        }
        c->up_cap = 0;
        if (c->stream) (void)hipStreamDestroy(c->stream);
        c->stream = nullptr;
    }
    // contexts stay allocated: their owning threads may still hold the pointer; the new generation tells them
    // that stream and buffers are gone
    g_generation.fetch_add(1, std::memory_order_acq_rel);
    g_device = -1;
}

int rmi_hip_set_forward_batched_mode(int mode) {
    if (mode != RMI_HIP_BATCHED_X86_ORDER && mode != RMI_HIP_BATCHED_AARCH64_ORDER && mode != RMI_HIP_BATCHED_FAST)
        return rmi_fail(RMI_HIP_E_INVALID, "unknown forward_batched mode %d", mode);
    g_batched_mode.store(mode, std::memory_order_relaxed);
    return RMI_HIP_OK;
}

int rmi_hip_get_forward_batched_mode(void) { return rmi_batched_mode(); }

size_t rmi_hip_thread_context_count(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    return g_ctxs.size();
}

int rmi_hip_device_info(char *name, size_t name_len, int *compute_units, size_t *hbm_bytes) {
    RMI_REQUIRE_INIT();
    if (name && name_len) snprintf(name, name_len, "%s", g_name);
    if (compute_units) *compute_units = g_cus;
    if (hbm_bytes) *hbm_bytes = g_hbm;
    return RMI_HIP_OK;
}

void *rmi_hip_malloc(size_t nbytes) {
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    if (!rmi_thread_ctx()) return nullptr;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, nbytes ? nbytes : 16);
    if (e != hipSuccess) {
        rmi_set_error("hipMalloc(%zu) failed: %s", nbytes, hipGetErrorString(e));
        return nullptr;
    }
    return p;
}

void rmi_hip_free(void *dptr) {
    if (dptr) (void)hipFree(dptr);
}

int rmi_hip_memcpy_h2d(void *dst, const void *src, size_t nbytes) {
    RMI_REQUIRE_INIT();
    if (!rmi_thread_ctx()) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice));
    return RMI_HIP_OK;
}

int rmi_hip_memcpy_d2h(void *dst, const void *src, size_t nbytes) {
    RMI_REQUIRE_INIT();
    if (!rmi_thread_ctx()) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost));
    return RMI_HIP_OK;
}

int rmi_hip_synchronize(void) {
    RMI_REQUIRE_INIT();
    if (!rmi_thread_ctx()) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipDeviceSynchronize());
    return RMI_HIP_OK;
}

// ------------------------------------------------------------------ weights

static rmi_hip_weight *alloc_weight(int dtype, uint32_t n_in, uint32_t n_out) {
    rmi_hip_weight *w = new rmi_hip_weight();
    w->dtype = dtype;
    w->n_in = n_in;
    w->n_out = n_out;
    w->n_tiles = (n_out + kTileRows - 1) / kTileRows;
    if (dtype == RMI_HIP_DTYPE_Q8_0 || dtype == RMI_HIP_DTYPE_Q4_0) {
        w->n_units = (n_in / 32 + 7) / 8;
        w->tile_bytes = size_t(w->n_units) * (dtype == RMI_HIP_DTYPE_Q8_0 ? kOctetBytes : kQ40OctetBytes);
    } else {
        w->n_units = n_in / 256;
        w->tile_bytes = size_t(w->n_units) * (dtype == RMI_HIP_DTYPE_Q6_K ? kQ6KSuperBytes : kQ4KSuperBytes);
    }
    w->nbytes = size_t(w->n_tiles) * w->tile_bytes;
    w->data = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->data), w->nbytes ? w->nbytes : 16);
    if (e != hipSuccess) {
        rmi_set_error("hipMalloc(%zu) for a weight failed: %s", w->nbytes, hipGetErrorString(e));
        delete w;
        return nullptr;
    }
    return w;
}

}  // extern "C"

static size_t row_bytes_of(int dtype, uint32_t n_in) {
    switch (dtype) {
        case RMI_HIP_DTYPE_Q8_0: return size_t(n_in / 32) * 34;
        case RMI_HIP_DTYPE_Q4_0: return size_t(n_in / 32) * 18;
        case RMI_HIP_DTYPE_Q6_K: return size_t(n_in / 256) * 210;
        default: return size_t(n_in / 256) * 144;
    }
}

static bool dtype_known(int dtype) {
    return dtype == RMI_HIP_DTYPE_Q8_0 || dtype == RMI_HIP_DTYPE_Q4_0 || dtype == RMI_HIP_DTYPE_Q4_K ||
           dtype == RMI_HIP_DTYPE_Q6_K;
}

// The staging pair of this thread: pinned host chunks the host fills while the previous chunk's copy and repack
// are still running, device chunks the repack kernel reads.  Grows when one 8-row tile is larger than a chunk.
static constexpr size_t kUploadChunkBytes = size_t(16) << 20;

static int upload_staging(RmiThreadCtx *c, size_t tile_src_bytes) {
    const size_t want = tile_src_bytes > kUploadChunkBytes ? tile_src_bytes : kUploadChunkBytes;
    if (c->up_cap >= want) return RMI_HIP_OK;
    RMI_HIP_CHECK(hipStreamSynchronize(c->stream));
    for (int i = 0; i < 2; i++) {
        if (c->up_pin[i]) (void)hipHostFree(c->up_pin[i]);
        if (c->up_dev[i]) (void)hipFree(c->up_dev[i]);
        c->up_pin[i] = c->up_dev[i] = nullptr;
    }
    c->up_cap = 0;
    for (int i = 0; i < 2; i++) {
        RMI_HIP_CHECK(hipHostMalloc(&c->up_pin[i], want, hipHostMallocDefault));
        RMI_HIP_CHECK(hipMalloc(&c->up_dev[i], want));
        if (!c->up_done[i]) RMI_HIP_CHECK(hipEventCreateWithFlags(&c->up_done[i], hipEventDisableTiming));
    }
    c->up_cap = want;
    return RMI_HIP_OK;
}

// host memcpy over a few threads: one core moves 5-10 GB/s (less while it also takes the page faults of a
// freshly mapped file), the link to the GPU several times that
static void copy_to_pinned(uint8_t *dst, const uint8_t *src, size_t n) {
    const size_t kPerThread = size_t(2) << 20;
    size_t n_thr = n / kPerThread;
    if (n_thr > 4) n_thr = 4;
    if (n_thr < 2) {
        memcpy(dst, src, n);
        return;
    }
    const size_t piece = ((n + n_thr - 1) / n_thr + 4095) & ~size_t(4095);
    std::vector<std::thread> pool;
    size_t handed = piece < n ? piece : n;  // bytes [0, handed) are this thread's or a helper's
    try {
        for (size_t t = 1; t < n_thr && handed < n; t++) {
            const size_t off = handed, len = n - off < piece ? n - off : piece;
            pool.emplace_back([=] { memcpy(dst + off, src + off, len); });
            handed = off + len;
        }
    } catch (...) {  // no more threads to be had: this one copies the rest
    }
    memcpy(dst, src, piece < n ? piece : n);
    if (handed < n) memcpy(dst + handed, src + handed, n - handed);
    for (std::thread &th : pool) th.join();
}

int rmi_upload_rows(RmiThreadCtx *c, rmi_hip_weight *w, uint32_t row0, const uint8_t *blocks, uint32_t n_rows) {
    if (row0 % kTileRows != 0 || row0 + n_rows > w->n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "upload of rows %u..%u into a weight of %u rows", row0, row0 + n_rows, w->n_out);
    if ((row0 + n_rows) % kTileRows != 0 && row0 + n_rows != w->n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "a row range that ends inside a tile must end the weight");
    const size_t row_bytes = row_bytes_of(w->dtype, w->n_in);
    if (n_rows == 0 || row_bytes == 0) return RMI_HIP_OK;
    int rc = upload_staging(c, row_bytes * kTileRows);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t rows_per_chunk = uint32_t(c->up_cap / (row_bytes * kTileRows)) * kTileRows;
    uint32_t i = 0;
    for (uint64_t done = 0; done < n_rows; done += rows_per_chunk, i++) {
        const int slot = int(i & 1);
        const uint32_t rows = n_rows - done < rows_per_chunk ? uint32_t(n_rows - done) : rows_per_chunk;
        const size_t nbytes = size_t(rows) * row_bytes;
        // the copy and the repack that last used this pair are done (at once for an event never recorded)
        RMI_HIP_CHECK(hipEventSynchronize(c->up_done[slot]));
        copy_to_pinned(static_cast<uint8_t *>(c->up_pin[slot]), blocks + size_t(done) * row_bytes, nbytes);
        RMI_HIP_CHECK(hipMemcpyAsync(c->up_dev[slot], c->up_pin[slot], nbytes, hipMemcpyHostToDevice, c->stream));
        const uint8_t *src = static_cast<const uint8_t *>(c->up_dev[slot]);
        const uint32_t tile0 = uint32_t((row0 + done) / kTileRows), n_tiles = (rows + kTileRows - 1) / kTileRows;
        rc = w->dtype == RMI_HIP_DTYPE_Q8_0   ? rmi_launch_repack_q8_0(src, w, tile0, n_tiles, c->stream)
             : w->dtype == RMI_HIP_DTYPE_Q4_0 ? rmi_launch_repack_q4_0(src, w, tile0, n_tiles, c->stream)
             : w->dtype == RMI_HIP_DTYPE_Q6_K ? rmi_launch_repack_q6_k(src, w, tile0, n_tiles, c->stream)
                                              : rmi_launch_repack_q4_k(src, w, tile0, n_tiles, c->stream);
        if (rc != RMI_HIP_OK) return rc;
        RMI_HIP_CHECK(hipEventRecord(c->up_done[slot], c->stream));
    }
    return RMI_HIP_OK;
}

rmi_hip_weight *rmi_upload_stack(int dtype, const uint8_t *const *parts, const uint32_t *rows, int n_parts,
                                 uint32_t n_in, bool wait) {
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    const uint32_t block_elems = dtype == RMI_HIP_DTYPE_Q8_0 || dtype == RMI_HIP_DTYPE_Q4_0 ? 32 : 256;
    if (!dtype_known(dtype) || n_parts < 1) {
        rmi_set_error("unknown weight type %d or no parts", dtype);
        return nullptr;
    }
    if (n_in == 0 || n_in % block_elems != 0) {
        rmi_set_error("n_in=%u is not a positive multiple of %u", n_in, block_elems);
        return nullptr;
    }
    uint64_t total = 0;
    bool aligned = true;  // every part but the last ends on a tile boundary
    for (int i = 0; i < n_parts; i++) {
        if (!parts[i] && rows[i]) {
            rmi_set_error("null weight slice");
            return nullptr;
        }
        if (i + 1 < n_parts && rows[i] % kTileRows != 0) aligned = false;
        total += rows[i];
    }
    if (total > 0xffffffffull) {
        rmi_set_error("stacked weight has %llu rows", (unsigned long long)total);
        return nullptr;
    }
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return nullptr;
    if (!aligned) {  // a part that starts inside a tile goes through the row copier
        rmi_hip_weight *acc = nullptr;
        for (int i = 0; i < n_parts; i++) {
            rmi_hip_weight *w = rmi_upload_stack(dtype, parts + i, rows + i, 1, n_in, true);
            rmi_hip_weight *f = w && acc ? rmi_hip_fuse_vstack(acc, w) : w;
            if (acc) {
                rmi_hip_free_weight(acc);
                if (w) rmi_hip_free_weight(w);
            }
            if (!f) return nullptr;
            acc = f;
        }
        return acc;
    }
    rmi_hip_weight *w = alloc_weight(dtype, n_in, uint32_t(total));
    if (!w) return nullptr;
    int rc = RMI_HIP_OK;
    uint32_t row0 = 0;
    for (int i = 0; i < n_parts && rc == RMI_HIP_OK; row0 += rows[i], i++)
        rc = rmi_upload_rows(c, w, row0, parts[i], rows[i]);
    if (rc == RMI_HIP_OK && wait) {
        hipError_t e = hipStreamSynchronize(c->stream);
        if (e != hipSuccess) rc = rmi_fail(RMI_HIP_E_RUNTIME, "weight upload failed: %s", hipGetErrorString(e));
    }
    if (rc != RMI_HIP_OK) {
        rmi_hip_free_weight(w);
        return nullptr;
    }
    return w;
}

extern "C" {

static rmi_hip_weight *upload(int dtype, const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out) {
    const uint32_t block_elems = dtype == RMI_HIP_DTYPE_Q8_0 || dtype == RMI_HIP_DTYPE_Q4_0 ? 32 : 256;
    if (n_in == 0 || n_in % block_elems != 0) {
        rmi_set_error("n_in=%u is not a positive multiple of %u", n_in, block_elems);
        return nullptr;
    }
    const size_t want = size_t(n_out) * row_bytes_of(dtype, n_in);
    if (nbytes < want || (!blocks && want)) {
        rmi_set_error("weight slice holds %zu bytes, %u x %u needs %zu", nbytes, n_out, n_in, want);
        return nullptr;
    }
    return rmi_upload_stack(dtype, &blocks, &n_out, 1, n_in, true);
}

rmi_hip_weight *rmi_hip_upload_q8_0(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out) {
    return upload(RMI_HIP_DTYPE_Q8_0, blocks, nbytes, n_in, n_out);
}

rmi_hip_weight *rmi_hip_upload_q4_k(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out) {
    return upload(RMI_HIP_DTYPE_Q4_K, blocks, nbytes, n_in, n_out);
}

rmi_hip_weight *rmi_hip_upload_q4_0(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out) {
    return upload(RMI_HIP_DTYPE_Q4_0, blocks, nbytes, n_in, n_out);
}

rmi_hip_weight *rmi_hip_upload_q6_k(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out) {
    return upload(RMI_HIP_DTYPE_Q6_K, blocks, nbytes, n_in, n_out);
}

rmi_hip_weight *rmi_hip_fuse_vstack(const rmi_hip_weight *a, const rmi_hip_weight *b) {
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    if (!a || !b || a->dtype != b->dtype || a->n_in != b->n_in) {
        rmi_set_error("fuse_vstack: dtype or n_in differ");
        return nullptr;
    }
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return nullptr;
    rmi_hip_weight *w = alloc_weight(a->dtype, a->n_in, a->n_out + b->n_out);
    if (!w) return nullptr;
    hipError_t e = hipSuccess;
    int rc = RMI_HIP_OK;
    if (w->nbytes) {
        // whole tiles of `a` move as bytes; a ragged last tile and all of `b`
        // when it starts inside a tile go through the row copier
        e = hipMemsetAsync(w->data, 0, w->nbytes, c->stream);
        if (e == hipSuccess) rc = rmi_launch_copy_rows(a, w, 0, c->stream);
        if (e == hipSuccess && rc == RMI_HIP_OK) rc = rmi_launch_copy_rows(b, w, a->n_out, c->stream);
        if (e == hipSuccess && rc == RMI_HIP_OK) e = hipStreamSynchronize(c->stream);
    }
    if (e != hipSuccess || rc != RMI_HIP_OK) {
        if (e != hipSuccess) rmi_set_error("fuse_vstack failed: %s", hipGetErrorString(e));
        rmi_hip_free_weight(w);
        return nullptr;
    }
    return w;
}

void rmi_hip_free_weight(rmi_hip_weight *w) {
    if (!w) return;
    if (w->data) (void)hipFree(w->data);
    delete w;
}

uint32_t rmi_hip_weight_n_in(const rmi_hip_weight *w) { return w ? w->n_in : 0; }
uint32_t rmi_hip_weight_n_out(const rmi_hip_weight *w) { return w ? w->n_out : 0; }
int rmi_hip_weight_dtype(const rmi_hip_weight *w) { return w ? w->dtype : 0; }
size_t rmi_hip_weight_device_bytes(const rmi_hip_weight *w) { return w ? w->nbytes : 0; }
const void *rmi_hip_weight_device_data(const rmi_hip_weight *w) { return w ? w->data : nullptr; }

}  // extern "C"
