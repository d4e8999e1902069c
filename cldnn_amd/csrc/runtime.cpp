// Engine / buffer / event half of the thin HIP layer: hipMalloc buffers with a pinned
// lock() shadow, one hipStream per engine, pooled hipEvents.
#include "kernels.h"
#include "runtime.h"

#include <chrono>
#include <cstring>
#include <thread>

namespace chip {

static thread_local std::string g_last_error;
void set_last_error(const std::string& m) { g_last_error = m; }

size_t dtype_size(int dt)
{
    switch (dt) {
    case CLDNN_HIP_S8:
    case CLDNN_HIP_U8: return 1;
    case CLDNN_HIP_I32:
    case CLDNN_HIP_F32: return 4;
    default: throw error(CLDNN_HIP_INVALID_ARG, "unknown data type");
    }
}

static int fsv_of(int format)
{
    switch (format) {
    case CLDNN_HIP_FMT_FS_B_YX_FSV16: return 16;
    case CLDNN_HIP_FMT_B_FS_YX_FSV4: return 4;
    default: return 1;
    }
}

static void check_tensor(const cldnn_hip_tensor& t)
{
    CHIP_REQUIRE(t.b > 0 && t.f > 0 && t.y > 0 && t.x > 0, CLDNN_HIP_INVALID_ARG, "tensor sizes must be positive");
    CHIP_REQUIRE(t.pad_lo_b >= 0 && t.pad_lo_f >= 0 && t.pad_lo_y >= 0 && t.pad_lo_x >= 0 && t.pad_hi_b >= 0
                     && t.pad_hi_f >= 0 && t.pad_hi_y >= 0 && t.pad_hi_x >= 0,
                 CLDNN_HIP_INVALID_ARG, "tensor padding must be non-negative");
    CHIP_REQUIRE(t.format >= CLDNN_HIP_FMT_BFYX && t.format <= CLDNN_HIP_FMT_B_FS_YX_FSV4, CLDNN_HIP_UNSUPPORTED_FORMAT,
                 "unknown tensor format");
    if (fsv_of(t.format) > 1)
        CHIP_REQUIRE(t.pad_lo_f == 0 && t.pad_hi_f == 0 && t.pad_lo_b == 0 && t.pad_hi_b == 0, CLDNN_HIP_UNSUPPORTED_FORMAT,
                     "blocked formats take spatial padding only");
}

Pitch make_pitch(const cldnn_hip_tensor& t)
{
    check_tensor(t);
    const int64_t B = t.b + t.pad_lo_b + t.pad_hi_b, F = t.f + t.pad_lo_f + t.pad_hi_f;
    const int64_t Y = t.y + t.pad_lo_y + t.pad_hi_y, X = t.x + t.pad_lo_x + t.pad_hi_x;
    Pitch p{};
    p.fsv = fsv_of(t.format);
    p.fs_count = (int32_t)((F + p.fsv - 1) / p.fsv);
    switch (t.format) {
    case CLDNN_HIP_FMT_BFYX: p.px = 1, p.py = X, p.pf = X * Y, p.pb = X * Y * F; break;
    case CLDNN_HIP_FMT_YXFB: p.pb = 1, p.pf = B, p.px = B * F, p.py = B * F * X; break;
    case CLDNN_HIP_FMT_BYXF: p.pf = 1, p.px = F, p.py = F * X, p.pb = F * X * Y; break;
    case CLDNN_HIP_FMT_FS_B_YX_FSV16: p.px = 16, p.py = 16 * X, p.pb = 16 * X * Y, p.pf = 16 * X * Y * B; break;
    case CLDNN_HIP_FMT_B_FS_YX_FSV4: p.px = 4, p.py = 4 * X, p.pf = 4 * X * Y, p.pb = 4 * X * Y * p.fs_count; break;
    }
    p.off = t.pad_lo_b * p.pb + (p.fsv == 1 ? t.pad_lo_f * p.pf : 0) + t.pad_lo_y * p.py + t.pad_lo_x * p.px;
    return p;
}

size_t tensor_elems(const cldnn_hip_tensor& t)
{
    check_tensor(t);
    const int64_t B = t.b + t.pad_lo_b + t.pad_hi_b, F = t.f + t.pad_lo_f + t.pad_hi_f;
    const int64_t Y = t.y + t.pad_lo_y + t.pad_hi_y, X = t.x + t.pad_lo_x + t.pad_hi_x;
    const int fsv = fsv_of(t.format);
    const int64_t Fp = (F + fsv - 1) / fsv * fsv;
    return (size_t)(B * Fp * Y * X);
}

}  // namespace chip

using namespace chip;

void cldnn_hip_engine_s::make_current() const { CHIP_CHECK(hipSetDevice(device)); }

hipEvent_t cldnn_hip_engine_s::take_event()
{
    {
        std::lock_guard<std::mutex> g(pool_mutex);
        if (!event_pool.empty()) {
            hipEvent_t ev = event_pool.back();
            event_pool.pop_back();
            return ev;
        }
    }
    hipEvent_t ev;
    make_current();
    CHIP_CHECK(hipEventCreateWithFlags(&ev, profiling ? hipEventDefault : hipEventDisableTiming));
    return ev;
}

void cldnn_hip_engine_s::give_event(hipEvent_t ev)
{
    std::lock_guard<std::mutex> g(pool_mutex);
    event_pool.push_back(ev);
}

extern "C" {

const char* cldnn_hip_last_error(void) { return g_last_error.c_str(); }

uint32_t cldnn_hip_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return (uint32_t)n;
}

cldnn_hip_status cldnn_hip_engine_create(uint32_t device, uint32_t enable_profiling, cldnn_hip_engine* out)
{
    return guarded([&] {
        CHIP_REQUIRE(out, CLDNN_HIP_INVALID_ARG, "null output handle");
        *out = nullptr;
        uint32_t n = cldnn_hip_device_count();
        CHIP_REQUIRE(n > 0, CLDNN_HIP_DEVICE_ERROR, "no HIP device available (this library has no host fallback)");
        CHIP_REQUIRE(device < n, CLDNN_HIP_INVALID_ARG, "device index out of range");
        auto* e = new cldnn_hip_engine_s();
        try {
            e->device = (int)device;
            e->profiling = enable_profiling != 0;
            e->make_current();
            CHIP_CHECK(hipGetDeviceProperties(&e->props, e->device));
            CHIP_CHECK(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
            e->static_scratch = mfma_static_scratch(e->device);
        } catch (...) {
            delete e;
            throw;
        }
        *out = e;
    });
}

cldnn_hip_status cldnn_hip_engine_retain(cldnn_hip_engine e)
{
    return guarded([&] {
        CHIP_REQUIRE(e, CLDNN_HIP_INVALID_ARG, "null engine");
        e->refs.fetch_add(1);
    });
}

cldnn_hip_status cldnn_hip_engine_release(cldnn_hip_engine e)
{
    return guarded([&] {
        CHIP_REQUIRE(e, CLDNN_HIP_INVALID_ARG, "null engine");
        if (e->refs.fetch_sub(1) == 1) {
            (void)hipSetDevice(e->device);
            (void)hipStreamSynchronize(e->stream);
            for (hipEvent_t ev : e->event_pool) (void)hipEventDestroy(ev);
            (void)hipStreamDestroy(e->stream);
            delete e;
        }
    });
}

cldnn_hip_status cldnn_hip_engine_get_info(cldnn_hip_engine e, cldnn_hip_engine_info* info)
{
    return guarded([&] {
        CHIP_REQUIRE(e && info, CLDNN_HIP_INVALID_ARG, "null argument");
        std::memset(info, 0, sizeof(*info));
        const hipDeviceProp_t& p = e->props;
        info->cores_count = (uint32_t)p.multiProcessorCount;
        info->core_frequency = (uint32_t)(p.clockRate / 1000);
        info->max_work_group_size = (uint64_t)p.maxThreadsPerBlock;
        info->max_local_mem_size = (uint64_t)p.sharedMemPerBlock;
        info->max_global_mem_size = (uint64_t)p.totalGlobalMem;
        info->max_alloc_mem_size = (uint64_t)p.totalGlobalMem;
        info->wavefront_size = (uint32_t)p.warpSize;
        info->xcd_count = 8;  // MI355X: 8 accelerator dies of 32 CUs
        std::strncpy(info->name, p.name, sizeof(info->name) - 1);
        std::strncpy(info->arch, p.gcnArchName, sizeof(info->arch) - 1);
    });
}

void* cldnn_hip_engine_stream(cldnn_hip_engine e) { return e ? (void*)e->stream : nullptr; }

cldnn_hip_status cldnn_hip_engine_flush(cldnn_hip_engine e)
{
    return guarded([&] {
        CHIP_REQUIRE(e, CLDNN_HIP_INVALID_ARG, "null engine");
        // HIP submits eagerly; querying the stream nudges any batched submission
        hipError_t r = hipStreamQuery(e->stream);
        if (r != hipSuccess && r != hipErrorNotReady) CHIP_CHECK(r);
    });
}

cldnn_hip_status cldnn_hip_engine_finish(cldnn_hip_engine e)
{
    return guarded([&] {
        CHIP_REQUIRE(e, CLDNN_HIP_INVALID_ARG, "null engine");
        e->make_current();
        CHIP_CHECK(hipStreamSynchronize(e->stream));
    });
}

int64_t cldnn_hip_engine_used_memory(cldnn_hip_engine e) { return e ? e->used.load() : -1; }
int64_t cldnn_hip_engine_max_used_memory(cldnn_hip_engine e) { return e ? e->max_used.load() : -1; }

// ------------------------------------------------------------------------------------------ buffers
cldnn_hip_status cldnn_hip_buffer_alloc(cldnn_hip_engine e, size_t bytes, cldnn_hip_buffer* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && out, CLDNN_HIP_INVALID_ARG, "null argument");
        *out = nullptr;
        CHIP_REQUIRE(bytes > 0, CLDNN_HIP_INVALID_ARG, "zero-sized buffer");
        e->make_current();
        auto* b = new cldnn_hip_buffer_s();
        // 256 spare bytes: vector loads of a tile's last slice may over-read a few bytes
        hipError_t r = hipMalloc(&b->dev, bytes + 256);
        if (r != hipSuccess) {
            delete b;
            (void)hipGetLastError();
            throw error(CLDNN_HIP_OUT_OF_RESOURCES, std::string("hipMalloc: ") + hipGetErrorString(r));
        }
        b->bytes = bytes;
        b->engine = e;
        e->refs.fetch_add(1);
        CHIP_CHECK(hipMemsetAsync(b->dev, 0, bytes + 256, e->stream));
        int64_t u = e->used.fetch_add((int64_t)bytes) + (int64_t)bytes;
        int64_t m = e->max_used.load();
        while (u > m && !e->max_used.compare_exchange_weak(m, u)) {}
        *out = b;
    });
}

cldnn_hip_status cldnn_hip_buffer_retain(cldnn_hip_buffer b)
{
    return guarded([&] {
        CHIP_REQUIRE(b, CLDNN_HIP_INVALID_ARG, "null buffer");
        b->refs.fetch_add(1);
    });
}

cldnn_hip_status cldnn_hip_buffer_release(cldnn_hip_buffer b)
{
    return guarded([&] {
        CHIP_REQUIRE(b, CLDNN_HIP_INVALID_ARG, "null buffer");
        if (b->refs.fetch_sub(1) == 1) {
            cldnn_hip_engine e = b->engine;
            (void)hipSetDevice(e->device);
            (void)hipStreamSynchronize(e->stream);
            if (b->shadow) (void)hipHostFree(b->shadow);
            (void)hipFree(b->dev);
            e->used.fetch_sub((int64_t)b->bytes);
            delete b;
            cldnn_hip_engine_release(e);
        }
    });
}

void* cldnn_hip_buffer_lock(cldnn_hip_buffer b)
{
    void* result = nullptr;
    guarded([&] {
        CHIP_REQUIRE(b, CLDNN_HIP_INVALID_ARG, "null buffer");
        std::lock_guard<std::mutex> g(b->lock_mutex);
        if (b->lock_count == 0) {
            b->engine->make_current();
            if (!b->shadow) CHIP_CHECK(hipHostMalloc(&b->shadow, b->bytes, hipHostMallocDefault));
            CHIP_CHECK(hipMemcpyAsync(b->shadow, b->dev, b->bytes, hipMemcpyDeviceToHost, b->engine->stream));
            CHIP_CHECK(hipStreamSynchronize(b->engine->stream));
        }
        ++b->lock_count;
        result = b->shadow;
    });
    return result;
}

cldnn_hip_status cldnn_hip_buffer_unlock(cldnn_hip_buffer b)
{
    return guarded([&] {
        CHIP_REQUIRE(b, CLDNN_HIP_INVALID_ARG, "null buffer");
        std::lock_guard<std::mutex> g(b->lock_mutex);
        CHIP_REQUIRE(b->lock_count > 0, CLDNN_HIP_ERROR, "unlock without lock");
        if (--b->lock_count == 0) {
            b->engine->make_current();
            CHIP_CHECK(hipMemcpyAsync(b->dev, b->shadow, b->bytes, hipMemcpyHostToDevice, b->engine->stream));
            CHIP_CHECK(hipStreamSynchronize(b->engine->stream));
        }
    });
}

cldnn_hip_status cldnn_hip_buffer_fill(cldnn_hip_buffer b, uint8_t pattern)
{
    return guarded([&] {
        CHIP_REQUIRE(b, CLDNN_HIP_INVALID_ARG, "null buffer");
        b->engine->make_current();
        CHIP_CHECK(hipMemsetAsync(b->dev, pattern, b->bytes, b->engine->stream));
    });
}

void* cldnn_hip_buffer_device_ptr(cldnn_hip_buffer b) { return b ? b->dev : nullptr; }
size_t cldnn_hip_buffer_size(cldnn_hip_buffer b) { return b ? b->bytes : 0; }

cldnn_hip_status cldnn_hip_buffer_write(cldnn_hip_buffer b, size_t offset, const void* host, size_t bytes)
{
    return guarded([&] {
        CHIP_REQUIRE(b && host, CLDNN_HIP_INVALID_ARG, "null argument");
        CHIP_REQUIRE(offset + bytes <= b->bytes, CLDNN_HIP_INVALID_ARG, "write beyond the end of the buffer");
        b->engine->make_current();
        CHIP_CHECK(hipMemcpyAsync((char*)b->dev + offset, host, bytes, hipMemcpyHostToDevice, b->engine->stream));
        CHIP_CHECK(hipStreamSynchronize(b->engine->stream));
    });
}

cldnn_hip_status cldnn_hip_buffer_read(cldnn_hip_buffer b, size_t offset, void* host, size_t bytes)
{
    return guarded([&] {
        CHIP_REQUIRE(b && host, CLDNN_HIP_INVALID_ARG, "null argument");
        CHIP_REQUIRE(offset + bytes <= b->bytes, CLDNN_HIP_INVALID_ARG, "read beyond the end of the buffer");
        b->engine->make_current();
        CHIP_CHECK(hipMemcpyAsync(host, (const char*)b->dev + offset, bytes, hipMemcpyDeviceToHost, b->engine->stream));
        CHIP_CHECK(hipStreamSynchronize(b->engine->stream));
    });
}

// ------------------------------------------------------------------------------------------ events
static cldnn_hip_event new_event(cldnn_hip_engine e, bool user)
{
    auto* ev = new cldnn_hip_event_s();
    ev->engine = e;
    ev->user = user;
    e->refs.fetch_add(1);
    return ev;
}

cldnn_hip_status cldnn_hip_event_create_user(cldnn_hip_engine e, uint32_t set, cldnn_hip_event* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && out, CLDNN_HIP_INVALID_ARG, "null argument");
        cldnn_hip_event ev = new_event(e, true);
        ev->user_set.store(set != 0);
        *out = ev;
    });
}

cldnn_hip_status cldnn_hip_event_record_begin(cldnn_hip_engine e, cldnn_hip_event* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && out, CLDNN_HIP_INVALID_ARG, "null argument");
        cldnn_hip_event ev = new_event(e, false);
        *out = ev;
        if (e->profiling) {
            ev->start = e->take_event();
            CHIP_CHECK(hipEventRecord(ev->start, e->stream));
        }
    });
}

cldnn_hip_status cldnn_hip_event_record_end(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev && !ev->user, CLDNN_HIP_INVALID_ARG, "not a recordable event");
        CHIP_REQUIRE(!ev->stop, CLDNN_HIP_ERROR, "event recorded twice");
        ev->stop = ev->engine->take_event();
        CHIP_CHECK(hipEventRecord(ev->stop, ev->engine->stream));
    });
}

cldnn_hip_status cldnn_hip_event_record(cldnn_hip_engine e, cldnn_hip_event* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && out, CLDNN_HIP_INVALID_ARG, "null argument");
        cldnn_hip_event ev = new_event(e, false);
        *out = ev;
        ev->stop = e->take_event();
        CHIP_CHECK(hipEventRecord(ev->stop, e->stream));
    });
}

cldnn_hip_status cldnn_hip_event_create_deferred(cldnn_hip_engine e, cldnn_hip_event* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && out, CLDNN_HIP_INVALID_ARG, "null argument");
        cldnn_hip_event ev = new_event(e, false);
        ev->deferred = true;
        ev->deferred_pending = true;
        *out = ev;
    });
}

cldnn_hip_status cldnn_hip_event_record_deferred(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev && ev->deferred, CLDNN_HIP_INVALID_ARG, "not a deferred event");
        hipError_t r = hipSuccess;
        {
            std::lock_guard<std::mutex> g(ev->deferred_mutex);
            CHIP_REQUIRE(ev->deferred_pending, CLDNN_HIP_ERROR, "deferred event recorded twice");
            ev->engine->make_current();
            ev->stop = ev->engine->take_event();
            r = hipEventRecord(ev->stop, ev->engine->stream);
            ev->deferred_pending = false;  // also after a failed record: nobody may wait for ever
        }
        ev->deferred_cv.notify_all();
        CHIP_CHECK(r);
    });
}

// a deferred event: block until the work it stands for has been submitted
static void await_submission(cldnn_hip_event ev)
{
    if (!ev->deferred) return;
    std::unique_lock<std::mutex> g(ev->deferred_mutex);
    ev->deferred_cv.wait(g, [&] { return !ev->deferred_pending; });
}

static bool submission_pending(cldnn_hip_event ev)
{
    if (!ev->deferred) return false;
    std::lock_guard<std::mutex> g(ev->deferred_mutex);
    return ev->deferred_pending;
}

cldnn_hip_status cldnn_hip_event_retain(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev, CLDNN_HIP_INVALID_ARG, "null event");
        ev->refs.fetch_add(1);
    });
}

cldnn_hip_status cldnn_hip_event_release(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev, CLDNN_HIP_INVALID_ARG, "null event");
        if (ev->refs.fetch_sub(1) == 1) {
            cldnn_hip_engine e = ev->engine;
            // an event still in flight must not be handed to the next user before it completes
            if (ev->stop) {
                (void)hipEventSynchronize(ev->stop);
                e->give_event(ev->stop);
            }
            if (ev->start) e->give_event(ev->start);
            delete ev;
            cldnn_hip_engine_release(e);
        }
    });
}

static void fire_handlers(cldnn_hip_event ev)
{
    std::vector<std::pair<cldnn_hip_event_handler, void*>> hs;
    {
        std::lock_guard<std::mutex> g(ev->handler_mutex);
        ev->handlers_fired = true;
        hs.swap(ev->handlers);
    }
    for (auto& h : hs) h.first(h.second);
}

cldnn_hip_status cldnn_hip_event_wait(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev, CLDNN_HIP_INVALID_ARG, "null event");
        if (ev->user) {
            while (!ev->user_set.load()) std::this_thread::sleep_for(std::chrono::microseconds(50));
        } else {
            await_submission(ev);
            if (ev->stop) CHIP_CHECK(hipEventSynchronize(ev->stop));
        }
        fire_handlers(ev);
    });
}

int32_t cldnn_hip_event_is_set(cldnn_hip_event ev)
{
    if (!ev) return 0;
    if (ev->user) return ev->user_set.load() ? 1 : 0;
    if (submission_pending(ev) || !ev->stop) return 0;
    hipError_t r = hipEventQuery(ev->stop);
    if (r == hipSuccess) return 1;
    (void)hipGetLastError();
    return 0;
}

int32_t cldnn_hip_event_is_user(cldnn_hip_event ev) { return ev && ev->user ? 1 : 0; }

cldnn_hip_status cldnn_hip_event_set(cldnn_hip_event ev)
{
    return guarded([&] {
        CHIP_REQUIRE(ev && ev->user, CLDNN_HIP_INVALID_ARG, "only user events can be set");
        ev->user_set.store(true);
        fire_handlers(ev);
    });
}

cldnn_hip_status cldnn_hip_event_add_handler(cldnn_hip_event ev, cldnn_hip_event_handler h, void* param)
{
    return guarded([&] {
        CHIP_REQUIRE(ev && h, CLDNN_HIP_INVALID_ARG, "null argument");
        bool fire_now = false;
        {
            std::lock_guard<std::mutex> g(ev->handler_mutex);
            if (ev->handlers_fired || cldnn_hip_event_is_set(ev)) fire_now = true;
            else ev->handlers.emplace_back(h, param);
        }
        if (fire_now) {
            h(param);
            return;
        }
        if (!ev->user) {
            // completion is observed from a helper thread, the way a driver thread would call back
            cldnn_hip_event_retain(ev);
            std::thread([ev] {
                (void)hipSetDevice(ev->engine->device);
                await_submission(ev);
                if (ev->stop) (void)hipEventSynchronize(ev->stop);
                fire_handlers(ev);
                cldnn_hip_event_release(ev);
            }).detach();
        }
    });
}

cldnn_hip_status cldnn_hip_event_elapsed_ns(cldnn_hip_event ev, uint64_t* ns)
{
    return guarded([&] {
        CHIP_REQUIRE(ev && ns, CLDNN_HIP_INVALID_ARG, "null argument");
        *ns = 0;
        if (!ev->start || !ev->stop) return;
        await_submission(ev);
        CHIP_CHECK(hipEventSynchronize(ev->stop));
        float ms = 0.f;
        CHIP_CHECK(hipEventElapsedTime(&ms, ev->start, ev->stop));
        *ns = (uint64_t)((double)ms * 1e6);
    });
}

cldnn_hip_status cldnn_hip_engine_wait_events(cldnn_hip_engine e, const cldnn_hip_event* evs, size_t n)
{
    return guarded([&] {
        CHIP_REQUIRE(e && (evs || n == 0), CLDNN_HIP_INVALID_ARG, "null argument");
        for (size_t i = 0; i < n; ++i) {
            cldnn_hip_event ev = evs[i];
            CHIP_REQUIRE(ev, CLDNN_HIP_INVALID_ARG, "null event in dependency list");
            if (ev->user) {
                // a stream cannot wait for a host flag: hold back submission until it is set
                while (!ev->user_set.load()) std::this_thread::sleep_for(std::chrono::microseconds(50));
            } else {
                await_submission(ev);
                if (ev->stop && ev->engine != e) CHIP_CHECK(hipStreamWaitEvent(e->stream, ev->stop, 0));
            }
            // same engine: the single in-order stream already orders the work
        }
    });
}

size_t cldnn_hip_tensor_bytes(const cldnn_hip_tensor* t)
{
    size_t r = 0;
    guarded([&] {
        CHIP_REQUIRE(t, CLDNN_HIP_INVALID_ARG, "null tensor");
        r = tensor_elems(*t) * dtype_size(t->dtype);
    });
    return r;
}

int64_t cldnn_hip_tensor_offset(const cldnn_hip_tensor* t, int32_t b, int32_t f, int32_t y, int32_t x)
{
    int64_t r = -1;
    guarded([&] {
        CHIP_REQUIRE(t, CLDNN_HIP_INVALID_ARG, "null tensor");
        r = make_pitch(*t).at(b, f, y, x);
    });
    return r;
}

}  // extern "C"
