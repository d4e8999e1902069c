// Engine, buffer and event objects behind the C handles of cldnn_hip.h.
#pragma once
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"

struct cldnn_hip_engine_s {
    std::atomic<int> refs{1};
    int device = 0;
    bool profiling = false;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
    std::atomic<int64_t> used{0}, max_used{0};
    std::mutex pool_mutex;
    std::vector<hipEvent_t> event_pool;  // recycled hipEvents (the reference pools its cl events too)
    // this device's copy of the scratch array inside the code object, looked up when the engine is created, so that
    // cldnn_hip_conv_enqueue_static_scratch only launches
    void* static_scratch = nullptr;

    hipEvent_t take_event();
    void give_event(hipEvent_t ev);
    void make_current() const;
};

struct cldnn_hip_buffer_s {
    std::atomic<int> refs{1};
    cldnn_hip_engine engine = nullptr;
    void* dev = nullptr;
    size_t bytes = 0;
    std::mutex lock_mutex;
    int lock_count = 0;
    void* shadow = nullptr;  // pinned host mirror, allocated on first lock
};

struct cldnn_hip_event_s {
    std::atomic<int> refs{1};
    cldnn_hip_engine engine = nullptr;
    bool user = false;
    std::atomic<bool> user_set{false};
    hipEvent_t start = nullptr;  // only with profiling
    hipEvent_t stop = nullptr;
    // a deferred event stands for work that has not been submitted yet: it is recorded later, and whoever waits for
    // it first waits for that
    bool deferred = false;
    std::mutex deferred_mutex;
    std::condition_variable deferred_cv;
    bool deferred_pending = false;
    std::mutex handler_mutex;
    bool handlers_fired = false;
    std::vector<std::pair<cldnn_hip_event_handler, void*>> handlers;
};

namespace chip {
// translate exceptions at the C boundary (same idea as the reference's exception_handler,
// src/include/api_impl.h:63-110)
template <class F>
cldnn_hip_status guarded(F&& f)
{
    try {
        f();
        return CLDNN_HIP_SUCCESS;
    } catch (const error& e) {
        set_last_error(e.what());
        return e.status;
    } catch (const std::bad_alloc&) {
        set_last_error("host allocation failed");
        return CLDNN_HIP_OUT_OF_RESOURCES;
    } catch (const std::exception& e) {
        set_last_error(e.what());
        return CLDNN_HIP_ERROR;
    }
}
}  // namespace chip
