// Slot pool for offloaded experts and the pinned-host -> HBM prefetch that feeds it.
//
// Replaces _UniMem (MOLE/cpp/umemory.cpp:92-183, MOLE/cpp/define.hpp:143-193),
// _CPUParamCore::prefetch_to (MOLE/cpp/uparameter.cpp:58-63), _ParamProxy::fetch
// (MOLE/cpp/umemory.cpp:189-205), _MOLECore::prefetch_fwd/bwd (MOLE/cpp/core.cpp:41-75),
// _BatchRecord::fetch_para (MOLE/cpp/core.cpp:110-143), the copy wrappers
// (MOLE/cpp/transfer.cu:9-12) and the "tran" stream with its events (MOLE/cpp/stream.cpp).
//
// The pool is four device arrays of pool_size slots (w1, b1, w2, b2).  Copies run on one
// library-owned stream at default priority; ordering against the caller's compute stream is by
// events only: a "parameters landed" event the compute stream waits on, and one "slot released"
// event per slot that the copy stream waits on before overwriting the slot.
#include "common.h"

#include <algorithm>
#include <array>
#include <vector>

namespace mole {

struct UniMem {
    int device = 0, pool_size = 0, dtype = 0;
    size_t slot_bytes[4] = {0, 0, 0, 0};
    char *pool[4] = {nullptr, nullptr, nullptr, nullptr};
    hipStream_t tran = nullptr, tranback = nullptr;
    hipEvent_t para_event = nullptr, grads_ready = nullptr, state_free = nullptr, state_ready = nullptr, wb_done = nullptr;
    bool para_recorded = false;
    std::vector<hipEvent_t> slot_event;
    std::vector<char> slot_pending;  // slot_event[s] was recorded and not yet waited on
    std::vector<hipEvent_t> landed_event;   // recorded on the copy stream once the slot's expert has arrived
    std::vector<char> landed_valid;
    std::vector<uint64_t> slot_tag;         // the caller's tag under which the slot was last filled (0: none)
    std::vector<const void *> slot_src;     // host address of the expert (its first parameter array) the slot holds
    uint64_t bytes_reused = 0;
    std::vector<std::array<int, 2>> stk;  // (layer, n)
    int virtual_offset = 0, view_pool_size = 0;
    // copy statistics
    std::vector<std::array<hipEvent_t, 2>> timers;
    size_t timers_used = 0;
    uint64_t bytes_open = 0, bytes_last = 0;
    float ms_last = 0.f;
    std::vector<std::array<hipEvent_t, 2>> wb_timers;
    size_t wb_timers_used = 0;
    uint64_t wb_bytes_open = 0, wb_bytes_last = 0;
    float wb_ms_last = 0.f;
    char *zeros = nullptr;           // one zeroed slot of the largest parameter kind (mole_unimem_zero_grads_ids)
    bool zeros_ready = false;
};

// The next event pair of a copy stream's statistics.  A caller that never synchronises the stream would
// grow the list without bound: past MAX_TIMERS pairs the last one is reused (the statistics then miss the
// copies in between; nothing else depends on them).
constexpr size_t MAX_TIMERS = 4096;
static int next_timer(std::vector<std::array<hipEvent_t, 2>> &timers, size_t &used, std::array<hipEvent_t, 2> **out) {
    if (used == MAX_TIMERS) --used;
    if (used == timers.size()) {
        std::array<hipEvent_t, 2> p;
        MOLE_HIP(hipEventCreate(&p[0]));
        MOLE_HIP(hipEventCreate(&p[1]));
        timers.push_back(p);
    }
    *out = &timers[used++];
    return 0;
}
static int next_timer(UniMem *u, std::array<hipEvent_t, 2> **out) { return next_timer(u->timers, u->timers_used, out); }

// Host -> pool copy of experts ids[0..n) (or base, base+1, .. when ids is null) into slots [slot0, slot0+n).
// Every expert travels as its own four copies followed by the slot's "landed" event, so that compute on the
// first experts of a large prefetch starts while the later ones are still on the bus (one event for the whole
// prefetch made a layer wait for all of it: 134 ms for 32 experts of 235 MB).  Before a slot is overwritten the
// copy stream waits for the compute that last used it, slot by slot, so that a prefetch trails the compute
// that still owns the later slots instead of waiting for all of it.
//
// tag != 0: a slot that was last filled under the same tag from the same host expert is left as it is (nothing is
// copied, its earlier "landed" event still stands): the caller vouches that the host arrays have not changed since -
// the host side hands out one tag per forward pass of a layer and uses it again for that pass's backward only.
static int copy_experts(UniMem *u, const void *const host_src[4], int slot0, const int32_t *ids, int base, int n,
                        uint64_t tag = 0) {
    if (n <= 0) return 0;
    auto id_of = [&](int i) { return ids ? (int)ids[i] : base + i; };
    int i = 0;
    while (i < n) {
        auto resident = [&](int j) {
            return tag != 0 && u->slot_tag[slot0 + j] == tag &&
                   u->slot_src[slot0 + j] == (const char *)host_src[0] + (size_t)id_of(j) * u->slot_bytes[0];
        };
        if (resident(i)) {
            for (int p = 0; p < 4; ++p) u->bytes_reused += u->slot_bytes[p];
            ++i;
            continue;
        }
        // a run: experts up to the next slot that is still waited for or already holds its expert (one pair of
        // timing events per run)
        int run = 1;
        while (i + run < n && !u->slot_pending[slot0 + i + run] && !resident(i + run)) ++run;
        if (u->slot_pending[slot0 + i]) {
            MOLE_HIP(hipStreamWaitEvent(u->tran, u->slot_event[slot0 + i], 0));
            u->slot_pending[slot0 + i] = 0;
        }
        std::array<hipEvent_t, 2> *tm;
        if (int rc = next_timer(u, &tm)) return rc;
        MOLE_HIP(hipEventRecord((*tm)[0], u->tran));
        // Small experts (below 1 MiB) with consecutive ids travel as one copy per parameter kind for up to 16 MiB at a
        // time: their slots and their host arrays are both contiguous, and four calls per expert cost more than the
        // bytes they move (hundreds of experts with 8-28 KB biases).  Every slot of a group still gets its own "landed"
        // event, recorded behind the group's copies.
        size_t expert_bytes = 0;
        for (int p = 0; p < 4; ++p) expert_bytes += u->slot_bytes[p];
        const int group_max = expert_bytes < ((size_t)1 << 20) ? (int)std::max<size_t>(1, ((size_t)16 << 20) / std::max<size_t>(expert_bytes, 1)) : 1;
        for (int j = i; j < i + run;) {
            int grp = 1;
            while (grp < group_max && j + grp < i + run && id_of(j + grp) == id_of(j) + grp) ++grp;
            for (int p = 0; p < 4; ++p) {
                const size_t sb = u->slot_bytes[p];
                MOLE_HIP(hipMemcpyAsync(u->pool[p] + (size_t)(slot0 + j) * sb, (const char *)host_src[p] + (size_t)id_of(j) * sb,
                                        sb * grp, hipMemcpyHostToDevice, u->tran));
                u->bytes_open += (uint64_t)sb * grp;
            }
            for (int q = j; q < j + grp; ++q) {
                MOLE_HIP(hipEventRecord(u->landed_event[slot0 + q], u->tran));
                u->landed_valid[slot0 + q] = 1;
                u->slot_tag[slot0 + q] = tag;
                u->slot_src[slot0 + q] = (const char *)host_src[0] + (size_t)id_of(q) * u->slot_bytes[0];
            }
            j += grp;
        }
        MOLE_HIP(hipEventRecord((*tm)[1], u->tran));
        i += run;
    }
    MOLE_HIP(hipEventRecord(u->para_event, u->tran));
    u->para_recorded = true;
    return 0;
}

static void destroy_members(UniMem *u) {
    for (auto &e : u->slot_event) if (e) (void)hipEventDestroy(e);
    for (auto &e : u->landed_event) if (e) (void)hipEventDestroy(e);
    for (auto &t : u->timers) { (void)hipEventDestroy(t[0]); (void)hipEventDestroy(t[1]); }
    for (auto &t : u->wb_timers) { (void)hipEventDestroy(t[0]); (void)hipEventDestroy(t[1]); }
    for (hipEvent_t e : {u->para_event, u->grads_ready, u->state_free, u->state_ready, u->wb_done}) if (e) (void)hipEventDestroy(e);
    if (u->tran) (void)hipStreamDestroy(u->tran);
    if (u->tranback) (void)hipStreamDestroy(u->tranback);
    for (int p = 0; p < 4; ++p) if (u->pool[p]) (void)hipFree(u->pool[p]);
    if (u->zeros) (void)hipFree(u->zeros);
    delete u;
}

// streams, events and slot events of a freshly allocated pool
static int create_members(UniMem *u) {
    MOLE_HIP(hipStreamCreateWithFlags(&u->tran, hipStreamNonBlocking));
    MOLE_HIP(hipStreamCreateWithFlags(&u->tranback, hipStreamNonBlocking));
    MOLE_HIP(hipEventCreateWithFlags(&u->para_event, hipEventDisableTiming));
    MOLE_HIP(hipEventCreateWithFlags(&u->grads_ready, hipEventDisableTiming));
    MOLE_HIP(hipEventCreateWithFlags(&u->state_free, hipEventDisableTiming));
    MOLE_HIP(hipEventCreateWithFlags(&u->state_ready, hipEventDisableTiming));
    MOLE_HIP(hipEventCreateWithFlags(&u->wb_done, hipEventDisableTiming));
    u->slot_event.assign(u->pool_size, nullptr);
    u->slot_pending.assign(u->pool_size, 0);
    for (int s = 0; s < u->pool_size; ++s) MOLE_HIP(hipEventCreateWithFlags(&u->slot_event[s], hipEventDisableTiming));
    u->landed_event.assign(u->pool_size, nullptr);
    u->landed_valid.assign(u->pool_size, 0);
    u->slot_tag.assign(u->pool_size, 0);
    u->slot_src.assign(u->pool_size, nullptr);
    for (int s = 0; s < u->pool_size; ++s) MOLE_HIP(hipEventCreateWithFlags(&u->landed_event[s], hipEventDisableTiming));
    return 0;
}

static bool ids_ok(const int32_t *ids, int n) {
    for (int i = 0; i < n; ++i) if (ids[i] < 0) return false;
    return true;
}

}  // namespace mole

using namespace mole;

#define UM(handle)                                                        \
    UniMem *u = (UniMem *)(handle);                                        \
    MOLE_REQUIRE(u != nullptr, "%s: null handle", __func__)

extern "C" int mole_unimem_create(int device, int pool_size, int dtype, int64_t F, int64_t M, void **handle) {
    MOLE_REQUIRE(handle != nullptr, "mole_unimem_create: null handle pointer");
    MOLE_REQUIRE(pool_size >= 0 && F > 0 && M > 0, "mole_unimem_create: bad sizes pool=%d F=%lld M=%lld", pool_size,
                 (long long)F, (long long)M);
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_unimem_create: bad dtype %d", dtype);
    MOLE_HIP(hipSetDevice(device));
    UniMem *u = new UniMem();
    u->device = device;
    u->pool_size = pool_size;
    u->dtype = dtype;
    const size_t es = dtype == MOLE_BF16 ? 2 : 4;
    u->slot_bytes[0] = (size_t)F * M * es;
    u->slot_bytes[1] = (size_t)F * es;
    u->slot_bytes[2] = (size_t)F * M * es;
    u->slot_bytes[3] = (size_t)M * es;
    u->view_pool_size = pool_size;
    for (int p = 0; p < 4 && pool_size > 0; ++p) {
        hipError_t e = hipMalloc((void **)&u->pool[p], u->slot_bytes[p] * pool_size);
        if (e != hipSuccess) {
            set_error("mole_unimem_create: hipMalloc of %zu bytes failed: %s", u->slot_bytes[p] * pool_size,
                      hipGetErrorString(e));
            destroy_members(u);
            return MOLE_E_NOMEM;
        }
    }
    if (int rc = create_members(u)) {   // nothing allocated so far outlives a failure
        destroy_members(u);
        return rc;
    }
    *handle = u;
    return 0;
}

extern "C" int mole_unimem_destroy(void *handle) {
    UM(handle);
    (void)hipSetDevice(u->device);
    (void)hipStreamSynchronize(u->tran);
    (void)hipStreamSynchronize(u->tranback);
    destroy_members(u);
    return 0;
}

extern "C" int mole_unimem_clear_virtual_mem(void *handle) {
    UM(handle);
    u->stk.clear();
    u->virtual_offset = 0;
    u->view_pool_size = u->pool_size;
    return 0;
}

extern "C" int mole_unimem_view_pool_size(void *handle, int *out) {
    UM(handle);
    *out = u->view_pool_size;
    return 0;
}

extern "C" int mole_unimem_virtual_offset(void *handle, int *out) {
    UM(handle);
    *out = u->virtual_offset;
    return 0;
}

extern "C" int mole_unimem_slot_ptr(void *handle, int p_id, int slot, void **out) {
    UM(handle);
    MOLE_REQUIRE(p_id >= 0 && p_id < 4 && slot >= 0 && slot < u->pool_size && out, "mole_unimem_slot_ptr: bad p_id %d / slot %d", p_id, slot);
    *out = u->pool[p_id] + (size_t)slot * u->slot_bytes[p_id];
    return 0;
}

static int prefetch_impl(UniMem *u, const char *who, int layer, const void *const host_src[4], const int32_t *ids, int base, int n,
                         uint64_t tag) {
    if (n == 0) return 0;
    MOLE_REQUIRE(n > 0 && base >= 0 && host_src && host_src[0] && host_src[1] && host_src[2] && host_src[3] && (!ids || ids_ok(ids, n)),
                 "%s: bad arguments (base=%d n=%d)", who, base, n);
    if (n > u->view_pool_size) {
        set_error("%s: %d experts do not fit the %d free pool slots", who, n, u->view_pool_size);
        return MOLE_E_STATE;
    }
    if (int rc = copy_experts(u, host_src, u->virtual_offset, ids, base, n, tag)) return rc;
    if (!u->stk.empty() && u->stk.back()[0] == layer) u->stk.back()[1] += n;
    else u->stk.push_back({layer, n});
    u->virtual_offset += n;
    u->view_pool_size -= n;
    return 0;
}

extern "C" int mole_unimem_prefetch(void *handle, int layer, const void *const host_src[4], int base, int n) {
    UM(handle);
    return prefetch_impl(u, "mole_unimem_prefetch", layer, host_src, nullptr, base, n, 0);
}

extern "C" int mole_unimem_prefetch_ids(void *handle, int layer, const void *const host_src[4], const int32_t *expert_ids, int n,
                                        uint64_t tag) {
    UM(handle);
    MOLE_REQUIRE(n == 0 || expert_ids, "mole_unimem_prefetch_ids: null expert list");
    return prefetch_impl(u, "mole_unimem_prefetch_ids", layer, host_src, expert_ids, 0, n, tag);
}

extern "C" int mole_unimem_reserve(void *handle, int layer, int n, void **slot_ptrs_out) {
    UM(handle);
    MOLE_REQUIRE(n >= 0 && slot_ptrs_out, "mole_unimem_reserve: bad arguments (n=%d)", n);
    if (n > u->view_pool_size) {
        set_error("mole_unimem_reserve: %d experts do not fit the %d free pool slots", n, u->view_pool_size);
        return MOLE_E_STATE;
    }
    for (int p = 0; p < 4; ++p) slot_ptrs_out[p] = u->pool_size > 0 ? u->pool[p] + (size_t)u->virtual_offset * u->slot_bytes[p] : nullptr;
    if (n == 0) return 0;
    for (int s = u->virtual_offset; s < u->virtual_offset + n; ++s) u->slot_tag[s] = 0;   // the caller fills them
    if (!u->stk.empty() && u->stk.back()[0] == layer) u->stk.back()[1] += n;
    else u->stk.push_back({layer, n});
    u->virtual_offset += n;
    u->view_pool_size -= n;
    return 0;
}

extern "C" int mole_unimem_fetch_top(void *handle, int layer, int *n_out) {
    UM(handle);
    MOLE_REQUIRE(n_out != nullptr, "mole_unimem_fetch_top: null output");
    *n_out = 0;
    if (!u->stk.empty() && u->stk.back()[0] == layer) {
        const int n = u->stk.back()[1];
        u->stk.pop_back();
        u->virtual_offset -= n;
        u->view_pool_size += n;
        *n_out = n;
    }
    return 0;
}

static int fetch_impl(UniMem *u, const char *who, const void *const host_src[4], int view_base, const int32_t *ids, int base, int n,
                      int prefetched, uint64_t tag, void **slot_ptrs_out) {
    const int slot0 = view_base + u->virtual_offset;
    MOLE_REQUIRE(n > 0 && slot0 >= 0 && base >= 0 && prefetched >= 0 && prefetched <= n && host_src && slot_ptrs_out &&
                     (!ids || ids_ok(ids, n)),
                 "%s: bad arguments (view_base=%d base=%d n=%d prefetched=%d)", who, view_base, base, n, prefetched);
    if (slot0 + n > u->pool_size) {
        set_error("%s: slots %d..%d exceed the pool of %d", who, slot0, slot0 + n, u->pool_size);
        return MOLE_E_STATE;
    }
    if (int rc = copy_experts(u, host_src, slot0 + prefetched, ids ? ids + prefetched : nullptr, base + prefetched, n - prefetched, tag)) return rc;
    for (int p = 0; p < 4; ++p) slot_ptrs_out[p] = u->pool[p] + (size_t)slot0 * u->slot_bytes[p];
    return 0;
}

extern "C" int mole_unimem_fetch(void *handle, const void *const host_src[4], int view_base, int base, int n,
                                 int prefetched, void **slot_ptrs_out) {
    UM(handle);
    return fetch_impl(u, "mole_unimem_fetch", host_src, view_base, nullptr, base, n, prefetched, 0, slot_ptrs_out);
}

extern "C" int mole_unimem_fetch_ids(void *handle, const void *const host_src[4], int view_base, const int32_t *expert_ids,
                                     int n, int prefetched, uint64_t tag, void **slot_ptrs_out) {
    UM(handle);
    MOLE_REQUIRE(expert_ids != nullptr, "mole_unimem_fetch_ids: null expert list");
    return fetch_impl(u, "mole_unimem_fetch_ids", host_src, view_base, expert_ids, 0, n, prefetched, tag, slot_ptrs_out);
}

extern "C" int mole_unimem_wait_params(void *handle, mole_stream_t compute_stream) {
    UM(handle);
    if (u->para_recorded) MOLE_HIP(hipStreamWaitEvent((hipStream_t)compute_stream, u->para_event, 0));
    return 0;
}

extern "C" int mole_unimem_wait_slots(void *handle, int view_base, int n, mole_stream_t compute_stream) {
    UM(handle);
    const int slot0 = view_base + u->virtual_offset;
    MOLE_REQUIRE(n >= 0 && slot0 >= 0 && slot0 + n <= u->pool_size, "mole_unimem_wait_slots: slots %d..%d outside the pool", slot0, slot0 + n);
    // the copy stream runs in order: within a stretch of slots filled by one call the last event covers the others,
    // but a chunk may mix slots prefetched earlier with slots fetched just now, so every slot's event is waited for
    for (int s = slot0; s < slot0 + n; ++s)
        if (u->landed_valid[s]) MOLE_HIP(hipStreamWaitEvent((hipStream_t)compute_stream, u->landed_event[s], 0));
    return 0;
}

extern "C" int mole_unimem_release(void *handle, int view_base, int n, mole_stream_t compute_stream) {
    UM(handle);
    const int slot0 = view_base + u->virtual_offset;
    MOLE_REQUIRE(n >= 0 && slot0 >= 0 && slot0 + n <= u->pool_size, "mole_unimem_release: slots %d..%d outside the pool", slot0, slot0 + n);
    for (int s = slot0; s < slot0 + n; ++s) {
        MOLE_HIP(hipEventRecord(u->slot_event[s], (hipStream_t)compute_stream));
        u->slot_pending[s] = 1;
    }
    return 0;
}

extern "C" int mole_unimem_sync_tran(void *handle) {
    UM(handle);
    MOLE_HIP(hipStreamSynchronize(u->tran));
    float total = 0.f;
    for (size_t i = 0; i < u->timers_used; ++i) {
        float ms = 0.f;
        MOLE_HIP(hipEventElapsedTime(&ms, u->timers[i][0], u->timers[i][1]));
        total += ms;
    }
    u->ms_last += total;
    u->bytes_last += u->bytes_open;
    u->bytes_open = 0;
    u->timers_used = 0;
    return 0;
}

// Device -> host copies of n experts' arrays of the four parameter kinds on the write-back stream, after the work
// already enqueued on compute_stream.  dev_src[p] holds the n experts back to back (every expert reads the same
// zeroed slot when zeros is set); expert i goes to host expert ids[i] (base + i when ids is null); runs of
// consecutive experts travel in one copy.
static int writeback_impl(UniMem *u, const char *who, void *const host_dst[4], const void *const dev_src[4], const int32_t *ids,
                          int base, int n, bool zeros, hipStream_t compute_stream) {
    MOLE_REQUIRE(host_dst && (zeros || dev_src) && base >= 0 && n >= 0 && (!ids || ids_ok(ids, n)), "%s: bad arguments base=%d n=%d", who, base, n);
    if (n == 0) return 0;
    for (int p = 0; p < 4; ++p)
        MOLE_REQUIRE(host_dst[p] && (zeros || dev_src[p]), "%s: null buffer for parameter kind %d", who, p);
    if (!zeros) {
        MOLE_HIP(hipEventRecord(u->grads_ready, compute_stream));
        MOLE_HIP(hipStreamWaitEvent(u->tranback, u->grads_ready, 0));
    }
    std::array<hipEvent_t, 2> *tmp;
    if (int rc = next_timer(u->wb_timers, u->wb_timers_used, &tmp)) return rc;
    auto &tm = *tmp;
    MOLE_HIP(hipEventRecord(tm[0], u->tranback));
    auto id_of = [&](int i) { return ids ? (int)ids[i] : base + i; };
    for (int i = 0; i < n;) {
        int run = 1;
        if (!zeros) while (i + run < n && id_of(i + run) == id_of(i) + run) ++run;
        for (int p = 0; p < 4; ++p) {
            const size_t sb = u->slot_bytes[p];
            const char *src = zeros ? u->zeros : (const char *)dev_src[p] + (size_t)i * sb;
            MOLE_HIP(hipMemcpyAsync((char *)host_dst[p] + (size_t)id_of(i) * sb, src, (size_t)run * sb, hipMemcpyDeviceToHost, u->tranback));
            u->wb_bytes_open += (uint64_t)run * sb;
        }
        i += run;
    }
    MOLE_HIP(hipEventRecord(tm[1], u->tranback));
    return 0;
}

extern "C" int mole_unimem_store_grads(void *handle, void *const host_dst[4], const void *const dev_src[4], int base,
                                       int n, mole_stream_t compute_stream) {
    UM(handle);
    return writeback_impl(u, "mole_unimem_store_grads", host_dst, dev_src, nullptr, base, n, false, (hipStream_t)compute_stream);
}

extern "C" int mole_unimem_store_grads_ids(void *handle, void *const host_dst[4], const void *const dev_src[4],
                                           const int32_t *expert_ids, int n, mole_stream_t compute_stream) {
    UM(handle);
    MOLE_REQUIRE(n == 0 || expert_ids, "mole_unimem_store_grads_ids: null expert list");
    return writeback_impl(u, "mole_unimem_store_grads_ids", host_dst, dev_src, expert_ids, 0, n, false, (hipStream_t)compute_stream);
}

extern "C" int mole_unimem_zero_grads_ids(void *handle, void *const host_dst[4], const int32_t *expert_ids, int n) {
    UM(handle);
    MOLE_REQUIRE(n == 0 || expert_ids, "mole_unimem_zero_grads_ids: null expert list");
    if (n == 0) return 0;
    if (!u->zeros_ready) {
        // one zeroed slot of the largest kind, made on first use and kept until the pool is destroyed; the fill runs
        // on the write-back stream, ahead of the copies that read it
        MOLE_HIP(hipSetDevice(u->device));
        if (!u->zeros) {
            hipError_t e = hipMalloc((void **)&u->zeros, u->slot_bytes[0]);
            if (e != hipSuccess) {
                u->zeros = nullptr;
                set_error("mole_unimem_zero_grads_ids: hipMalloc of %zu bytes failed: %s", u->slot_bytes[0], hipGetErrorString(e));
                return MOLE_E_NOMEM;
            }
        }
        MOLE_HIP(hipMemsetAsync(u->zeros, 0, u->slot_bytes[0], u->tranback));
        u->zeros_ready = true;
    }
    return writeback_impl(u, "mole_unimem_zero_grads_ids", host_dst, nullptr, expert_ids, 0, n, true, nullptr);
}

extern "C" int mole_unimem_load_state(void *handle, void *const dev_dst[], const void *const host_src[],
                                      const size_t bytes[], int count, int after_writeback,
                                      mole_stream_t compute_stream) {
    UM(handle);
    MOLE_REQUIRE(dev_dst && host_src && bytes && count >= 0, "mole_unimem_load_state: bad arguments count=%d", count);
    if (count == 0) return 0;
    for (int i = 0; i < count; ++i)
        MOLE_REQUIRE(bytes[i] == 0 || (dev_dst[i] && host_src[i]), "mole_unimem_load_state: null buffer %d", i);
    // the destination may have been in use by work already enqueued on the compute stream
    MOLE_HIP(hipEventRecord(u->state_free, (hipStream_t)compute_stream));
    MOLE_HIP(hipStreamWaitEvent(u->tran, u->state_free, 0));
    // the host arrays may still be the target of an earlier write-back (gradients of the previous micro-step):
    // then the copies also wait for the write-back stream, which costs the overlap of the two directions
    if (after_writeback) {
        MOLE_HIP(hipEventRecord(u->wb_done, u->tranback));
        MOLE_HIP(hipStreamWaitEvent(u->tran, u->wb_done, 0));
    }
    std::array<hipEvent_t, 2> *tm;
    if (int rc = next_timer(u, &tm)) return rc;
    MOLE_HIP(hipEventRecord((*tm)[0], u->tran));
    for (int i = 0; i < count; ++i) {
        if (bytes[i] == 0) continue;
        MOLE_HIP(hipMemcpyAsync(dev_dst[i], host_src[i], bytes[i], hipMemcpyHostToDevice, u->tran));
        u->bytes_open += bytes[i];
    }
    MOLE_HIP(hipEventRecord((*tm)[1], u->tran));
    MOLE_HIP(hipEventRecord(u->state_ready, u->tran));
    MOLE_HIP(hipStreamWaitEvent((hipStream_t)compute_stream, u->state_ready, 0));
    return 0;
}

extern "C" int mole_unimem_store_state(void *handle, void *const host_dst[], const void *const dev_src[],
                                       const size_t bytes[], int count, mole_stream_t compute_stream) {
    UM(handle);
    MOLE_REQUIRE(host_dst && dev_src && bytes && count >= 0, "mole_unimem_store_state: bad arguments count=%d", count);
    if (count == 0) return 0;
    for (int i = 0; i < count; ++i)
        MOLE_REQUIRE(bytes[i] == 0 || (host_dst[i] && dev_src[i]), "mole_unimem_store_state: null buffer %d", i);
    MOLE_HIP(hipEventRecord(u->grads_ready, (hipStream_t)compute_stream));
    MOLE_HIP(hipStreamWaitEvent(u->tranback, u->grads_ready, 0));
    std::array<hipEvent_t, 2> *tmp;
    if (int rc = next_timer(u->wb_timers, u->wb_timers_used, &tmp)) return rc;
    auto &tm = *tmp;
    MOLE_HIP(hipEventRecord(tm[0], u->tranback));
    for (int i = 0; i < count; ++i) {
        if (bytes[i] == 0) continue;
        MOLE_HIP(hipMemcpyAsync(host_dst[i], dev_src[i], bytes[i], hipMemcpyDeviceToHost, u->tranback));
        u->wb_bytes_open += bytes[i];
    }
    MOLE_HIP(hipEventRecord(tm[1], u->tranback));
    return 0;
}

extern "C" int mole_unimem_sync_tranback(void *handle) {
    UM(handle);
    MOLE_HIP(hipStreamSynchronize(u->tranback));
    float total = 0.f;
    for (size_t i = 0; i < u->wb_timers_used; ++i) {
        float ms = 0.f;
        MOLE_HIP(hipEventElapsedTime(&ms, u->wb_timers[i][0], u->wb_timers[i][1]));
        total += ms;
    }
    u->wb_ms_last += total;
    u->wb_bytes_last += u->wb_bytes_open;
    u->wb_bytes_open = 0;
    u->wb_timers_used = 0;
    return 0;
}

extern "C" int mole_unimem_tranback_stream(void *handle, mole_stream_t *out) {
    UM(handle);
    *out = (mole_stream_t)u->tranback;
    return 0;
}

extern "C" int mole_unimem_writeback_stats(void *handle, uint64_t *bytes, float *busy_ms) {
    UM(handle);
    if (bytes) *bytes = u->wb_bytes_last;
    if (busy_ms) *busy_ms = u->wb_ms_last;
    u->wb_bytes_last = 0;
    u->wb_ms_last = 0.f;
    return 0;
}

extern "C" int mole_unimem_tran_stream(void *handle, mole_stream_t *out) {
    UM(handle);
    *out = (mole_stream_t)u->tran;
    return 0;
}

extern "C" int mole_unimem_reuse_stats(void *handle, uint64_t *bytes) {
    UM(handle);
    if (bytes) *bytes = u->bytes_reused;
    u->bytes_reused = 0;
    return 0;
}

extern "C" int mole_unimem_copy_stats(void *handle, uint64_t *bytes, float *busy_ms) {
    UM(handle);
    if (bytes) *bytes = u->bytes_last;
    if (busy_ms) *busy_ms = u->ms_last;
    u->bytes_last = 0;
    u->ms_last = 0.f;
    return 0;
}

extern "C" int mole_fast_assign_prefetch(int P, const int *Fv, const int *Ev, int n, int *lp_out, int *gp_out,
                                         int gp_cap, int *gp_n) {
    MOLE_REQUIRE(n >= 0 && Fv && Ev && lp_out && gp_out && gp_n, "mole_fast_assign_prefetch: null pointer");
    // Layers with spare fetch time lend it to later layers that cannot hide their own fetches.
    // `lenders` is a stack of (layer, spare experts it may still fetch for others); `pool_free`
    // is the number of pool slots not yet promised.
    std::vector<std::array<int, 2>> lenders;
    int pool_free = P, written = 0;
    auto emit = [&](int from, int to, int cnt) -> bool {
        if (written >= gp_cap) return false;
        gp_out[3 * written] = from; gp_out[3 * written + 1] = to; gp_out[3 * written + 2] = cnt;
        ++written;
        return true;
    };
    for (int i = 0; i < n; ++i) {
        const int can = pool_free < Fv[i] ? pool_free : Fv[i];
        if (can > Ev[i]) {                 // spare capacity: lend it
            lp_out[i] = Ev[i];
            lenders.push_back({i, can - Ev[i]});
            pool_free -= can - Ev[i];
            continue;
        }
        lp_out[i] = can;
        int need = Ev[i] - can;
        while (need > 0 && !lenders.empty()) {
            auto &top = lenders.back();
            const int take = top[1] > need ? need : top[1];
            if (!emit(top[0], i, take)) { set_error("mole_fast_assign_prefetch: gp_out too small"); return MOLE_E_WORKSPACE; }
            pool_free += take;
            need -= take;
            if (top[1] > take) top[1] -= take; else lenders.pop_back();
        }
    }
    *gp_n = written;
    return 0;
}
