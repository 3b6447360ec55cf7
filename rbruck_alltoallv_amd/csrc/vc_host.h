// vc_host.h — what the host-side translation units of librbruck_vc share: the communicator, its grow-only device buffers,
// error reporting, and the few helpers of vc_api.hip the tools in vc_tools.hip need.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/rbruck_vc.h"
#include "vc_common.h"
#include "vc_dispatch.h"
#include "vc_sched.h"
#include "vc_plan_math.h"
#include "vc_scan.h"

extern thread_local std::string g_last_error;      // text of the calling thread's last failure (vc_last_error_string)

inline int fail_hip(hipError_t e, const char *what, int line, const char *file = "vc_api.hip") {
    char buf[256];
    snprintf(buf, sizeof buf, "%s failed at %s:%d: %s", what, file, line, hipGetErrorString(e));
    g_last_error = buf;
    return VC_ERR_HIP;
}

#define HIP_TRY(expr)                                                   \
    do {                                                                \
        hipError_t e_ = (expr);                                         \
        if (e_ != hipSuccess) return fail_hip(e_, #expr, __LINE__, __FILE_NAME__);     \
    } while (0)

inline int fail_arg(const char *msg, int code = VC_ERR_ARG) {
    g_last_error = msg;
    return code;
}

// Grow-only device buffer.
struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes) {
        if (bytes <= cap) return hipSuccess;
        if (p) { hipError_t e = hipFree(p); p = nullptr; cap = 0; if (e != hipSuccess) return e; }
        size_t want = std::max(bytes, (size_t)256);
        hipError_t e = hipMalloc(&p, want);
        if (e == hipSuccess) cap = want;
        return e;
    }
    void release() { if (p) (void)hipFree(p); p = nullptr; cap = 0; }
    template <class T> T *as() const { return static_cast<T *>(p); }
};

// Device buffers a call plans into: the communicator's grow-only allocations, or slices of memory the caller of the
// planning functions carved elsewhere.
struct PlanBufs {
    int64_t *slot_off = nullptr, *row_tot = nullptr, *row_base = nullptr, *org_run_base = nullptr, *item_row_tot = nullptr,
            *item_row_base = nullptr, *row_bytes = nullptr, *chain_row_tot = nullptr, *chain_row_base = nullptr, *header = nullptr;
    VcLaunchInfo *launches = nullptr;
    int *rd_packed = nullptr;
};

// What a call asked for: enough to derive its schedule again in the other execution mode.
struct CallParams {
    VcFunc f;
    int n, r, batch, esz, uniform, batch2;
};

struct vc_comm {
    int P = 0;
    int device = 0;
    hipStream_t stream = nullptr;
    const int64_t *sbase = nullptr, *rbase = nullptr;
    bool timing = false;
    int forward = 1;                      // vc_comm_set_forwarding: 0 launch per digit, 1 forwarded (list or listless as the last
                                          // call suggests), 2 forwarded through a work-item list, 3 / 4 forwarded, listless with a
                                          // workgroup / a quarter of a wavefront per pair of ranks
    VcHint hint = {0, 0, 0, 0, 0};        // what the last forwarded call on this communicator looked like
    int plan_end = 2;                     // which event marks the end of the planning kernels of the call in progress
    int waits = 0;                        // times the host has waited for the stream in the call in progress
    int64_t items_before_last = 0;        // block pieces of the forwarded call before the one `hint` describes (0: there was none)
    DevBuf chain_row_tot, chain_row_base;
    DevBuf strided_headers;               // fixed-stride calls: two headers used in turn
    bool strided_clean = false;           // ... and the one the next call will use is known to be zero
    int strided_turn = 0;
    DevBuf slot_off, row_tot, row_base, org_run_base, item_row_tot, item_row_base, row_bytes, desc, header, launches, stage, rd_packed,
        uni_counts, uni_displs, scratch;
    double cal_copy_bytes_per_s = 0, cal_launch_s = 0, cal_sync_s = 0;   // calibrate(): the plain copy's rate, the cost of a
                                          // launch, of a launch the host waits for
    int bound_staging = 1;                // vc_comm_set_staging_bound
    int64_t staging_allowance = 0;        // bytes of staging a forwarded call may take whatever its payload (set with the bound)
    int live_plans = 0;                   // plans created on this communicator and not yet freed
    std::vector<void *> retired_stage;    // staging arenas that were outgrown while plans existed: a HIP graph captured from
                                          // vc_plan_execute_async holds the arena's address, so they stay until the plans go
    std::atomic_flag busy = ATOMIC_FLAG_INIT;   // a call is in progress (a communicator serves one call at a time)
    struct {                              // a call enqueued by an _async entry point that vc_comm_wait has not collected yet
        bool active = false;
        VcSched S;
        VcTables T;
        const char *sendbuf = nullptr;
        char *recvbuf = nullptr;
        int lanes = 0;
        int n_launch_infos = 0;
        hipStream_t own_stream = nullptr; // the communicator's stream while the call runs on the caller's
        CallParams q;                     // what was asked for (the call may have to be run again another way)
    } pending;
    PlanBufs B;                           // where the current call's plan lives
    const void *last_stage = nullptr;     // staging arena of the last call
    int64_t *h_header = nullptr;          // pinned, coherent: the planner writes its header straight into it
    int64_t *h_header_dev = nullptr;      // the same memory as the device sees it
    int *h_flags = nullptr, *h_flags_dev = nullptr;   // pinned, coherent: the two flags of vc_displs_from_counts, as host and device see them
    VcLaunchInfo *h_launches = nullptr;   // pinned
    std::vector<hipEvent_t> events;
    vc_stats_t stats;
    int last_nlaunch = 0;
    int64_t launch_first[VC_MAX_LAUNCHES], launch_items[VC_MAX_LAUNCHES];   // work items of the last call
    const VcDesc *last_items = nullptr;
};

// Grows the staging arena.  While plans exist the outgrown arena is kept (not freed): graphs captured from their
// launches write to its address.
inline hipError_t reserve_stage(vc_comm *c, size_t bytes) {
    if (bytes <= c->stage.cap) return hipSuccess;
    if (c->live_plans > 0 && c->stage.p) {
        c->retired_stage.push_back(c->stage.p);
        c->stage.p = nullptr;
        c->stage.cap = 0;
    }
    return c->stage.reserve(bytes);
}

inline void free_retired_stage(vc_comm *c) {
    for (void *p : c->retired_stage) (void)hipFree(p);
    c->retired_stage.clear();
}

// One call at a time per communicator: a second host thread gets VC_ERR_BUSY instead of a race on the plan buffers.
struct BusyGuard {
    vc_comm *c;
    bool mine;
    explicit BusyGuard(vc_comm *comm) : c(comm), mine(comm && !comm->busy.test_and_set(std::memory_order_acquire)) {
        if (mine) c->waits = 0;
    }
    ~BusyGuard() { if (mine) c->busy.clear(std::memory_order_release); }
    bool ok() const { return !c || mine; }
    void keep() { mine = false; }         // the call stays in progress after the entry point returns (vc_comm_wait ends it)
};
// the host waits for the communicator's stream (counted: vc_stats_t.host_waits)
#define VC_WAIT(c) ((c)->waits++, hipStreamSynchronize((c)->stream))

#define VC_ONE_CALL(c)                                                                                              \
    BusyGuard busy_guard_(c);                                                                                       \
    if (!busy_guard_.ok()) return fail_arg("the communicator is serving another call (one call at a time)", VC_ERR_BUSY)

// ---- defined in vc_api.hip, used by vc_tools.hip ----
int ensure_events(vc_comm *c, size_t n);
bool staging_out_of_bound(const vc_comm *c, int64_t stage_bytes, int64_t payload_bytes);
VcTables make_tables(vc_comm *c, const int *sc, const int *sd, const int *rc, const int *rd);
