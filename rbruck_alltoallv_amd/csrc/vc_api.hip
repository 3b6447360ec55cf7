// vc_api.hip — host side of librbruck_vc: the C ABI declared in include/rbruck_vc.h.
//
// Every collective entry point does what the reference function of the same name
// does on each of the P ranks, for all ranks at once:
//   1. clamp / validate the tunables exactly as the reference does,
//   2. derive the schedule: which digit phases exist, which rounds share a launch,
//   3. plan on the device (staging prefix sums, one copy descriptor per block hop),
//   4. run one copy kernel per launch,
//   5. synchronise the stream (the reference functions are blocking).
#include "vc_host.h"

thread_local std::string g_last_error;

extern "C" const char *vc_last_error_string(void) { return g_last_error.c_str(); }

// Device memory of the entry point that allocates nothing (twophase_rbruck_alltoallv_noalloc): its plan tables and its
// staging arena are slices of this array.  Every GPU the library runs on holds its own copy, at its own address, until
// the process ends; `scratch` itself is only the host-side name of the symbol and never a device address: host code
// uses the pointer hipGetSymbolAddress returned for the device, resolved once per device in vc_comm_create.
static __device__ __align__(256) unsigned char scratch[VC_NOALLOC_SCRATCH_BYTES];
#define VC_MAX_DEVICES 64
static unsigned char *g_scratch_ptr[VC_MAX_DEVICES];       // per device: where its copy of `scratch` lives (null: not resolved)
static std::mutex g_scratch_mutex;                         // guards the resolution (communicators may be created from several threads)
static std::atomic_flag g_scratch_busy[VC_MAX_DEVICES];    // per device: a call is using the array (all communicators on a GPU share it)

// ------------------------------------------------------------------ communicator

static int64_t default_staging_allowance();

extern "C" int vc_comm_create(int nranks, vc_comm_t *comm_out) {
    if (!comm_out || nranks < 1) return fail_arg("vc_comm_create: need nranks >= 1 and an output pointer");
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) return fail_arg("no HIP device", VC_ERR_NO_DEVICE);
    if (nranks > 32768) return fail_arg("vc_comm_create: at most 32768 ranks (P x P int32 tables)");
    vc_comm *c = new vc_comm();
    c->P = nranks;
    memset(&c->stats, 0, sizeof c->stats);
    hipError_t e = hipGetDevice(&c->device);
    if (e == hipSuccess && c->device >= 0 && c->device < VC_MAX_DEVICES) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[c->device]) {
            void *ptr = nullptr;                          // this device's copy of the static scratch array
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e == hipSuccess) g_scratch_ptr[c->device] = static_cast<unsigned char *>(ptr);
        }
    }
    if (e == hipSuccess) e = hipHostMalloc((void **)&c->h_header, sizeof(int64_t) * VC_HEADER_WORDS(VC_MAX_LAUNCHES), hipHostMallocCoherent);
    if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&c->h_header_dev, c->h_header, 0);
    if (e == hipSuccess) e = hipHostMalloc((void **)&c->h_launches, sizeof(VcLaunchInfo) * VC_MAX_LAUNCHES, hipHostMallocDefault);
    if (e == hipSuccess) e = hipHostMalloc((void **)&c->h_flags, 2 * sizeof(int), hipHostMallocCoherent);
    if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&c->h_flags_dev, c->h_flags, 0);
    if (e != hipSuccess) {
        (void)vc_comm_free(c);
        return fail_hip(e, "vc_comm_create", __LINE__);
    }
    c->staging_allowance = default_staging_allowance();
    *comm_out = c;
    return VC_OK;
}

extern "C" int vc_comm_free(vc_comm_t c) {
    if (!c) return VC_OK;
    (void)hipStreamSynchronize(c->stream);
    c->pending.active = false;
    for (DevBuf *b : {&c->slot_off, &c->row_tot, &c->row_base, &c->org_run_base, &c->item_row_tot, &c->item_row_base, &c->row_bytes, &c->desc, &c->header, &c->launches, &c->stage, &c->rd_packed,
                      &c->uni_counts, &c->uni_displs, &c->scratch, &c->chain_row_tot, &c->chain_row_base, &c->strided_headers})
        b->release();
    free_retired_stage(c);
    for (hipEvent_t e : c->events) (void)hipEventDestroy(e);
    if (c->h_header) (void)hipHostFree(c->h_header);
    if (c->h_launches) (void)hipHostFree(c->h_launches);
    if (c->h_flags) (void)hipHostFree(c->h_flags);
    delete c;
    return VC_OK;
}

extern "C" int vc_comm_size(vc_comm_t c) { return c ? c->P : VC_ERR_ARG; }

extern "C" int vc_comm_set_stream(vc_comm_t c, void *hip_stream) {
    if (!c) return fail_arg("null communicator");
    c->stream = static_cast<hipStream_t>(hip_stream);
    return VC_OK;
}

extern "C" int vc_comm_set_bases(vc_comm_t c, const int64_t *sbase, const int64_t *rbase) {
    if (!c || !sbase || !rbase) return fail_arg("vc_comm_set_bases: null argument");
    c->sbase = sbase;
    c->rbase = rbase;
    return VC_OK;
}

extern "C" int vc_comm_set_timing(vc_comm_t c, int enable) {
    if (!c) return fail_arg("null communicator");
    c->timing = enable != 0;
    return VC_OK;
}

extern "C" int vc_comm_set_forwarding(vc_comm_t c, int enable) {
    if (!c) return fail_arg("null communicator");
    if (enable < 0 || enable > 5) return fail_arg("vc_comm_set_forwarding: 0 .. 5");
    c->forward = enable;
    return VC_OK;
}

// An eighth of the device's memory, at least 1 GiB: what a forwarded call may keep in staging before its ratio to the
// payload is looked at.
static int64_t default_staging_allowance() {
    size_t free_bytes = 0, total = 0;
    if (hipMemGetInfo(&free_bytes, &total) != hipSuccess) { (void)hipGetLastError(); total = 0; }
    return std::max<int64_t>((int64_t)1 << 30, (int64_t)(total / 8));
}

extern "C" int vc_comm_set_staging_bound(vc_comm_t c, int enable) {
    if (!c) return fail_arg("null communicator");
    if (enable < 0) return fail_arg("vc_comm_set_staging_bound: 0, 1 or an allowance in MiB");
    c->bound_staging = enable != 0;
    c->staging_allowance = enable > 1 ? (int64_t)enable << 20 : default_staging_allowance();
    return VC_OK;
}

extern "C" int vc_comm_last_stats(vc_comm_t c, vc_stats_t *out) {
    if (!c || !out) return fail_arg("vc_comm_last_stats: null argument");
    *out = c->stats;
    return VC_OK;
}

// ------------------------------------------------------------- plan and run

int ensure_events(vc_comm *c, size_t n) {
    while (c->events.size() < n) {
        hipEvent_t e;
        HIP_TRY(hipEventCreate(&e));
        c->events.push_back(e);
    }
    return VC_OK;
}

static int schedule_error(int code);

// The schedule of a call in one of the two execution modes.  Launch-per-digit execution reuses staging memory when the
// communicator bounds its staging (the default) and there is something to reuse: with fewer than three staging regions
// no sub-region is written after another one has been read for the last time.
// reuse: launch-per-digit execution on reused staging memory (where the schedule allows it).
static int make_schedule(const vc_comm *c, const CallParams &q, bool forward, VcSched &S, std::vector<VcLaunchInfo> &L, bool reuse = false) {
    const int rc = vc_make_schedule(q.f, c->P, q.n, q.r, q.batch, q.esz, q.uniform, S, L, q.batch2, forward);
    if (rc) return rc;
    const int nreg = S.w + S.w2;
    if (!forward && reuse && c->bound_staging && nreg >= 3 && nreg + 1 <= VC_RECYCLE_MAX_SLOTS) S.recycle = 1;
    return VC_OK;
}

// Reused staging costs planning time (one prefix sum per pair of hop slots, the allocator on one thread: 0.05 ms on 64
// ranks), so a launch-per-digit call is planned with a region per digit first and planned again on reused staging
// only when that would take more than a thirty-second of the communicator's staging allowance (about 1 GiB).
static bool worth_reusing(const vc_comm *c, const VcSched &S, int64_t stage_bytes) {
    const int nreg = S.w + S.w2;
    return c->bound_staging && !S.recycle && nreg >= 3 && nreg + 1 <= VC_RECYCLE_MAX_SLOTS && stage_bytes > (c->staging_allowance >> 5);
}

// Forwarded execution keeps every hop's copy of every block (nothing reads them, so nothing says when one could be
// overwritten): its staging is the sum over the blocks of (hops - 1) x bytes, 3.5 x the payload for a radix-2 Bruck
// over 512 ranks.  A communicator that bounds its staging runs such a call one launch per digit instead, where staging
// memory is reused (and stays below about twice the payload): beyond three times the payload, and only when it
// matters (more than an eighth of the device's memory, 36 GB here; vc_comm_set_staging_bound takes another allowance).
// Measured on MI355X: configuration 5 with radix 2, 60 GB forwarded in 17.4 ms against 30 GB in 25.5 ms; a radix-4
// two-layer Bruck at configuration 4 (13 GB, 3.1 x its payload) stays forwarded: 4.8 ms against 6.8.
bool staging_out_of_bound(const vc_comm *c, int64_t stage_bytes, int64_t payload_bytes) {
    return c->bound_staging && stage_bytes > c->staging_allowance && stage_bytes > 3 * payload_bytes;
}

// What the planner leaves behind for the copy launches.
struct PlanInfo {
    int nl = 0, n_digits = 0;
    int recv_lo = 0;
    int64_t stage_bytes = 0, payload_bytes = 0;
    std::vector<int64_t> first, count, bytes;       // per launch: first work item, item count, bytes moved
    std::vector<char> inter;                        // per launch: its messages cross nodes
    std::vector<int> lanes;                         // per launch: lanes per work item of the copy kernel
    int chain_lanes = VC_THREADS;                   // the same for the one launch of forwarded execution
    int64_t items_total = 0;                        // work items of all launches
    bool chain = false;                             // forwarded execution: `items` holds chain items instead
    int chain_stride = 0;                           // int64 words per chain item
    int64_t chain_items = 0, max_pieces = 0;        // (max_pieces: the most pieces any block is cut into)
    int64_t max_len = 0;                            // forwarded execution: the longest block
    bool strided = false;                           // ... that went without the list on fixed-stride staging
    bool listless = false;                          // forwarded execution that went without the item list
};

static int plan_sizes(vc_comm *c, const VcSched &S, std::vector<VcLaunchInfo> &L, VcTables &T, bool forward);

// Sizes (bytes) of the plan buffers of a call, in the order of PlanBufs' members.
struct PlanBufSizes { size_t slot_off, row_tot, row_base, org_run_base, item_row_tot, item_row_base, row_bytes, chain_row_tot, chain_row_base, header, launches, rd_packed; };

static PlanBufSizes plan_buf_sizes(const VcSched &S, int nl, bool forward) {
    const size_t P = (size_t)S.P, PP = P * P;
    const size_t wmax = (size_t)std::max(vc_regions(S), 1) + 1;      // staging regions
    PlanBufSizes z;
    z.slot_off = sizeof(int64_t) * PP * wmax;
    z.row_tot = z.row_base = sizeof(int64_t) * P * std::max(wmax, (size_t)vc_row_families(S) + 1);
    z.org_run_base = sizeof(int64_t) * P * (size_t)std::max(S.G, 1);
    z.item_row_tot = z.item_row_base = sizeof(int64_t) * P * (size_t)std::max(nl, 1);
    z.row_bytes = sizeof(int64_t) * P * (size_t)(std::max(nl, S.w + S.w2) + 3);
    z.chain_row_tot = forward ? sizeof(int64_t) * (2 + VC_TILES(P)) * P : 0;
    z.chain_row_base = forward ? sizeof(int64_t) * P : 0;
    z.header = sizeof(int64_t) * VC_HEADER_WORDS(VC_MAX_LAUNCHES);
    z.launches = sizeof(VcLaunchInfo) * VC_MAX_LAUNCHES;
    z.rd_packed = S.packed_recv ? sizeof(int) * PP : 0;
    return z;
}

// The communicator's own buffers, grown to what the call needs.
static int reserve_plan_bufs(vc_comm *c, const VcSched &S, int nl, bool forward) {
    const PlanBufSizes z = plan_buf_sizes(S, nl, forward);
    HIP_TRY(c->slot_off.reserve(z.slot_off));
    HIP_TRY(c->row_tot.reserve(z.row_tot));
    HIP_TRY(c->row_base.reserve(z.row_base));
    HIP_TRY(c->org_run_base.reserve(z.org_run_base));
    HIP_TRY(c->item_row_tot.reserve(z.item_row_tot));
    HIP_TRY(c->item_row_base.reserve(z.item_row_base));
    HIP_TRY(c->row_bytes.reserve(z.row_bytes));
    HIP_TRY(c->header.reserve(z.header));
    HIP_TRY(c->launches.reserve(z.launches));
    if (forward) {
        HIP_TRY(c->chain_row_tot.reserve(z.chain_row_tot));
        HIP_TRY(c->chain_row_base.reserve(z.chain_row_base));
    }
    if (S.packed_recv) HIP_TRY(c->rd_packed.reserve(z.rd_packed));
    PlanBufs &B = c->B;
    B.slot_off = c->slot_off.as<int64_t>(); B.row_tot = c->row_tot.as<int64_t>(); B.row_base = c->row_base.as<int64_t>();
    B.org_run_base = c->org_run_base.as<int64_t>(); B.item_row_tot = c->item_row_tot.as<int64_t>();
    B.item_row_base = c->item_row_base.as<int64_t>(); B.row_bytes = c->row_bytes.as<int64_t>();
    B.chain_row_tot = forward ? c->chain_row_tot.as<int64_t>() : nullptr;
    B.chain_row_base = forward ? c->chain_row_base.as<int64_t>() : nullptr;
    B.header = c->header.as<int64_t>(); B.launches = c->launches.as<VcLaunchInfo>(); B.rd_packed = c->rd_packed.as<int>();
    return VC_OK;
}

// Step 3a: enqueues the planning kernels that size everything (staging prefix sums, item counts, table check) into the
// buffers c->B names; their result lands in the pinned header.
static int enqueue_plan_sizes(vc_comm *c, const VcSched &S, std::vector<VcLaunchInfo> &L, VcTables &T, bool forward, bool timing) {
    const int P = S.P;
    const int nl = (int)L.size();
    hipStream_t st = c->stream;
    const PlanBufs &B = c->B;
    if (timing) HIP_TRY(hipEventRecord(c->events[0], st));
    if (!forward && nl > VC_LAUNCH_PACK) {                 // a short launch table travels as a kernel argument instead
        memcpy(c->h_launches, L.data(), sizeof(VcLaunchInfo) * nl);
        HIP_TRY(hipMemcpyAsync(B.launches, c->h_launches, sizeof(VcLaunchInfo) * nl, hipMemcpyHostToDevice, st));
    }
    if (S.packed_recv) {
        HIP_TRY(vc_launch_row_scan(T.rc, B.rd_packed, nullptr, nullptr, P, st));
        T.rd_packed = B.rd_packed;
    }
    HIP_TRY(vc_launch_plan_sizes(S, L.data(), B.launches, nl, T, B.slot_off, B.row_tot, B.row_base, B.org_run_base, B.item_row_tot,
                                 B.item_row_base, B.row_bytes, forward ? B.chain_row_tot : nullptr,
                                 forward ? B.chain_row_base : nullptr, B.header, c->h_header_dev, st));
    return VC_OK;
}

static int plan_sizes(vc_comm *c, const VcSched &S, std::vector<VcLaunchInfo> &L, VcTables &T, bool forward) {
    const int nl = (int)L.size();
    if (nl > VC_MAX_LAUNCHES) return fail_arg("more than VC_MAX_LAUNCHES launches: raise b / bblock");
    if (forward && vc_hop_slots(S) > VC_MAX_HOP_SLOTS) return fail_arg("too many digits for forwarded execution");
    int rc = reserve_plan_bufs(c, S, nl, forward);
    if (rc) return rc;
    if (c->timing) { rc = ensure_events(c, (size_t)nl + 4); if (rc) return rc; }
    c->plan_end = 2;                                      // the planning ends where the first copy launch begins: one event for both
    return enqueue_plan_sizes(c, S, L, T, forward, c->timing);
}

// Step 3b, after the stream has been synchronised: what the planning kernels found.
static int plan_read(vc_comm *c, const VcSched &S, const std::vector<VcLaunchInfo> &L, PlanInfo &out, bool forward) {
    const int nl = forward ? 1 : (int)L.size();           // forwarded execution: one launch, one set of totals
    const int64_t *h = c->h_header;
    out = PlanInfo();                                     // (a plan that is derived again in the other execution mode reuses `out`)
    c->stats.bad_table_entries = h[VC_HEADER_BAD];
    if (h[VC_HEADER_BAD] >= VC_BAD_OVERFLOW)
        return fail_arg("a rank receives more than INT_MAX elements: the packed receive displacements of TTPL_BT_alltoallv do not fit an int",
                        VC_ERR_OVERFLOW);
    if (h[VC_HEADER_BAD] != 0)    // such tables would send the copy kernels outside the arenas
        return fail_arg("sendcounts / sdispls / recvcounts / rdispls hold negative entries, or recvcounts[t][s] != sendcounts[s][t]",
                        VC_ERR_TABLES);
    out.nl = nl; out.n_digits = S.w + S.w2; out.recv_lo = S.recv_lo;
    out.stage_bytes = h[0]; out.payload_bytes = h[1];
    out.first.assign(nl, 0); out.count.assign(nl, 0); out.bytes.assign(nl, 0); out.inter.assign(nl, 0); out.lanes.assign(nl, VC_THREADS);
    if (forward) {
        out.bytes[0] = h[VC_HEADER_FIXED];
        out.chain = true;
        out.chain_stride = VC_CHAIN_HEAD + vc_hop_slots(S);
        out.chain_items = h[2];
        out.chain_lanes = vc_lanes_for_items(out.payload_bytes, out.chain_items);      // every chain item carries one piece of the payload
        out.max_pieces = h[VC_HEADER_MAX_PIECES];
        out.max_len = h[VC_HEADER_MAX_LEN];
        return VC_OK;
    }
    int64_t nitems = 0;
    for (int k = 0; k < nl; k++) {
        out.inter[k] = L[k].kind == 1 || L[k].kind == 3 || L[k].kind == 4 || (L[k].kind == 2 && L[k].x == 2);
        out.bytes[k] = h[VC_HEADER_FIXED + k];
        out.first[k] = nitems;
        out.count[k] = h[VC_HEADER_FIXED + nl + k];
        out.lanes[k] = vc_lanes_for_items(out.bytes[k], out.count[k]);
        nitems += out.count[k];
    }
    out.items_total = nitems;
    return VC_OK;
}

// Step 3c: the work items into `items` (sized from the plan).
static int plan_emit(vc_comm *c, const VcSched &S, std::vector<VcLaunchInfo> &L, const VcTables &T, DevBuf &items, const PlanInfo &pi) {
    hipStream_t st = c->stream;
    if (pi.chain) {
        if (!c->B.chain_row_base || !c->B.chain_row_tot) return fail_arg("internal: chain items asked for a plan that was not sized for them", VC_ERR_HIP);
        HIP_TRY(items.reserve(sizeof(int64_t) * (size_t)pi.chain_stride * (size_t)std::max<int64_t>(pi.chain_items, 1)));
        HIP_TRY(vc_launch_chain_plan(S, T, c->B.slot_off, c->B.row_base, c->B.chain_row_tot + 2 * (size_t)S.P, items.as<int64_t>(),
                                     pi.chain_items, st));
    } else {
        HIP_TRY(items.reserve(sizeof(VcDesc) * (size_t)std::max<int64_t>(pi.items_total, 1)));
        HIP_TRY(vc_launch_plan_emit(S, L.data(), c->B.launches, pi.nl, T, c->B.slot_off, c->B.row_base, c->B.item_row_base, c->B.header,
                                    items.as<VcDesc>(), pi.items_total, st));
    }
    return VC_OK;
}

static int build_plan(vc_comm *c, const CallParams &q, int recv_lo, VcTables T, DevBuf &items, PlanInfo &out, bool forward, bool reuse = false) {
    VcSched S;
    std::vector<VcLaunchInfo> L;
    int rc = make_schedule(c, q, forward, S, L, reuse);
    if (rc) return schedule_error(rc);
    S.recv_lo = recv_lo;
    rc = plan_sizes(c, S, L, T, forward);
    if (rc) return rc;
    HIP_TRY(VC_WAIT(c));     // the staging arena and the item list are sized from the plan
    rc = plan_read(c, S, L, out, forward);
    if (rc) return rc;
    if (forward && staging_out_of_bound(c, out.stage_bytes, out.payload_bytes)) return build_plan(c, q, recv_lo, T, items, out, false, true);
    if (!forward && worth_reusing(c, S, out.stage_bytes)) return build_plan(c, q, recv_lo, T, items, out, false, true);
    return plan_emit(c, S, L, T, items, out);
}

// Steps 4-5: one copy kernel per launch, then the blocking synchronisation.  `planned_now` says whether events 0 and 1
// (the planner's) belong to this call.
// Only the launches: no allocation, no synchronisation, no host-side bookkeeping (safe under stream capture).
static int launch_items(vc_comm *c, const PlanInfo &pi, const void *items_any, const char *sendbuf, char *recvbuf) {
    if (c->stage.cap < (size_t)pi.stage_bytes + 64) return fail_arg("staging arena smaller than the plan needs");
    if (pi.chain) {
        HIP_TRY(vc_launch_copy_chains(static_cast<const int64_t *>(items_any), pi.chain_stride, pi.chain_items,
                                      pi.chain_lanes, sendbuf, recvbuf, c->stage.as<char>(), c->stream));
        return VC_OK;
    }
    const VcDesc *items = static_cast<const VcDesc *>(items_any);
    for (int k = 0; k < pi.nl; k++)
        HIP_TRY(vc_launch_copy_items(items + pi.first[k], pi.count[k], pi.lanes[k], sendbuf, recvbuf, c->stage.as<char>(), c->stream));
    return VC_OK;
}

// After the final synchronisation: the statistics of the call.
static int finish_stats(vc_comm *c, const PlanInfo &pi, const void *items_any, bool planned_now) {
    const int nl = pi.chain ? 1 : pi.nl;              // kernel launches of this execution
    vc_stats_t &s = c->stats;
    s.n_launches = nl;
    s.n_digits = pi.n_digits;
    s.staging_bytes = pi.stage_bytes;
    s.payload_bytes = pi.payload_bytes;
    s.moved_bytes = 0;
    s.execution = pi.chain ? (pi.listless ? (pi.strided ? 3 : 2) : 1) : 0;
    s.block_pieces = pi.chain ? pi.chain_items : 0;
    s.max_block_pieces = pi.chain ? pi.max_pieces : 0;
    s.max_block_bytes = pi.chain ? pi.max_len : 0;
    s.bad_table_entries = 0;
    s.host_waits = c->waits;
    s.plan_ms = s.total_ms = s.intra_ms = s.inter_ms = 0.f;
    if (pi.chain) {                                   // one launch that performs the hops of every digit
        for (int k = 0; k < pi.nl; k++) s.moved_bytes += pi.bytes[k];
        s.launch_bytes[0] = s.moved_bytes;
        s.launch_ms[0] = 0.f;
        if (c->timing) HIP_TRY(hipEventElapsedTime(&s.launch_ms[0], c->events[2], c->events[3]));
        s.intra_ms = s.launch_ms[0];
        s.lanes_per_item = pi.chain_lanes;
        c->items_before_last = c->hint.valid ? c->hint.items : 0;
        c->hint = VcHint{1, pi.chain_items, pi.payload_bytes, pi.max_pieces, pi.max_len};
    } else {
        int64_t most = -1;
        for (int k = 0; k < nl; k++) {
            if (pi.bytes[k] > most) { most = pi.bytes[k]; s.lanes_per_item = pi.lanes[k]; }
            s.launch_bytes[k] = pi.bytes[k];
            s.moved_bytes += pi.bytes[k];
            s.launch_ms[k] = 0.f;
            c->launch_first[k] = pi.first[k];
            c->launch_items[k] = pi.count[k];
            if (c->timing) HIP_TRY(hipEventElapsedTime(&s.launch_ms[k], c->events[2 + k], c->events[3 + k]));
            (pi.inter[k] ? s.inter_ms : s.intra_ms) += s.launch_ms[k];
        }
    }
    if (c->timing) {
        if (planned_now) HIP_TRY(hipEventElapsedTime(&s.plan_ms, c->events[0], c->events[c->plan_end]));
        HIP_TRY(hipEventElapsedTime(&s.total_ms, c->events[planned_now ? 0 : 2], c->events[2 + nl]));
    }
    c->last_nlaunch = pi.chain ? 0 : nl;              // per-launch traffic can only be inspected after launch-per-digit execution
    c->last_items = static_cast<const VcDesc *>(items_any);
    c->last_stage = c->stage.p;
    return VC_OK;
}

static int run_items(vc_comm *c, const PlanInfo &pi, const void *items_any, const char *sendbuf, char *recvbuf, bool planned_now) {
    hipStream_t st = c->stream;
    const int nl = pi.chain ? 1 : pi.nl;              // kernel launches of this execution
    const VcDesc *items = static_cast<const VcDesc *>(items_any);
    HIP_TRY(reserve_stage(c, (size_t)pi.stage_bytes + 64));
    if (c->timing) { int rc = ensure_events(c, (size_t)nl + 4); if (rc) return rc; }
    if (pi.chain) {
        if (c->timing) HIP_TRY(hipEventRecord(c->events[2], st));
        int rc = launch_items(c, pi, items_any, sendbuf, recvbuf);
        if (rc) return rc;
    } else {
        for (int k = 0; k < nl; k++) {
            if (c->timing) HIP_TRY(hipEventRecord(c->events[2 + k], st));
            HIP_TRY(vc_launch_copy_items(items + pi.first[k], pi.count[k], pi.lanes[k], sendbuf, recvbuf, c->stage.as<char>(), st));
        }
    }
    if (c->timing) HIP_TRY(hipEventRecord(c->events[2 + nl], st));
    HIP_TRY(VC_WAIT(c));
    return finish_stats(c, pi, items_any, planned_now);
}

// One launch on fixed-stride staging (vc_dispatch chose it: a small call in the default mode, after a call the listless
// kernels could serve): no planner before the copy kernel, one host synchronisation.  The first wavefronts of the copy kernel
// add up what the host wants to know afterwards (validation, totals, the longest block); every pair of ranks checks its
// own table entries, and that its block fits a slot, before it forms an address from them, and holds its stores back
// until all of those wavefronts have reported the tables in order (their verdict comes after one round of loads, about
// when the copying wavefronts have their data): as everywhere else, a call with bad tables has touched nothing when it
// returns.  A call with a longer block than the stride holds is redone the general way (the blocks that did fit have
// been delivered by then, and are delivered again).
// Returns 1 when the call has been served, 0 when it must go the general way, < 0 on errors.
static int try_strided(vc_comm *c, VcSched S, std::vector<VcLaunchInfo> &L, const char *sendbuf, char *recvbuf, VcTables T, const VcDispatch &d) {
    if (d.stride <= 0) return 0;
    const int pair_lanes = d.stride_lanes;
    S.stride = d.stride;
    const int64_t need = vc_strided_stage_bytes(S);
    hipStream_t st = c->stream;
    // two headers in turn: the planner adds up into one (with atomics, so it must start from zero) while the copy kernel
    // clears the other one for the next call
    const size_t header_bytes = sizeof(int64_t) * 16;
    if (!c->strided_headers.p) {
        HIP_TRY(c->strided_headers.reserve(2 * header_bytes));
        c->strided_clean = false;
    }
    HIP_TRY(reserve_stage(c, (size_t)need + 64));
    if (S.packed_recv) HIP_TRY(c->rd_packed.reserve(sizeof(int) * (size_t)S.P * S.P));
    if (c->timing) { int rc = ensure_events(c, 5); if (rc) return rc; HIP_TRY(hipEventRecord(c->events[0], st)); }
    if (!c->strided_clean) HIP_TRY(hipMemsetAsync(c->strided_headers.p, 0, 2 * header_bytes, st));
    c->strided_clean = false;                             // until the copy kernel that clears the other header is enqueued
    int64_t *header = c->strided_headers.as<int64_t>() + (c->strided_turn ? 16 : 0);
    int64_t *header_next = c->strided_headers.as<int64_t>() + (c->strided_turn ? 0 : 16);
    c->strided_turn ^= 1;
    if (S.packed_recv) {
        HIP_TRY(vc_launch_row_scan(T.rc, c->rd_packed.as<int>(), nullptr, nullptr, S.P, st));
        T.rd_packed = c->rd_packed.as<int>();
    }
    VcListlessGuard guard = d.guard;
    guard.stage_cap = (int64_t)c->stage.cap - 64;
    if (c->timing) HIP_TRY(hipEventRecord(c->events[2], st));
    c->h_header[VC_HEADER_STALLED] = 0;
    // the one launch of the call: its first wavefronts check the tables and add their totals up into `header`; every pair
    // checks its own entries and the length of its block before it forms an address, and stores nothing before all of
    // the tables have been found in order
    HIP_TRY(vc_launch_copy_blocks(S, T, nullptr, nullptr, header, guard, pair_lanes, sendbuf, recvbuf, c->stage.as<char>(), st, c->h_header_dev,
                                  header_next, header));
    c->strided_clean = true;
    if (c->timing) HIP_TRY(hipEventRecord(c->events[3], st));
    HIP_TRY(VC_WAIT(c));
    PlanInfo pi;
    int rc = plan_read(c, S, L, pi, true);
    if (rc) return rc;
    if (c->h_header[VC_HEADER_STALLED]) return 0;          // a copying wavefront gave up waiting for the verdict and moved nothing
    if (!vc_listless_ok(c->h_header, guard)) return 0;     // longer blocks than the last call's, or not a call for this kernel
    pi.listless = pi.strided = true;
    pi.chain_lanes = pair_lanes;
    rc = finish_stats(c, pi, nullptr, true);
    return rc ? rc : 1;
}

// A forwarded call through the work-item list, without the host's look at the plan in mid-call (a round trip of ~10 us):
// the list kernel and the copy kernel go out right behind the sizing kernels, the list's length guessed from the last
// forwarded call on the communicator, and check on the device what the host checks otherwise — tables in order, the list
// and the staging arena large enough, the staging within the communicator's bound (VcChainGuard).  The host reads the
// same header after the one synchronisation of the call: a plan the launches could not serve has moved nothing and goes
// the general way; a list longer than guessed gets a second launch for the rest.
// Returns 1: served; 0: nothing moved, `pi` holds the plan (the stream is synchronised); 2: not tried; < 0: errors.
static int try_enqueued_list(vc_comm *c, const VcSched &S, std::vector<VcLaunchInfo> &L, const VcTables &T, const char *sendbuf, char *recvbuf,
                             PlanInfo &pi) {
    const int stride = VC_CHAIN_HEAD + vc_hop_slots(S);
    VcChainGuard guard;
    guard.cap_items = (int64_t)(c->desc.cap / (sizeof(int64_t) * (size_t)stride));
    guard.stage_cap = c->stage.cap >= 64 ? (int64_t)c->stage.cap - 64 : 0;
    guard.allowance = c->bound_staging ? c->staging_allowance : INT64_MAX;
    const int64_t guess = std::min<int64_t>(c->hint.items, guard.cap_items);
    if (!c->hint.valid || guess <= 0 || !c->B.chain_row_tot) return 2;
    // with per-launch timing on the host keeps its look at the plan: an event between the list kernel and the copy kernel
    // would sit in the stream's critical path (4 - 8 us a piece) and be counted as time of the copy kernel
    if (c->timing) return 2;
    // a guess far above the call's real length costs a workgroup that starts and ends for every item there is not: only
    // while the communicator's calls stay of a kind (the last one no more than twice the one before)
    if (c->hint.items > 2 * c->items_before_last) return 2;
    hipStream_t st = c->stream;
    const int lanes = vc_lanes_for_items(c->hint.payload, c->hint.items);
    HIP_TRY(vc_launch_chain_plan(S, T, c->B.slot_off, c->B.row_base, c->B.chain_row_tot + 2 * (size_t)S.P, c->desc.as<int64_t>(), guess, st,
                                 c->B.header, guard.cap_items));
    if (c->timing) HIP_TRY(hipEventRecord(c->events[2], st));
    int64_t done = 0;                                     // items the guarded launch was sized for
    HIP_TRY(vc_launch_copy_chains_guarded(c->desc.as<int64_t>(), stride, guess, lanes, sendbuf, recvbuf, c->stage.as<char>(), st, c->B.header,
                                          guard, &done));
    if (c->timing) HIP_TRY(hipEventRecord(c->events[3], st));
    HIP_TRY(VC_WAIT(c));
    int rc = plan_read(c, S, L, pi, true);
    if (rc) return rc;                                    // (bad tables: the launches have moved nothing)
    if (!vc_chain_guard_ok(c->h_header, guard)) return 0;
    pi.chain_lanes = lanes;
    if (pi.chain_items > done) {                          // more pieces than the last call had
        HIP_TRY(vc_launch_copy_chains(c->desc.as<int64_t>() + done * stride, stride, pi.chain_items - done, lanes, sendbuf, recvbuf,
                                      c->stage.as<char>(), st));
        if (c->timing) HIP_TRY(hipEventRecord(c->events[3], st));
        HIP_TRY(VC_WAIT(c));
    }
    rc = finish_stats(c, pi, c->desc.p, true);
    return rc ? rc : 1;
}

static int run_schedule(vc_comm *c, const CallParams &q, const char *sendbuf, char *recvbuf, VcTables T, bool forward, bool reuse = false) {
    VcSched S;
    std::vector<VcLaunchInfo> L;
    const int rc_sched = make_schedule(c, q, forward, S, L, reuse);
    if (rc_sched) return schedule_error(rc_sched);
    S.recv_lo = (int)((uintptr_t)recvbuf & 4095);
    PlanInfo pi;
    hipStream_t st = c->stream;
    const VcDispatch d = forward ? vc_dispatch(c->forward, VC_CALL_BLOCKING, c->hint, S) : VcDispatch{0, 0, 0, {0, 0, 0, 0, 0}};
    const int pair_lanes = d.lanes;
    int rc = try_strided(c, S, L, sendbuf, recvbuf, T, d);
    if (rc) return rc < 0 ? rc : VC_OK;
    rc = plan_sizes(c, S, L, T, forward);
    if (rc) return rc;
    bool synced = false;
    if (pair_lanes) {
        // the copy kernel goes out right behind the planning kernels and checks their verdict on the device: when the
        // staging arena turns out too small it has touched nothing and goes out once more behind a larger arena; when the
        // call is not of the kind the last one made the host expect, the call continues through the list
        VcListlessGuard guard = d.guard;
        guard.max_len = 0;                                // (the limit of fixed-stride slots: compact ones hold any block)
        for (int attempt = 0; attempt < 2 && !pi.listless; attempt++) {
            guard.stage_cap = c->stage.cap >= 64 ? (int64_t)c->stage.cap - 64 : 0;
            if (c->timing) {
                // (the planning ended where the first attempt began: its event stays as events[1])
                if (attempt == 1) { std::swap(c->events[1], c->events[2]); c->plan_end = 1; }
                HIP_TRY(hipEventRecord(c->events[2], st));
            }
            HIP_TRY(vc_launch_copy_blocks(S, T, c->B.slot_off, c->B.row_base, c->B.header, guard, pair_lanes, sendbuf, recvbuf,
                                          c->stage.as<char>(), st));
            if (c->timing) HIP_TRY(hipEventRecord(c->events[3], st));
            HIP_TRY(VC_WAIT(c));
            synced = true;
            rc = plan_read(c, S, L, pi, true);
            if (rc) return rc;
            if (vc_listless_ok(c->h_header, guard)) { pi.listless = true; pi.chain_lanes = pair_lanes; break; }
            if (pi.stage_bytes <= guard.stage_cap) break;          // not a call for this kernel
            if (staging_out_of_bound(c, pi.stage_bytes, pi.payload_bytes)) break;
            HIP_TRY(reserve_stage(c, (size_t)pi.stage_bytes + 64));
        }
        if (pi.listless) return finish_stats(c, pi, nullptr, true);
    }
    if (!synced && forward) {
        rc = try_enqueued_list(c, S, L, T, sendbuf, recvbuf, pi);
        if (rc == 1) return VC_OK;
        if (rc < 0) return rc;
        synced = rc == 0;
    }
    if (!synced) {
        HIP_TRY(VC_WAIT(c));         // the staging arena and the item list are sized from the plan
        rc = plan_read(c, S, L, pi, forward);
        if (rc) return rc;
    }
    if (forward && staging_out_of_bound(c, pi.stage_bytes, pi.payload_bytes)) return run_schedule(c, q, sendbuf, recvbuf, T, false, true);
    if (!forward && worth_reusing(c, S, pi.stage_bytes)) return run_schedule(c, q, sendbuf, recvbuf, T, false, true);
    rc = plan_emit(c, S, L, T, c->desc, pi);
    if (rc) return rc;
    return run_items(c, pi, c->desc.p, sendbuf, recvbuf, true);
}

// The _async entry points: planning kernels and the listless copy kernel are enqueued and the call returns.  The copy
// kernel checks the planner's verdict on the device (tables, staging arena) and touches nothing when it is bad;
// vc_comm_wait reads the same verdict and reports it, or grows the arena and runs the copy again.
static int enqueue_async(vc_comm *c, const CallParams &q, const VcSched &S, std::vector<VcLaunchInfo> &L, const char *sendbuf, char *recvbuf,
                         VcTables T) {
    int rc = plan_sizes(c, S, L, T, true);
    if (rc) return rc;
    hipStream_t st = c->stream;
    const int lanes = vc_dispatch(c->forward, VC_CALL_LISTLESS_ONLY, c->hint, S).lanes;
    const VcListlessGuard guard = {c->stage.cap >= 64 ? (int64_t)c->stage.cap - 64 : 0, 0, 0, 0, 0};
    if (c->timing) HIP_TRY(hipEventRecord(c->events[2], st));
    HIP_TRY(vc_launch_copy_blocks(S, T, c->B.slot_off, c->B.row_base, c->B.header, guard, lanes, sendbuf, recvbuf, c->stage.as<char>(), st));
    if (c->timing) HIP_TRY(hipEventRecord(c->events[3], st));
    c->pending.active = true;
    c->pending.S = S; c->pending.T = T; c->pending.sendbuf = sendbuf; c->pending.recvbuf = recvbuf; c->pending.lanes = lanes;
    c->pending.n_launch_infos = (int)L.size();
    c->pending.q = q;
    return VC_OK;
}

extern "C" int vc_comm_wait(vc_comm_t c) {
    if (!c) return fail_arg("null communicator");
    if (!c->pending.active) {
        HIP_TRY(VC_WAIT(c));
        return VC_OK;
    }
    // whatever happens below, the call is over when this function returns: the communicator is free again and launches
    // on its own stream, not on the caller's (which the caller may destroy once the call has been collected)
    c->pending.active = false;
    struct Release {
        vc_comm *c;
        ~Release() {
            c->stream = c->pending.own_stream;
            c->busy.clear(std::memory_order_release);
        }
    } release{c};
    HIP_TRY(VC_WAIT(c));
    const VcSched &S = c->pending.S;
    std::vector<VcLaunchInfo> L((size_t)c->pending.n_launch_infos);     // plan_read only needs their number here
    PlanInfo pi;
    int rc = plan_read(c, S, L, pi, true);
    if (rc) return rc;
    VcListlessGuard guard = {c->stage.cap >= 64 ? (int64_t)c->stage.cap - 64 : 0, 0, 0, 0, 0};
    if (!vc_listless_ok(c->h_header, guard)) {            // the arena was too small: nothing has been moved yet
        // a call whose forwarded staging is out of the communicator's bound runs one launch per digit on reused staging,
        // like its blocking twin
        if (staging_out_of_bound(c, pi.stage_bytes, pi.payload_bytes))
            return run_schedule(c, c->pending.q, c->pending.sendbuf, c->pending.recvbuf, c->pending.T, false, true);
        HIP_TRY(reserve_stage(c, (size_t)pi.stage_bytes + 64));
        guard.stage_cap = (int64_t)c->stage.cap - 64;
        if (c->timing) {
            std::swap(c->events[1], c->events[2]);        // (the planning ended where the first attempt began)
            c->plan_end = 1;
            HIP_TRY(hipEventRecord(c->events[2], c->stream));
        }
        HIP_TRY(vc_launch_copy_blocks(S, c->pending.T, c->B.slot_off, c->B.row_base, c->B.header, guard, c->pending.lanes,
                                      c->pending.sendbuf, c->pending.recvbuf, c->stage.as<char>(), c->stream));
        if (c->timing) HIP_TRY(hipEventRecord(c->events[3], c->stream));
        HIP_TRY(VC_WAIT(c));
    }
    pi.listless = true;
    pi.chain_lanes = c->pending.lanes;
    return finish_stats(c, pi, nullptr, true);
}

static int check_common(vc_comm *c, const void *sendbuf, const void *recvbuf, int esz) {
    if (!c) return fail_arg("null communicator");
    if (!sendbuf || !recvbuf) return fail_arg("null buffer");
    if (esz < 1) return fail_arg("element size must be >= 1");
    if (!c->sbase || !c->rbase) return fail_arg("vc_comm_set_bases has not been called");
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev != c->device)
        return fail_arg("the communicator was created on another HIP device than the current one");
    return VC_OK;
}

VcTables make_tables(vc_comm *c, const int *sc, const int *sd, const int *rc, const int *rd) {
    VcTables T;
    T.sc = sc; T.sd = sd; T.rc = rc; T.rd = rd; T.sbase = c->sbase; T.rbase = c->rbase; T.rd_packed = nullptr;
    return T;
}

static int schedule_error(int code) {
    switch (code) {
    case VC_ERR_RADIX: g_last_error = "radix must be >= 2 (exclisive_or_alltoallv: the rank count must be a power of 2)"; break;
    case VC_ERR_GROUP: g_last_error = "the ranks per node must divide the rank count (uniform functions: 2 <= n < P)"; break;
    case VC_ERR_TOO_FEW_RANKS: g_last_error = "tuna_algorithm needs at least 3 ranks"; break;
    default: break;
    }
    return code;
}

// The alltoallv-shaped functions.
// `async_stream` (null: the blocking call): the stream the call is enqueued on; vc_comm_wait collects it.
static int run_v(VcFunc f, int n, int r, int batch, vc_comm *c, char *sendbuf, int *sendcounts, int *sdispls, int esz,
                 char *recvbuf, int *recvcounts, int *rdispls, int batch2 = 0, void **async_stream = nullptr) {
    int rc = check_common(c, sendbuf, recvbuf, esz);
    if (rc) return rc;
    VC_ONE_CALL(c);
    if (!sendcounts || !sdispls || !recvcounts || (f != VC_F_TTPL && !rdispls)) return fail_arg("null table");
    const CallParams q = {f, n, r, batch, esz, 0, batch2};
    const bool forward = c->forward != 0 || async_stream;
    if (!async_stream) return run_schedule(c, q, sendbuf, recvbuf, make_tables(c, sendcounts, sdispls, recvcounts, rdispls), forward);
    VcSched S;
    std::vector<VcLaunchInfo> L;
    rc = make_schedule(c, q, true, S, L);
    if (rc) return schedule_error(rc);
    S.recv_lo = (int)((uintptr_t)recvbuf & 4095);
    c->pending.own_stream = c->stream;
    c->stream = static_cast<hipStream_t>(*async_stream);
    rc = enqueue_async(c, q, S, L, sendbuf, recvbuf, make_tables(c, sendcounts, sdispls, recvcounts, rdispls));
    if (rc == VC_OK) busy_guard_.keep();
    else c->stream = c->pending.own_stream;
    return rc;
}

extern "C" int twophase_rbruck_alltoallv(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                         int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TWOPHASE, 0, r, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int twophase_rbruck_alltoallv_om(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                            int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_OM, 0, r, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int tuna_algorithm(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                              int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TUNA, 0, r, b, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int tuna2_algorithm(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                               int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TUNA2, 0, r, b, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int TTPL_BT_alltoallv(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                                 char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TTPL, n, r, bblock, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int TTPL_BT_alltoallv_s1(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                                    char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TTPL_S1, n, r, bblock, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int TTPL_rbruck_alltoallv(int n, int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                     int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TTPL_RBRUCK, n, r, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

// ---- the entry point that allocates nothing ----
// twophase_rbruck_alltoallv for callers that cannot allocate (code under HIP graph capture of its surroundings, tight
// serving loops, harnesses that forbid hipMalloc): the same schedule, planning kernels and copy kernel as the forwarded,
// listless execution of twophase_rbruck_alltoallv, with the plan tables and the staging arena carved out of the static
// device array `scratch` instead of the communicator's grow-only buffers.  No hipMalloc, hipFree, event or stream
// creation happens here; the pinned header the planner reports through was allocated by vc_comm_create.  Every call on
// a GPU uses that GPU's one array, so calls that overlap on one GPU race.  Nothing in the array needs to start at
// zero: the planning kernels overwrite every word they or the copy kernel later read.
static size_t carve(size_t &at, size_t bytes) {
    const size_t here = at;
    at += (bytes + 255) & ~(size_t)255;
    return here;
}

extern "C" int twophase_rbruck_alltoallv_noalloc(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                                 int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    int rc = check_common(c, sendbuf, recvbuf, sendtype_size);
    if (rc) return rc;
    VC_ONE_CALL(c);
    if (!sendcounts || !sdispls || !recvcounts || !rdispls) return fail_arg("null table");
    unsigned char *base = nullptr;
    if (c->device < VC_MAX_DEVICES) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        base = g_scratch_ptr[c->device];
    }
    if (!base) return fail_arg("the static scratch array was not resolved on this device", VC_ERR_HIP);
    // every communicator on this GPU shares the one array: a second call that would overlap this one is refused
    struct ScratchLock {
        std::atomic_flag &f;
        bool mine;
        explicit ScratchLock(std::atomic_flag &flag) : f(flag), mine(!flag.test_and_set(std::memory_order_acquire)) {}
        ~ScratchLock() { if (mine) f.clear(std::memory_order_release); }
    } scratch_lock(g_scratch_busy[c->device]);
    if (!scratch_lock.mine)
        return fail_arg("twophase_rbruck_alltoallv_noalloc: another call on this GPU is using the static scratch array", VC_ERR_BUSY);
    VcSched S;
    std::vector<VcLaunchInfo> L;
    rc = vc_make_schedule(VC_F_TWOPHASE, c->P, 0, r, 0, sendtype_size, 0, S, L, 0, true);
    if (rc) return schedule_error(rc);
    if (vc_hop_slots(S) > VC_MAX_HOP_SLOTS) return fail_arg("too many digits for forwarded execution");
    S.recv_lo = (int)((uintptr_t)recvbuf & 4095);
    // slices of the scratch array: plan tables first, the rest is the staging arena
    const PlanBufSizes z = plan_buf_sizes(S, 1, true);
    size_t at = 0;
    PlanBufs &B = c->B;
    B = PlanBufs();
    B.header = reinterpret_cast<int64_t *>(base + carve(at, z.header));
    B.slot_off = reinterpret_cast<int64_t *>(base + carve(at, z.slot_off));
    B.row_tot = reinterpret_cast<int64_t *>(base + carve(at, z.row_tot));
    B.row_base = reinterpret_cast<int64_t *>(base + carve(at, z.row_base));
    B.row_bytes = reinterpret_cast<int64_t *>(base + carve(at, z.row_bytes));
    B.chain_row_tot = reinterpret_cast<int64_t *>(base + carve(at, z.chain_row_tot));
    B.chain_row_base = reinterpret_cast<int64_t *>(base + carve(at, z.chain_row_base));
    if (at + 64 > (size_t)VC_NOALLOC_SCRATCH_BYTES) {
        char msg[200];
        snprintf(msg, sizeof msg, "twophase_rbruck_alltoallv_noalloc: the plan tables of %d ranks with radix %d need %zu bytes, the static "
                 "scratch array has %zu", c->P, S.r, at, (size_t)VC_NOALLOC_SCRATCH_BYTES);
        return fail_arg(msg, VC_ERR_SCRATCH);
    }
    char *stage = reinterpret_cast<char *>(base + at);
    VcListlessGuard guard = {(int64_t)((size_t)VC_NOALLOC_SCRATCH_BYTES - at - 64), 0, 0, 0, 0};
    VcTables T = make_tables(c, sendcounts, sdispls, recvcounts, rdispls);
    rc = enqueue_plan_sizes(c, S, L, T, true, false);
    if (rc) return rc;
    const int lanes = vc_dispatch(c->forward, VC_CALL_LISTLESS_ONLY, c->hint, S).lanes;
    HIP_TRY(vc_launch_copy_blocks(S, T, B.slot_off, B.row_base, B.header, guard, lanes, sendbuf, recvbuf, stage, c->stream));
    HIP_TRY(VC_WAIT(c));
    PlanInfo pi;
    rc = plan_read(c, S, L, pi, true);
    if (rc) return rc;
    if (!vc_listless_ok(c->h_header, guard)) {            // the copy kernel saw the same header and has touched nothing
        char msg[200];
        snprintf(msg, sizeof msg, "twophase_rbruck_alltoallv_noalloc: the call needs %lld bytes of staging, the static scratch array "
                 "has %lld left after the plan tables", (long long)pi.stage_bytes, (long long)guard.stage_cap);
        return fail_arg(msg, VC_ERR_SCRATCH);
    }
    pi.listless = true;
    pi.chain_lanes = lanes;
    const bool timing = c->timing;
    c->timing = false;                                    // no events were recorded
    rc = finish_stats(c, pi, nullptr, true);
    c->timing = timing;
    c->last_stage = stage;
    return rc;
}

// The linear comparators (src/MPICH_scattered.cpp, src/OpenMPI_basic_linear.cpp, src/OpenMPI_pairwise.cpp,
// src/exclusive_or_alltoallv.cpp, benchmarks/common.cpp): one hop per block.
extern "C" int MPICH_intra_scattered(int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                     int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_MPICH_SCATTERED, 0, 2, bblock, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int ompi_alltoallv_intra_basic_linear(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                                 int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_OMPI_LINEAR, 0, 2, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int ompi_alltoallv_intra_pairwise(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                             int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_OMPI_PAIRWISE, 0, 2, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int exclisive_or_alltoallv(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                      int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_XOR, 0, 2, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int spreadout_alltoallv(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                   int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_SPREADOUT, 0, 2, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

// src/twolayer_communicator_linear.cpp: node-local messages first, then the messages between nodes; one hop each.
extern "C" int twolayer_communicator_linear(int n, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                            int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TWOLAYER_LINEAR, n, 2, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls);
}

extern "C" int twolayer_communicator_linear_s2(int n, int bblock1, int bblock2, char *sendbuf, int *sendcounts, int *sdispls,
                                               int sendtype_size, char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size,
                                               vc_comm_t c) {
    (void)recvtype_size;
    return run_v(VC_F_TWOLAYER_LINEAR_S2, n, 2, bblock1, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls,
                 bblock2);
}

// The alltoall-shaped (equal blocks) functions: the count tables are implied.
static int run_uniform(VcFunc f, int n, int r, vc_comm *c, char *sendbuf, int sendcount, int esz, char *recvbuf, void **async_stream = nullptr) {
    int rc = check_common(c, sendbuf, recvbuf, esz);
    if (rc) return rc;
    VC_ONE_CALL(c);
    if (sendcount < 0) return fail_arg("negative block length");
    if ((int64_t)sendcount * c->P > 0x7FFFFFFF) return fail_arg("sendcount * P must fit the reference's int displacements");
    const CallParams q = {f, n, r, 0, esz, sendcount, 0};
    VcSched S;
    std::vector<VcLaunchInfo> L;
    const bool forward = c->forward != 0 || async_stream;
    rc = make_schedule(c, q, forward, S, L);              // (validates the tunables before anything is enqueued)
    if (rc) return schedule_error(rc);
    S.recv_lo = (int)((uintptr_t)recvbuf & 4095);
    const size_t PP = (size_t)c->P * c->P;
    HIP_TRY(c->uni_counts.reserve(sizeof(int) * PP));
    HIP_TRY(c->uni_displs.reserve(sizeof(int) * PP));
    hipStream_t const own = c->stream;
    if (async_stream) c->stream = static_cast<hipStream_t>(*async_stream);
    const int *cnt = c->uni_counts.as<int>(), *dsp = c->uni_displs.as<int>();
    hipError_t e = vc_launch_uniform_tables(c->uni_counts.as<int>(), c->uni_displs.as<int>(), sendcount, c->P, c->stream);
    if (e != hipSuccess) { c->stream = own; return fail_hip(e, "vc_launch_uniform_tables", __LINE__); }
    if (!async_stream) return run_schedule(c, q, sendbuf, recvbuf, make_tables(c, cnt, dsp, cnt, dsp), forward);
    c->pending.own_stream = own;
    rc = enqueue_async(c, q, S, L, sendbuf, recvbuf, make_tables(c, cnt, dsp, cnt, dsp));
    if (rc == VC_OK) busy_guard_.keep();
    else c->stream = own;
    return rc;
}

extern "C" int uniform_spreadout_twolayer(int n, int r, char *sendbuf, int sendcount, int sendtype_size, char *recvbuf,
                                          int recvcount, int recvtype_size, vc_comm_t c) {
    (void)recvcount; (void)recvtype_size;
    return run_uniform(VC_F_UNIFORM_SPREADOUT, n, r, c, sendbuf, sendcount, sendtype_size, recvbuf);
}

extern "C" int uniform_inverse_isplit_r_bruck(int n, int r1, int r2, char *sendbuf, int sendcount, int sendtype_size,
                                              char *recvbuf, int recvcount, int recvtype_size, vc_comm_t c) {
    (void)recvcount; (void)recvtype_size; (void)r2;          // r2 is overwritten with the group count (:158)
    return run_uniform(VC_F_UNIFORM_ISPLIT, n, r1, c, sendbuf, sendcount, sendtype_size, recvbuf);
}

// ---- the _async twins of the seven collectives: enqueue on `hip_stream` (which becomes the communicator's stream) and
// return; vc_comm_wait completes the call and reports what the planner found.
extern "C" int twophase_rbruck_alltoallv_async(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                               int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvtype_size;
    return run_v(VC_F_TWOPHASE, 0, r, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls, 0, &hip_stream);
}

extern "C" int twophase_rbruck_alltoallv_om_async(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                                  int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvtype_size;
    return run_v(VC_F_OM, 0, r, 0, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls, 0, &hip_stream);
}

extern "C" int tuna_algorithm_async(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                    int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvtype_size;
    return run_v(VC_F_TUNA, 0, r, b, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls, 0, &hip_stream);
}

extern "C" int TTPL_BT_alltoallv_async(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                                       char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvtype_size;
    return run_v(VC_F_TTPL, n, r, bblock, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls, 0, &hip_stream);
}

extern "C" int TTPL_BT_alltoallv_s1_async(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                                          char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvtype_size;
    return run_v(VC_F_TTPL_S1, n, r, bblock, c, sendbuf, sendcounts, sdispls, sendtype_size, recvbuf, recvcounts, rdispls, 0, &hip_stream);
}

extern "C" int uniform_spreadout_twolayer_async(int n, int r, char *sendbuf, int sendcount, int sendtype_size, char *recvbuf,
                                                int recvcount, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvcount; (void)recvtype_size;
    return run_uniform(VC_F_UNIFORM_SPREADOUT, n, r, c, sendbuf, sendcount, sendtype_size, recvbuf, &hip_stream);
}

extern "C" int uniform_inverse_isplit_r_bruck_async(int n, int r1, int r2, char *sendbuf, int sendcount, int sendtype_size,
                                                    char *recvbuf, int recvcount, int recvtype_size, vc_comm_t c, void *hip_stream) {
    (void)recvcount; (void)recvtype_size; (void)r2;
    return run_uniform(VC_F_UNIFORM_ISPLIT, n, r1, c, sendbuf, sendcount, sendtype_size, recvbuf, &hip_stream);
}

// ------------------------------------------------------------- persistent plans

struct vc_plan {
    vc_comm *comm = nullptr;
    PlanInfo info;
    DevBuf items;
};

static bool func_by_name(const char *name, VcFunc &f) {
    static const struct { const char *name; VcFunc f; } table[] = {
        {"twophase_rbruck_alltoallv", VC_F_TWOPHASE}, {"twophase_rbruck_alltoallv_om", VC_F_OM}, {"tuna_algorithm", VC_F_TUNA}, {"tuna2_algorithm", VC_F_TUNA2},
        {"TTPL_BT_alltoallv", VC_F_TTPL}, {"TTPL_BT_alltoallv_s1", VC_F_TTPL_S1}, {"TTPL_rbruck_alltoallv", VC_F_TTPL_RBRUCK},
        {"twolayer_communicator_linear", VC_F_TWOLAYER_LINEAR}, {"spreadout_alltoallv", VC_F_SPREADOUT},
        {"MPICH_intra_scattered", VC_F_MPICH_SCATTERED}, {"ompi_alltoallv_intra_basic_linear", VC_F_OMPI_LINEAR},
        {"ompi_alltoallv_intra_pairwise", VC_F_OMPI_PAIRWISE}, {"exclisive_or_alltoallv", VC_F_XOR},
        {"uniform_spreadout_twolayer", VC_F_UNIFORM_SPREADOUT}, {"uniform_inverse_isplit_r_bruck", VC_F_UNIFORM_ISPLIT}};
    for (const auto &e : table)
        if (strcmp(name, e.name) == 0) { f = e.f; return true; }
    return false;
}

extern "C" int vc_plan_create(const char *function, int n, int r, int batch, int *sendcounts, int *sdispls, int elem_size,
                              int *recvcounts, int *rdispls, int recvbuf_low_bits, vc_comm_t c, vc_plan_t *plan_out) {
    if (!c || !function || !plan_out) return fail_arg("vc_plan_create: null argument");
    if (elem_size < 1) return fail_arg("element size must be >= 1");
    if (!c->sbase || !c->rbase) return fail_arg("vc_comm_set_bases has not been called");
    VC_ONE_CALL(c);
    VcFunc f;
    if (!func_by_name(function, f)) return fail_arg("vc_plan_create: unknown function name");
    const bool uniform = f == VC_F_UNIFORM_SPREADOUT || f == VC_F_UNIFORM_ISPLIT;      // `batch` is the block length, tables implied
    if (!uniform && (!sendcounts || !sdispls || !recvcounts || (f != VC_F_TTPL && !rdispls))) return fail_arg("null table");
    if (uniform && (batch < 0 || (int64_t)batch * c->P > 0x7FFFFFFF)) return fail_arg("block length * P must fit the reference's int displacements");
    const CallParams q = {f, n, r, uniform ? 0 : batch, elem_size, uniform ? batch : 0, 0};
    const bool forward = c->forward != 0;
    int rc = VC_OK;
    {
        VcSched S;
        std::vector<VcLaunchInfo> L;
        rc = make_schedule(c, q, forward, S, L);          // validates the tunables before anything is allocated
        if (rc) return schedule_error(rc);
    }
    if (uniform) {
        const size_t PP = (size_t)c->P * c->P;
        HIP_TRY(c->uni_counts.reserve(sizeof(int) * PP));
        HIP_TRY(c->uni_displs.reserve(sizeof(int) * PP));
        HIP_TRY(vc_launch_uniform_tables(c->uni_counts.as<int>(), c->uni_displs.as<int>(), batch, c->P, c->stream));
        sendcounts = recvcounts = c->uni_counts.as<int>();
        sdispls = rdispls = c->uni_displs.as<int>();
    }
    vc_plan *p = new vc_plan();
    p->comm = c;
    rc = build_plan(c, q, recvbuf_low_bits & 4095, make_tables(c, sendcounts, sdispls, recvcounts, rdispls), p->items, p->info, forward);
    if (rc == VC_OK && hipStreamSynchronize(c->stream) != hipSuccess) rc = fail_arg("vc_plan_create: stream error", VC_ERR_HIP);
    if (rc == VC_OK && reserve_stage(c, (size_t)p->info.stage_bytes + 64) != hipSuccess)       // so that executing never allocates
        rc = fail_arg("vc_plan_create: cannot allocate the staging arena", VC_ERR_HIP);
    if (rc) { p->items.release(); delete p; return rc; }
    c->live_plans++;
    *plan_out = p;
    return VC_OK;
}

extern "C" int vc_plan_execute(vc_plan_t p, char *sendbuf, char *recvbuf) {
    if (!p || !sendbuf || !recvbuf) return fail_arg("vc_plan_execute: null argument");
    if ((int)((uintptr_t)recvbuf & (VC_LINE - 1)) != (p->info.recv_lo & (VC_LINE - 1)))
        return fail_arg("vc_plan_execute: recvbuf must have the low address bits the plan was made for");
    VC_ONE_CALL(p->comm);
    return run_items(p->comm, p->info, p->items.p, sendbuf, recvbuf, false);
}

extern "C" int vc_plan_execute_async(vc_plan_t p, char *sendbuf, char *recvbuf) {
    if (!p || !sendbuf || !recvbuf) return fail_arg("vc_plan_execute_async: null argument");
    if ((int)((uintptr_t)recvbuf & (VC_LINE - 1)) != (p->info.recv_lo & (VC_LINE - 1)))
        return fail_arg("vc_plan_execute_async: recvbuf must have the low address bits the plan was made for");
    return launch_items(p->comm, p->info, p->items.p, sendbuf, recvbuf);
}

extern "C" int vc_plan_free(vc_plan_t p) {
    if (!p) return VC_OK;
    (void)hipStreamSynchronize(p->comm->stream);
    if (p->comm->last_items == p->items.as<VcDesc>()) { p->comm->last_items = nullptr; p->comm->last_nlaunch = 0; }
    p->items.release();
    if (--p->comm->live_plans == 0) free_retired_stage(p->comm);
    delete p;
    return VC_OK;
}
