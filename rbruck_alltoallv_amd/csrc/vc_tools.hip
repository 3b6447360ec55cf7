// vc_tools.hip — what stands beside the collectives in the C ABI (include/rbruck_vc.h): the caller-side metadata steps of the
// reference's drivers, the choice of radix, inspection of the last call, and the harness utilities.
#include "vc_host.h"

// ------------------------------------------------------------ caller-side steps

extern "C" int vc_alltoall_counts(const int *sendcounts, int *recvcounts, vc_comm_t c) {
    if (!c || !sendcounts || !recvcounts) return fail_arg("vc_alltoall_counts: null argument");
    HIP_TRY(vc_launch_transpose(sendcounts, recvcounts, c->P, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

extern "C" int vc_displs_from_counts(const int *counts, int *displs, int64_t *extent_out, vc_comm_t c) {
    if (!c || !counts || !displs) return fail_arg("vc_displs_from_counts: null argument");
    VC_ONE_CALL(c);
    // the kernel raises the two flags in pinned host memory: no clearing launch before it, no copy back after it
    c->h_flags[0] = c->h_flags[1] = 0;
    HIP_TRY(vc_launch_row_scan(counts, displs, extent_out, c->h_flags_dev, c->P, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    if (c->h_flags[1]) return fail_arg("vc_displs_from_counts: negative count", VC_ERR_TABLES);
    if (c->h_flags[0]) return fail_arg("vc_displs_from_counts: a rank's counts sum past INT_MAX elements", VC_ERR_OVERFLOW);
    return VC_OK;
}

extern "C" int vc_bases_from_extents(const int64_t *extent, int elem_size, int64_t align, int64_t *base_out, int64_t *total_out,
                                     vc_comm_t c) {
    if (!c || !extent || !base_out || elem_size < 1 || align < 1) return fail_arg("vc_bases_from_extents: bad argument");
    HIP_TRY(vc_launch_bases(extent, elem_size, align, base_out, total_out, c->P, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

extern "C" int vc_allreduce_max_count(const int *sendcounts, int *max_out, vc_comm_t c) {
    if (!c || !sendcounts || !max_out) return fail_arg("vc_allreduce_max_count: null argument");
    HIP_TRY(vc_launch_max(sendcounts, max_out, (int64_t)c->P * c->P, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

// ------------------------------------------------------------------ radix choice

// Launches a schedule of radix r needs: one per digit that has rounds, plus the inter-node launch.
static int launches_for(int span, int r, bool inter) {
    int w, d;
    vc_radix_params(span, r, w, d);
    int n = 0;
    for (int x = 0; x < w; x++) n += ((x == w - 1) ? r - d : r) - 1 >= 1;
    return n + (inter ? 1 : 0);
}

// What this GPU sustains, measured once per communicator: a plain copy of 256 MiB (best of 3) and the cost of one more
// kernel launch on the stream (a row of 64 empty kernels).  The model below is priced in these two figures.
static int calibrate(vc_comm *c) {
    if (c->cal_copy_bytes_per_s > 0) return VC_OK;
    int rc = ensure_events(c, 2);
    if (rc) return rc;
    // 2 x 256 MiB where the device has room, 2 x 16 MiB where it is nearly full; with no room at all the figures of an idle
    // MI355X stand in (the suggestion then prices candidates with constants instead of measurements)
    size_t nb = (size_t)256 << 20;
    char *buf = nullptr;
    if (hipMalloc((void **)&buf, 2 * nb) != hipSuccess) {
        (void)hipGetLastError();
        nb = (size_t)16 << 20;
        if (hipMalloc((void **)&buf, 2 * nb) != hipSuccess) {
            (void)hipGetLastError();
            c->cal_copy_bytes_per_s = 6.0e12;
            c->cal_launch_s = 4.0e-6;
            c->cal_sync_s = 15.0e-6;
            return VC_OK;
        }
    }
    float best = 0.f, ms = 0.f;
    hipError_t e = hipSuccess;
    for (int rep = 0; rep < 4 && e == hipSuccess; rep++) {         // the first one warms up
        e = hipEventRecord(c->events[0], c->stream);
        if (e == hipSuccess) e = vc_launch_calibration_copy(buf, buf + nb, nullptr, (int64_t)nb, c->stream);
        if (e == hipSuccess) e = hipEventRecord(c->events[1], c->stream);
        if (e == hipSuccess) e = hipEventSynchronize(c->events[1]);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, c->events[0], c->events[1]);
        if (rep > 0 && (best == 0.f || ms < best)) best = ms;
    }
    const int row = 64;
    if (e == hipSuccess) e = hipEventRecord(c->events[0], c->stream);
    for (int k = 0; k < row && e == hipSuccess; k++) e = vc_launch_empty(c->stream);
    if (e == hipSuccess) e = hipEventRecord(c->events[1], c->stream);
    if (e == hipSuccess) e = hipEventSynchronize(c->events[1]);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, c->events[0], c->events[1]);
    (void)hipFree(buf);
    // a launch the host waits for, by the host's clock: what each of a blocking call's synchronisations costs
    const auto t0 = std::chrono::steady_clock::now();
    const int waits = 16;
    for (int k = 0; k < waits && e == hipSuccess; k++) {
        e = vc_launch_empty(c->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    }
    const double waited = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (e != hipSuccess) return fail_hip(e, "calibrate", __LINE__, __FILE_NAME__);
    c->cal_copy_bytes_per_s = 2.0 * (double)nb / (best * 1e-3);
    c->cal_launch_s = (double)ms * 1e-3 / row;
    c->cal_sync_s = waited / waits;
    return VC_OK;
}

extern "C" int vc_comm_calibration(vc_comm_t c, double *copy_bytes_per_s_out, double *launch_seconds_out) {
    if (!c) return fail_arg("null communicator");
    VC_ONE_CALL(c);
    int rc = calibrate(c);
    if (rc) return rc;
    if (copy_bytes_per_s_out) *copy_bytes_per_s_out = c->cal_copy_bytes_per_s;
    if (launch_seconds_out) *launch_seconds_out = c->cal_launch_s;
    return VC_OK;
}

#define VC_MAX_CANDIDATES 64
// the block movers sustain this share of the plain copy's rate on scattered, unaligned blocks (0.80 - 0.97 measured)
#define VC_BLOCK_COPY_EFFICIENCY 0.85

extern "C" int vc_suggest_tunables(const int *sendcounts, int elem_size, int n, const int *candidates, int ncand, int *r_out, int *b_out,
                                   double *seconds_out, int64_t *moved_bytes_out, vc_comm_t c) {
    if (!c || !sendcounts || !r_out || elem_size < 1 || ncand < 0 || ncand > VC_MAX_CANDIDATES || (ncand > 0 && !candidates))
        return fail_arg("vc_suggest_tunables: bad argument (0..64 candidates)");
    VC_ONE_CALL(c);
    const int P = c->P;
    if (n <= 0) n = P;
    if (P % n != 0) return fail_arg("n must divide the number of ranks", VC_ERR_GROUP);
    const int span = std::max(n, 2);
    int given[VC_MAX_CANDIDATES], cand[VC_MAX_CANDIDATES];
    if (ncand == 0) {                                     // every radix from 2 to min(span, 64), and the span itself (one hop)
        for (int r = 2; r <= std::min(span, VC_MAX_CANDIDATES - 1); r++) given[ncand++] = r;
        if (span > VC_MAX_CANDIDATES - 1) given[ncand++] = span;
    } else {
        for (int k = 0; k < ncand; k++) given[k] = candidates[k];
    }
    for (int k = 0; k < ncand; k++) {
        if (given[k] < 2) return fail_arg("radix must be >= 2", VC_ERR_RADIX);
        cand[k] = std::min(given[k], span);
    }
    int rc = calibrate(c);
    if (rc) return rc;
    const int words = 2 * (ncand + 1);
    HIP_TRY(c->scratch.reserve(sizeof(unsigned long long) * 2 * (VC_MAX_CANDIDATES + 1) + sizeof(int) * VC_MAX_CANDIDATES));
    unsigned long long *moved_dev = c->scratch.as<unsigned long long>();
    int *cand_dev = reinterpret_cast<int *>(moved_dev + 2 * (VC_MAX_CANDIDATES + 1));
    HIP_TRY(hipMemsetAsync(moved_dev, 0, sizeof(unsigned long long) * words, c->stream));
    HIP_TRY(hipMemcpyAsync(cand_dev, cand, sizeof(int) * ncand, hipMemcpyHostToDevice, c->stream));
    HIP_TRY(vc_launch_hop_bytes(sendcounts, elem_size, P, n, cand_dev, ncand, moved_dev, c->stream));
    unsigned long long got[2 * (VC_MAX_CANDIDATES + 1)];
    HIP_TRY(hipMemcpyAsync(got, moved_dev, sizeof(unsigned long long) * words, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    // Time model.  A blocking call waits for the stream twice (after sizing the plan, at the end) and launches three planning
    // kernels besides its copy kernels.  Every launch costs one launch latency; bytes move at the rate
    // of the plain copy times what the block movers keep of it.  One launch per digit: every hop reads and writes its
    // bytes and its 32-byte work items are written and read once.  Forwarded execution: one launch; the payload is read
    // once, every hop writes its bytes, and every piece has one item of 24 + 8 x (hop slots) bytes.  The planning kernels
    // read the count tables once per staging region.
    const double rate = c->cal_copy_bytes_per_s * VC_BLOCK_COPY_EFFICIENCY, launch = c->cal_launch_s;
    const double payload = (double)got[ncand], pieces = (double)got[2 * ncand + 1];
    double best = 0;
    int best_k = 0;
    for (int k = 0; k < ncand; k++) {
        const double moved = (double)got[k], hop_pieces = (double)got[ncand + 1 + k];
        int w, d;
        vc_radix_params(n, cand[k], w, d);
        const double plan = 2 * c->cal_sync_s + 3 * launch + (double)P * P * (w + 2) * 16.0 / rate;
        // (a forwarded call whose staging, the bytes of all hops but the last, is out of bound runs per digit)
        const bool forwarded = c->forward != 0 && !staging_out_of_bound(c, (int64_t)(moved - payload), (int64_t)payload);
        const double t = forwarded
            ? plan + launch + (payload + moved + 2.0 * pieces * (24 + 8 * (w + 1))) / rate
            : plan + launch * launches_for(n, cand[k], n < P) + (2.0 * moved + 2.0 * 32 * hop_pieces) / rate;
        if (moved_bytes_out) moved_bytes_out[k] = (int64_t)got[k];
        if (seconds_out) seconds_out[k] = t;
        if (k == 0 || t < best) { best = t; best_k = k; }
    }
    *r_out = given[best_k];
    // rounds of a digit per launch (b of tuna_algorithm): on one GPU the rounds of a digit are independent copies, so
    // splitting them over launches only adds launch latencies; all of them (r - 1) share a launch
    if (b_out) *b_out = std::max(cand[best_k] - 1, 1);
    return VC_OK;
}

extern "C" int vc_suggest_radix(const int *sendcounts, int elem_size, int n, const int *candidates, int ncand, int *best_out,
                                int64_t *moved_bytes_out, vc_comm_t c) {
    if (!candidates || ncand < 1) return fail_arg("vc_suggest_radix: bad argument (1..64 candidates)");
    return vc_suggest_tunables(sendcounts, elem_size, n, candidates, ncand, best_out, nullptr, nullptr, moved_bytes_out, c);
}

// ------------------------------------------------------------------ inspection

extern "C" int vc_comm_last_traffic(vc_comm_t c, int launch, int64_t *matrix_out) {
    if (!c || !matrix_out) return fail_arg("vc_comm_last_traffic: null argument");
    if (launch < 0 || launch >= c->last_nlaunch)
        return fail_arg("vc_comm_last_traffic: no such launch (forwarded execution has no per-digit launches to inspect)");
    const size_t PP = (size_t)c->P * c->P;
    HIP_TRY(c->scratch.reserve(sizeof(int64_t) * PP));
    HIP_TRY(hipMemsetAsync(c->scratch.p, 0, sizeof(int64_t) * PP, c->stream));
    HIP_TRY(vc_launch_traffic(c->last_items + c->launch_first[launch], c->launch_items[launch], c->scratch.as<int64_t>(), c->P,
                              c->stream));
    HIP_TRY(hipMemcpyAsync(matrix_out, c->scratch.p, sizeof(int64_t) * PP, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

extern "C" int vc_comm_staging(vc_comm_t c, void **ptr_out, int64_t *bytes_out) {
    if (!c || !ptr_out || !bytes_out) return fail_arg("vc_comm_staging: null argument");
    *ptr_out = const_cast<void *>(c->last_stage);
    *bytes_out = c->stats.staging_bytes;
    return VC_OK;
}

// ------------------------------------------------------------ harness utilities

extern "C" int vc_fill_payload(int mode, uint64_t seed, char *sendbuf, const int *sendcounts, const int *sdispls, int elem_size,
                               vc_comm_t c) {
    if (!c || !sendbuf || !sendcounts || !sdispls || elem_size < 1 || !c->sbase) return fail_arg("vc_fill_payload: bad argument");
    HIP_TRY(vc_launch_fill_payload(mode, seed, sendbuf, sendcounts, sdispls, c->sbase, elem_size, c->P, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

extern "C" int vc_verify_alltoallv(const char *sendbuf, const int *sendcounts, const int *sdispls, int elem_size,
                                   const char *recvbuf, const int *recvcounts, const int *rdispls, int packed_recv,
                                   int64_t *mismatch_out, vc_comm_t c) {
    if (!c || !sendbuf || !recvbuf || !sendcounts || !sdispls || !recvcounts || !mismatch_out || elem_size < 1 || !c->sbase)
        return fail_arg("vc_verify_alltoallv: bad argument");
    if (!packed_recv && !rdispls) return fail_arg("vc_verify_alltoallv: rdispls needed");
    const size_t PP = (size_t)c->P * c->P;
    VcTables T = make_tables(c, sendcounts, sdispls, recvcounts, rdispls);
    if (packed_recv) {
        HIP_TRY(c->rd_packed.reserve(sizeof(int) * PP));
        HIP_TRY(vc_launch_row_scan(recvcounts, c->rd_packed.as<int>(), nullptr, nullptr, c->P, c->stream));
        T.rd_packed = c->rd_packed.as<int>();
    }
    HIP_TRY(c->scratch.reserve(sizeof(int64_t) * PP));
    HIP_TRY(hipMemsetAsync(c->scratch.p, 0, sizeof(unsigned long long), c->stream));
    HIP_TRY(vc_launch_verify(sendbuf, recvbuf, T, elem_size, c->P, packed_recv, c->scratch.as<unsigned long long>(), c->stream));
    unsigned long long bad = 0;
    HIP_TRY(hipMemcpyAsync(&bad, c->scratch.p, sizeof bad, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    *mismatch_out = (int64_t)bad;
    return VC_OK;
}

extern "C" int vc_calibration_copy(char *dst, const char *src, int64_t nbytes, vc_comm_t c) {
    if (!c || !dst || !src || nbytes < 0 || (nbytes & 15) || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15))
        return fail_arg("vc_calibration_copy: 16-byte aligned pointers and size needed");
    HIP_TRY(vc_launch_calibration_copy(src, dst, nullptr, nbytes, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}

extern "C" int vc_calibration_copy2(char *dst, char *dst2, const char *src, int64_t nbytes, vc_comm_t c) {
    if (!c || !dst || !dst2 || !src || nbytes < 0 || (nbytes & 15) || ((uintptr_t)dst & 15) || ((uintptr_t)dst2 & 15) || ((uintptr_t)src & 15))
        return fail_arg("vc_calibration_copy2: 16-byte aligned pointers and size needed");
    HIP_TRY(vc_launch_calibration_copy(src, dst, dst2, nbytes, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    return VC_OK;
}
