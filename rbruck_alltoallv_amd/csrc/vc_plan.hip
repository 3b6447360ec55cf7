// vc_plan.hip — turns the count tables into the list of block copies of every
// launch.
//
// The reference learns the size of each incoming block from a metadata
// MPI_Sendrecv before every data round ("two-phase", src/twophase_tunable_rbruckv.cpp:110).
// With all P ranks' tables in one address space the size of a block is simply
// sendcounts[s][t] of the (s, t) it belongs to, and which (s, t) sits in slot
// `id` of rank p before digit x follows from the residency invariant:
//   least significant digit first: s is (j mod r^x) ranks above the holder,
//   most significant digit first:  s is (j div r^(x+1)) * r^(x+1) ranks above it.
// Staging offsets (the reference's fixed-stride extra_buffer, :59) become
// exclusive prefix sums over the blocks that arrive in a rank's staging area in a
// digit phase, so the staging arena is compact.
#include "vc_common.h"
#include "vc_scan.h"

#include "vc_plan_math.h"

// ---- pass 1: per (digit, receiving rank) exclusive scan of the staging sizes ----
// grid (P, w).  slot_off[(x*P + to)*P + id] = offset of the slot inside the row.
__global__ __launch_bounds__(VC_THREADS) void vc_plan_stage_rows(VcSched S, VcTables T, int64_t *__restrict__ slot_off,
                                                                 int64_t *__restrict__ row_tot) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int to = blockIdx.x, x = blockIdx.y, P = S.P;
    int dist = 1;
    for (int k = 0; k < x; k++) dist *= S.r;
    int64_t carry = 0;
    for (int base = 0; base < P; base += VC_THREADS) {
        const int id = base + threadIdx.x;
        int64_t total;
        const int64_t v = (id < P) ? vc_stage_slot_size(S, T, x, dist, to, id) : 0;
        int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (id < P) slot_off[((int64_t)x * P + to) * P + id] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) row_tot[(int64_t)x * P + to] = carry;
}

// ---- pass 2: exclusive scan of the row totals; one workgroup ----
__global__ __launch_bounds__(VC_THREADS) void vc_plan_stage_bases(const int64_t *__restrict__ row_tot, int64_t *__restrict__ row_base,
                                                                  int64_t nrows, int64_t *__restrict__ header, int nheader) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    int64_t carry = 0;
    for (int64_t b0 = 0; b0 < nrows; b0 += VC_THREADS) {
        int64_t i = b0 + threadIdx.x, total;
        int64_t v = (i < nrows) ? row_tot[i] : 0;
        int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (i < nrows) row_base[i] = carry + ex;
        carry += total;
    }
    for (int i = threadIdx.x; i < nheader; i += VC_THREADS) header[i] = (i == 0) ? carry : 0;
}

// ---- pass 3: one descriptor per (launch, receiving rank, slot) ----
// grid (P, nlaunch).  Inactive entries get len = 0.
__global__ __launch_bounds__(VC_THREADS) void vc_plan_emit(VcSched S, const VcLaunchInfo *__restrict__ launches, VcTables T,
                                                           const int64_t *__restrict__ slot_off, const int64_t *__restrict__ row_base,
                                                           VcDesc *__restrict__ desc, int64_t *__restrict__ header) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int to = blockIdx.x, L = blockIdx.y, P = S.P;
    const VcLaunchInfo info = launches[L];
    int64_t moved = 0, payload = 0;
    for (int id = threadIdx.x; id < P; id += VC_THREADS) {
        if (L == 0) payload += (int64_t)T.rc[(int64_t)to * P + id] * S.esz;
        const VcDesc d = vc_emit_entry(S, info, T, slot_off, row_base, to, id);
        moved += d.len;
        desc[((int64_t)L * P + to) * P + id] = d;
    }
    moved = vc_block_sum(moved, lds);
    if (threadIdx.x == 0 && moved) atomicAdd((unsigned long long *)&header[2 + L], (unsigned long long)moved);
    if (L == 0) {
        payload = vc_block_sum(payload, lds);
        if (threadIdx.x == 0 && payload) atomicAdd((unsigned long long *)&header[1], (unsigned long long)payload);
    }
}

hipError_t vc_launch_plan(const VcSched &S, const VcLaunchInfo *launches_dev, int nlaunch, VcTables T, int64_t *slot_off,
                          int64_t *row_tot, int64_t *row_base, VcDesc *desc, int64_t *header, hipStream_t st) {
    if (S.w > 0)
        hipLaunchKernelGGL(vc_plan_stage_rows, dim3(S.P, S.w), dim3(VC_THREADS), 0, st, S, T, slot_off, row_tot);
    hipLaunchKernelGGL(vc_plan_stage_bases, dim3(1), dim3(VC_THREADS), 0, st, row_tot, row_base, (int64_t)S.w * S.P, header, 2 + nlaunch);
    hipLaunchKernelGGL(vc_plan_emit, dim3(S.P, nlaunch), dim3(VC_THREADS), 0, st, S, launches_dev, T, slot_off, row_base, desc, header);
    return hipGetLastError();
}

// ---- route inspection: bytes sent from every rank to every rank in one launch ----
__global__ __launch_bounds__(VC_THREADS) void vc_traffic_kernel(const VcDesc *__restrict__ desc, int64_t ndesc, int64_t *__restrict__ matrix, int P) {
    int64_t i = (int64_t)blockIdx.x * VC_THREADS + threadIdx.x;
    if (i >= ndesc) return;
    VcDesc d = desc[i];
    if (d.len > 0 && d.from >= 0)
        atomicAdd((unsigned long long *)&matrix[(int64_t)d.from * P + d.to], (unsigned long long)d.len);
}

hipError_t vc_launch_traffic(const VcDesc *desc, int64_t ndesc, int64_t *matrix, int P, hipStream_t st) {
    int64_t nb = (ndesc + VC_THREADS - 1) / VC_THREADS;
    if (nb < 1) nb = 1;
    hipLaunchKernelGGL(vc_traffic_kernel, dim3((unsigned)nb), dim3(VC_THREADS), 0, st, desc, ndesc, matrix, P);
    return hipGetLastError();
}
