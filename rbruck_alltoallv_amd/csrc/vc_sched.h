// vc_sched.h — host-side derivation of the schedule of one collective call: the
// reference's clamping and validation of its tunables, the digit phases, and which
// rounds share a kernel launch.  Plain C++ (no HIP calls) so that it can also be
// compiled into a CPU-only check of the plan.
#pragma once

#include <algorithm>
#include <cstring>
#include <vector>

#include "../../include/rbruck_vc.h"
#include "vc_common.h"

enum VcFunc {
    VC_F_TWOPHASE,           // twophase_rbruck_alltoallv
    VC_F_OM,                 // twophase_rbruck_alltoallv_om
    VC_F_TUNA,               // tuna_algorithm
    VC_F_TTPL,               // TTPL_BT_alltoallv
    VC_F_TTPL_S1,            // TTPL_BT_alltoallv_s1
    VC_F_UNIFORM_SPREADOUT,  // uniform_spreadout_twolayer
    VC_F_UNIFORM_ISPLIT,     // uniform_inverse_isplit_r_bruck
    // the linear comparators the reference times next to the Bruck variants: every block goes straight from
    // its source's sendbuf to its destination's recvbuf
    VC_F_SPREADOUT,          // spreadout_alltoallv
    VC_F_MPICH_SCATTERED,    // MPICH_intra_scattered
    VC_F_OMPI_LINEAR,        // ompi_alltoallv_intra_basic_linear
    VC_F_OMPI_PAIRWISE,      // ompi_alltoallv_intra_pairwise
    VC_F_XOR,                // exclisive_or_alltoallv
    VC_F_TUNA2,              // tuna2_algorithm: TuNA's rounds with the unpack deferred to the end of each digit
    VC_F_TWOLAYER_LINEAR,    // twolayer_communicator_linear
    VC_F_TWOLAYER_LINEAR_S2, // twolayer_communicator_linear_s2
    VC_F_TTPL_RBRUCK         // TTPL_rbruck_alltoallv: intra-node Bruck, then a Bruck over the nodes
};

// Digits of span-1 in base r and the number of unused values of the top digit, in
// integer arithmetic (src/tuna.cpp:28-31).  The float-log form of
// src/twophase_tunable_rbruckv.cpp:30-32 gives the same rounds: where it differs it
// adds a top digit with no rounds.
inline void vc_radix_params(int span, int r, int &w, int &d) {
    w = 0;
    for (int top = span - 1; top; top /= r) w++;
    int nlpow = 1;
    for (int i = 0; i < w - 1; i++) nlpow *= r;
    d = w ? (nlpow * r - span) / nlpow : 0;
}

// One launch per digit, or per `batch` rounds of a digit (TuNA's b, src/tuna.cpp:69).
inline void vc_add_intra_launches(std::vector<VcLaunchInfo> &out, const VcSched &S, int d, int batch) {
    for (int k = 0; k < S.w; k++) {
        const int x = S.msd ? S.w - 1 - k : k;
        int dist = 1;
        for (int i = 0; i < x; i++) dist *= S.r;
        const int ze = (x == S.w - 1) ? S.r - d : S.r;      // digit values 1 .. ze-1 occur
        if (ze - 1 < 1) continue;
        const int step = (batch <= 0 || batch > ze - 1) ? ze - 1 : batch;
        for (int zlo = 1; zlo < ze; zlo += step) {
            VcLaunchInfo li;
            memset(&li, 0, sizeof li);
            li.kind = 0; li.x = x; li.dist = dist; li.zlo = zlo; li.zhi = std::min(zlo + step - 1, ze - 1);
            out.push_back(li);
        }
    }
}

// Inter-node Bruck: one launch per digit of the group offset, least significant first.
inline void vc_add_inter_bruck_launches(std::vector<VcLaunchInfo> &out, const VcSched &S, int d2) {
    int dist = 1;
    for (int x = 0; x < S.w2; x++, dist *= S.r) {
        const int ze = (x == S.w2 - 1) ? S.r - d2 : S.r;
        if (ze - 1 < 1) continue;
        VcLaunchInfo li;
        memset(&li, 0, sizeof li);
        li.kind = 4; li.x = x; li.dist = dist; li.zlo = 1; li.zhi = ze - 1;
        out.push_back(li);
    }
}

// Inter-node messages, `qstep` (group distance, source local index) pairs per launch.
inline void vc_add_inter_launches(std::vector<VcLaunchInfo> &out, const VcSched &S, int qstep) {
    if (S.G <= 1) return;
    if (qstep <= 0 || qstep > S.P) qstep = S.P;
    for (int q = 0; q < S.P; q += qstep) {
        VcLaunchInfo li;
        memset(&li, 0, sizeof li);
        li.kind = 1; li.x = -1; li.qlo = q; li.qhi = std::min(q + qstep, S.P);
        out.push_back(li);
    }
}

// Direct (one-hop) messages, `qstep` rank distances (source - destination) mod P per launch.
inline void vc_add_direct_launches(std::vector<VcLaunchInfo> &out, int P, int qstep) {
    if (qstep <= 0 || qstep > P) qstep = P;
    for (int q = 0; q < P; q += qstep) {
        VcLaunchInfo li;
        memset(&li, 0, sizeof li);
        li.kind = 2; li.x = -1; li.qlo = q; li.qhi = std::min(q + qstep, P);
        out.push_back(li);
    }
}

// Direct messages of the linear two-layer comparators: `scope` 1 = inside the node, batches of the local rank
// distance; `scope` 2 = between nodes, batches of (group distance)*n + source local index.
inline void vc_add_scoped_direct_launches(std::vector<VcLaunchInfo> &out, int scope, int qfirst, int qend, int qstep) {
    if (qstep <= 0 || qstep > qend) qstep = qend;
    for (int q = qfirst; q < qend; q += qstep) {
        VcLaunchInfo li;
        memset(&li, 0, sizeof li);
        li.kind = 2; li.x = scope; li.qlo = q; li.qhi = std::min(q + qstep, qend);
        out.push_back(li);
    }
}

// Fills S and L for function f.  `r`, `batch` (b of tuna_algorithm, bblock of the TTPL functions; with batch2 the two
// bblocks of twolayer_communicator_linear_s2) and `n`
// are the caller's raw values; `forward`: the schedule is for forwarded execution (one work item per block piece
// through all hops).  Returns VC_OK or the code the entry point must return.
inline int vc_make_schedule(VcFunc f, int P, int n, int r, int batch, int esz, int uniform_count, VcSched &S,
                            std::vector<VcLaunchInfo> &L, int batch2 = 0, bool forward = false) {
    memset(&S, 0, sizeof S);
    L.clear();
    S.P = P; S.esz = esz; S.uniform = uniform_count;
    if (forward) batch = batch2 = 0;                        // one kernel performs every hop: batches of rounds mean nothing

    int d = 0;
    switch (f) {
    case VC_F_TWOPHASE:
    case VC_F_OM:
        if (r < 2) return VC_ERR_RADIX;                     // src/twophase_tunable_rbruckv.cpp:16, -om.cpp:13
        if (r > P) r = P;                                   // :22, :19
        S.n = P; S.G = 1; S.r = r; S.msd = (f == VC_F_TWOPHASE); S.last_hop = 0;
        vc_radix_params(P, S.r, S.w, d);
        vc_add_intra_launches(L, S, d, 0);
        break;
    case VC_F_TUNA:
    case VC_F_TUNA2:                                        // src/tuna2.cpp:13-21: the same clamps; one launch per batch is already
                                                            // "all rounds received, then unpacked together" (:202-223)
        if (P < 3) return VC_ERR_TOO_FEW_RANKS;             // src/tuna.cpp:20,28 never returns
        if (r < 2) r = 2;                                   // :13
        if (r > P - 1) r = P - 1;                           // :20
        if (batch <= 0 || batch > P) batch = P;             // :21
        S.n = P; S.G = 1; S.r = r; S.msd = 0; S.last_hop = 0;
        vc_radix_params(P, S.r, S.w, d);
        vc_add_intra_launches(L, S, d, batch);
        break;
    case VC_F_TTPL:
    case VC_F_TTPL_S1:
        if (r < 2) return VC_ERR_RADIX;                     // src/twophase_twolayer_rbruck.cpp:242, :472
        if (n < 1 || P % n != 0) return VC_ERR_GROUP;       // the reference truncates P/n (:260) and hangs
        if (r > n) r = n;                                   // :248
        S.n = n; S.G = P / n; S.r = std::max(r, 2); S.msd = 0; S.last_hop = 1;
        S.packed_recv = (f == VC_F_TTPL);                   // the coalesced variant never reads rdispls
        vc_radix_params(n, S.r, S.w, d);
        vc_add_intra_launches(L, S, d, 0);
        if (f == VC_F_TTPL_S1) {
            vc_add_inter_launches(L, S, (batch <= 0 || batch > P) ? P : batch);                 // :621
        } else {
            const int groups = (batch <= 0 || batch > S.G) ? S.G : batch;                      // :421
            const size_t first_inter = L.size();
            vc_add_inter_launches(L, S, groups * n);
            // coalesced messages need the organized region, which the intra-node launches fill; forwarded execution
            // carries every block on its own and keeps the per-block inter-node messages
            if (S.w > 0 && S.G > 1 && !forward) {
                S.coalesce = 1;
                for (size_t k = first_inter; k < L.size(); k++) L[k].kind = 3;
            }
        }
        break;
    case VC_F_TTPL_RBRUCK: {
        if (r < 2) return VC_ERR_RADIX;                     // src/twophase_twolayer_rbruck.cpp:20
        if (n < 1 || P % n != 0) return VC_ERR_GROUP;
        if (r > n) r = n;                                   // :26
        S.n = n; S.G = P / n; S.r = std::max(r, 2); S.msd = 0; S.last_hop = 0;
        vc_radix_params(n, S.r, S.w, d);                    // :42
        vc_add_intra_launches(L, S, d, 0);
        if (L.empty()) {                                    // n == 1: the copies to self need a launch of their own (the
            VcLaunchInfo li;                                // entries of an inter-node launch are not indexed by source rank)
            memset(&li, 0, sizeof li);
            li.kind = 0; li.dist = 1; li.zlo = 1; li.zhi = 0;
            L.push_back(li);
        }
        int d2 = 0;
        vc_radix_params(S.G, S.r, S.w2, d2);                // :45, the same radix for the digits of the group offset
        vc_add_inter_bruck_launches(L, S, d2);
        break;
    }
    case VC_F_UNIFORM_SPREADOUT:
    case VC_F_UNIFORM_ISPLIT:
        if (f == VC_F_UNIFORM_SPREADOUT && r < 2) return VC_ERR_RADIX;   // src/twolayer_rbruck.cpp:12
        if (r < 2) r = 2;                                                // :143
        if (n < 2 || n >= P || P % n != 0) return VC_ERR_GROUP;          // :18-22, :145-149 MPI_Abort
        if (r > n) r = n;
        S.n = n; S.G = P / n; S.r = r; S.msd = 1; S.last_hop = 1;   // intra-node phase is most significant digit first (:69)
        vc_radix_params(n, S.r, S.w, d);
        vc_add_intra_launches(L, S, d, 0);
        vc_add_inter_launches(L, S, P);                     // every group at once (:107-128; :243-274 with r2 = ngroup)
        break;
    case VC_F_XOR:
        if ((P & (P - 1)) != 0) return VC_ERR_RADIX;        // src/exclusive_or_alltoallv.cpp:31 returns -1 unless P is a power of 2
        /* fall through */
    case VC_F_SPREADOUT:                                    // benchmarks/common.cpp:10-37: all 2P requests, one Waitall
    case VC_F_OMPI_LINEAR:                                  // src/OpenMPI_basic_linear.cpp:10-77: self copy, then everything at once
    case VC_F_OMPI_PAIRWISE:                                // src/OpenMPI_pairwise.cpp:32-58: P steps; independent, so one launch
        S.n = P; S.G = 1; S.r = 2; S.msd = 0; S.w = 0; S.last_hop = 2;
        vc_add_direct_launches(L, P, P);
        break;
    case VC_F_TWOLAYER_LINEAR:                              // src/twolayer_communicator_linear.cpp:13-88
    case VC_F_TWOLAYER_LINEAR_S2:                           // :92-192; batch = bblock1, batch2 = bblock2
        if (n < 1 || n >= P || P % n != 0) return VC_ERR_GROUP;           // :24-28 MPI_Abort (and misses n that does not divide P)
        S.n = n; S.G = P / n; S.r = 2; S.msd = 0; S.w = 0; S.last_hop = 2;
        // intra-node: MPICH_intra_scattered on the node's communicator, all at once (:45) or bblock1 at a time (:118-123)
        vc_add_scoped_direct_launches(L, 1, 0, n, f == VC_F_TWOLAYER_LINEAR ? n : ((batch <= 0 || batch > n) ? n : batch));
        // inter-node: one Waitall for everything (:55-83), or bblock2 (group distance, local index) pairs at a time (:140-181)
        vc_add_scoped_direct_launches(L, 2, f == VC_F_TWOLAYER_LINEAR ? n : 1, P,
                                      f == VC_F_TWOLAYER_LINEAR ? P : ((batch2 <= 0 || batch2 > P) ? P : batch2));
        break;
    case VC_F_MPICH_SCATTERED:                              // src/MPICH_scattered.cpp:31-70: bblock requests in flight
        S.n = P; S.G = 1; S.r = 2; S.msd = 0; S.w = 0; S.last_hop = 2;
        vc_add_direct_launches(L, P, (batch <= 0 || batch > P) ? P : batch);
        break;
    }
    if (L.empty()) {                                        // a single rank: only the copy to itself
        VcLaunchInfo li;
        memset(&li, 0, sizeof li);
        li.kind = 0; li.dist = 1; li.zlo = 1; li.zhi = 0;
        L.push_back(li);
    }
    if (L[0].kind != 2) L[0].self = 1;                      // direct launches carry the self block as distance 0
    vc_set_divisors(S);
    return VC_OK;
}
