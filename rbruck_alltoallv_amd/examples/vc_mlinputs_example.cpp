// vc_mlinputs_example.cpp — the reference's examples/MLinputs_example.cpp on the virtual communicator.
//
// Reads a communication-pattern matrix in the reference's text format (inputs/<P>proc/global_comm_pattern_<P>proc.txt:
// P lines of P byte counts, row = sender; examples/MLinputs_example.cpp:119-145), builds the displacements as the
// reference does (:52-62, packed, MPI_CHAR elements), and times the one-pass exchange ("MPI_Alltoallv" line of the
// reference, here spreadout_alltoallv) and twophase_rbruck_alltoallv for every base (:88-104), with the reference's
// result lines.  The payload is generated and checked on the device (the matrices move 5 - 13 GB).
//
//   vc_mlinputs_example <matrix.txt> <nranks> <loop-count> <base-list>
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <vector>

#include "../../include/rbruck_vc.h"

#define CHECK_HIP(expr)                                                                                   \
    do {                                                                                                  \
        hipError_t e_ = (expr);                                                                           \
        if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_)); exit(2); }     \
    } while (0)
#define CHECK_VC(expr)                                                                                    \
    do {                                                                                                  \
        int rc_ = (expr);                                                                                 \
        if (rc_ != 0) { fprintf(stderr, "%s returned %d: %s\n", #expr, rc_, vc_last_error_string()); exit(2); } \
    } while (0)

int main(int argc, char **argv) {
    if (argc < 5) {
        printf("Usage: %s <matrix.txt> <nranks> <loop-count> <base-list>\n", argv[0]);
        return -1;
    }
    const int P = atoi(argv[2]), loopcount = atoi(argv[3]);
    std::vector<int> bases;
    for (int i = 4; i < argc; i++) bases.push_back(atoi(argv[i]));

    // read_file (:119-145): the whole matrix; rank p's sendcounts are row p
    std::vector<int> h_sc((size_t)P * P);
    {
        std::ifstream file(argv[1]);
        if (!file.is_open()) { fprintf(stderr, "cannot open %s\n", argv[1]); return 2; }
        for (size_t i = 0; i < h_sc.size(); i++) {
            long long v;
            if (!(file >> v) || v < 0 || v > 0x7FFFFFFF) { fprintf(stderr, "%s: entry %zu missing or out of range\n", argv[1], i); return 2; }
            h_sc[i] = (int)v;
        }
    }

    vc_comm_t comm;
    CHECK_VC(vc_comm_create(P, &comm));
    const size_t table_bytes = sizeof(int) * (size_t)P * P;
    int *sc, *sd, *rc, *rd;
    int64_t *ext, *sbase, *rbase, *total;
    CHECK_HIP(hipMalloc(&sc, table_bytes)); CHECK_HIP(hipMalloc(&sd, table_bytes));
    CHECK_HIP(hipMalloc(&rc, table_bytes)); CHECK_HIP(hipMalloc(&rd, table_bytes));
    CHECK_HIP(hipMalloc(&ext, 2 * sizeof(int64_t) * P)); CHECK_HIP(hipMalloc(&sbase, sizeof(int64_t) * P));
    CHECK_HIP(hipMalloc(&rbase, sizeof(int64_t) * P)); CHECK_HIP(hipMalloc(&total, 2 * sizeof(int64_t)));
    CHECK_HIP(hipMemcpy(sc, h_sc.data(), table_bytes, hipMemcpyHostToDevice));
    CHECK_VC(vc_alltoall_counts(sc, rc, comm));                 // the column of the matrix (:140-144)
    CHECK_VC(vc_displs_from_counts(sc, sd, ext, comm));         // :56-61
    CHECK_VC(vc_displs_from_counts(rc, rd, ext + P, comm));
    CHECK_VC(vc_bases_from_extents(ext, 1, 256, sbase, total, comm));
    CHECK_VC(vc_bases_from_extents(ext + P, 1, 256, rbase, total + 1, comm));
    int64_t h_total[2];
    CHECK_HIP(hipMemcpy(h_total, total, sizeof h_total, hipMemcpyDeviceToHost));
    CHECK_VC(vc_comm_set_bases(comm, sbase, rbase));
    long long send_tsize = 0;
    for (int v : h_sc) send_tsize += v;

    char *sendbuf, *recvbuf;
    CHECK_HIP(hipMalloc(&sendbuf, h_total[0] + 16)); CHECK_HIP(hipMalloc(&recvbuf, h_total[1] + 16));
    CHECK_VC(vc_fill_payload(0, 1, sendbuf, sc, sd, 1, comm));  // the reference fills random letters (:66-67)

    long long errors = 0;
    auto timed = [&](int (*call)(int, char *, int *, int *, int, char *, int *, int *, int, vc_comm_t), int base) {
        CHECK_HIP(hipMemset(recvbuf, 0, h_total[1]));
        const auto st = std::chrono::steady_clock::now();
        const int rcode = call(base, sendbuf, sc, sd, 1, recvbuf, rc, rd, 1, comm);
        const double t = std::chrono::duration<double>(std::chrono::steady_clock::now() - st).count();
        int64_t bad = -1;
        if (rcode != 0) { printf("call fails (%d: %s)\n", rcode, vc_last_error_string()); errors++; return t; }
        CHECK_VC(vc_verify_alltoallv(sendbuf, sc, sd, 1, recvbuf, rc, rd, 0, &bad, comm));
        if (bad) { printf("%lld bytes differ from the definition of alltoallv\n", (long long)bad); errors += bad; }
        return t;
    };
    auto one_pass = [](int, char *s, int *c1, int *d1, int e1, char *r, int *c2, int *d2, int e2, vc_comm_t cm) {
        return spreadout_alltoallv(s, c1, d1, e1, r, c2, d2, e2, cm);
    };

    for (int t = 0; t < loopcount; t++) {
        const double comm_time = timed(one_pass, 0);
        printf("MPI_Alltoallv, %d %g %lld %lld\n", P, comm_time, send_tsize, send_tsize);       // :75-80
    }
    for (size_t i = 0; i < bases.size(); i++)
        for (int it = 0; it < loopcount; it++) {
            printf("%zu %d twophase_rbruck_alltoallv\n", i, it);                                 // :91-93
            const double comm_time = timed(twophase_rbruck_alltoallv, bases[i]);
            printf("TUNA, %d %d %g %lld %lld\n", P, bases[i], comm_time, send_tsize, send_tsize); // :99-103
        }
    printf("errors: %lld\n", errors);

    CHECK_HIP(hipFree(sendbuf)); CHECK_HIP(hipFree(recvbuf));
    vc_comm_free(comm);
    for (void *p : {(void *)sc, (void *)sd, (void *)rc, (void *)rd, (void *)ext, (void *)sbase, (void *)rbase, (void *)total}) CHECK_HIP(hipFree(p));
    return errors != 0;
}
