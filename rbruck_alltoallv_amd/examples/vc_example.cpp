// vc_example.cpp — the reference's example drivers on the virtual communicator.
//
// One process plays all ranks.  The loop structure, the payload (element = destination + 10 * source), the sweep
// over block sizes (n = 2 .. 2048 elements of 8 bytes, a random share of n per pair) and the result lines follow
// examples/rbruckv_example.cpp:49-131, examples/twophaseLayer_example.cpp:48-225 and, for the equal-block functions,
// examples/twolayer_example.cpp:49-140 of the reference; where those
// call MPI_Alltoall / the displacement loops / a collective, this calls the function of librbruck_vc that replaces it.
// The error check compares every received element with the value its sender wrote (the reference's check_errors,
// src/utils.cpp:31-46, only tests the last decimal digit).
//
//   vc_example <nranks> <loop-count> <ncores-per-node> <base-list>
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
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

static uint64_t mix(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

int main(int argc, char **argv) {
    if (argc < 5) {
        printf("Usage: %s <nranks> <loop-count> <ncores-per-node> <base-list>\n", argv[0]);
        return -1;
    }
    const int P = atoi(argv[1]), loopcount = atoi(argv[2]), ncores = atoi(argv[3]);
    std::vector<int> bases;
    for (int i = 4; i < argc; i++) bases.push_back(atoi(argv[i]));
    typedef unsigned long long elem_t;
    const int esz = (int)sizeof(elem_t);

    vc_comm_t comm;
    CHECK_VC(vc_comm_create(P, &comm));
    const size_t table_bytes = sizeof(int) * (size_t)P * P;
    int *sc, *sd, *rc, *rd;
    int64_t *ext, *sbase, *rbase, *total;
    CHECK_HIP(hipMalloc(&sc, table_bytes)); CHECK_HIP(hipMalloc(&sd, table_bytes));
    CHECK_HIP(hipMalloc(&rc, table_bytes)); CHECK_HIP(hipMalloc(&rd, table_bytes));
    CHECK_HIP(hipMalloc(&ext, 2 * sizeof(int64_t) * P)); CHECK_HIP(hipMalloc(&sbase, sizeof(int64_t) * P));
    CHECK_HIP(hipMalloc(&rbase, sizeof(int64_t) * P)); CHECK_HIP(hipMalloc(&total, 2 * sizeof(int64_t)));

    long long errors = 0;
    std::vector<int> h_sc((size_t)P * P), h_sd((size_t)P * P), h_rc((size_t)P * P), h_rd((size_t)P * P);
    std::vector<int64_t> h_sbase(P), h_rbase(P);
    for (int n = 2; n <= 2048; n *= 2) {
        // sendcounts[i] = n * (rand() % 100) / 100 on every rank (twophaseLayer_example.cpp:60-63), from a fixed seed
        for (int s = 0; s < P; s++)
            for (int d = 0; d < P; d++) h_sc[(size_t)s * P + d] = (int)((n * (mix(mix((uint64_t)s * P + d) + n) % 100)) / 100);
        CHECK_HIP(hipMemcpy(sc, h_sc.data(), table_bytes, hipMemcpyHostToDevice));
        CHECK_VC(vc_alltoall_counts(sc, rc, comm));                     // MPI_Alltoall of the counts (:76)
        CHECK_VC(vc_displs_from_counts(sc, sd, ext, comm));             // the sdispls loop (:69-72)
        CHECK_VC(vc_displs_from_counts(rc, rd, ext + P, comm));         // the rdispls loop (:77-82)
        CHECK_VC(vc_bases_from_extents(ext, esz, 256, sbase, total, comm));
        CHECK_VC(vc_bases_from_extents(ext + P, esz, 256, rbase, total + 1, comm));
        int64_t h_total[2];
        CHECK_HIP(hipMemcpy(h_total, total, sizeof h_total, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(h_sd.data(), sd, table_bytes, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(h_rc.data(), rc, table_bytes, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(h_rd.data(), rd, table_bytes, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(h_sbase.data(), sbase, sizeof(int64_t) * P, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(h_rbase.data(), rbase, sizeof(int64_t) * P, hipMemcpyDeviceToHost));
        CHECK_VC(vc_comm_set_bases(comm, sbase, rbase));

        // send_buffer[index++] = i + rank * 10 (:91-95)
        std::vector<elem_t> h_send((size_t)h_total[0] / esz + 1, 0), h_recv((size_t)h_total[1] / esz + 1);
        for (int s = 0; s < P; s++)
            for (int d = 0; d < P; d++) {
                elem_t *at = h_send.data() + h_sbase[s] / esz + h_sd[(size_t)s * P + d];
                for (int k = 0; k < h_sc[(size_t)s * P + d]; k++) at[k] = (elem_t)d + (elem_t)s * 10;
            }
        char *sendbuf, *recvbuf;
        CHECK_HIP(hipMalloc(&sendbuf, h_total[0] + 16)); CHECK_HIP(hipMalloc(&recvbuf, h_total[1] + 16));
        CHECK_HIP(hipMemcpy(sendbuf, h_send.data(), h_total[0], hipMemcpyHostToDevice));

        // one timed call + the check, as every block of the reference's drivers does
        auto timed = [&](const char *tag, const std::function<int()> &call, const std::function<void(double)> &report) {
            for (int it = 0; it < loopcount; it++) {
                CHECK_HIP(hipMemset(recvbuf, 0, h_total[1]));
                const auto st = std::chrono::steady_clock::now();
                const int rcode = call();
                const double t = std::chrono::duration<double>(std::chrono::steady_clock::now() - st).count();
                if (rcode != 0) { printf("%s fail! (%d: %s)\n", tag, rcode, vc_last_error_string()); errors++; continue; }
                CHECK_HIP(hipMemcpy(h_recv.data(), recvbuf, h_total[1], hipMemcpyDeviceToHost));
                long long bad = 0;
                for (int t_ = 0; t_ < P; t_++)
                    for (int s = 0; s < P; s++) {
                        const elem_t *at = h_recv.data() + h_rbase[t_] / esz + h_rd[(size_t)t_ * P + s];
                        for (int k = 0; k < h_rc[(size_t)t_ * P + s]; k++) bad += at[k] != (elem_t)t_ + (elem_t)s * 10;
                    }
                if (bad) { printf("[%s] %d has errors %lld\n", tag, n, bad); errors += bad; }
                report(t);
            }
        };

        timed("Spreadout", [&] { return spreadout_alltoallv(sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
              [&](double t) { printf("[Spreadout] %d %d %g\n", P, n, t); });
        timed("MPICH_scattered", [&] { return MPICH_intra_scattered(ncores, sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
              [&](double t) { printf("[MPICH_scattered] %d %d %d %g\n", P, n, ncores, t); });
        timed("OMPI_linear", [&] { return ompi_alltoallv_intra_basic_linear(sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
              [&](double t) { printf("[OMPI_linear] %d %d %g\n", P, n, t); });
        timed("OMPI_pairwise", [&] { return ompi_alltoallv_intra_pairwise(sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
              [&](double t) { printf("[OMPI_pairwise] %d %d %g\n", P, n, t); });
        if ((P & (P - 1)) == 0)
            timed("ExcOr", [&] { return exclisive_or_alltoallv(sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
                  [&](double t) { printf("[ExcOr] %d %d %g\n", P, n, t); });
        for (int base : bases) {
            const int b = 1;
            timed("Rbruckv", [&] { return tuna2_algorithm(base, b, sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
                  [&](double t) { printf("[Rbruckv] %d, %d, %d, %d, %g\n", P, n, b, base, t); });
            if (ncores >= 1 && P % ncores == 0) {
                // TTPL_BT_alltoallv writes packed in source order; rdispls here are packed, so the check above holds
                timed("TTPL", [&] { return TTPL_BT_alltoallv(ncores, base, 0, sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
                      [&](double t) { printf("[TTPL] %d, %d, %d, %d, %g\n", P, n, 0, base, t); });
                timed("TTPL_S1", [&] { return TTPL_BT_alltoallv_s1(ncores, base, 0, sendbuf, sc, sd, esz, recvbuf, rc, rd, esz, comm); },
                      [&](double t) { printf("[TTPL_S1] %d, %d, %d, %d, %g\n", P, n, 0, base, t); });
            }
        }
        CHECK_HIP(hipFree(sendbuf)); CHECK_HIP(hipFree(recvbuf));

        // examples/twolayer_example.cpp:49-140: the equal-block functions, n elements per pair
        if (ncores >= 2 && ncores < P && P % ncores == 0 && (long long)n * P <= 0x7FFFFFFF) {
            std::vector<int64_t> h_ext((size_t)P, (int64_t)P * n);
            CHECK_HIP(hipMemcpy(ext, h_ext.data(), sizeof(int64_t) * P, hipMemcpyHostToDevice));
            CHECK_VC(vc_bases_from_extents(ext, esz, 256, sbase, total, comm));
            CHECK_VC(vc_bases_from_extents(ext, esz, 256, rbase, total + 1, comm));
            CHECK_HIP(hipMemcpy(h_total, total, sizeof h_total, hipMemcpyDeviceToHost));
            CHECK_HIP(hipMemcpy(h_sbase.data(), sbase, sizeof(int64_t) * P, hipMemcpyDeviceToHost));
            CHECK_VC(vc_comm_set_bases(comm, sbase, rbase));            // same layout on both sides
            std::vector<elem_t> u_send((size_t)h_total[0] / esz + 1, 0), u_recv((size_t)h_total[1] / esz + 1);
            for (int s = 0; s < P; s++)
                for (int d = 0; d < P; d++)
                    for (int k = 0; k < n; k++) u_send[h_sbase[s] / esz + (size_t)d * n + k] = (elem_t)d + (elem_t)s * 10;
            char *usend, *urecv;
            CHECK_HIP(hipMalloc(&usend, h_total[0] + 16)); CHECK_HIP(hipMalloc(&urecv, h_total[1] + 16));
            CHECK_HIP(hipMemcpy(usend, u_send.data(), h_total[0], hipMemcpyHostToDevice));
            auto timed_uniform = [&](const char *tag, int base, const std::function<int()> &call) {
                for (int it = 0; it < loopcount; it++) {
                    CHECK_HIP(hipMemset(urecv, 0, h_total[1]));
                    const auto st = std::chrono::steady_clock::now();
                    const int rcode = call();
                    const double t = std::chrono::duration<double>(std::chrono::steady_clock::now() - st).count();
                    if (rcode != 0) { printf("%s fail! (%d: %s)\n", tag, rcode, vc_last_error_string()); errors++; continue; }
                    CHECK_HIP(hipMemcpy(u_recv.data(), urecv, h_total[1], hipMemcpyDeviceToHost));
                    long long bad = 0;
                    for (int t_ = 0; t_ < P; t_++)
                        for (int s = 0; s < P; s++)
                            for (int k = 0; k < n; k++) bad += u_recv[h_sbase[t_] / esz + (size_t)s * n + k] != (elem_t)t_ + (elem_t)s * 10;
                    if (bad) { printf("[%s] %d has errors %lld\n", tag, base, bad); errors += bad; }
                    printf("[%s] %d, %d, %d, %g\n", tag, P, n, base, t);
                }
            };
            for (int base : bases) {
                timed_uniform("SOR_alltoall", base, [&] { return uniform_spreadout_twolayer(ncores, base, usend, n, esz, urecv, n, esz, comm); });
                timed_uniform("BR_alltoall", base, [&] { return uniform_inverse_isplit_r_bruck(ncores, base, base, usend, n, esz, urecv, n, esz, comm); });
            }
            CHECK_HIP(hipFree(usend)); CHECK_HIP(hipFree(urecv));
        }
    }
    printf("errors: %lld\n", errors);
    vc_comm_free(comm);
    for (void *p : {(void *)sc, (void *)sd, (void *)rc, (void *)rd, (void *)ext, (void *)sbase, (void *)rbase, (void *)total}) CHECK_HIP(hipFree(p));
    return errors != 0;
}
