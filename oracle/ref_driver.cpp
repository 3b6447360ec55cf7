/*
 * ref_driver.cpp — MPI driver around the REAL reference functions.
 *
 * TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/ together
 * with the reference's own sources, compiled where they lie under
 * /root/reference (never copied).  It plays the role of the reference's example
 * drivers (examples/rbruckv_example.cpp:49-131): every rank derives its row and
 * column of a P x P count matrix, fills its send blocks, calls one reference
 * function, and the slowest rank's time is reported (MPI_Allreduce MAX, as in
 * examples/rbruckv_example.cpp:123-131).  Unlike those drivers the payload pins
 * source, destination and position (oracle/vc_synth.h) and the result is also
 * compared with MPI_Alltoallv.
 *
 * usage: mpiexec -n P ref_driver FUNC COUNTS ESZ R B N BBLOCK LAYOUT PAYLOAD SEED ITERS OUT
 *   FUNC    twophase | om | tuna | tuna2 | ttpl | ttpl_s1 | uniform_spreadout | uniform_isplit |
 *           scattered | ompi_linear | ompi_pairwise | xor | spreadout | ttpl_rbruck (blocks from the own node only) | tl_linear | tl_linear_s2 (B = bblock1,
 *           BBLOCK = bblock2) | mpi_alltoallv
 *   COUNTS  file of P*P int32 (row = sender); for the uniform functions the decimal block count
 *   LAYOUT  0 packed ascending displacements, 1 reversed order with gaps
 *   OUT     prefix: OUT.digests (one hex FNV-1a per rank), OUT.recv.bin (all recv extents, rank
 *           order) when the total is below 16 MiB, OUT.times (seconds, max over ranks, per iteration)
 */
#include <mpi.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "rbruckv.h"   /* found through -I/root/reference/src */
#include "vc_synth.h"

static int rank_, nprocs_;

static void layout_displs(const std::vector<int> &counts, int layout, std::vector<int> &displs, int &extent) {
    int P = (int)counts.size();
    displs.assign(P, 0);
    int off = 0;
    if (layout == 0) {
        for (int i = 0; i < P; i++) { displs[i] = off; off += counts[i]; }
    } else {
        for (int i = P - 1; i >= 0; i--) { off += (i + rank_) % 3; displs[i] = off; off += counts[i]; }
    }
    extent = off;
}

int main(int argc, char **argv) {
    MPI_Init(&argc, &argv);
    MPI_Comm_size(MPI_COMM_WORLD, &nprocs_);
    MPI_Comm_rank(MPI_COMM_WORLD, &rank_);
    if (argc < 13) {
        if (rank_ == 0) fprintf(stderr, "usage: ref_driver FUNC COUNTS ESZ R B N BBLOCK LAYOUT PAYLOAD SEED ITERS OUT\n");
        MPI_Finalize();
        return 2;
    }
    std::string func = argv[1];
    const char *counts_arg = argv[2];
    int esz = atoi(argv[3]), r = atoi(argv[4]), b = atoi(argv[5]), n = atoi(argv[6]), bblock = atoi(argv[7]);
    int layout = atoi(argv[8]), payload = atoi(argv[9]);
    uint64_t seed = strtoull(argv[10], NULL, 10);
    int iters = atoi(argv[11]);
    std::string out = argv[12];
    int P = nprocs_;
    bool uniform = func.rfind("uniform", 0) == 0;

    std::vector<int> sendcounts(P), recvcounts(P), sdispls, rdispls;
    if (uniform) {
        int cnt = atoi(counts_arg);
        for (int i = 0; i < P; i++) sendcounts[i] = recvcounts[i] = cnt;
        layout = 0;
    } else {
        std::vector<int> matrix((size_t)P * P);
        FILE *f = fopen(counts_arg, "rb");
        if (!f || fread(matrix.data(), sizeof(int), (size_t)P * P, f) != (size_t)P * P) {
            fprintf(stderr, "rank %d: cannot read %d x %d counts from %s\n", rank_, P, P, counts_arg);
            MPI_Abort(MPI_COMM_WORLD, 3);
        }
        fclose(f);
        for (int i = 0; i < P; i++) {
            sendcounts[i] = matrix[(size_t)rank_ * P + i];
            recvcounts[i] = matrix[(size_t)i * P + rank_];
        }
    }
    int sext, rext;
    layout_displs(sendcounts, layout, sdispls, sext);
    layout_displs(recvcounts, func == "ttpl" ? 0 : layout, rdispls, rext);

    MPI_Datatype dtype;
    MPI_Type_contiguous(esz, MPI_CHAR, &dtype);
    MPI_Type_commit(&dtype);

    std::vector<unsigned char> sendbuf((size_t)sext * esz + 1), sendcopy, recvbuf((size_t)rext * esz + 1),
        expect((size_t)rext * esz + 1);
    for (int i = 0; i < P; i++)
        vc_fill_block(payload, seed, rank_, i, sendbuf.data() + (size_t)sdispls[i] * esz, (int64_t)sendcounts[i] * esz);
    sendcopy = sendbuf;

    memset(expect.data(), 0xEE, expect.size());
    MPI_Alltoallv(sendbuf.data(), sendcounts.data(), sdispls.data(), dtype, expect.data(), recvcounts.data(),
                  rdispls.data(), dtype, MPI_COMM_WORLD);

    std::vector<double> times;
    int ret = 0;
    for (int it = 0; it < iters; it++) {
        memset(recvbuf.data(), 0xEE, recvbuf.size());
        if (uniform) sendbuf = sendcopy;      /* the uniform functions use sendbuf as scratch */
        MPI_Barrier(MPI_COMM_WORLD);
        double st = MPI_Wtime();
        char *sb = (char *)sendbuf.data(), *rb = (char *)recvbuf.data();
        int *sc = sendcounts.data(), *sd = sdispls.data(), *rc = recvcounts.data(), *rd = rdispls.data();
        if (func == "twophase") ret = twophase_rbruck_alltoallv(r, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "om") ret = twophase_rbruck_alltoallv_om(r, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "tuna") ret = tuna_algorithm(r, b, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "tuna2") ret = tuna2_algorithm(r, b, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "ttpl") ret = TTPL_BT_alltoallv(n, r, bblock, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "ttpl_s1") ret = TTPL_BT_alltoallv_s1(n, r, bblock, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "uniform_spreadout") ret = uniform_spreadout_twolayer(n, r, sb, sendcounts[0], dtype, rb, recvcounts[0], dtype, MPI_COMM_WORLD);
        else if (func == "uniform_isplit") uniform_inverse_isplit_r_bruck(n, r, b, sb, sendcounts[0], dtype, rb, recvcounts[0], dtype, MPI_COMM_WORLD);
        else if (func == "scattered") ret = MPICH_intra_scattered(bblock, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "ompi_linear") ret = ompi_alltoallv_intra_basic_linear(sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "ompi_pairwise") ret = ompi_alltoallv_intra_pairwise(sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "xor") ret = exclisive_or_alltoallv(sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "spreadout") spreadout_alltoallv(sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "ttpl_rbruck") ret = TTPL_rbruck_alltoallv(n, r, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "tl_linear") ret = twolayer_communicator_linear(n, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "tl_linear_s2") ret = twolayer_communicator_linear_s2(n, b, bblock, sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else if (func == "mpi_alltoallv") ret = MPI_Alltoallv(sb, sc, sd, dtype, rb, rc, rd, dtype, MPI_COMM_WORLD);
        else { if (rank_ == 0) fprintf(stderr, "unknown FUNC %s\n", func.c_str()); MPI_Abort(MPI_COMM_WORLD, 2); }
        double el = MPI_Wtime() - st, mx = 0;
        MPI_Allreduce(&el, &mx, 1, MPI_DOUBLE, MPI_MAX, MPI_COMM_WORLD);
        times.push_back(mx);
    }

    /* TTPL_rbruck_alltoallv never unpacks what its inter-node phase exchanges (src/twophase_twolayer_rbruck.cpp:222-231):
     * only the blocks from the own node reach recvbuf, so only those are compared and digested */
    if (func == "ttpl_rbruck")
        for (int i = 0; i < P; i++)
            if (i / n != rank_ / n) recvcounts[i] = 0;

    /* mismatch against MPI_Alltoallv, over the receive blocks only */
    long long bad = 0, badsum = 0;
    for (int i = 0; i < P; i++)
        for (int64_t k = 0; k < (int64_t)recvcounts[i] * esz; k++)
            bad += recvbuf[(size_t)rdispls[i] * esz + k] != expect[(size_t)rdispls[i] * esz + k];
    long long send_changed = uniform ? 0 : (long long)(memcmp(sendbuf.data(), sendcopy.data(), sendbuf.size()) != 0);
    bad += send_changed;
    MPI_Allreduce(&bad, &badsum, 1, MPI_LONG_LONG, MPI_SUM, MPI_COMM_WORLD);

    uint64_t h = VC_FNV_OFFSET;
    for (int i = 0; i < P; i++) h = vc_fnv1a64(recvbuf.data() + (size_t)rdispls[i] * esz, (int64_t)recvcounts[i] * esz, h);
    std::vector<uint64_t> digests(P);
    MPI_Gather(&h, 1, MPI_UINT64_T, digests.data(), 1, MPI_UINT64_T, 0, MPI_COMM_WORLD);

    long long mybytes = (long long)rext * esz, total = 0;
    MPI_Allreduce(&mybytes, &total, 1, MPI_LONG_LONG, MPI_SUM, MPI_COMM_WORLD);
    std::vector<int> ext_all(P), ext_disp(P);
    std::vector<unsigned char> dump;
    bool do_dump = total < (16ll << 20);
    if (do_dump) {
        int mine = (int)mybytes;
        MPI_Gather(&mine, 1, MPI_INT, ext_all.data(), 1, MPI_INT, 0, MPI_COMM_WORLD);
        int off = 0;
        for (int i = 0; i < P; i++) { ext_disp[i] = off; off += ext_all[i]; }
        if (rank_ == 0) dump.resize((size_t)off + 1);
        MPI_Gatherv(recvbuf.data(), mine, MPI_CHAR, dump.data(), ext_all.data(), ext_disp.data(), MPI_CHAR, 0, MPI_COMM_WORLD);
    }
    if (rank_ == 0) {
        FILE *f = fopen((out + ".digests").c_str(), "w");
        for (int i = 0; i < P; i++) fprintf(f, "%016llx\n", (unsigned long long)digests[i]);
        fclose(f);
        f = fopen((out + ".times").c_str(), "w");
        for (double t : times) fprintf(f, "%.9f\n", t);
        fclose(f);
        if (do_dump) {
            f = fopen((out + ".recv.bin").c_str(), "wb");
            fwrite(dump.data(), 1, (size_t)total, f);
            fclose(f);
        }
        printf("ref_driver func=%s P=%d esz=%d r=%d b=%d n=%d bblock=%d layout=%d ret=%d mismatch_vs_MPI_Alltoallv=%lld\n",
               func.c_str(), P, esz, r, b, n, bblock, layout, ret, badsum);
        fflush(stdout);
    }
    MPI_Type_free(&dtype);
    MPI_Finalize();
    return badsum == 0 && ret == 0 ? 0 : 1;
}
