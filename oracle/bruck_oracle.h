/*
 * bruck_oracle.h — CPU oracle for the radix-r Bruck alltoallv family.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * per-rank algorithms (KokoFan16/rbruck_alltoallv, the .cpp files under src/) in which P
 * "virtual" MPI ranks live in one process and every MPI_Sendrecv / Isend /
 * Irecv becomes a mailbox hand-over between two ranks' private buffers.  Only
 * tests, the smoke check and the benchmark's CPU-baseline leg may link or load
 * it; the product library never does.
 *
 * Calling convention (shared by every function below): one call serves all P
 * ranks.  `sendarena + sbase[p]` is what rank p would have passed as sendbuf,
 * `recvarena + rbase[p]` its recvbuf; the four tables are [P][P] row-major
 * int32 with row p = the array rank p would have passed; counts and
 * displacements are in elements of `esz` bytes.
 *
 * Parity pins: every function is checked (tests/test_oracle_*.py) against the
 * textbook MPI_Alltoallv definition on brute-force inputs, against the golden
 * digests produced by the real reference under mpiexec (tests/golden/), and
 * its round structure against the closed forms for K, ns and the residency
 * invariants.  No function is "parity unpinned"; ora_tuna2_algorithm is pinned by
 * the reference for b = 1 and by the definition for b > 1, where the reference
 * itself is defective; ora_TTPL_rbruck_alltoallv is pinned by the reference for
 * the blocks that stay inside a node (the reference drops the others after
 * exchanging them) and by the definition for all of them.
 */
#ifndef BRUCK_ORACLE_H_
#define BRUCK_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One record per simulated data message (the tag-1 MPI_Sendrecv, a direct
 * Isend/Irecv pair, or an inter-node message). */
typedef struct {
    int32_t kind;    /* 0 staged Bruck round, 1 direct single-block round, 2 inter-node coalesced,
                        3 inter-node staggered, 4 self copy, 5 direct message of a linear comparator,
                        6 round of the Bruck over the nodes */
    int32_t digit;   /* x for kind 0/1/6, -1 otherwise */
    int32_t z;       /* digit value of the round (kind 0/1/6), group distance otherwise */
    int32_t from, to;
    int32_t nblocks;
    int64_t bytes;
} ora_trace_rec;

/* Tracing is off by default.  ora_trace_begin() clears and enables it;
 * ora_trace_get() returns the records of the calls made since. */
void ora_trace_begin(void);
void ora_trace_end(void);
int64_t ora_trace_count(void);
const ora_trace_rec *ora_trace_data(void);

/* integer power (src/utils.cpp:9-16) */
int ora_pow(int x, unsigned int p);

/* radix parameters, float-log form (src/twophase_tunable_rbruckv.cpp:30-32) */
void ora_radix_params_float(int P, int r, int *w, int *nlpow, int *d);
/* radix parameters, integer form (src/tuna.cpp:28-31); also returns K */
void ora_radix_params_int(int P, int r, int *w, int *nlpow, int *d, int *K);

/* src/twophase_tunable_rbruckv.cpp:13-152 */
int ora_twophase_rbruck_alltoallv(int r, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                  const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                                  const int *recvcounts, const int *rdispls, int P);

/* src/twophase_tunable_rbruckv-om.cpp:10-157 */
int ora_twophase_rbruck_alltoallv_om(int r, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                     const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                                     const int *recvcounts, const int *rdispls, int P);

/* src/tuna.cpp:10-177.  Returns -3 for P < 3, where the reference never returns. */
int ora_tuna_algorithm(int r, int b, char *sendarena, const int64_t *sbase, const int *sendcounts,
                       const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                       const int *recvcounts, const int *rdispls, int P);

/* src/tuna2.cpp:10-239 with its send-buffer reuse (:175-185) repaired; see the note at the definition. */
int ora_tuna2_algorithm(int r, int b, char *sendarena, const int64_t *sbase, const int *sendcounts,
                        const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                        const int *recvcounts, const int *rdispls, int P);
int ora_compact_slot_float(int j, int r);

/* src/twophase_twolayer_rbruck.cpp:237-463 (coalesced; ignores rdispls).
 * Returns -2 when n does not divide P, where the reference hangs. */
int ora_TTPL_BT_alltoallv(int n, int r, int bblock, char *sendarena, const int64_t *sbase,
                          const int *sendcounts, const int *sdispls, int esz, char *recvarena,
                          const int64_t *rbase, const int *recvcounts, const int *rdispls, int P);

/* src/twophase_twolayer_rbruck.cpp:467-681 (staggered) */
int ora_TTPL_BT_alltoallv_s1(int n, int r, int bblock, char *sendarena, const int64_t *sbase,
                             const int *sendcounts, const int *sdispls, int esz, char *recvarena,
                             const int64_t *rbase, const int *recvcounts, const int *rdispls, int P);

/* src/twolayer_rbruck.cpp:10-134.  Equal blocks of sendcount*esz bytes; rank p's
 * buffers are P blocks long.  MUTATES sendarena like the reference does. */
int ora_uniform_spreadout_twolayer(int n, int r, char *sendarena, const int64_t *sbase, int sendcount,
                                   int esz, char *recvarena, const int64_t *rbase, int P);

/* src/twolayer_rbruck.cpp:137-277 */
int ora_uniform_inverse_isplit_r_bruck(int n, int r1, int r2, char *sendarena, const int64_t *sbase,
                                       int sendcount, int esz, char *recvarena, const int64_t *rbase, int P);

/* The linear comparators (kind 5 in the trace: one direct message per pair; z = the step or distance). */
int ora_spreadout_alltoallv(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls, int esz,
                            char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P);   /* benchmarks/common.cpp:10-37 */
int ora_MPICH_intra_scattered(int bblock, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                              int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P); /* src/MPICH_scattered.cpp:11-76 */
int ora_ompi_alltoallv_intra_basic_linear(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                          int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                          const int *rdispls, int P);                                              /* src/OpenMPI_basic_linear.cpp:10-77 */
int ora_ompi_alltoallv_intra_pairwise(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                      int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                      const int *rdispls, int P);                                                  /* src/OpenMPI_pairwise.cpp:14-64 */
int ora_exclisive_or_alltoallv(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls, int esz,
                               char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P);  /* src/exclusive_or_alltoallv.cpp:12-51 */

/* src/twophase_twolayer_rbruck.cpp:15-235.  The reference's inter-node Bruck (:179-227) exchanges its messages and
 * drops them; here the received blocks are kept (per-rank slots indexed by group offset and source local index) and
 * delivered after the last non-zero digit of their group offset.  Pinned by the reference for the blocks that stay
 * inside a node, by the definition of alltoallv for the rest. */
int ora_TTPL_rbruck_alltoallv(int n, int r, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                              int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P);

int ora_twolayer_communicator_linear(int n, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                     int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P); /* src/twolayer_communicator_linear.cpp:13-88 */
int ora_twolayer_communicator_linear_s2(int n, int bblock1, int bblock2, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                        const int *sdispls, int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                        const int *rdispls, int P);                                                              /* :92-192 */

/* Synthetic payload (oracle/vc_synth.h) written into every rank's send blocks. */
void ora_fill_payload(int mode, uint64_t seed, char *sendarena, const int64_t *sbase, const int *sendcounts,
                      const int *sdispls, int esz, int P);

/* FNV-1a 64 digest of each rank's receive blocks, in source-rank order. */
void ora_digest_recv(const char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls,
                     int esz, int P, uint64_t *digest_out);

#ifdef __cplusplus
}
#endif
#endif /* BRUCK_ORACLE_H_ */
