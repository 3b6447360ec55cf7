/*
 * rbruck_vc.h — C ABI of the MI355X-native radix-r Bruck alltoallv library
 * (librbruck_vc.so): the alltoallv data path of KokoFan16/rbruck_alltoallv for
 * a VIRTUAL COMMUNICATOR of P ranks whose send, receive and staging buffers all
 * live in the HBM of one GPU.
 *
 * The collective entry points keep the reference's names and argument order
 * (src/rbruckv.h).  Three things change, uniformly:
 *   - one call serves all P ranks.  `sendbuf` / `recvbuf` are DEVICE pointers
 *     to arenas; rank p's buffer starts at sbase[p] / rbase[p] bytes into them
 *     (vc_comm_set_bases).  `sendcounts`, `sdispls`, `recvcounts`, `rdispls`
 *     are DEVICE pointers to [P][P] row-major int32 tables whose row p is the
 *     array rank p would have passed; units are elements, as in the reference;
 *   - MPI_Datatype becomes the element size in bytes (the reference only ever
 *     calls MPI_Type_size on it, src/twophase_tunable_rbruckv.cpp:28; the
 *     receive type is ignored there and here);
 *   - MPI_Comm becomes a vc_comm_t handle.
 * Calls are blocking like the reference's: the result is in `recvbuf` when the
 * function returns (the comm's stream has been synchronised).
 *
 * Return codes: 0 success; -1 radix < 2 where the reference returns -1;
 * further negative codes below for conditions under which the reference hangs,
 * aborts or overflows.
 */
#ifndef RBRUCK_VC_H_
#define RBRUCK_VC_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct vc_comm *vc_comm_t;

#define VC_OK 0
#define VC_ERR_RADIX (-1)      /* r < 2 (src/twophase_tunable_rbruckv.cpp:16, twophase_twolayer_rbruck.cpp:242,472) */
#define VC_ERR_GROUP (-2)      /* n does not divide P (the reference truncates P/n and hangs), or n >= P for the uniform functions (MPI_Abort, src/twolayer_rbruck.cpp:18-22) */
#define VC_ERR_TOO_FEW_RANKS (-3) /* tuna_algorithm with P < 3 (src/tuna.cpp:20,28 never returns) */
#define VC_ERR_HIP (-4)        /* a HIP runtime call failed; vc_last_error_string() says which */
#define VC_ERR_ARG (-5)        /* null handle / pointer, element size < 1, bases not set */
#define VC_ERR_NO_DEVICE (-6)  /* no HIP device */
#define VC_ERR_TABLES (-7)     /* a negative count or displacement in the tables, or recvcounts[t][s] != sendcounts[s][t] (the reference
                                  fails with an MPI truncation error); found on the device before anything is copied:
                                  recvbuf is untouched */
#define VC_ERR_OVERFLOW (-8)   /* a rank's counts sum past INT_MAX elements, where the reference's int displacements wrap
                                  (examples/rbruckv_example.cpp:69-72): vc_displs_from_counts, and the packed receive layout of
                                  TTPL_BT_alltoallv (src/twophase_twolayer_rbruck.cpp:406-418) */
#define VC_ERR_BUSY (-10)      /* the communicator is serving another call (a second host thread): one call at a time */
#define VC_ERR_SCRATCH (-9)    /* twophase_rbruck_alltoallv_noalloc: the call needs more than VC_NOALLOC_SCRATCH_BYTES */

/* ---- communicator (replaces MPI_Comm; MPI_Comm_size/MPI_Comm_rank have no per-rank analogue) ---- */

/* Creates a virtual communicator of `nranks` ranks on the current HIP device.  A communicator serves one call at a time
 * (it owns the staging arena and the planning buffers the calls reuse); use one per host thread or stream. */
int vc_comm_create(int nranks, vc_comm_t *comm_out);
/* Waits for the communicator's stream, then releases its device and pinned memory.  Free its plans first. */
int vc_comm_free(vc_comm_t comm);
int vc_comm_size(vc_comm_t comm);

/* Stream every kernel of this communicator is launched on (a hipStream_t; NULL = the default stream). */
int vc_comm_set_stream(vc_comm_t comm, void *hip_stream);

/* Where each rank's buffers start inside the arenas: two DEVICE arrays of P int64 byte offsets.  They are
 * read on the device at every call (not copied), so they must stay valid.  Required before any collective. */
int vc_comm_set_bases(vc_comm_t comm, const int64_t *sbase_bytes, const int64_t *rbase_bytes);

/* How the collectives execute (no counterpart in the reference, whose ranks are separate processes).
 * 1 (default): forwarded execution.  One launch for the whole call; the workgroup that moves a piece of a block performs
 *    all the hops of that block one after the other and keeps the piece in registers in between, so the data is read
 *    once (from sendbuf) and written once per hop (into the staging slot of every intermediate holder, then into
 *    recvbuf).  The batching tunables (b, bblock) then have no effect, and TTPL_BT_alltoallv sends its inter-node data
 *    per block instead of coalesced.  The copy kernel normally works through a list of block pieces that a planning
 *    kernel writes first, after the host has learnt its size (vc_stats_t.host_waits 2).  Once two calls in a row on the
 *    communicator were of a kind (the second no more than twice the pieces of the first), list and copy kernel are
 *    enqueued right behind the size computation, the list's length taken from the last call, and check the plan on the
 *    device instead (tables, room in the list and in the staging arena, the staging bound: host_waits 1); a call they
 *    cannot serve has moved nothing and is redone the usual way, a longer list than guessed gets a second launch.
 *    When the last call on the communicator consisted of
 *    short blocks, the next one goes without the list: every pair of ranks gets a workgroup (at most 128 ranks) or a
 *    quarter of a wavefront (short blocks: average piece below 768 B on any number of ranks, below 1.75 - 3 KiB on 33 - 128) that derives its block's route itself; the
 *    kernel is enqueued right behind the size computation and the call needs one host synchronisation instead of two.
 *    Such a call also gets the reference's own staging layout, every slot as long as the longest block
 *    (src/twophase_tunable_rbruckv.cpp:59; the stride comes from the last call's longest block): slot addresses are then
 *    closed forms and the call is a single kernel launch, without a planner before it.  Every pair of ranks checks its own
 *    table entries, and that its block fits a slot, before it forms an address from them; the kernel's first wavefronts
 *    check all of the tables and add up what the host needs afterwards, and the copying wavefronts hold their stores
 *    back until those have reported the tables in order (a call that returns VC_ERR_TABLES has written nothing here
 *    either); a call with a longer block is redone the general way.  Only on at most 192 ranks and while
 *    regions x P x P x stride stays below 256 MiB.
 *    On more than 192 ranks and blocks below 384 B on average a wavefront takes a batch of 16 - 64 pairs instead: a lane per
 *    pair works out the route, then the quarters of the wavefront carry the blocks one after the other.
 * 2: forwarded, always through the list.   3 / 4 / 5: forwarded, always without it, a workgroup / a quarter of a
 *    wavefront per pair of ranks / a batch of pairs per wavefront (any sizes; not the fastest choice everywhere).
 * 0: one kernel launch per digit phase (or per batch of its rounds, as b / bblock say); every hop reads the block
 *    where the previous hop left it.  This is the mode whose launches vc_comm_last_stats and vc_comm_last_traffic
 *    describe one by one.
 * Results are the same in all of them, and so are the staging contents wherever two modes use the same staging layout
 * (a region per digit phase: staging bound off, no fixed stride).  Applies to calls and to plans created afterwards
 * (plans always hold a list). */
int vc_comm_set_forwarding(vc_comm_t comm, int enable);

/* Whether the communicator bounds its staging memory (1, the default; a larger value: bounded, with an allowance of that many
 * MiB instead of an eighth of the device's memory, see below) or not (0).  The reference keeps one fixed-stride slot
 * per multi-hop offset and reuses it in every round (src/twophase_tunable_rbruckv-om.cpp:52-75).  Here, bounded:
 *  - one launch per digit: a staged block arrives in one digit phase and leaves in a later one; blocks with the same
 *    (arrival, departure) pair form a sub-region of the arena, and a sub-region is placed over the memory of sub-regions
 *    whose blocks have all left before it is written (first fit).  Calls with at least three staging regions whose
 *    separate regions would take more than a thirty-second of the allowance below (about 1 GiB: planning for reuse costs
 *    some tens of microseconds, and such a call is planned twice); the
 *    peak then stays below about 1.5 x the payload where separate regions need the sum over the blocks of
 *    (hops - 1) x bytes (configuration 5 with radix 2: 60 GB);
 *  - forwarded execution keeps every hop's copy of every block, because nothing reads them and so nothing says when one
 *    may be overwritten.  A call whose staging would pass both the allowance (an eighth of the device's memory, at least
 *    1 GiB) and three times its payload is therefore run one launch per digit instead (vc_stats_t.execution says so).
 * Unbounded: every digit phase has its own region and forwarded calls stay forwarded, whatever they need. */
int vc_comm_set_staging_bound(vc_comm_t comm, int enable);

/* Text of the most recent failure on this thread ("" if none). */
const char *vc_last_error_string(void);

/* ---- caller-side steps of the reference drivers, as kernels ---- */

/* MPI_Alltoall of one int per pair (examples/rbruckv_example.cpp:76): recvcounts[t][s] = sendcounts[s][t].
 * LDS-tiled P x P transpose. */
int vc_alltoall_counts(const int *sendcounts, int *recvcounts, vc_comm_t comm);

/* Exclusive prefix sum of every rank's counts (examples/rbruckv_example.cpp:69-72,77-82): displs[p][i] =
 * sum_{k<i} counts[p][k].  extent_out (may be NULL) receives each rank's total, P int64 elements.  Returns VC_ERR_TABLES
 * for a negative count and VC_ERR_OVERFLOW when a total does not fit an int (displs and extent_out are written anyway). */
int vc_displs_from_counts(const int *counts, int *displs, int64_t *extent_out, vc_comm_t comm);

/* Packed arena bases: base[p] = sum_{q<p} roundup(extent[q] * elem_size, align); total_out (device, 1 int64,
 * may be NULL) receives the arena size in bytes. */
int vc_bases_from_extents(const int64_t *extent, int elem_size, int64_t align, int64_t *base_out, int64_t *total_out,
                          vc_comm_t comm);

/* The reference's MPI_Allreduce(MAX) of the block length (src/twophase_tunable_rbruckv.cpp:40-44): max_out is
 * one device int.  Kept for interface parity; the GPU path sizes its staging by prefix sums instead. */
int vc_allreduce_max_count(const int *sendcounts, int *max_out, vc_comm_t comm);

/* ---- the alltoallv family (reference: src/rbruckv.h:24-26, 84-96, 39-45, 28-33) ---- */

/* src/twophase_tunable_rbruckv.cpp:13-152 — radix-r Bruck, most significant digit first. */
int twophase_rbruck_alltoallv(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                              int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twophase_tunable_rbruckv-om.cpp:10-157 — least significant digit first; single-block rounds go straight
 * from sendbuf to recvbuf. */
int twophase_rbruck_alltoallv_om(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                 int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/tuna.cpp:10-177 — as _om with r clamped to [2, P-1] and b rounds of a digit in flight together
 * (here: b rounds per kernel launch; b <= 0 or b > P means all of them). */
int tuna_algorithm(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                   int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/tuna2.cpp:10-239 — TuNA with the received rounds of a digit unpacked together at the end of the digit
 * (:202-223).  On the GPU that is what a launch per batch already does, so the schedule is tuna_algorithm's.  The
 * reference corrupts messages for b > 1 (one send buffer reused under in-flight sends, :175-185); this does not. */
int tuna2_algorithm(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                    int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twophase_twolayer_rbruck.cpp:237-463 — two-layer, coalesced inter-node messages, bblock groups in flight.
 * Like the reference it ignores rdispls: rank t's blocks land back to back in source-rank order. */
int TTPL_BT_alltoallv(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                      char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twophase_twolayer_rbruck.cpp:467-681 — two-layer, one inter-node message per block ("staggered"),
 * bblock of them in flight; honours rdispls. */
int TTPL_BT_alltoallv_s1(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                         char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twophase_twolayer_rbruck.cpp:15-235 — two-layer with a radix-r Bruck over the nodes as well: after the
 * intra-node phase (:88-168) the n blocks a rank holds per destination node travel together down the digits of the
 * group offset, least significant first, between ranks of equal local index (:179-227).  The reference stops after
 * exchanging those messages and never unpacks them (only blocks from the own node reach its recvbuf); this entry
 * point completes the phase: a block whose group offset has further non-zero digits waits in staging, otherwise it
 * lands in recvbuf at rdispls. */
int TTPL_rbruck_alltoallv(int n, int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                          int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twolayer_rbruck.cpp:10-134 — equal blocks of sendcount elements; rank p's buffers hold P blocks.
 * The reference scrambles sendbuf (and needs recvbuf[0..P) free of '1' bytes); this one leaves sendbuf intact. */
int uniform_spreadout_twolayer(int n, int r, char *sendbuf, int sendcount, int sendtype_size, char *recvbuf,
                               int recvcount, int recvtype_size, vc_comm_t comm);

/* src/twolayer_rbruck.cpp:137-277 — as above with a group-level Bruck whose radix the reference forces to the
 * number of groups (:158), i.e. one digit of direct rounds.  The reference returns void; this returns a code. */
int uniform_inverse_isplit_r_bruck(int n, int r1, int r2, char *sendbuf, int sendcount, int sendtype_size,
                                   char *recvbuf, int recvcount, int recvtype_size, vc_comm_t comm);

/* ---- the linear comparators the reference drivers time beside the Bruck variants
 * (examples/twophaseLayer_example.cpp:99-113).  On one GPU each is a single pass: every block goes straight from
 * its source's sendbuf to its destination's recvbuf.  Same argument order as the reference. ---- */

/* src/MPICH_scattered.cpp:11-76 — bblock messages per rank in flight (here: bblock rank distances per launch). */
int MPICH_intra_scattered(int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                          int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/OpenMPI_basic_linear.cpp:10-77 */
int ompi_alltoallv_intra_basic_linear(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                      int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/OpenMPI_pairwise.cpp:14-64 — the P pairwise steps are independent here and share one launch. */
int ompi_alltoallv_intra_pairwise(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                  int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/exclusive_or_alltoallv.cpp:12-51 (name as spelled there) — returns -1 unless P is a power of two (:31). */
int exclisive_or_alltoallv(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                           int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twolayer_communicator_linear.cpp:13-88 — node-local messages (MPICH_intra_scattered on the node's ranks), then
 * every message between nodes; returns -2 where the reference aborts (n >= P) or misbehaves (n does not divide P). */
int twolayer_communicator_linear(int n, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                 int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* src/twolayer_communicator_linear.cpp:92-192 — the same with bblock1 node-local and bblock2 inter-node messages in
 * flight.  (twolayer_communicator_linear_s3, :196-318, never delivers a rank's block to itself and is not provided.) */
int twolayer_communicator_linear_s2(int n, int bblock1, int bblock2, char *sendbuf, int *sendcounts, int *sdispls,
                                    int sendtype_size, char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size,
                                    vc_comm_t comm);

/* benchmarks/common.cpp:10-37 (declared in src/rbruckv.h:88-89; returns void there). */
int spreadout_alltoallv(char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                        int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* ---- _async twins of the seven collectives above (same reference functions: src/rbruckv.h:24-26, 28-33, 39-45, 84-93).
 * The reference's calls are blocking; on a GPU a caller wants to enqueue a collective behind its producer kernels, time it
 * with its own events, or overlap two communicators on two streams.  Same arguments plus the stream (a hipStream_t; it
 * becomes the communicator's stream): the planning kernels and the copy kernel are enqueued and the call returns without
 * having waited for the device.  The execution is the forwarded one without a work-item list (the copy kernel derives
 * every block's route itself and checks the planner's verdict on the device before it touches anything), so the batching
 * tunables have no effect; a workgroup serves each pair of ranks, or a quarter of a wavefront after a call of short blocks.
 * Calls of very long blocks are served faster by a persistent plan (vc_plan_execute_async).
 * Until vc_comm_wait the communicator is busy (other calls on it return VC_ERR_BUSY) and the tables, bases and buffers
 * must stay valid.  The return code covers what the host can check (0, -1, -2, -3, -5); vc_comm_wait reports the rest. */
int twophase_rbruck_alltoallv_async(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                    int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm, void *hip_stream);
int twophase_rbruck_alltoallv_om_async(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                       int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm, void *hip_stream);
int tuna_algorithm_async(int r, int b, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                         int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm, void *hip_stream);
int TTPL_BT_alltoallv_async(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                            char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm, void *hip_stream);
int TTPL_BT_alltoallv_s1_async(int n, int r, int bblock, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size,
                               char *recvbuf, int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm, void *hip_stream);
int uniform_spreadout_twolayer_async(int n, int r, char *sendbuf, int sendcount, int sendtype_size, char *recvbuf,
                                     int recvcount, int recvtype_size, vc_comm_t comm, void *hip_stream);
int uniform_inverse_isplit_r_bruck_async(int n, int r1, int r2, char *sendbuf, int sendcount, int sendtype_size,
                                         char *recvbuf, int recvcount, int recvtype_size, vc_comm_t comm, void *hip_stream);
/* Waits for the communicator's stream and completes the call an _async entry point enqueued: returns VC_ERR_TABLES /
 * VC_ERR_OVERFLOW when the planner refused the tables (recvbuf is then untouched), VC_ERR_HIP for a runtime failure; when the
 * staging arena was too small for the call (the copy kernel has then moved nothing) it grows the arena and runs the copy
 * kernel again before returning.  0 with nothing pending.  vc_comm_last_stats describes the call afterwards. */
int vc_comm_wait(vc_comm_t comm);

/* No counterpart in the reference.  twophase_rbruck_alltoallv for callers that cannot allocate device memory: code whose
 * surroundings are under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments, same
 * result (byte for byte) as twophase_rbruck_alltoallv in its forwarded execution, but the plan tables and the staging
 * arena are slices of one static device array of VC_NOALLOC_SCRATCH_BYTES that each GPU holds for the life of the
 * process: the call performs no hipMalloc / hipFree and creates no events or streams.  A call whose plan tables
 * (about 8 * P * P * (digits + 1) bytes) plus staging (the bytes of all blocks that make more than one hop, once per
 * intermediate hop, each rounded up to 128) exceed the array returns VC_ERR_SCRATCH and leaves recvbuf untouched.  All
 * calls on one GPU share that GPU's array: calls that overlap on one GPU (two host threads, two streams) race.
 * Blocking; vc_comm_set_timing has no effect on it. */
#define VC_NOALLOC_SCRATCH_BYTES (64u << 20)
int twophase_rbruck_alltoallv_noalloc(int r, char *sendbuf, int *sendcounts, int *sdispls, int sendtype_size, char *recvbuf,
                                      int *recvcounts, int *rdispls, int recvtype_size, vc_comm_t comm);

/* ---- persistent plans: the analogue of MPI-4 persistent collectives (MPI_Alltoallv_init / MPI_Start).
 * The reference re-exchanges its metadata in every call (src/twophase_tunable_rbruckv.cpp:110); when the same tables are
 * used again, a plan keeps the schedule, the staging layout and the work items, and executing it launches only the
 * copy kernels (no planning kernels, no host synchronisation before the final one).  No counterpart in the reference. ---- */

typedef struct vc_plan *vc_plan_t;

/* `function` is the name of one of the alltoallv-shaped entry points above ("twophase_rbruck_alltoallv", "tuna_algorithm",
 * "TTPL_BT_alltoallv", "spreadout_alltoallv", ...); n, r and batch (b / bblock) are that function's tunables, ignored where
 * it has none; for "uniform_spreadout_twolayer" and "uniform_inverse_isplit_r_bruck" batch is the block length in elements
 * and the four tables are implied (pass NULL).  The tables are read now and not needed afterwards; the communicator's
 * bases are read now too.
 * recvbuf_low_bits = (address of the recvbuf that will be passed) & 4095: the low 7 bits must match at execution, the
 * rest only decides where long copies are cut.  Same return codes as the function itself. */
int vc_plan_create(const char *function, int n, int r, int batch, int *sendcounts, int *sdispls, int elem_size,
                   int *recvcounts, int *rdispls, int recvbuf_low_bits, vc_comm_t comm, vc_plan_t *plan_out);

/* Runs the planned collective; blocking.  One plan (or call) per communicator at a time. */
int vc_plan_execute(vc_plan_t plan, char *sendbuf, char *recvbuf);
/* Only enqueues the copy kernels on the communicator's stream and returns: no synchronisation, no allocation, no
 * host-side bookkeeping — usable while the stream is being captured into a HIP graph.  The staging arena was sized
 * when the plan was created and stays where it is for as long as any plan of the communicator exists (a later, larger
 * call gets a second arena; the outgrown one is released with the last plan), so a graph captured from this call stays
 * valid until its plan is freed.  The caller orders later work after it (same stream, or an event). */
int vc_plan_execute_async(vc_plan_t plan, char *sendbuf, char *recvbuf);
/* Waits for the communicator's stream and releases the plan's work items; before vc_comm_free of its communicator. */
int vc_plan_free(vc_plan_t plan);

/* ---- tunables.  The reference leaves r and b to the caller; its drivers sweep a list of bases and batch sizes and time
 * every combination (examples/rbruckv_example.cpp:33-35, 98-103; src/tuna.cpp:21, 69).  vc_suggest_tunables replaces the
 * sweep by a model priced in figures measured once per communicator (vc_comm_calibration): the rate of a plain copy on
 * this GPU, the cost of one more kernel launch, and of a launch the host waits for.  For every candidate radix it evaluates on the device the bytes and
 * work items the call would move (sum over blocks of hops x bytes; hops = non-zero base-r digits of the offset inside the
 * node, + 1 if the node differs) and models the call in the communicator's execution mode (vc_comm_set_forwarding):
 *   one launch per digit:  (planning) + launches x launch cost + (2 x moved bytes + 64 x moved items) / rate
 *   forwarded:             (planning) + launch cost + (payload + moved bytes + 2 x items x (24 + 8 x hop slots)) / rate
 * with rate = 0.85 x the plain copy's.  n = ranks per node for the two-layer functions, 0 or P for the one-layer ones.
 * candidates / ncand: HOST array of radices; ncand = 0 searches every radix from 2 to min(n, 63) and n itself.
 * r_out: the candidate with the smallest modelled time; b_out (may be NULL): rounds of a digit per launch for
 * tuna_algorithm: always all of them (r - 1), because on one GPU the rounds of a digit are independent copies and
 * splitting them over launches only adds launch costs; seconds_out / moved_bytes_out (HOST, ncand entries, may be NULL;
 * pass NULL with ncand = 0): modelled time and hop-weighted bytes per candidate. ---- */
int vc_suggest_tunables(const int *sendcounts, int elem_size, int n, const int *candidates, int ncand, int *r_out, int *b_out,
                        double *seconds_out, int64_t *moved_bytes_out, vc_comm_t comm);
/* The radix alone, from a non-empty candidate list (vc_suggest_tunables without b and the modelled times). */
int vc_suggest_radix(const int *sendcounts, int elem_size, int n, const int *candidates, int ncand, int *best_out,
                     int64_t *moved_bytes_out, vc_comm_t comm);
/* Measures (once per communicator, then remembered) what the model is priced in: bytes per second of a plain 256 MiB copy
 * (read + written bytes) and seconds per kernel launch in a row of empty launches.  Allocates 512 MiB for the moment. */
int vc_comm_calibration(vc_comm_t comm, double *copy_bytes_per_s_out, double *launch_seconds_out);

/* ---- measurement and inspection (the reference's global phase timers, src/rbruckv.h:13-18) ---- */

#define VC_MAX_LAUNCHES 1024

typedef struct {
    int32_t n_launches;          /* data-moving kernel launches of the last call (1 in forwarded execution) */
    int32_t n_digits;            /* digit phases among them */
    int64_t payload_bytes;       /* S: sum of all blocks */
    int64_t moved_bytes;         /* sum over all hops of the bytes copied (each hop counted once) */
    int64_t staging_bytes;       /* staging arena the call needed */
    float plan_ms;               /* metadata kernels (valid when timing is on) */
    float total_ms;              /* whole call on the stream (valid when timing is on) */
    float intra_ms;              /* launches inside the nodes: the digit rounds (the reference's getBlock_time ... replace_time) */
    float inter_ms;              /* launches between the nodes (orgData_time, prepSP_time, SP_time; intra_time / iteration_time of
                                    src/twolayer_communicator_linear.cpp:10-11 likewise).  Forwarded execution has one launch
                                    for both: its time is in intra_ms and inter_ms is 0. */
    int64_t launch_bytes[VC_MAX_LAUNCHES];   /* bytes the hops of a launch copy (forwarded execution: [0] = moved_bytes) */
    float launch_ms[VC_MAX_LAUNCHES];  /* per data-moving launch, HIP events on the comm's stream */
    int32_t execution;           /* how the call ran: 0 launch per digit, 1 forwarded through a work-item list, 2 forwarded
                                    without one, 3 forwarded without one on fixed-stride staging (see vc_comm_set_forwarding) */
    int32_t lanes_per_item;      /* 256: the copy kernel gave every work item (without a list: every pair of ranks) a
                                    workgroup; 64: a wavefront (short pieces); 16: a quarter of one (pieces of a
                                    few hundred bytes); 1: a wavefront took a batch of pairs of ranks (many very short
                                    blocks).  Launch-per-digit execution: of the launch that moved the most bytes. */
    int64_t block_pieces;        /* forwarded execution: pieces the blocks were cut into (the work items of the list); else 0 */
    int64_t max_block_pieces;    /* ... the most pieces of one block */
    int64_t max_block_bytes;     /* ... the longest block */
    int64_t bad_table_entries;   /* table entries no set of ranks could have passed (negative ones, recvcounts[t][s] !=
                                    sendcounts[s][t]; + 2^40 per rank whose packed receive layout overflows), as the device
                                    counted them: 0 after a call that returned VC_OK, set by one that returned VC_ERR_TABLES
                                    or VC_ERR_OVERFLOW (the other fields then still describe the call before it) */
    int64_t host_waits;          /* times the host waited for the device inside the call: 1 when everything the call needed was
                                    enqueued at once, 2 when the host looked at the plan in mid-call to size the work-item list
                                    and the staging arena, more when a launch had to be repeated behind larger buffers */
} vc_stats_t;

/* Per-launch HIP-event timing of the following calls (0 = off, default).  While it is on, a list-driven call keeps the
 * host's look at the plan in mid-call (host_waits 2), so that the events bracket the copy kernel alone. */
int vc_comm_set_timing(vc_comm_t comm, int enable);
int vc_comm_last_stats(vc_comm_t comm, vc_stats_t *out);

/* Route of the last call: for launch `launch`, the bytes sent from every rank to every rank, as a HOST
 * [P][P] int64 matrix (row = sender).  For tests that pin the route against the oracle's message trace.  Only after a
 * call in the launch-per-digit mode (vc_comm_set_forwarding(comm, 0)). */
int vc_comm_last_traffic(vc_comm_t comm, int launch, int64_t *matrix_out);

/* The staging arena as the last call left it: DEVICE pointer and the bytes that call used (what the reference keeps in
 * extra_buffer / temp_recv_buffer between rounds, src/twophase_tunable_rbruckv.cpp:59-61).  Both execution modes leave
 * the same bytes there; tests compare them.  The pointer is valid until a call on this communicator needs more. */
int vc_comm_staging(vc_comm_t comm, void **ptr_out, int64_t *bytes_out);

/* ---- harness utilities (payload of the reference drivers, examples/rbruckv_example.cpp:88-92, and a
 * receiver-side check in the spirit of src/utils.cpp:31-46, but exact) ---- */

/* Fills every send block: mode 0: byte k of block (s,d) = byte (k & 7) of H(seed, s, d, k >> 3), H = three chained
 * splitmix64 rounds; mode 1: int32 word idx = s*2^20 + d*2^10 + idx. */
int vc_fill_payload(int mode, uint64_t seed, char *sendbuf, const int *sendcounts, const int *sdispls, int elem_size,
                    vc_comm_t comm);

/* Counts the bytes of recvbuf that differ from the textbook definition recv_t[rdispls_t[s] + k] =
 * send_s[sdispls_s[t] + k] into *mismatch_out (host).  packed_recv != 0 checks the packed layout of TTPL_BT_alltoallv. */
int vc_verify_alltoallv(const char *sendbuf, const int *sendcounts, const int *sdispls, int elem_size,
                        const char *recvbuf, const int *recvcounts, const int *rdispls, int packed_recv,
                        int64_t *mismatch_out, vc_comm_t comm);

/* Plain contiguous copy of nbytes (multiple of 16, 16-byte aligned pointers) with the same 16-byte non-temporal
 * accesses the block mover uses: the transfer of known size against which hardware byte counters are scaled. */
int vc_calibration_copy(char *dst, const char *src, int64_t nbytes, vc_comm_t comm);

/* The same with every vector stored twice (to dst and to dst2): one read, two writes, the mix of the forwarded
 * kernel on two-hop routes (the pack and unpack memcpys of src/twophase_twolayer_rbruck.cpp:334-343,368-377 in one
 * pass).  The contiguous ceiling that kernel is held against. */
int vc_calibration_copy2(char *dst, char *dst2, const char *src, int64_t nbytes, vc_comm_t comm);

#ifdef __cplusplus
}
#endif
#endif /* RBRUCK_VC_H_ */
