// vc_common.h — types shared by the host side and the kernels of librbruck_vc.
//
// Vocabulary (follows the reference): a *block* is the data one rank sends to one
// other rank; its *offset* is j = (source - destination) mod span and never
// changes; the *slot* a block occupies on whichever rank currently holds it is
// id = g*n + (j + local_rank) % n (src/twophase_twolayer_rbruck.cpp:322; with one
// group this is (j + rank) % P, src/twophase_tunable_rbruckv.cpp:81).  A *digit
// phase* x moves every block whose base-r digit x of j is non-zero by z*r^x ranks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define VC_THREADS 256
// lanes of a work item in the copy kernels for short pieces: a wavefront (VC_WAVE, vc_scan.h) or a quarter of one
#define VC_QUARTER 16
// lane code of the listless copy kernel that gives a wavefront a batch of pairs: a lane per pair works out the route, then
// the quarters of the wavefront carry the blocks one after the other
#define VC_BATCHED 1
// window of one workgroup of the copy kernel: 256 lanes x 2 vectors x 16 bytes, starting at a cache-line boundary
#define VC_CHUNK 8192
#define VC_LINE 128
// piece size for copies longer than that: 256 lanes x 1 vector x 16 bytes
#define VC_PIECE 4096

// Location of a byte range: which arena (top bits) and the byte offset inside it.
#define VC_SPACE_SHIFT 60
#define VC_SPACE_SEND (0ll << VC_SPACE_SHIFT)
#define VC_SPACE_RECV (1ll << VC_SPACE_SHIFT)
#define VC_SPACE_STAGE (2ll << VC_SPACE_SHIFT)
#define VC_OFFSET_MASK ((1ll << VC_SPACE_SHIFT) - 1)

// One block copy: `len` bytes from `src` to `dst` (space-tagged offsets), sent by
// virtual rank `from` to virtual rank `to`.
struct VcDesc {
    int64_t src;
    int64_t dst;
    int64_t len;
    int32_t from;
    int32_t to;
};

#if defined(__HIPCC__)
#define VC_HD __host__ __device__ __forceinline__
#else
#define VC_HD inline
#endif

// Division of a non-negative int (below 2^31) by a divisor that is the same for the whole call — ranks per node, nodes,
// the radix, ranks — as a multiplication and a shift with constants the host works out once per call: an integer
// division is 30-odd instructions on this chip, and the route of one block takes a dozen of them.
// floor(x / d) = (x * mul) >> shift for all 0 <= x < 2^31, with shift = 31 + ceil(log2 d) and mul = floor(2^shift / d) + 1 < 2^32
// (2^shift <= mul * d <= 2^shift + 2^ceil(log2 d)).
struct VcDivisor {
    int d;
    unsigned mul;
    int shift;
};

VC_HD VcDivisor vc_make_divisor(int d) {          // d >= 1
    int l = 0;
    while (((int64_t)1 << l) < d) l++;
    VcDivisor v;
    v.d = d;
    v.shift = 31 + l;
    v.mul = (unsigned)((((uint64_t)1 << v.shift) / (uint64_t)d) + 1);
    return v;
}

VC_HD int vc_div(int x, const VcDivisor &v) { return (int)(((uint64_t)(unsigned)x * v.mul) >> v.shift); }
VC_HD int vc_mod(int x, const VcDivisor &v) { return x - vc_div(x, v) * v.d; }

// What kind of algorithm the call runs; fixed for the whole call.
struct VcSched {
    int P;            // ranks
    int n;            // ranks per node (P for the one-layer variants)
    int G;            // nodes = P / n
    int r;            // radix of the intra-node digits (already clamped)
    int w;            // digits of n-1 in base r (0 when n == 1)
    int w2;           // digits of G-1 in base r when the inter-node phase is a Bruck over the nodes too
                      // (TTPL_rbruck_alltoallv), else 0.  Its digit x stages in region w + x.
    int msd;          // 1: most significant digit first (twophase_rbruck_alltoallv, uniform intra phase)
    int esz;          // element size in bytes
    int packed_recv;  // 1: receive side is the packed source-ordered layout (TTPL_BT_alltoallv ignores rdispls)
    int uniform;      // >0: equal blocks of this many elements, tables are implied (uniform_* functions)
    int recv_lo;      // low 12 bits of the recvbuf pointer: staging slots copy the final destination's cache-line phase,
                      // long copies into recvbuf are cut at its 4 KiB boundaries
    int last_hop;     // which blocks make a hop that is no digit round and ends in recvbuf, besides every rank's block to
                      // itself: 0 none (one-layer Bruck; Bruck over the nodes), 1 those that change node (inter-node
                      // messages), 2 all (direct one-hop functions)
    int stride;       // > 0: staging slots at a fixed stride of this many bytes (a multiple of VC_LINE that holds the longest block
                      //    at any cache-line phase), the reference's own layout (src/twophase_tunable_rbruckv.cpp:59): slot `id`
                      //    of rank `holder` in region x starts at ((x P + holder) P + id) stride, a closed form, and the planner's
                      //    prefix sums and slot tables are not needed.  0: compact slots at prefix-sum offsets.
    int recycle;      // 1 (launch-per-digit execution only): staging memory is reused.  A staged block arrives in one hop slot and
                      //    leaves in a later one; blocks with the same (arrival, departure) pair of hop slots form a sub-region,
                      //    and a sub-region may take the memory of another one whose blocks have all left before it is written
                      //    (the reference reuses its extra_buffer slots the same way, src/twophase_tunable_rbruckv-om.cpp:52-75).
    int coalesce;     // 1: blocks that are about to leave their node wait in "organized" runs — the n blocks one rank
                      //    holds for one destination rank back to back in source order — so that an inter-node message
                      //    is a contiguous copy (TTPL_BT_alltoallv, src/twophase_twolayer_rbruck.cpp:388-398, 430-453).
                      //    The organized region is staging region number w.
    // set by vc_set_divisors once n, G, r and P are final:
    VcDivisor dn, dG, dr, dP;                     // division by n, G, r, P
};

VC_HD void vc_set_divisors(VcSched &S) {
    S.dn = vc_make_divisor(S.n > 0 ? S.n : 1);
    S.dG = vc_make_divisor(S.G > 0 ? S.G : 1);
    S.dr = vc_make_divisor(S.r > 0 ? S.r : 1);
    S.dP = vc_make_divisor(S.P > 0 ? S.P : 1);
}

// Staging regions of a call: one per intra-node digit, one per inter-node digit, the organized region.
VC_HD int vc_regions(const VcSched &S) { return S.w + S.w2 + S.coalesce; }

// Reused staging (S.recycle): hop slots a call may have at most, and rows of the row tables per rank: one per (arrival,
// departure) pair of hop slots plus one for the organized region.
#define VC_RECYCLE_MAX_SLOTS 12
#define VC_RECYCLE_MAX_PAIRS (VC_RECYCLE_MAX_SLOTS * VC_RECYCLE_MAX_SLOTS + 1)
VC_HD int vc_row_families(const VcSched &S) {
    const int ns = S.w + S.w2 + 1;
    return S.recycle ? ns * ns + 1 : vc_regions(S);
}

// One data-moving kernel launch.
struct VcLaunchInfo {
    int kind;      // 0: rounds of intra-node digit x with digit value in [zlo, zhi]; 1: inter-node messages, one per block;
                   // 2: direct messages; 3: inter-node messages, coalesced (entries are (source group, part) pairs);
                   // 4: rounds of inter-node digit x with digit value in [zlo, zhi]
    int x;         // digit; for direct launches the scope: 0 all pairs by rank distance, 1 inside a node, 2 between nodes
    int dist;      // r^x (ranks inside the node for kind 0, nodes for kind 4)
    int zlo, zhi;
    int qlo, qhi;  // inter-node: (group distance)*n + source local index in [qlo, qhi); direct: rank distance in [qlo, qhi)
    int self;      // also performs every rank's copy to itself
};

// Forwarded execution lists its chain items in tiles of VC_TILE_RANKS receivers x VC_TILE_RANKS sources (receiver by
// receiver inside a tile) instead of all sources of a receiver in a row: neighbours in the list then read from few send
// buffers and write to few receive buffers, each in runs of consecutive blocks.
#define VC_TILE_RANKS 32
#define VC_TILES(P) (((P) + VC_TILE_RANKS - 1) / VC_TILE_RANKS)

#define VC_LAUNCH_PACK 16
struct VcLaunchPack { VcLaunchInfo info[VC_LAUNCH_PACK]; };

struct VcTables {
    const int *sc, *sd, *rc, *rd;    // [P][P] row-major, elements
    const int64_t *sbase, *rbase;    // [P] bytes
    const int *rd_packed;            // [P][P] exclusive scan of rc rows (only when packed_recv)
};

// ---- launchers implemented in the .hip files (all asynchronous on `st`) ----

// vc_meta.hip
hipError_t vc_launch_transpose(const int *in, int *out, int P, hipStream_t st);
// flags (device, 2 ints the caller has zeroed, or null): [0] set when a row's total passes INT_MAX, [1] when a count is negative
hipError_t vc_launch_row_scan(const int *counts, int *displs, int64_t *extent, int *flags, int P, hipStream_t st);
hipError_t vc_launch_bases(const int64_t *extent, int esz, int64_t align, int64_t *base, int64_t *total, int P, hipStream_t st);
hipError_t vc_launch_max(const int *counts, int *out, int64_t nelem, hipStream_t st);
hipError_t vc_launch_fill_payload(int mode, uint64_t seed, char *sendbuf, const int *sc, const int *sd, const int64_t *sbase,
                                  int esz, int P, hipStream_t st);
hipError_t vc_launch_verify(const char *sendbuf, const char *recvbuf, VcTables t, int esz, int P, int packed,
                            unsigned long long *mismatch, hipStream_t st);
// moved_dev: 2 (ncand + 1) words the caller has zeroed: hop-weighted bytes per candidate, the payload, hop-weighted work
// items per candidate, the work items of the payload
hipError_t vc_launch_hop_bytes(const int *sc, int esz, int P, int n, const int *cand_dev, int ncand, unsigned long long *moved_dev,
                               hipStream_t st);
hipError_t vc_launch_uniform_tables(int *counts, int *displs, int count, int P, hipStream_t st);
hipError_t vc_launch_empty(hipStream_t st);

// vc_plan.hip
// header layout (int64), nl = number of launches:
//   [0] staging bytes   [1] payload bytes   [2] chain items (forwarded execution)
//   [3] entries of the count / displacement tables no set of ranks could have passed: negative ones, recvcounts[t][s] that
//       differ from sendcounts[s][t]; plus VC_BAD_OVERFLOW per rank whose packed receive layout overflows an int
//   [4] the most pieces any block is cut into (forwarded execution)
//   [5 + L] bytes moved by launch L   [5 + nl + L] work items of launch L
//   (forwarded execution: [5] all moved bytes, [6] the longest block, no per-launch words)
#define VC_HEADER_FIXED 5
// forwarded execution: the longest block of the call, bytes
#define VC_HEADER_MAX_LEN (VC_HEADER_FIXED + 1)
#define VC_HEADER_BAD 3
// added to header[VC_HEADER_BAD] once per rank whose packed receive displacements would pass INT_MAX elements
#define VC_BAD_OVERFLOW (1ll << 40)
#define VC_HEADER_MAX_PIECES 4
// fixed-stride staging: wavefronts that have added their part of the tables' totals into the header
#define VC_HEADER_SYNC (VC_HEADER_MAX_LEN + 1)
// ... wavefronts that have checked their part of the tables and added what they found to VC_HEADER_BAD: the copying
// wavefronts of the same launch store nothing before all of them have
#define VC_HEADER_CHECKED (VC_HEADER_SYNC + 1)
// ... set (in the host's copy of the header only) by a copying wavefront that gave up waiting for that: the call is redone
#define VC_HEADER_STALLED (VC_HEADER_SYNC + 2)
#define VC_HEADER_WORDS(nl) (VC_HEADER_FIXED + 2 * (nl))
// Passes 1 and 2: staging prefix sums and the number of work items of every launch (sizes only).  The launch table
// travels as a kernel argument when it has at most VC_LAUNCH_PACK entries (launches_dev is then not read).  With chain_row_tot /
// chain_row_base ((2 + VC_TILES(P)) P and P int64, or null) also the chain items per final receiver, the first item of every
// (receiver, tile of sources) in the list's tiled order (behind chain_row_tot's first 2 P words), their total in header[2] and the most
// pieces of any block in header[4].
hipError_t vc_launch_plan_sizes(const VcSched &S, const VcLaunchInfo *launches_host, const VcLaunchInfo *launches_dev, int nlaunch,
                                VcTables T, int64_t *slot_off,
                                int64_t *row_tot, int64_t *row_base, int64_t *org_run_base, int64_t *item_row_tot,
                                int64_t *item_row_base, int64_t *row_bytes, int64_t *chain_row_tot, int64_t *chain_row_base,
                                int64_t *header, int64_t *header_host, hipStream_t st);
// Forwarded execution: the chain items (every block's route in closed form, staging addresses from the plan tables).
// chain_tile_base: [P][VC_TILES(P)] first item of every (receiver, tile of sources) (vc_launch_plan_sizes leaves it behind
// chain_row_tot's first 2 P words).
// header + cap_items (optional): the launch was enqueued before the host knew the plan; it writes nothing unless the
// device header the sizing kernels left says the tables are in order and the list holds all header[2] items.
hipError_t vc_launch_chain_plan(const VcSched &S, VcTables T, const int64_t *slot_off, const int64_t *row_base,
                                const int64_t *chain_tile_base, int64_t *items, int64_t nitems, hipStream_t st,
                                const int64_t *header = nullptr, int64_t cap_items = 0);
// Pass 3: writes the work items (needs the item buffer, sized from the header).
hipError_t vc_launch_plan_emit(const VcSched &S, const VcLaunchInfo *launches_host, const VcLaunchInfo *launches_dev, int nlaunch,
                               VcTables T, const int64_t *slot_off,
                               const int64_t *row_base, const int64_t *item_row_base, const int64_t *header, VcDesc *items,
                               int64_t nitems, hipStream_t st);
hipError_t vc_launch_traffic(const VcDesc *desc, int64_t ndesc, int64_t *matrix, int P, hipStream_t st);

// vc_copy.hip
// lanes: VC_THREADS (a workgroup per item), VC_WAVE (a wavefront per item, for lists of short pieces) or VC_QUARTER (a quarter of
// a wavefront, for lists of pieces of a few hundred bytes)
hipError_t vc_launch_copy_items(const VcDesc *items, int64_t nitems, int lanes, const char *sendbuf, char *recvbuf, char *stage,
                                hipStream_t st);
hipError_t vc_launch_copy_chains(const int64_t *items, int stride, int64_t nitems, int lanes, const char *sendbuf, char *recvbuf,
                                 char *stage, hipStream_t st);
// What the plan of a call must look like for a list and a copy launch that were enqueued right behind the sizing kernels,
// before the host had seen the plan, to do their work.  Kernels and host evaluate it on the same header, so both agree on
// whether anything was moved.
struct VcChainGuard {
    int64_t cap_items;      // chain items the list has room for
    int64_t stage_cap;      // bytes of staging arena there are
    int64_t allowance;      // staging a forwarded call may take before its ratio to the payload counts (INT64_MAX: no bound)
};

VC_HD bool vc_chain_guard_ok(const int64_t *header, const VcChainGuard &g) {
    if (header[VC_HEADER_BAD] != 0 || header[2] > g.cap_items || header[0] > g.stage_cap) return false;
    return !(header[0] > g.allowance && header[0] > 3 * header[1]);
}

// The same launch for a list whose length the host only guesses (grid_items: work items the grid is sized for): every
// workgroup checks vc_chain_guard_ok on the device header and takes an item only if there is one at its index
// (header[2] items exist).  Items beyond `covered` (grid_items, or what one launch holds) are left for a second, ordinary launch.
hipError_t vc_launch_copy_chains_guarded(const int64_t *items, int stride, int64_t grid_items, int lanes, const char *sendbuf,
                                         char *recvbuf, char *stage, hipStream_t st, const int64_t *header, VcChainGuard guard, int64_t *covered);
// What the plan of a call must look like for the listless kernels to run it; 0 = no limit.  The kernels evaluate it on
// the device header, the host on its copy after the synchronisation: both then agree on whether anything was moved.
struct VcListlessGuard {
    int64_t stage_cap;      // bytes of staging arena there are
    int64_t max_pieces;     // most pieces of one block
    int64_t max_items;      // block pieces in all
    int64_t max_average;    // average piece, bytes
    int64_t max_len;        // longest block, bytes (fixed-stride staging: what a slot holds at any phase)
};

VC_HD bool vc_listless_ok(const int64_t *header, const VcListlessGuard &g) {
    if (header[0] > g.stage_cap || header[VC_HEADER_BAD] != 0) return false;
    if (g.max_len && header[VC_HEADER_MAX_LEN] > g.max_len) return false;
    if (g.max_pieces && header[VC_HEADER_MAX_PIECES] > g.max_pieces) return false;
    if (g.max_items && header[2] > g.max_items) return false;
    return !(g.max_average && header[1] > g.max_average * header[2]);
}

// Forwarded execution without a work-item list: one workgroup (or a quarter of a wavefront) per (source, destination)
// pair works out the route of its block from the plan tables and carries it through.  Reads the device `header` the
// planning kernels before it on the stream have written and does nothing unless vc_listless_ok(header, guard).
// lanes: VC_THREADS (a workgroup per pair), VC_WAVE (a wavefront per pair, blocks of a KiB or two) or VC_QUARTER (a quarter of a
// wavefront per pair, for blocks of a few hundred bytes).
// header_host (pinned, may be null): the first workgroup copies the fixed words of `header` there, for planners that add
// the header up with atomics and cannot write it to the host themselves.  header_zero (may be null): ... and clears the
// fixed words there: the header the next call's planner will add up into.
// totals (device, non-null: fixed-stride staging, S.stride > 0, at most VC_MAX_GRID pairs): the kernel needs no planner
// before it.  Its first wavefronts add up the tables' totals — validation, payload, block pieces, longest block,
// hop-weighted bytes — into `totals` (words 0 .. VC_HEADER_SYNC zeroed by the caller) and the last of them to finish
// copies the words to header_host, with [0] = the bytes the fixed-stride arena takes; `header` is not read.  Every pair
// checks its own table entries and the guard's max_len / max_pieces and leaves its block alone when one of them fails, so
// no address is formed from a bad entry; the host, which evaluates the same conditions on the totals afterwards, reports
// the call as refused then.  With bad table entries nothing has been stored by then: the copying wavefronts hold their
// stores back until the totalling ones have reported on all of the tables.  With a block longer than a slot the blocks of
// the other pairs may already have been delivered; they are delivered again when the host redoes the call.
hipError_t vc_launch_copy_blocks(const VcSched &S, VcTables T, const int64_t *slot_off, const int64_t *row_base, const int64_t *header,
                                 VcListlessGuard guard, int lanes, const char *sendbuf, char *recvbuf, char *stage, hipStream_t st,
                                 int64_t *header_host = nullptr, int64_t *header_zero = nullptr, int64_t *totals = nullptr);
// dst2 non-null: every vector is stored twice (one read, two writes)
hipError_t vc_launch_calibration_copy(const char *src, char *dst, char *dst2, int64_t nbytes, hipStream_t st);
