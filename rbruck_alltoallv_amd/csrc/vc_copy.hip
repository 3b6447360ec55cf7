// vc_copy.hip — the data mover.  A Bruck round on P virtual ranks is a set of
// independent block copies inside HBM: the reference's pack (memcpy into
// temp_send_buffer), MPI_Sendrecv and unpack (memcpy out of temp_recv_buffer)
// (src/twophase_tunable_rbruckv.cpp:90-100,119,126-139) collapse into one read of
// the block where the sender holds it and one write where the receiver wants it.
//
// Shape of the kernels, chosen by measurement on MI355X: one work item = a piece of one block that fits a window of
// VC_CHUNK = 8 KiB; every lane moves 16-byte vectors whose loads are all issued before the stores, non-temporal on both
// sides (the data is touched once per hop).  For pieces of several KiB a 256-lane workgroup per item is fastest (many
// small workgroups beat persistent or wider ones for a plain copy on this chip, and the same holds for the scattered
// variable-size blocks of an alltoallv); lists of short pieces are bound by the number of items in flight and get a
// wavefront, or a quarter of one, per item.  The host chooses per launch (vc_lanes_for_items in vc_dispatch.h).
//
// Workgroups are handed to the 8 XCDs of the chip in turn (workgroup b runs on XCD
// b mod 8) and every XCD has its own L2.  Work items that follow each other in the
// list are neighbours in memory (pieces of one block, blocks of one run), so each
// XCD takes a contiguous eighth of the list instead of every eighth item: cache
// lines shared by two neighbouring items then meet in one L2, and every XCD streams
// through its own range of addresses.  Measured: +3 % on 4 KiB blocks, +15 % on
// 1 MiB blocks cut into pieces.
#include "vc_common.h"
#include "vc_dispatch.h"
#include "vc_plan_math.h"
#include "vc_scan.h"

typedef unsigned int vc_u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(1))) VcU128 { vc_u32x4 v; };

// 16-byte load from any byte address (one global_load_dwordx4; the hardware handles the misalignment)
__device__ __forceinline__ vc_u32x4 vc_load16(const char *p) {
    return __builtin_nontemporal_load(&reinterpret_cast<const VcU128 *>(p)->v);
}

// 16-byte store to a 16-byte aligned address
__device__ __forceinline__ void vc_store16(char *p, vc_u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<vc_u32x4 *>(p));
}

__device__ __forceinline__ char *vc_resolve(int64_t loc, const char *sendbuf, char *recvbuf, char *stage) {
    const int64_t off = loc & VC_OFFSET_MASK;
    const int space = (int)(loc >> VC_SPACE_SHIFT);
    char *base = space == 0 ? const_cast<char *>(sendbuf) : (space == 1 ? recvbuf : stage);
    return base + off;
}

#define VC_XCDS 8
// Workgroups of one launch: a dispatch counts its grid in work-items in 32 bits, so gridDim.x * VC_THREADS must stay
// below 2^32 (a larger grid is not refused: it runs truncated); longer lists go out in several launches.  A multiple of
// VC_XCDS.
#define VC_MAX_GRID ((int64_t)((1ull << 32) / VC_THREADS) - VC_XCDS)

// One workgroup (or one wavefront) of LANES lanes moves one piece.  Lane t owns the t-th, (t + LANES)-th, ... 16-byte vector
// of the window that starts at the 128-byte boundary at or below dst, so every wave stores whole cache lines whatever
// the byte phase of the block (measured: +4 % over counting vectors from the first 16-byte boundary of dst).  Vectors
// that lie fully inside the block are moved by (possibly unaligned) 16-byte loads and aligned stores; the < 16 bytes
// before the first and after the last of them are moved byte-wise (lanes 0..15 the head, lanes 16..31 the tail: one byte
// load and one byte store each).  The planner guarantees len + (dst & 127) <= VC_CHUNK.
// With nhop > 1 this is forwarded execution: the piece is read once, from sendbuf, and every hop stores the same
// registers (all destinations of a block share the offset inside their cache line, so one mapping of lanes to window
// vectors serves them all).  dst_of(k) is where hop k puts the piece.
// go() is asked once, after the loads have been issued and before the first store: false leaves the piece where it is.
struct VcAlwaysGo { __device__ __forceinline__ bool operator()() const { return true; } };

template <int LANES, class DstOf, class Go = VcAlwaysGo>
__device__ __forceinline__ void vc_forward_piece(const char *src, int64_t len, int nhop, DstOf dst_of, Go go = Go()) {
    constexpr int VECS = VC_CHUNK / 16 / LANES;           // window vectors per lane: 2 for a workgroup of 256, 8 for one wavefront
    char *dst = dst_of(0);
    const int t = threadIdx.x;
    const int64_t w = (int64_t)((uintptr_t)dst & (VC_LINE - 1));
    const int64_t first_full = (w + 15) >> 4, end_full = (w + len) >> 4;
    const char *sw = src - w;
    vc_u32x4 v[VECS];
    bool has[VECS];
#pragma unroll
    for (int i = 0; i < VECS; i++) {
        const int64_t j = t + i * LANES;
        has[i] = (i > 0 || j >= first_full) && j < end_full;
        if (has[i]) v[i] = vc_load16(sw + (j << 4));
    }
    int64_t head = (first_full << 4) - w;
    if (head > len) head = len;
    int64_t done = (end_full << 4) - w;
    if (done < head) done = head;
    const int64_t edge = t < 16 ? (t < head ? t : -1) : (t < 32 && done + (t - 16) < len ? done + (t - 16) : -1);
    char edge_byte = 0;
    if (edge >= 0) edge_byte = src[edge];
    if (!go()) return;
    for (int k = 0; k < nhop; k++) {
        if (k) dst = dst_of(k);
        char *dw = dst - w;
        if (edge >= 0) dst[edge] = edge_byte;
#pragma unroll
        for (int i = 0; i < VECS; i++)
            if (has[i]) vc_store16(dw + ((int64_t)(t + i * LANES) << 4), v[i]);
    }
}

// LANES = VC_THREADS: one workgroup of four wavefronts per item, the shape that moves blocks of several KiB fastest.
// LANES = VC_WAVE: one wavefront per item, for lists of short pieces: four times as many items in flight per compute
// unit, and no wavefronts that start only to find nothing left for them in a piece of a few hundred bytes.
// GUARDED: the launch was enqueued before the host had seen the plan (see VcChainGuard): `nitems` is a guess, header[2] the
// truth, and nothing moves unless the plan is one this launch can serve.
template <int LANES, bool GUARDED = false>
__global__ __launch_bounds__(LANES) void vc_copy_chains_kernel(const int64_t *__restrict__ items, int stride, unsigned nitems,
                                                               const char *__restrict__ sendbuf, char *__restrict__ recvbuf,
                                                               char *__restrict__ stage, const int64_t *__restrict__ header = nullptr,
                                                               VcChainGuard guard = VcChainGuard()) {
    const unsigned per = gridDim.x / VC_XCDS;
    const unsigned idx = (blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    if (idx >= nitems) return;
    if (GUARDED && (!vc_chain_guard_ok(header, guard) || (int64_t)idx >= header[2])) return;
    const int64_t *it = items + (int64_t)idx * stride;
    const int64_t len = it[VC_CHAIN_LEN];
    const int nhop = (int)it[VC_CHAIN_NHOP];
    if (len <= 0 || nhop <= 0) return;
    vc_forward_piece<LANES>(vc_resolve(it[VC_CHAIN_SRC], sendbuf, recvbuf, stage), len, nhop,
                            [&](int k) { return vc_resolve(it[VC_CHAIN_HEAD + k], sendbuf, recvbuf, stage); });
}

// Launch-per-digit execution: one hop of one piece per item.
template <int LANES>
__global__ __launch_bounds__(LANES) void vc_copy_items_kernel(const VcDesc *__restrict__ items, unsigned nitems,
                                                              const char *__restrict__ sendbuf, char *__restrict__ recvbuf,
                                                              char *__restrict__ stage) {
    // gridDim.x is a multiple of VC_XCDS; XCD k = blockIdx.x % VC_XCDS works through items [k * per, (k + 1) * per)
    const unsigned per = gridDim.x / VC_XCDS;
    const unsigned idx = (blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    if (idx >= nitems) return;
    const VcDesc d = items[idx];
    if (d.len <= 0) return;
    char *dst = vc_resolve(d.dst, sendbuf, recvbuf, stage);
    vc_forward_piece<LANES>(vc_resolve(d.src, sendbuf, recvbuf, stage), d.len, 1, [&](int) { return dst; });
}

// A quarter of a wavefront (16 lanes) per item, four items per wavefront, for lists of pieces of a few hundred bytes:
// such a launch is bound by how many items are in flight, not by HBM, and a piece of 100 bytes has work for 7 lanes.
// Every group of 16 lanes reads its own item; lane t of the group owns window vectors t, t + 16 of every 512-byte pass
// (most items need one pass; longer ones loop), and moves head byte t and tail byte t.
template <class DstOf, class Go = VcAlwaysGo>
__device__ __forceinline__ void vc_forward_piece_quarter(const char *src, int64_t len, int nhop, DstOf dst_of, Go go = Go()) {
    const int t = threadIdx.x & 15;
    char *dst = dst_of(0);
    const int64_t w = (int64_t)((uintptr_t)dst & (VC_LINE - 1));
    const int64_t first_full = (w + 15) >> 4, end_full = (w + len) >> 4;
    int64_t head = (first_full << 4) - w;
    if (head > len) head = len;
    int64_t done = (end_full << 4) - w;
    if (done < head) done = head;
    const bool has_head = t < head, has_tail = done + t < len;
    char head_byte = 0, tail_byte = 0;
    if (has_head) head_byte = src[t];
    if (has_tail) tail_byte = src[done + t];
    const char *sw = src - w;
    bool first_pass = true;                               // the pass that also stores the head and tail bytes: there is
    for (int64_t j = t; first_pass || j < end_full; j += 32) {     // always one, also for a block without a full vector
        const bool has0 = j >= first_full && j < end_full, has1 = j + 16 >= first_full && j + 16 < end_full;
        vc_u32x4 v0, v1;
        if (has0) v0 = vc_load16(sw + (j << 4));
        if (has1) v1 = vc_load16(sw + ((j + 16) << 4));
        if (first_pass && !go()) return;
        for (int k = 0; k < nhop; k++) {
            if (k || !first_pass) dst = dst_of(k);
            char *dw = dst - w;
            if (first_pass && has_head) dst[t] = head_byte;
            if (first_pass && has_tail) dst[done + t] = tail_byte;
            if (has0) vc_store16(dw + (j << 4), v0);
            if (has1) vc_store16(dw + ((j + 16) << 4), v1);
        }
        first_pass = false;
    }
}

#define VC_ITEMS_PER_WAVE (VC_WAVE / VC_QUARTER)

// gridDim.x wavefronts, a multiple of VC_XCDS; XCD k works through the k-th eighth of them, each taking four items in a row
// `rounds`: groups of four items in a row a wavefront takes, one after the other (long lists of very short pieces: fewer
// wavefronts, each paying its start-up once for more items)
template <bool GUARDED = false>
__global__ __launch_bounds__(VC_WAVE) void vc_copy_chains_quarter_kernel(const int64_t *__restrict__ items, int stride, unsigned nitems,
                                                                         int rounds, const char *__restrict__ sendbuf,
                                                                         char *__restrict__ recvbuf, char *__restrict__ stage,
                                                                         const int64_t *__restrict__ header = nullptr,
                                                                         VcChainGuard guard = VcChainGuard()) {
    const unsigned per = gridDim.x / VC_XCDS;
    const unsigned wave = (blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    if (GUARDED && !vc_chain_guard_ok(header, guard)) return;
    for (int round = 0; round < rounds; round++) {
        const int64_t idx = ((int64_t)wave * rounds + round) * VC_ITEMS_PER_WAVE + threadIdx.x / VC_QUARTER;
        if (idx >= nitems || (GUARDED && idx >= header[2])) continue;
        const int64_t *it = items + idx * stride;
        const int64_t len = it[VC_CHAIN_LEN];
        const int nhop = (int)it[VC_CHAIN_NHOP];
        if (len <= 0 || nhop <= 0) continue;
        vc_forward_piece_quarter(vc_resolve(it[VC_CHAIN_SRC], sendbuf, recvbuf, stage), len, nhop,
                                 [&](int k) { return vc_resolve(it[VC_CHAIN_HEAD + k], sendbuf, recvbuf, stage); });
    }
}

__global__ __launch_bounds__(VC_WAVE) void vc_copy_items_quarter_kernel(const VcDesc *__restrict__ items, unsigned nitems, int rounds,
                                                                        const char *__restrict__ sendbuf, char *__restrict__ recvbuf,
                                                                        char *__restrict__ stage) {
    const unsigned per = gridDim.x / VC_XCDS;
    const unsigned wave = (blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    for (int round = 0; round < rounds; round++) {
        const int64_t idx = ((int64_t)wave * rounds + round) * VC_ITEMS_PER_WAVE + threadIdx.x / VC_QUARTER;
        if (idx >= nitems) continue;
        const VcDesc d = items[idx];
        if (d.len <= 0) continue;
        char *dst = vc_resolve(d.dst, sendbuf, recvbuf, stage);
        vc_forward_piece_quarter(vc_resolve(d.src, sendbuf, recvbuf, stage), d.len, 1, [&](int) { return dst; });
    }
}

// ---- fixed-stride staging in one launch (the `totals` of vc_launch_copy_blocks) ----
__device__ __forceinline__ int64_t vc_wave_sum(int64_t v) {
#pragma unroll
    for (int o = VC_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, VC_WAVE);
    return v;
}

__device__ __forceinline__ int64_t vc_wave_max(int64_t v) {
#pragma unroll
    for (int o = VC_WAVE / 2; o > 0; o >>= 1) {
        const int64_t u = __shfl_xor(v, o, VC_WAVE);
        v = u > v ? u : v;
    }
    return v;
}

// The wavefronts of the first vc_totals_blocks workgroups of the grid: four pairs of ranks per lane (by receiver, then
// source; the atomics on the same few words are what limits this at many ranks), the wavefront's
// sums and maxima added into `totals` with one atomic each: [1] payload, [2] block pieces, [3] table entries no rank could
// have passed, [4] the most pieces of a block, [5] hop-weighted bytes, [6] the longest block.  The wavefront that finishes
// last hands the words to the host.
#define VC_TOTALS_PER_LANE 4
// wavefronts that add up the totals of a call on P ranks
__host__ __device__ __forceinline__ int64_t vc_totals_waves(int P) {
    const int64_t per_wave = VC_WAVE * VC_TOTALS_PER_LANE;
    return ((int64_t)P * P + per_wave - 1) / per_wave;
}

__device__ __forceinline__ void vc_add_totals(const VcSched &S, const VcTables &T, int64_t *totals, int64_t *header_host) {
    const int P = S.P;
    const int64_t pairs = (int64_t)P * P, per_wave = VC_WAVE * VC_TOTALS_PER_LANE, nwaves = vc_totals_waves(P);
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / VC_WAVE) + threadIdx.x / VC_WAVE;
    if (wave >= nwaves) return;
    const int lane = threadIdx.x & (VC_WAVE - 1);
    unsigned long long *h = reinterpret_cast<unsigned long long *>(totals);
    int64_t payload = 0, items = 0, bad = 0, most = 0, moved = 0, longest = 0;
    // The verdict on the tables first, with nothing but one round of loads in front of it: the copying wavefronts of this
    // launch hold their stores back until every totalling wavefront has reported (vc_wait_verdict).
#pragma unroll
    for (int u = 0; u < VC_TOTALS_PER_LANE; u++) {
        const int64_t idx = wave * per_wave + u * VC_WAVE + lane;
        if (idx >= pairs) continue;
        const int to = vc_div((int)idx, S.dP), s = (int)idx - to * P;      // (idx < P^2 <= 2^30)
        const int64_t i = (int64_t)to * P + s;
        bad += vc_pair_bad_entries(S, T, s, to);          // the same count the planner's row kernel makes
        // (a packed receive layout past INT_MAX elements shows as a negative packed displacement of a later source)
        if (S.packed_recv && (T.rd_packed[i] < 0 || (s == P - 1 && (int64_t)T.rd_packed[i] + T.rc[i] > 0x7FFFFFFF))) bad += VC_BAD_OVERFLOW;
    }
    bad = vc_wave_sum(bad);
    // one word says it all, so one atomic publishes it: wavefronts that have reported in the low half, wavefronts that
    // found something wrong in the high half
    if (lane == 0) atomicAdd(&h[VC_HEADER_CHECKED], 1ull | (bad ? 1ull << 32 : 0ull));
#pragma unroll
    for (int u = 0; u < VC_TOTALS_PER_LANE; u++) {
        const int64_t idx = wave * per_wave + u * VC_WAVE + lane;
        if (idx >= pairs) continue;
        const int to = vc_div((int)idx, S.dP), s = (int)idx - to * P;      // (idx < P^2 <= 2^30)
        const int64_t i = (int64_t)to * P + s, k = (int64_t)s * P + to;
        const int sc = T.sc[k], rc = T.rc[i];
        const int64_t len = (int64_t)sc * S.esz;
        const int64_t cnt = sc > 0 ? vc_chain_count(S, T, s, to) : 0;
        payload += (int64_t)rc * S.esz;                   // (what the receivers expect, as the planner counts it)
        items += cnt;
        moved += len * vc_block_hops(S, s, to);
        most = cnt > most ? cnt : most;
        longest = len > longest ? len : longest;
    }
    payload = vc_wave_sum(payload);
    items = vc_wave_sum(items);
    moved = vc_wave_sum(moved);
    most = vc_wave_max(most);
    longest = vc_wave_max(longest);
    int last = 0;
    if (lane == 0) {
        // The count below must not be seen before the words above.  A release fence would do, but at device scope it writes
        // this XCD's L2 back, once per wavefront here.  Instead every atomic returns its old value: when the values are
        // back the atomics have been performed where the count is kept too, and the count's operand is made from them.
        unsigned long long seen = 0;
        if (payload) seen += atomicAdd(&h[1], (unsigned long long)payload);
        if (items) seen += atomicAdd(&h[2], (unsigned long long)items);
        if (bad) seen += atomicAdd(&h[VC_HEADER_BAD], (unsigned long long)bad);
        if (moved) seen += atomicAdd(&h[VC_HEADER_FIXED], (unsigned long long)moved);
        if (most) seen += atomicMax(&h[VC_HEADER_MAX_PIECES], (unsigned long long)most);
        if (longest) seen += atomicMax(&h[VC_HEADER_MAX_LEN], (unsigned long long)longest);
        unsigned zero;
        asm volatile("v_mov_b32 %0, 0" : "=v"(zero) : "v"((unsigned)seen), "v"((unsigned)(seen >> 32)));      // (opaque to the compiler)
        last = atomicAdd(&h[VC_HEADER_SYNC], 1ull + zero) == (unsigned long long)(nwaves - 1);
    }
    last = __shfl(last, 0, VC_WAVE);
    if (last && lane <= VC_HEADER_MAX_LEN)
        header_host[lane] = lane == 0 ? vc_strided_stage_bytes(S)
                                      : (int64_t)__hip_atomic_load(&h[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A copying wavefront of the single launch asks before its first store: have all totalling wavefronts checked their part of
// the tables, and did they find them in order?  The totalling workgroups are the first of the grid, so they are resident
// before any copying one; the wait is bounded all the same (VC_CHECK_SPINS polls, a few milliseconds): a wavefront that
// gives up moves nothing and says so in the host's copy of the header, and the host redoes the call the general way.
#define VC_CHECK_SPINS (1 << 15)
__device__ __forceinline__ unsigned long long vc_verdict_word(int64_t *totals) {
    return __hip_atomic_load(reinterpret_cast<unsigned long long *>(totals) + VC_HEADER_CHECKED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Asked by the piece movers between their loads and their stores (see vc_forward_piece).  Without `totals` there is nothing
// to wait for (the planner's verdict was checked before the block's route was worked out).  look() reads the word once
// ahead of the block's loads, so that a verdict that is already in costs no round trip of its own.
struct VcVerdictGate {
    int64_t *totals, *header_host;
    unsigned long long nwaves, word;
    int state;                                            // 0 not known yet, 1 go, 2 leave everything where it is
    __device__ __forceinline__ void look() { if (totals) word = vc_verdict_word(totals); }
    __device__ __forceinline__ bool operator()() {
        if (!totals) return true;
        for (int spin = 0; state == 0; spin++) {
            if ((word & 0xFFFFFFFFull) >= nwaves) state = (word >> 32) ? 2 : 1;
            else if (spin >= VC_CHECK_SPINS) { header_host[VC_HEADER_STALLED] = 1; state = 2; }
            else { __builtin_amdgcn_s_sleep(4); word = vc_verdict_word(totals); }
        }
        return state == 1;
    }
};

// Workgroups at the head of the grid that only add up the totals (none without `totals`): their round trips run beside the
// copying instead of in front of it.  A multiple of VC_XCDS, so that the workgroups behind them keep their XCDs.
__host__ __device__ __forceinline__ unsigned vc_totals_blocks(const VcSched &S, const int64_t *totals, int lanes) {
    if (!totals) return 0;
    const int64_t per_wave = VC_WAVE * VC_TOTALS_PER_LANE;
    const int64_t waves = ((int64_t)S.P * S.P + per_wave - 1) / per_wave, per = lanes / VC_WAVE;
    return (unsigned)(((waves + per - 1) / per + VC_XCDS - 1) / VC_XCDS * VC_XCDS);
}

// Whether the pair's own table entries allow its block to be moved: none negative, the receiver expecting what the
// source sends, the block no longer than a slot and cut into no more pieces than the kernel was chosen for.
__device__ __forceinline__ bool vc_pair_allowed(const VcSched &S, const VcTables &T, const VcListlessGuard &g, int s, int t) {
    const int64_t i = (int64_t)t * S.P + s, k = (int64_t)s * S.P + t;
    const int sc = T.sc[k];
    if (sc < 0 || T.rc[i] != sc || T.sd[k] < 0 || (S.packed_recv ? T.rd_packed[i] < 0 : T.rd[i] < 0)) return false;
    if (S.packed_recv && (int64_t)T.rd_packed[i] + sc > 0x7FFFFFFF) return false;
    const int64_t len = (int64_t)sc * S.esz;
    if (g.max_len && len > g.max_len) return false;
    return !(g.max_pieces && sc > 0 && vc_chain_count(S, T, s, t) > g.max_pieces);
}

// Forwarded execution without a work-item list, for calls whose planning would otherwise cost more than their copying:
// one workgroup per (source, destination) pair, in the order of the chain items (by destination, then source, an eighth
// of the pairs per XCD).  The workgroup works out the route of its block in closed form from the plan tables (lane k
// evaluates hop slot k), then carries the block through it piece by piece.  The kernel is enqueued right behind the
// planning kernels, before the host has seen their result, so it checks that result itself: nothing is touched when the
// plan needs more staging than there is, the tables hold negative entries, or the call is not of the kind the host
// expected when it chose this kernel (the host, which evaluates the same condition afterwards, then takes another path).
// LANES = VC_THREADS: a workgroup of four wavefronts per pair; LANES = VC_WAVE: one wavefront per pair, for blocks of a
// KiB or two (a quarter of the wavefronts to start, all of them with work).
template <int LANES>
__global__ __launch_bounds__(LANES) void vc_copy_blocks_kernel(VcSched S, VcTables T, const int64_t *__restrict__ slot_off,
                                                               const int64_t *__restrict__ row_base,
                                                               const int64_t *__restrict__ header, VcListlessGuard guard,
                                                               int64_t first_pair, const char *__restrict__ sendbuf,
                                                               char *__restrict__ recvbuf, char *__restrict__ stage,
                                                               int64_t *__restrict__ header_host, int64_t *__restrict__ header_zero,
                                                               int64_t *totals) {
    __shared__ int64_t route[VC_MAX_HOP_SLOTS];
    __shared__ int route_len;
    const unsigned head = vc_totals_blocks(S, totals, LANES);
    if (blockIdx.x < head) { vc_add_totals(S, T, totals, header_host); return; }
    const unsigned block = blockIdx.x - head;
    const int64_t per = (gridDim.x - head) / VC_XCDS;
    const int64_t idx = first_pair + (int64_t)(block % VC_XCDS) * per + block / VC_XCDS;
    const bool inside = idx < (int64_t)S.P * S.P;
    const int t = inside ? vc_div((int)idx, S.dP) : 0, s = inside ? (int)idx - t * S.P : 0;       // (idx < P^2 <= 2^30)
    // Everything the block's addresses depend on is loaded before the planner's verdict is looked at: the loads are
    // independent of each other and of the verdict (tables are always readable), so they travel together instead of one
    // memory round trip after the other; nothing is stored before the verdict is known.
    const int64_t len = (int64_t)T.sc[(int64_t)s * S.P + t] * S.esz;
    const int64_t send_off = vc_send_offset(S, T, s, t);
    const int64_t recv_off = vc_recv_offset(S, T, s, t);
    int64_t dst = 0;
    const bool moves = threadIdx.x < VC_WAVE && (int)threadIdx.x < vc_hop_slots(S) && vc_block_hop(S, T, slot_off, row_base, s, t, threadIdx.x, dst);
    if (block == 0 && first_pair == 0 && threadIdx.x <= VC_HEADER_CHECKED) {
        if (header_host && !totals && threadIdx.x <= VC_HEADER_MAX_LEN) header_host[threadIdx.x] = header[threadIdx.x];
        if (header_zero) header_zero[threadIdx.x] = 0;    // the header the next call will add up into
    }
    if (!inside || len <= 0) return;
    if (totals ? !vc_pair_allowed(S, T, guard, s, t) : !vc_listless_ok(header, guard)) return;
    if (threadIdx.x < VC_WAVE) {                          // hop slots <= VC_MAX_HOP_SLOTS < lanes of the first wavefront
        const unsigned long long mask = __ballot(moves);
        if (moves) route[__popcll(mask & ((1ull << threadIdx.x) - 1))] = dst;
        if (threadIdx.x == 0) route_len = __popcll(mask);
    }
    __syncthreads();
    const int nhop = route_len;
    if (nhop <= 0) return;
    const char *src = sendbuf + send_off;
    const int phase = (int)((recv_off + S.recv_lo) & (VC_LINE - 1)), cut = (int)((recv_off + S.recv_lo) & (VC_PIECE - 1));
    const int64_t pieces = vc_chunk_count(len, phase, cut);
    VcVerdictGate gate = {totals, header_host, (unsigned long long)vc_totals_waves(S.P), 0, 0};
    gate.look();
    for (int64_t c = 0; c < pieces; c++) {                // the same cuts as the chain items of this block
        int64_t lo, hi;
        vc_piece_range(len, phase, cut, c, lo, hi);
        vc_forward_piece<LANES>(src + lo, hi - lo, nhop, [&](int k) { return vc_resolve(route[k] + lo, sendbuf, recvbuf, stage); },
                                [&]() { return gate(); });
    }
}

// The same for pairs whose blocks are a few hundred bytes: a quarter of a wavefront per pair, four pairs in a row per
// wavefront.  Lane q of a group evaluates hop slots q and q + 16; the four routes of the wavefront go through LDS.
__global__ __launch_bounds__(VC_WAVE) void vc_copy_blocks_quarter_kernel(VcSched S, VcTables T, const int64_t *__restrict__ slot_off,
                                                                         const int64_t *__restrict__ row_base,
                                                                         const int64_t *__restrict__ header, VcListlessGuard guard,
                                                                         int64_t first_pair, const char *__restrict__ sendbuf,
                                                                         char *__restrict__ recvbuf, char *__restrict__ stage,
                                                                         int64_t *__restrict__ header_host, int64_t *__restrict__ header_zero,
                                                                         int64_t *totals) {
    __shared__ int64_t route[VC_ITEMS_PER_WAVE][VC_MAX_HOP_SLOTS];
    const unsigned head = vc_totals_blocks(S, totals, VC_WAVE);
    if (blockIdx.x < head) { vc_add_totals(S, T, totals, header_host); return; }
    const unsigned block = blockIdx.x - head;
    const int64_t per = (gridDim.x - head) / VC_XCDS;
    const int64_t wave = (int64_t)(block % VC_XCDS) * per + block / VC_XCDS;
    const int g = threadIdx.x / VC_QUARTER, q = threadIdx.x % VC_QUARTER;
    const int64_t idx = first_pair + wave * VC_ITEMS_PER_WAVE + g;
    const bool inside = idx < (int64_t)S.P * S.P;
    const int t = inside ? vc_div((int)idx, S.dP) : 0, s = inside ? (int)idx - t * S.P : 0;       // (idx < P^2 <= 2^30)
    // all loads the addresses depend on go out before the planner's verdict is looked at (see vc_copy_blocks_kernel)
    const int64_t len = inside ? (int64_t)T.sc[(int64_t)s * S.P + t] * S.esz : 0;
    const int64_t send_off = vc_send_offset(S, T, s, t);
    const int64_t recv_off = vc_recv_offset(S, T, s, t);
    // no lane leaves before the barrier below
    const bool active = len > 0 && (!totals || vc_pair_allowed(S, T, guard, s, t));
    const int nslots = vc_hop_slots(S);
    int64_t d0 = 0, d1 = 0;
    const bool m0 = active && q < nslots && vc_block_hop(S, T, slot_off, row_base, s, t, q, d0);
    const bool m1 = active && q + VC_QUARTER < nslots && vc_block_hop(S, T, slot_off, row_base, s, t, q + VC_QUARTER, d1);
    if (block == 0 && first_pair == 0 && threadIdx.x <= VC_HEADER_CHECKED) {
        if (header_host && !totals && threadIdx.x <= VC_HEADER_MAX_LEN) header_host[threadIdx.x] = header[threadIdx.x];
        if (header_zero) header_zero[threadIdx.x] = 0;
    }
    if (!totals && !vc_listless_ok(header, guard)) return;      // the same for every lane of the grid
    const unsigned g0 = (unsigned)(__ballot(m0) >> (g * VC_QUARTER)) & 0xFFFFu;      // the group's hops among slots 0..15
    const unsigned g1 = (unsigned)(__ballot(m1) >> (g * VC_QUARTER)) & 0xFFFFu;      // ... among slots 16..31
    if (m0) route[g][__popc(g0 & ((1u << q) - 1))] = d0;
    if (m1) route[g][__popc(g0) + __popc(g1 & ((1u << q) - 1))] = d1;
    __syncthreads();
    const int nhop = __popc(g0) + __popc(g1);
    if (!active || nhop <= 0) return;
    const char *src = sendbuf + send_off;
    const int phase = (int)((recv_off + S.recv_lo) & (VC_LINE - 1)), cut = (int)((recv_off + S.recv_lo) & (VC_PIECE - 1));
    const int64_t pieces = vc_chunk_count(len, phase, cut);
    VcVerdictGate gate = {totals, header_host, (unsigned long long)vc_totals_waves(S.P), 0, 0};
    gate.look();
    for (int64_t c = 0; c < pieces; c++) {
        int64_t lo, hi;
        vc_piece_range(len, phase, cut, c, lo, hi);
        vc_forward_piece_quarter(src + lo, hi - lo, nhop, [&](int k) { return vc_resolve(route[g][k] + lo, sendbuf, recvbuf, stage); },
                                 [&]() { return gate(); });
    }
}

// The same again for calls of many short blocks, where the wavefronts above live for one pass over four blocks and the
// round trips and the arithmetic of working out a route, not the bytes, set the pace: a wavefront takes BATCH pairs in a
// row.  64 / BATCH lanes per pair evaluate its hop slots, one lane per pair compacts the route in LDS, then every quarter
// of the wavefront carries BATCH / 4 of the blocks, one after the other.  Measured on MI355X, 1024 ranks, blocks of 0 - 16
// bytes (two hops each): 211 us with a quarter of a wavefront per pair, 105 / 87 / 79 us with BATCH = 16 / 32 / 64.
template <int BATCH>
__global__ __launch_bounds__(VC_WAVE) void vc_copy_blocks_batch_kernel(VcSched S, VcTables T, const int64_t *__restrict__ slot_off,
                                                                       const int64_t *__restrict__ row_base,
                                                                       const int64_t *__restrict__ header, VcListlessGuard guard,
                                                                       int64_t first_pair, const char *__restrict__ sendbuf,
                                                                       char *__restrict__ recvbuf, char *__restrict__ stage,
                                                                       int64_t *__restrict__ header_host, int64_t *__restrict__ header_zero) {
    extern __shared__ int64_t batch_lds[];
    const int nslots = vc_hop_slots(S);
    int64_t *route = batch_lds;                           // [BATCH][nslots]
    int64_t *b_len = route + BATCH * nslots, *b_src = b_len + BATCH;
    int *b_nhop = reinterpret_cast<int *>(b_src + BATCH), *b_cut = b_nhop + BATCH;
    const int64_t per = gridDim.x / VC_XCDS;
    const int64_t wave = (int64_t)(blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    const int p = threadIdx.x % BATCH, kq = threadIdx.x / BATCH;
    const int64_t idx = first_pair + wave * BATCH + p;
    const bool inside = idx < (int64_t)S.P * S.P;
    const int t = inside ? vc_div((int)idx, S.dP) : 0, s = inside ? (int)idx - t * S.P : 0;       // (idx < P^2 <= 2^30)
    // all loads the addresses depend on go out before the planner's verdict is looked at (see vc_copy_blocks_kernel)
    const int64_t len = inside ? (int64_t)T.sc[(int64_t)s * S.P + t] * S.esz : 0;
    const int64_t send_off = vc_send_offset(S, T, s, t);
    const int64_t recv_off = vc_recv_offset(S, T, s, t);
    const bool active = len > 0;
    for (int k = kq; k < nslots; k += VC_WAVE / BATCH) {
        int64_t d = 0;
        const bool moves = active && vc_block_hop(S, T, slot_off, row_base, s, t, k, d);
        route[p * nslots + k] = moves ? d : -1;           // destinations carry their space in bits 60 and 61: never negative
    }
    if (blockIdx.x == 0 && first_pair == 0 && threadIdx.x <= VC_HEADER_MAX_LEN) {
        if (header_host) header_host[threadIdx.x] = header[threadIdx.x];
        if (header_zero) header_zero[threadIdx.x] = 0;
    }
    if (!vc_listless_ok(header, guard)) return;           // the same for every lane of the grid
    __syncthreads();
    if (kq == 0) {
        int nhop = 0;
        for (int k = 0; k < nslots; k++) {
            const int64_t d = route[p * nslots + k];
            if (d >= 0) route[p * nslots + nhop++] = d;
        }
        b_len[p] = len;
        b_src[p] = send_off;
        b_nhop[p] = active ? nhop : 0;
        b_cut[p] = (int)((recv_off + S.recv_lo) & (VC_PIECE - 1));
    }
    __syncthreads();
    for (int it = 0; it < BATCH / VC_ITEMS_PER_WAVE; it++) {
        const int b = it * VC_ITEMS_PER_WAVE + threadIdx.x / VC_QUARTER;
        const int64_t blen = b_len[b];
        const int nhop = b_nhop[b];
        if (blen <= 0 || nhop <= 0) continue;
        const char *src = sendbuf + b_src[b];
        const int cut = b_cut[b], phase = cut & (VC_LINE - 1);
        const int64_t *dsts = route + b * nslots;
        const int64_t pieces = vc_chunk_count(blen, phase, cut);
        for (int64_t c = 0; c < pieces; c++) {            // the same cuts as the chain items of this block
            int64_t lo, hi;
            vc_piece_range(blen, phase, cut, c, lo, hi);
            vc_forward_piece_quarter(src + lo, hi - lo, nhop, [&](int k) { return vc_resolve(dsts[k] + lo, sendbuf, recvbuf, stage); });
        }
    }
}

template <int BATCH>
static void vc_launch_batch(int64_t pairs, const VcSched &S, VcTables T, const int64_t *slot_off, const int64_t *row_base, const int64_t *header,
                            VcListlessGuard guard, int64_t first_pair, const char *sendbuf, char *recvbuf, char *stage, hipStream_t st,
                            int64_t *header_host, int64_t *header_zero) {
    const int64_t waves = (pairs + BATCH - 1) / BATCH;
    const size_t lds = sizeof(int64_t) * BATCH * (vc_hop_slots(S) + 2) + sizeof(int) * BATCH * 2;
    hipLaunchKernelGGL(vc_copy_blocks_batch_kernel<BATCH>, dim3((unsigned)((waves + VC_XCDS - 1) / VC_XCDS * VC_XCDS)), dim3(VC_WAVE), lds, st, S,
                       T, slot_off, row_base, header, guard, first_pair, sendbuf, recvbuf, stage, header_host, header_zero);
}

hipError_t vc_launch_copy_blocks(const VcSched &S, VcTables T, const int64_t *slot_off, const int64_t *row_base, const int64_t *header,
                                 VcListlessGuard guard, int lanes, const char *sendbuf, char *recvbuf, char *stage, hipStream_t st,
                                 int64_t *header_host, int64_t *header_zero, int64_t *totals) {
    const int64_t npairs = (int64_t)S.P * S.P;
    const int64_t step = lanes == VC_QUARTER || lanes == VC_BATCHED ? VC_MAX_GRID * VC_ITEMS_PER_WAVE : VC_MAX_GRID;
    for (int64_t done = 0; done < npairs; done += step) {
        const int64_t now = npairs - done < step ? npairs - done : step;
        const int64_t units = lanes == VC_QUARTER ? (now + VC_ITEMS_PER_WAVE - 1) / VC_ITEMS_PER_WAVE : now;
        if (totals && done) return hipErrorInvalidValue;    // the totals belong to a call that one launch takes
        const dim3 grid((unsigned)((units + VC_XCDS - 1) / VC_XCDS * VC_XCDS) + vc_totals_blocks(S, totals, lanes == VC_THREADS ? VC_THREADS : VC_WAVE));
        if (lanes == VC_BATCHED) {
            if (totals) return hipErrorInvalidValue;      // the batches are for more pairs than one launch with totals takes
            const int batch = vc_batch_pairs(npairs);
            if (batch == 64)
                vc_launch_batch<64>(now, S, T, slot_off, row_base, header, guard, done, sendbuf, recvbuf, stage, st, header_host, header_zero);
            else if (batch == 32)
                vc_launch_batch<32>(now, S, T, slot_off, row_base, header, guard, done, sendbuf, recvbuf, stage, st, header_host, header_zero);
            else
                vc_launch_batch<16>(now, S, T, slot_off, row_base, header, guard, done, sendbuf, recvbuf, stage, st, header_host, header_zero);
        } else if (lanes == VC_QUARTER)
            hipLaunchKernelGGL(vc_copy_blocks_quarter_kernel, grid, dim3(VC_WAVE), 0, st, S, T, slot_off, row_base, header, guard, done,
                               sendbuf, recvbuf, stage, header_host, header_zero, totals);
        else if (lanes == VC_WAVE)
            hipLaunchKernelGGL(vc_copy_blocks_kernel<VC_WAVE>, grid, dim3(VC_WAVE), 0, st, S, T, slot_off, row_base, header, guard, done,
                               sendbuf, recvbuf, stage, header_host, header_zero, totals);
        else
            hipLaunchKernelGGL(vc_copy_blocks_kernel<VC_THREADS>, grid, dim3(VC_THREADS), 0, st, S, T, slot_off, row_base, header, guard,
                               done, sendbuf, recvbuf, stage, header_host, header_zero, totals);
    }
    return hipGetLastError();
}

// Items of one launch: as many as VC_MAX_GRID workgroups or wavefronts take.
static int64_t vc_items_per_launch(int lanes) { return lanes == VC_QUARTER ? VC_MAX_GRID * VC_ITEMS_PER_WAVE : VC_MAX_GRID; }

static unsigned vc_grid_for(int64_t items, int lanes) {
    const int64_t per = lanes == VC_QUARTER ? VC_ITEMS_PER_WAVE * vc_quarter_rounds(items) : 1;
    const int64_t units = (items + per - 1) / per;
    return (unsigned)((units + VC_XCDS - 1) / VC_XCDS * VC_XCDS);
}

hipError_t vc_launch_copy_chains(const int64_t *items, int stride, int64_t nitems, int lanes, const char *sendbuf, char *recvbuf,
                                 char *stage, hipStream_t st) {
    const int64_t step = vc_items_per_launch(lanes);
    for (int64_t done = 0; done < nitems; done += step) {
        const int64_t now = nitems - done < step ? nitems - done : step;
        const dim3 grid(vc_grid_for(now, lanes));
        const int64_t *first = items + done * stride;
        if (lanes == VC_QUARTER)
            hipLaunchKernelGGL(vc_copy_chains_quarter_kernel<false>, grid, dim3(VC_WAVE), 0, st, first, stride, (unsigned)now,
                               vc_quarter_rounds(now), sendbuf, recvbuf, stage, nullptr, VcChainGuard());
        else if (lanes == VC_WAVE)
            hipLaunchKernelGGL((vc_copy_chains_kernel<VC_WAVE, false>), grid, dim3(VC_WAVE), 0, st, first, stride, (unsigned)now, sendbuf, recvbuf,
                               stage, nullptr, VcChainGuard());
        else
            hipLaunchKernelGGL((vc_copy_chains_kernel<VC_THREADS, false>), grid, dim3(VC_THREADS), 0, st, first, stride, (unsigned)now, sendbuf,
                               recvbuf, stage, nullptr, VcChainGuard());
    }
    return hipGetLastError();
}

// One launch (a guessed list longer than a launch holds is cut to what one holds; the rest is the caller's second launch).
hipError_t vc_launch_copy_chains_guarded(const int64_t *items, int stride, int64_t grid_items, int lanes, const char *sendbuf,
                                         char *recvbuf, char *stage, hipStream_t st, const int64_t *header, VcChainGuard guard, int64_t *covered) {
    const int64_t step = vc_items_per_launch(lanes);
    const int64_t now = grid_items < step ? grid_items : step;
    *covered = now > 0 ? now : 0;
    if (now <= 0) return hipSuccess;
    const dim3 grid(vc_grid_for(now, lanes));
    if (lanes == VC_QUARTER)
        hipLaunchKernelGGL(vc_copy_chains_quarter_kernel<true>, grid, dim3(VC_WAVE), 0, st, items, stride, (unsigned)now, vc_quarter_rounds(now),
                           sendbuf, recvbuf, stage, header, guard);
    else if (lanes == VC_WAVE)
        hipLaunchKernelGGL((vc_copy_chains_kernel<VC_WAVE, true>), grid, dim3(VC_WAVE), 0, st, items, stride, (unsigned)now, sendbuf, recvbuf,
                           stage, header, guard);
    else
        hipLaunchKernelGGL((vc_copy_chains_kernel<VC_THREADS, true>), grid, dim3(VC_THREADS), 0, st, items, stride, (unsigned)now, sendbuf,
                           recvbuf, stage, header, guard);
    return hipGetLastError();
}

hipError_t vc_launch_copy_items(const VcDesc *items, int64_t nitems, int lanes, const char *sendbuf, char *recvbuf, char *stage,
                                hipStream_t st) {
    const int64_t step = vc_items_per_launch(lanes);
    for (int64_t done = 0; done < nitems; done += step) {
        const int64_t now = nitems - done < step ? nitems - done : step;
        const dim3 grid(vc_grid_for(now, lanes));
        if (lanes == VC_QUARTER)
            hipLaunchKernelGGL(vc_copy_items_quarter_kernel, grid, dim3(VC_WAVE), 0, st, items + done, (unsigned)now, vc_quarter_rounds(now),
                               sendbuf, recvbuf, stage);
        else if (lanes == VC_WAVE)
            hipLaunchKernelGGL(vc_copy_items_kernel<VC_WAVE>, grid, dim3(VC_WAVE), 0, st, items + done, (unsigned)now, sendbuf, recvbuf, stage);
        else
            hipLaunchKernelGGL(vc_copy_items_kernel<VC_THREADS>, grid, dim3(VC_THREADS), 0, st, items + done, (unsigned)now, sendbuf, recvbuf,
                               stage);
    }
    return hipGetLastError();
}

// Plain contiguous copy of a known size: one 16-byte vector per lane, 4 KiB per workgroup, WRITES stores per load.  It exists so
// that hardware counters (bytes fetched / written per dispatch) can be scaled against a transfer whose size is known, and as
// the ceiling the block movers are held against: WRITES = 1 for launch-per-digit execution (one read, one write per hop),
// WRITES = 2 for the forwarded kernel on two-hop routes (one read, two writes).
template <int WRITES>
__global__ __launch_bounds__(VC_THREADS) void vc_calibration_copy_kernel(const vc_u32x4 *__restrict__ src, vc_u32x4 *__restrict__ dst,
                                                                         vc_u32x4 *__restrict__ dst2, int64_t nvec) {
    const int64_t i = (int64_t)blockIdx.x * VC_THREADS + threadIdx.x;
    if (i >= nvec) return;
    const vc_u32x4 v = __builtin_nontemporal_load(&src[i]);
    __builtin_nontemporal_store(v, &dst[i]);
    if (WRITES == 2) __builtin_nontemporal_store(v, &dst2[i]);
}

hipError_t vc_launch_calibration_copy(const char *src, char *dst, char *dst2, int64_t nbytes, hipStream_t st) {
    const int64_t nvec = nbytes / 16;
    for (int64_t done = 0; done < nvec; done += VC_MAX_GRID * VC_THREADS) {
        const int64_t now = nvec - done < VC_MAX_GRID * VC_THREADS ? nvec - done : VC_MAX_GRID * VC_THREADS;
        const dim3 grid((unsigned)((now + VC_THREADS - 1) / VC_THREADS));
        if (dst2)
            hipLaunchKernelGGL(vc_calibration_copy_kernel<2>, grid, dim3(VC_THREADS), 0, st, reinterpret_cast<const vc_u32x4 *>(src) + done,
                               reinterpret_cast<vc_u32x4 *>(dst) + done, reinterpret_cast<vc_u32x4 *>(dst2) + done, now);
        else
            hipLaunchKernelGGL(vc_calibration_copy_kernel<1>, grid, dim3(VC_THREADS), 0, st, reinterpret_cast<const vc_u32x4 *>(src) + done,
                               reinterpret_cast<vc_u32x4 *>(dst) + done, static_cast<vc_u32x4 *>(nullptr), now);
    }
    return hipGetLastError();
}
