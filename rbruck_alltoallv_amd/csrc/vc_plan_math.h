// vc_plan_math.h — index arithmetic of the Bruck family, shared by the planning
// kernels and by host code (the CPU build used to check the plan without a GPU).
//
// Which block sits in slot `id` of rank p before digit x follows from the
// residency invariant of the digit order:
//   least significant digit first: its source is (j mod r^x) ranks above the holder,
//   most significant digit first:  its source is (j div r^(x+1)) * r^(x+1) ranks above.
#pragma once

#include "vc_common.h"

struct VcBlock {
    int s, t;        // source and destination rank of the block
    int from;        // rank that holds it before this hop
    int z;           // digit value (0: does not move in this digit)
    int xprev;       // digit in which it last moved (-1: still in sendbuf)
    int id_from;     // its slot on `from`
    bool to_stage;   // lands in the receiver's staging area (else in recvbuf)
    bool to_org;     // ... in its organized region (last intra-node hop of a block that still has to change node)
};

VC_HD int vc_top_digit(int v, const VcDivisor &r) {     // position of the highest non-zero digit, v > 0
    int x = -1;
    while (v) { v = vc_div(v, r); x++; }
    return x;
}

VC_HD int vc_low_digit(int v, const VcDivisor &r) {     // position of the lowest non-zero digit, v > 0
    int x = 0;
    for (;;) {
        const int q = vc_div(v, r);
        if (q * r.d != v) return x;
        v = q; x++;
    }
}

// a mod n for 0 <= a < 2n
VC_HD int vc_wrap(int a, int n) { return a >= n ? a - n : a; }

// Offset j < span without its x lowest base-r digits (j div r^x), and r^x in `dist`: x divisions by the radix.  The power
// stops growing once it has reached the span (spans are at most 32768 ranks, the radix no more than the span: r^x and
// r^(x+1) stay below 2^30); the quotient is 0 then, as no offset reaches it.
VC_HD int vc_upper_digits(const VcSched &S, int j, int x, int span, int &dist) {
    int upper = j;
    dist = 1;
    for (int i = 0; i < x && dist < span; i++) { upper = vc_div(upper, S.dr); dist *= S.r; }
    return upper;
}

// Block that arrives in slot `id` of rank `to` during digit x (dist = r^x), if any.
VC_HD bool vc_intra_block(const VcSched &S, int x, int dist, int to, int id, VcBlock &b) {
    const int n = S.n;
    const int gs = vc_div(to, S.dn), lr = to - gs * n;
    const int g = vc_div(id, S.dn);
    const int j = vc_wrap(id - g * n - lr + n, n);
    b.z = 0;
    if (j == 0) return false;
    const int upper = vc_upper_digits(S, j, x, n, dist);  // the digits from x upwards (dist = r^x as the launch says, or past n)
    const int higher = vc_div(upper, S.dr);               // ... from x + 1 upwards
    const int z = upper - higher * S.r;
    if (z == 0) return false;
    const int nd = dist * S.r;                            // z != 0: dist <= j < n
    const int lfrom = vc_wrap(lr + z * dist, n);          // z r^x <= j < n
    int above;        // how far the source is above the sender
    bool last;
    if (!S.msd) {
        above = j - upper * dist;
        last = higher == 0;
        b.xprev = above ? vc_top_digit(above, S.dr) : -1;
    } else {
        above = higher * nd;
        last = upper * dist == j;
        b.xprev = above ? vc_low_digit(above, S.dr) : -1;
    }
    const int ls = vc_wrap(lfrom + above, n);             // above <= j < n
    b.s = gs * n + ls;
    b.t = g * n + vc_wrap(ls - j + n, n);
    b.from = gs * n + lfrom;
    b.z = z;
    b.id_from = g * n + vc_wrap(j + lfrom, n);
    b.to_stage = !(last && g == gs);
    b.to_org = S.coalesce && last && g != gs;
    return true;
}

// One entry of a launch before addresses are known: which block it moves and between which arenas.
struct VcEntry {
    int s, t;          // the block
    int from;          // rank that holds it before the hop
    int xprev;         // staging region in which it waits on `from` (-1: still in sendbuf)
    int id_from;       // its slot there
    int xdst;          // staging region that receives it (-1: it goes to recvbuf)
    int id_to;         // its slot on the receiver
    int nblk;          // 1, or the number of consecutive source blocks of a coalesced inter-node message part
};

// Inter-node Bruck over the group offset jg = (source node - destination node) mod G, least significant digit
// first, between ranks of equal local index (src/twophase_twolayer_rbruck.cpp:179-227: send to the rank
// spoint*n below, group slots (j + gid) % ngroup, n blocks per group slot).  Entry id = jg*n + jj of rank `to`
// is the block of source local index jj that arrives there in digit x (dist = r^x nodes), if any.
VC_HD bool vc_inter_block(const VcSched &S, int x, int dist, int to, int id, VcEntry &e, int &z) {
    const int n = S.n, G = S.G;
    const int gto = vc_div(to, S.dn), l = to - gto * n;
    const int jg = vc_div(id, S.dn), jj = id - jg * n;
    const int upper = vc_upper_digits(S, jg, x, G, dist);
    const int higher = vc_div(upper, S.dr);
    z = upper - higher * S.r;
    if (z == 0) return false;
    const int low = jg - upper * dist;                // part of the offset travelled in earlier digits
    const int gfrom = vc_wrap(gto + z * dist, G);
    const int gs = vc_wrap(gfrom + low, G);
    const int gt = vc_wrap(gs - jg + G, G);
    e.s = gs * n + jj; e.t = gt * n + l; e.from = gfrom * n + l; e.nblk = 1;
    if (low) {
        e.xprev = S.w + vc_top_digit(low, S.dr); e.id_from = id;
    } else {                                          // still where the intra-node phase left it
        const int j = vc_wrap(jj - l + n, n);
        e.xprev = j == 0 ? -1 : vc_top_digit(j, S.dr);
        e.id_from = gt * n + jj;
    }
    e.xdst = higher == 0 ? -1 : S.w + x;
    e.id_to = id;
    return true;
}

VC_HD int64_t vc_recv_offset(const VcSched &S, const VcTables &T, int s, int t) {
    const int *rd = S.packed_recv ? T.rd_packed : T.rd;
    return T.rbase[t] + (int64_t)rd[(int64_t)t * S.P + s] * S.esz;
}

// Staging slots start cache-line (VC_LINE) aligned; the data inside starts at the line phase
// of the block's final address in recvbuf, so that every later hop copies between
// equally aligned addresses.
VC_HD int vc_phase(const VcSched &S, const VcTables &T, int s, int t) {
    return (int)((vc_recv_offset(S, T, s, t) + S.recv_lo) & (VC_LINE - 1));
}


// Bytes the staging slot `id` of rank `to` needs for the block that arrives in digit x
// (0 if nothing arrives there, or if it goes to recvbuf).  Always a multiple of VC_LINE.  st (optional) receives the
// block's source and destination rank.
VC_HD int64_t vc_stage_slot_size(const VcSched &S, const VcTables &T, int x, int dist, int to, int id, int64_t *data_len = nullptr,
                                 int *st = nullptr) {
    VcBlock b;
    if (data_len) *data_len = 0;
    if (!vc_intra_block(S, x, dist, to, id, b) || !b.to_stage || b.to_org) return 0;
    if (st) { st[0] = b.s; st[1] = b.t; }
    const int64_t len = (int64_t)T.sc[(int64_t)b.s * S.P + b.t] * S.esz;
    if (data_len) *data_len = len;
    return len ? ((len + vc_phase(S, T, b.s, b.t) + VC_LINE - 1) & ~(int64_t)(VC_LINE - 1)) : 0;
}

// The same for staging region y of a call: intra-node digits first, then inter-node digits.  data_len (optional)
// receives the bytes of the block itself.
VC_HD int64_t vc_region_slot_size(const VcSched &S, const VcTables &T, int y, int to, int id, int64_t *data_len = nullptr, int *st = nullptr) {
    int dist = 1;
    if (y < S.w) {
        for (int k = 0; k < y; k++) dist *= S.r;
        return vc_stage_slot_size(S, T, y, dist, to, id, data_len, st);
    }
    for (int k = S.w; k < y; k++) dist *= S.r;
    VcEntry e;
    int z;
    if (data_len) *data_len = 0;
    if (!vc_inter_block(S, y - S.w, dist, to, id, e, z) || e.xdst < 0) return 0;
    if (st) { st[0] = e.s; st[1] = e.t; }
    const int64_t len = (int64_t)T.sc[(int64_t)e.s * S.P + e.t] * S.esz;
    if (data_len) *data_len = len;
    return len ? ((len + vc_phase(S, T, e.s, e.t) + VC_LINE - 1) & ~(int64_t)(VC_LINE - 1)) : 0;
}

// Address (inside the staging arena) of the data of block (s, t) while it sits in slot `id`
// of `holder` in staging region x.
// With reused staging (S.recycle) the rows of a region are split by the hop slot in which their blocks leave again:
// row family (arrival slot) * slots + (departure slot), the organized region last.
VC_HD int vc_next_hop(const VcSched &S, int s, int t, int k);
VC_HD int64_t vc_stage_addr(const VcSched &S, const VcTables &T, const int64_t *slot_off, const int64_t *row_base,
                            int x, int holder, int id, int s, int t) {
    const int64_t row = (int64_t)x * S.P + holder;
    if (S.stride) return (row * S.P + id) * S.stride + vc_phase(S, T, s, t);
    if (S.recycle) {
        const int ns = S.w + S.w2 + 1;
        const int family = (S.coalesce && x == S.w) ? ns * ns : x * ns + vc_next_hop(S, s, t, x);
        return row_base[(int64_t)family * S.P + holder] + slot_off[row * S.P + id] + vc_phase(S, T, s, t);
    }
    return row_base[row] + slot_off[row * S.P + id] + vc_phase(S, T, s, t);
}

// Bytes of staging arena a fixed-stride layout takes.
VC_HD int64_t vc_strided_stage_bytes(const VcSched &S) { return (int64_t)(S.w + S.w2) * S.P * S.P * S.stride; }

// Hops of block (s, t): the digit rounds it moves in, plus the hop that is no digit round (vc_block_hop's last slot).
VC_HD int vc_block_hops(const VcSched &S, int s, int t) {
    if (s == t) return 1;
    const int n = S.n, G = S.G;
    const int gs = vc_div(s, S.dn), gt = vc_div(t, S.dn);
    int hops = (S.last_hop == 2 || (S.last_hop == 1 && gs != gt)) ? 1 : 0;
    if (S.w)
        for (int j = vc_wrap((s - gs * n) - (t - gt * n) + n, n); j;) {
            const int q = vc_div(j, S.dr);
            hops += q * S.r != j;
            j = q;
        }
    if (S.w2)
        for (int j = vc_wrap(gs - gt + G, G); j;) {
            const int q = vc_div(j, S.dr);
            hops += q * S.r != j;
            j = q;
        }
    return hops;
}

VC_HD int64_t vc_send_offset(const VcSched &S, const VcTables &T, int s, int t) {
    return T.sbase[s] + (int64_t)T.sd[(int64_t)s * S.P + t] * S.esz;
}

// ---- organized region (S.coalesce) ----
// Rank `to` = (gs, l) keeps, for every other group g, a run that mirrors byte for byte the part of rank (g, l)'s
// packed recvbuf that comes from group gs: n blocks in source order.  The block of local rank l itself never
// moves inside the node and leaves a hole of its length.  A run starts line aligned plus the line phase of
// its image in recvbuf, so that the inter-node copy of a run is a copy between equally aligned addresses.

// byte offset, inside rank t's recvbuf, of the first block coming from group gs (packed receive layout)
VC_HD int64_t vc_org_run_dst(const VcSched &S, const VcTables &T, int gs, int t) {
    return T.rbase[t] + (int64_t)T.rd_packed[(int64_t)t * S.P + gs * S.n] * S.esz;
}

// bytes of blocks [0, m) of the run, m in [0, n]
VC_HD int64_t vc_org_run_prefix(const VcSched &S, const VcTables &T, int gs, int t, int m) {
    const int64_t row = (int64_t)t * S.P, s0 = gs * S.n;
    const int64_t end = m < S.n ? T.rd_packed[row + s0 + m] : (int64_t)T.rd_packed[row + s0 + S.n - 1] + T.rc[row + s0 + S.n - 1];
    return (end - T.rd_packed[row + s0]) * S.esz;
}

// size of the run rank `to` keeps for group g (multiple of VC_LINE; 0 for its own group)
VC_HD int64_t vc_org_run_size(const VcSched &S, const VcTables &T, int to, int g) {
    const int gs = vc_div(to, S.dn), t = g * S.n + (to - gs * S.n);
    if (g == gs) return 0;
    const int64_t phase = (vc_org_run_dst(S, T, gs, t) + S.recv_lo) & (VC_LINE - 1);
    return (phase + vc_org_run_prefix(S, T, gs, t, S.n) + VC_LINE - 1) & ~(int64_t)(VC_LINE - 1);
}

// line-aligned part of the offset of slot id = g*n + m inside the run (vc_stage_addr adds the block's own phase)
VC_HD int64_t vc_org_slot_rel(const VcSched &S, const VcTables &T, int to, int id) {
    const int gs = vc_div(to, S.dn), g = vc_div(id, S.dn), m = id - g * S.n, t = g * S.n + (to - gs * S.n);
    if (g == gs) return 0;
    const int64_t phase = (vc_org_run_dst(S, T, gs, t) + S.recv_lo) & (VC_LINE - 1);
    return (phase + vc_org_run_prefix(S, T, gs, t, m)) & ~(int64_t)(VC_LINE - 1);
}


// Number of entries per receiving rank in a launch of this kind.
VC_HD int vc_entries_per_rank(const VcSched &S, const VcLaunchInfo &info) { return info.kind == 3 ? 3 * S.G : S.P; }

// Entry (`to`, `id`) of a launch: intra-node launches index by the receiver's slot, inter-node
// launches by the source rank.  Returns false if the entry moves nothing in this launch.
VC_HD bool vc_entry_block(const VcSched &S, const VcLaunchInfo &info, int to, int id, VcEntry &e) {
    const int n = S.n;
    e.nblk = 1;
    if (info.kind == 3) {
        // coalesced inter-node message from rank (gs, lt) to rank `to` = (gt, lt), in three contiguous parts: the
        // blocks of local ranks below lt (organized region), the block of lt itself (still in sendbuf), those above
        const int gs = id / 3, part = id % 3, gt = vc_div(to, S.dn), lt = to - gt * n;
        if (gs == gt) return false;
        const int q = vc_wrap(gs - gt + S.G, S.G) * n;
        if (q < info.qlo || q >= info.qhi) return false;
        const int m0 = part == 0 ? 0 : (part == 1 ? lt : lt + 1);
        const int m1 = part == 0 ? lt : (part == 1 ? lt + 1 : n);
        if (m1 <= m0) return false;
        e.s = gs * n + m0; e.t = to; e.from = gs * n + lt; e.nblk = m1 - m0;
        e.xprev = part == 1 ? -1 : S.w; e.id_from = gt * n + m0; e.xdst = -1; e.id_to = id;
        return true;
    }
    if (info.kind == 2) {
        // direct: `id` is the source rank; launches are batches of the distance (source - destination) mod P
        // (src/MPICH_scattered.cpp:44-45: receive from rank + i + ii)
        int q;
        if (info.x == 1) {                                  // inside the node: local rank distance (twolayer_communicator_linear.cpp:45)
            const int gi = vc_div(id, S.dn), gt = vc_div(to, S.dn);
            if (gi != gt) return false;
            q = vc_wrap((id - gi * n) - (to - gt * n) + n, n);
        } else if (info.x == 2) {                           // between nodes: (group distance)*n + source local index (:146-153)
            const int gi = vc_div(id, S.dn), gt = vc_div(to, S.dn);
            if (gi == gt) return false;
            q = vc_wrap(gt - gi + S.G, S.G) * n + (id - gi * n);
        } else {
            q = vc_wrap(id - to + S.P, S.P);
        }
        if (q < info.qlo || q >= info.qhi) return false;
        e.s = id; e.t = to; e.from = id; e.xprev = -1; e.id_from = to; e.xdst = -1; e.id_to = id;
        return true;
    }
    if (info.self && id == to) {
        // a rank's block to itself (src/twophase_tunable_rbruckv.cpp:63)
        e.s = e.t = e.from = to; e.xprev = -1; e.id_from = id; e.xdst = -1; e.id_to = id;
        return true;
    }
    if (info.kind == 4) {
        int z;
        return vc_inter_block(S, info.x, info.dist, to, id, e, z) && z >= info.zlo && z <= info.zhi;
    }
    if (info.kind == 0) {
        VcBlock b;
        if (!vc_intra_block(S, info.x, info.dist, to, id, b) || b.z < info.zlo || b.z > info.zhi) return false;
        e.s = b.s; e.t = b.t; e.from = b.from; e.xprev = b.xprev; e.id_from = b.id_from;
        e.xdst = b.to_org ? S.w : (b.to_stage ? info.x : -1); e.id_to = id;
        return true;
    }
    // inter-node: `id` is the source rank s; the block waits on the rank of s's node that has
    // the receiver's local index (src/twophase_twolayer_rbruck.cpp:430-453, 634-671)
    const int s = id, t = to;
    const int gs = vc_div(s, S.dn), gt = vc_div(t, S.dn), ls = s - gs * n, lt = t - gt * n;
    if (gs == gt) return false;
    const int q = vc_wrap(gs - gt + S.G, S.G) * n + ls;
    if (q < info.qlo || q >= info.qhi) return false;
    const int j = vc_wrap(ls - lt + n, n);
    e.s = s; e.t = t; e.from = gs * n + lt;
    e.xprev = j == 0 ? -1 : (S.msd ? vc_low_digit(j, S.dr) : vc_top_digit(j, S.dr));
    e.id_from = gt * n + ls; e.xdst = -1; e.id_to = id;
    return true;
}

VC_HD int64_t vc_entry_len(const VcSched &S, const VcTables &T, const VcEntry &e) {
    if (e.nblk == 1) return (int64_t)T.sc[(int64_t)e.s * S.P + e.t] * S.esz;
    const int gs = vc_div(e.s, S.dn), m0 = e.s - gs * S.n;
    return vc_org_run_prefix(S, T, gs, e.t, m0 + e.nblk) - vc_org_run_prefix(S, T, gs, e.t, m0);
}

// The whole-block copy an entry stands for.
VC_HD VcDesc vc_entry_desc(const VcSched &S, const VcTables &T, const int64_t *slot_off, const int64_t *row_base,
                           const VcEntry &e, int to) {
    VcDesc d;
    d.len = vc_entry_len(S, T, e);
    d.from = e.from; d.to = to;
    d.src = e.xprev < 0 ? (VC_SPACE_SEND | vc_send_offset(S, T, e.s, e.t))
                        : (VC_SPACE_STAGE | vc_stage_addr(S, T, slot_off, row_base, e.xprev, e.from, e.id_from, e.s, e.t));
    d.dst = e.xdst < 0 ? (VC_SPACE_RECV | vc_recv_offset(S, T, e.s, e.t))
                       : (VC_SPACE_STAGE | vc_stage_addr(S, T, slot_off, row_base, e.xdst, to, e.id_to, e.s, e.t));
    return d;
}

// Blocks are copied in pieces of at most VC_CHUNK bytes, one work item (a workgroup, a wavefront or a quarter of one)
// each.  Pieces are cut where the DESTINATION address is a multiple of the cache line, so that only the first piece of
// a block has a byte-wise head and only the last one a tail; every piece in between is whole aligned vectors.

// Cache-line phase of the destination address of an entry's copy.  Staging slots and organized runs are laid out at
// the phase of the block's final address, so this holds whichever arena the copy writes to.
VC_HD int vc_entry_phase(const VcSched &S, const VcTables &T, const VcEntry &e) { return vc_phase(S, T, e.s, e.t); }

// Where a long copy is cut: pieces end where the destination address is a multiple of VC_PIECE when the destination
// is recvbuf (whole 4 KiB-aligned pieces, no cache line shared between two workgroups), and at multiples of VC_PIECE
// from the line boundary below the start otherwise (staging addresses are not known when pieces are counted).
// Always congruent to the line phase.
VC_HD int vc_entry_cut(const VcSched &S, const VcTables &T, const VcEntry &e) {
    if (e.xdst < 0) return (int)((vc_recv_offset(S, T, e.s, e.t) + S.recv_lo) & (VC_PIECE - 1));
    return vc_phase(S, T, e.s, e.t);
}

// A copy that fits one work item (VC_CHUNK bytes from the cache-line boundary below its destination) stays whole; a
// longer one is cut into pieces of at most VC_PIECE bytes, the size at which a plain copy runs fastest on this chip
// (one vector per lane of a 256-lane workgroup).  Only the first piece has a byte-wise head and only the last one a tail.
// The copy kernel's window starts at the cache-line boundary at or below the destination: `phase` bytes before it.
VC_HD bool vc_fits_one_item(int64_t len, int phase) { return len + phase <= VC_CHUNK; }

VC_HD int64_t vc_chunk_count(int64_t len, int phase, int cut) {
    if (len <= 0) return 0;
    return vc_fits_one_item(len, phase) ? 1 : (len + cut + VC_PIECE - 1) / VC_PIECE;
}

// Bytes [lo, hi) of a copy of `len` bytes that piece c of its vc_chunk_count(len, phase, cut) pieces moves.
VC_HD void vc_piece_range(int64_t len, int phase, int cut, int64_t c, int64_t &lo, int64_t &hi) {
    if (vc_fits_one_item(len, phase)) { lo = 0; hi = len; return; }
    lo = c == 0 ? 0 : c * VC_PIECE - cut;
    hi = (c + 1) * VC_PIECE - cut;
    if (hi > len) hi = len;
}

VC_HD VcDesc vc_chunk_of(const VcDesc &whole, int64_t c, int phase, int cut) {
    int64_t lo, hi;
    vc_piece_range(whole.len, phase, cut, c, lo, hi);
    VcDesc d = whole;
    d.src += lo; d.dst += lo; d.len = hi - lo;
    return d;
}

// ---- forwarded execution: one work item carries a piece of a block through all its hops ----
// The hops of one block depend only on each other: hop k + 1 reads what hop k wrote.  When one workgroup performs all
// of them it keeps the piece in registers between the hops: the data is read once (from sendbuf) and written once per
// hop (to the staging slot of every intermediate holder, then to recvbuf).  Every block ends up in the same places as
// after the launch-per-digit execution.
//
// A block moves at most once per digit, so its hops are indexed by "hop slots": intra-node digit x, inter-node digit
// S.w + x, and one last slot for what goes straight to recvbuf by an inter-node or direct message (or stays on its rank).
#define VC_MAX_HOP_SLOTS 32

VC_HD int vc_hop_slots(const VcSched &S) { return S.w + S.w2 + 1; }

// Hop slot of an entry of a launch (the CPU check of the plan derives every block's route from the launches' entries
// this way and compares it with vc_block_hop).
VC_HD int vc_hop_slot(const VcSched &S, const VcLaunchInfo &info, const VcEntry &e) {
    if (e.s == e.t) return S.w + S.w2;
    return info.kind == 0 ? info.x : (info.kind == 4 ? S.w + info.x : S.w + S.w2);
}

// All hops of a block cut it at the same places: where its image in recvbuf crosses a multiple of VC_PIECE.
VC_HD int vc_chain_cut(const VcSched &S, const VcTables &T, int s, int t) {
    return (int)((vc_recv_offset(S, T, s, t) + S.recv_lo) & (VC_PIECE - 1));
}

VC_HD int64_t vc_chain_count(const VcSched &S, const VcTables &T, int s, int t) {
    const int64_t len = (int64_t)T.sc[(int64_t)s * S.P + t] * S.esz;
    return vc_chunk_count(len, vc_phase(S, T, s, t), vc_chain_cut(S, T, s, t));
}

// Entries of the tables around the pair (source s, receiver t) that no set of ranks could have passed: the receiver must
// expect exactly what the source sends (the reference fails with an MPI truncation error), and no count or displacement
// of the receiver's own row may be negative.  Summed over all pairs this is header word VC_HEADER_BAD, whoever adds it
// up (the planner's row kernel, or the copy kernel that plans nothing).
VC_HD int vc_pair_bad_entries(const VcSched &S, const VcTables &T, int s, int t) {
    const int64_t i = (int64_t)t * S.P + s;
    const int expected = T.rc[i], sent = T.sc[(int64_t)s * S.P + t];
    return (expected != sent) + (int)((T.sc[i] < 0) | (T.sd[i] < 0) | (expected < 0) | (!S.packed_recv && T.rd[i] < 0));
}

// Layout of a chain item, in int64 words; `stride` = VC_CHAIN_HEAD + hop slots of the call.
#define VC_CHAIN_SRC 0    // space-tagged source offset of the piece (always in sendbuf)
#define VC_CHAIN_LEN 1
#define VC_CHAIN_NHOP 2
#define VC_CHAIN_HEAD 3   // followed by the space-tagged destination of the piece at every hop

// Hop slots in the order in which a call works through them: the intra-node digits (most significant first for the
// functions that run them that way), the inter-node digits, the last slot.  The mapping is its own inverse.
VC_HD int vc_slot_time(const VcSched &S, int k) { return (k < S.w && S.msd) ? S.w - 1 - k : k; }

// Whether block (s, t) moves in hop slot k (vc_block_hop without the destination).
VC_HD bool vc_block_moves(const VcSched &S, int s, int t, int k) {
    const int n = S.n, G = S.G, final_slot = S.w + S.w2;
    if (s == t) return k == final_slot;
    const int gs = vc_div(s, S.dn), gt = vc_div(t, S.dn);
    if (k == final_slot) return S.last_hop == 2 || (S.last_hop == 1 && gs != gt);
    const bool intra = k < S.w;
    const int x = intra ? k : k - S.w;
    const int span = intra ? n : G;
    const int j = intra ? vc_wrap((s - gs * n) - (t - gt * n) + n, n) : vc_wrap(gs - gt + G, G);
    int dist;
    const int upper = vc_upper_digits(S, j, x, span, dist);
    return dist < span && vc_mod(upper, S.dr) != 0;
}

// The hop slot in which block (s, t) moves next after hop slot k (in the call's order), or -1.
VC_HD int vc_next_hop(const VcSched &S, int s, int t, int k) {
    const int ns = S.w + S.w2 + 1;
    for (int time = vc_slot_time(S, k) + 1; time < ns; time++) {
        const int k2 = vc_slot_time(S, time);
        if (vc_block_moves(S, s, t, k2)) return k2;
    }
    return -1;
}

// Where the sub-regions of reused staging go.  A sub-region (family = arrival slot * slots + departure slot; the organized
// region at slots * slots) is written in the launches of its arrival slot and read for the last time in those of its
// departure slot, so its memory is free for sub-regions that arrive in any later slot.  A hole seldom has the size of a
// whole sub-region, so sub-regions are placed in VC_RECYCLE_SEGMENTS pieces, each the rows of a run of consecutive
// receiving ranks: size[family * VC_RECYCLE_SEGMENTS + g] are the bytes of the pieces (multiples of VC_LINE), base[...]
// receives their offsets in the arena; returns the arena's size.  First fit from the low end of the arena, the
// longest-lived sub-regions of an arrival slot first; the holes are kept sorted and merged, so the pieces of a sub-region
// that leaves become one hole again where they were neighbours.  This is the reference's economy — only the P - K - 1
// multi-hop slots, reused every round (src/twophase_tunable_rbruckv-om.cpp:52-86, src/tuna.cpp:36-52,93-97) — for compact
// slots of variable length.  hole_lo / hole_hi: work space of VC_RECYCLE_MAX_HOLES entries each.
#define VC_RECYCLE_SEGMENTS 8
#define VC_RECYCLE_MAX_HOLES 256

VC_HD void vc_hole_add(int64_t *lo, int64_t *hi, int &nh, int64_t a, int64_t b, int64_t &top) {
    if (a >= b) return;
    int i = 0;
    while (i < nh && lo[i] < a) i++;
    if (i > 0 && hi[i - 1] == a) {
        hi[--i] = b;                                      // grows the hole below it
    } else {
        if (nh == VC_RECYCLE_MAX_HOLES) return;           // (the bytes stay unused for the rest of the call)
        for (int k = nh; k > i; k--) { lo[k] = lo[k - 1]; hi[k] = hi[k - 1]; }
        lo[i] = a; hi[i] = b; nh++;
    }
    if (i + 1 < nh && hi[i] == lo[i + 1]) {               // ... and meets the hole above it
        hi[i] = hi[i + 1];
        for (int k = i + 1; k + 1 < nh; k++) { lo[k] = lo[k + 1]; hi[k] = hi[k + 1]; }
        nh--;
    }
    if (hi[nh - 1] == top) top = lo[--nh];                // the top of the arena comes back
}

VC_HD int64_t vc_hole_take(int64_t *lo, int64_t *hi, int &nh, int64_t size, int64_t &top, int64_t &peak) {
    for (int i = 0; i < nh; i++)
        if (hi[i] - lo[i] >= size) {
            const int64_t at = lo[i];
            lo[i] += size;
            if (lo[i] == hi[i]) {
                for (int k = i; k + 1 < nh; k++) { lo[k] = lo[k + 1]; hi[k] = hi[k + 1]; }
                nh--;
            }
            return at;
        }
    const int64_t at = top;
    top += size;
    if (top > peak) peak = top;
    return at;
}

VC_HD int64_t vc_allocate_staging(const VcSched &S, const int64_t *size, int64_t *base, int64_t *hole_lo, int64_t *hole_hi) {
    const int ns = S.w + S.w2 + 1, org = ns * ns, nseg = VC_RECYCLE_SEGMENTS;
    int nh = 0;
    int64_t top = 0, peak = 0;
    for (int g = 0; g < nseg; g++)                        // the organized region lives from the first launch to the last
        base[org * nseg + g] = size[org * nseg + g] > 0 ? vc_hole_take(hole_lo, hole_hi, nh, size[org * nseg + g], top, peak) : 0;
    for (int ta = 0; ta < ns; ta++) {
        if (ta >= 1) {                                    // what the launches of the slot before have read for the last time
            const int kd = vc_slot_time(S, ta - 1);
            for (int ka = 0; ka < ns - 1; ka++)
                if (vc_slot_time(S, ka) < ta - 1)
                    for (int g = 0; g < nseg; g++) {
                        const int u = (ka * ns + kd) * nseg + g;
                        if (size[u] > 0) vc_hole_add(hole_lo, hole_hi, nh, base[u], base[u] + size[u], top);
                    }
        }
        const int ka = vc_slot_time(S, ta);
        if (ka >= ns - 1) continue;                       // the last slot has no staging region
        for (int td = ns - 1; td > ta; td--) {
            const int f = ka * ns + vc_slot_time(S, td);
            for (int g = 0; g < nseg; g++)
                base[f * nseg + g] = size[f * nseg + g] > 0 ? vc_hole_take(hole_lo, hole_hi, nh, size[f * nseg + g], top, peak) : 0;
        }
    }
    return peak;
}

// Receiving ranks per piece of a sub-region, and the piece a rank's row belongs to.
VC_HD int vc_recycle_rows_per_segment(int P) { return (P + VC_RECYCLE_SEGMENTS - 1) / VC_RECYCLE_SEGMENTS; }

// The route of block (s, t) in closed form: does it move in hop slot k, and where to?  After digit x of a Bruck that
// runs least significant digit first a block has travelled (offset mod r^(x+1)) ranks down from its source, most
// significant first (offset div r^x) * r^x; it sits in slot (destination group) * n + (local offset + local rank) % n
// of its holder (src/twophase_twolayer_rbruck.cpp:322), and lands in recvbuf when no digit is left and it is on its
// destination's node.  The CPU check of the plan compares this with what the launches' entries say, block by block.
VC_HD bool vc_block_hop(const VcSched &S, const VcTables &T, const int64_t *slot_off, const int64_t *row_base, int s, int t, int k,
                        int64_t &dst) {
    const int n = S.n, G = S.G, final_slot = S.w + S.w2;
    const int64_t to_recv = VC_SPACE_RECV | vc_recv_offset(S, T, s, t);
    if (s == t) { dst = to_recv; return k == final_slot; }
    const int gs = vc_div(s, S.dn), gt = vc_div(t, S.dn), ls = s - gs * n, lt = t - gt * n;
    if (k == final_slot) { dst = to_recv; return S.last_hop == 2 || (S.last_hop == 1 && gs != gt); }
    const bool intra = k < S.w;
    const int x = intra ? k : k - S.w;
    const int span = intra ? n : G;
    const int j = intra ? vc_wrap(ls - lt + n, n) : vc_wrap(gs - gt + G, G);      // offset inside the node / between the nodes
    int dist;
    const int upper = vc_upper_digits(S, j, x, span, dist);       // the digits from x upwards
    if (dist >= span) return false;
    const int higher = vc_div(upper, S.dr);                       // ... from x + 1 upwards
    if (upper == higher * S.r) return false;
    const bool msd = intra && S.msd;
    const int travelled = msd ? upper * dist : j - higher * dist * S.r;           // at most j < span
    const bool last = msd ? upper * dist == j : higher == 0;
    const int pos = vc_wrap((intra ? ls : gs) - travelled + span, span);            // local rank / node of the holder after the hop
    const int to = intra ? gs * n + pos : pos * n + lt;
    const int id = intra ? gt * n + vc_wrap(j + pos, n) : j * n + ls;
    dst = (last && (intra ? gs == gt : true)) ? to_recv : (VC_SPACE_STAGE | vc_stage_addr(S, T, slot_off, row_base, k, to, id, s, t));
    return true;
}

// Piece c of a block whose source and hop destinations (whole block) are known.
VC_HD void vc_chain_piece(int64_t src, int64_t len, int phase, int cut, int64_t c, const int64_t *dst, int nhop, int64_t *item) {
    VcDesc whole;
    whole.src = src; whole.dst = 0; whole.len = len; whole.from = 0; whole.to = 0;
    const VcDesc piece = vc_chunk_of(whole, c, phase, cut);      // piece.dst = offset of the piece inside the block
    item[VC_CHAIN_SRC] = piece.src;
    item[VC_CHAIN_LEN] = piece.len;
    item[VC_CHAIN_NHOP] = nhop;
    for (int k = 0; k < nhop; k++) item[VC_CHAIN_HEAD + k] = dst[k] + piece.dst;
}

// Hop destinations of block (s, t) in slot order; returns their number.
VC_HD int vc_chain_route(const VcSched &S, const VcTables &T, const int64_t *slot_off, const int64_t *row_base, int s, int t,
                         int64_t *dst) {
    int nhop = 0;
    const int nslots = vc_hop_slots(S);
    for (int k = 0; k < nslots; k++) {
        int64_t d;
        if (vc_block_hop(S, T, slot_off, row_base, s, t, k, d)) dst[nhop++] = d;
    }
    return nhop;
}

// Writes piece c of block (s, t) to `item`.
VC_HD void vc_chain_item(const VcSched &S, const VcTables &T, const int64_t *slot_off, const int64_t *row_base, int s, int t, int64_t c,
                         int64_t *item) {
    const int64_t len = (int64_t)T.sc[(int64_t)s * S.P + t] * S.esz;
    const int nhop = vc_chain_route(S, T, slot_off, row_base, s, t, item + VC_CHAIN_HEAD);   // whole-block destinations first
    vc_chain_piece(VC_SPACE_SEND | vc_send_offset(S, T, s, t), len, vc_phase(S, T, s, t), vc_chain_cut(S, T, s, t), c,
                   item + VC_CHAIN_HEAD, nhop, item);
}
