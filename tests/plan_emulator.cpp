// plan_emulator.cpp — CPU build of the library's schedule and plan arithmetic.
//
// Test infrastructure: compiles the SAME headers the GPU library uses
// (csrc/vc_sched.h for the schedule, csrc/vc_plan_math.h for the per-entry index
// arithmetic) as host code, replaces the three planning kernels by plain loops
// and the copy kernel by memcpy, and checks every copy before doing it:
//   - source and destination ranges lie inside their arenas,
//   - staged bytes are read only after they were written,
//   - within one launch no destination overlaps another destination or a source.
// Copies are cut into the same pieces (work items) the copy kernel gets.
// This is how indexing mistakes are found without a GPU.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../rbruck_alltoallv_amd/csrc/vc_dispatch.h"
#include "../rbruck_alltoallv_amd/csrc/vc_plan_math.h"
#include "../rbruck_alltoallv_amd/csrc/vc_sched.h"

struct Range { int64_t lo, hi; int space; };

static int count_overlaps(std::vector<Range> &dst, std::vector<Range> &src) {
    int bad = 0;
    auto key = [](const Range &a, const Range &b) { return a.space != b.space ? a.space < b.space : a.lo < b.lo; };
    std::sort(dst.begin(), dst.end(), key);
    for (size_t i = 1; i < dst.size(); i++)
        if (dst[i].space == dst[i - 1].space && dst[i].lo < dst[i - 1].hi) bad++;
    // a source against the sorted destinations: only the last destination that starts below the source's end can reach
    // into it once the destinations do not overlap each other
    for (const Range &s : src) {
        const Range probe{s.hi, 0, s.space};
        auto it = std::lower_bound(dst.begin(), dst.end(), probe, key);      // first destination with lo >= s.hi
        if (it == dst.begin()) continue;
        --it;
        if (it->space == s.space && it->lo < s.hi && s.lo < it->hi) bad++;
    }
    return bad;
}

extern "C" int plan_emulate(int func, int P, int n, int r, int batch, int esz, int uniform_count, const char *send,
                            int64_t send_bytes, char *recv, int64_t recv_bytes, const int64_t *sbase, const int64_t *rbase,
                            const int *sc, const int *sd, const int *rc, const int *rd, int recv_lo, int64_t *stats_out,
                            int64_t *traffic_out, int max_launches, int batch2, int forward, int stride, int recycle) {
    VcSched S;
    std::vector<VcLaunchInfo> L;
    int code = vc_make_schedule((VcFunc)func, P, n, r, batch, esz, uniform_count, S, L, batch2, forward != 0);
    if (code) return code;
    S.recv_lo = recv_lo;
    const int64_t PP = (int64_t)P * P;
    if (stride > 0 && S.coalesce) return -100;            // fixed-stride staging has no organized region
    S.stride = stride > 0 ? stride : 0;
    // reused staging under the library's own rule (make_schedule in csrc/vc_api.hip): launch-per-digit execution with at
    // least three staging regions
    if (recycle && !forward && !S.stride && S.w + S.w2 >= 3 && S.w + S.w2 + 1 <= VC_RECYCLE_MAX_SLOTS) S.recycle = 1;

    std::vector<int> ucnt, udsp, rdp;
    VcTables T;
    T.sbase = sbase; T.rbase = rbase; T.rd_packed = nullptr;
    if (uniform_count > 0 || func == VC_F_UNIFORM_SPREADOUT || func == VC_F_UNIFORM_ISPLIT) {
        ucnt.assign(PP, uniform_count); udsp.resize(PP);
        for (int64_t i = 0; i < PP; i++) udsp[i] = (int)(i % P) * uniform_count;
        T.sc = T.rc = ucnt.data(); T.sd = T.rd = udsp.data();
    } else {
        T.sc = sc; T.sd = sd; T.rc = rc; T.rd = rd;
    }
    if (S.packed_recv) {
        rdp.resize(PP);
        for (int t = 0; t < P; t++) { int acc = 0; for (int s = 0; s < P; s++) { rdp[(int64_t)t * P + s] = acc; acc += T.rc[(int64_t)t * P + s]; } }
        T.rd_packed = rdp.data();
    }

    // passes 1 and 2 of the planner
    const int w = std::max(vc_regions(S), 1) + 1;         // staging regions
    std::vector<int64_t> slot_off(PP * w, 0), row_base((int64_t)P * std::max(w, vc_row_families(S) + 1), 0);
    int64_t stage_bytes = S.stride ? vc_strided_stage_bytes(S) : 0;
    if (S.recycle) {
        // the planner's passes for reused staging: slots numbered per (arrival, departure) family, rows inside a family,
        // families placed by the allocator the planning kernel uses
        const int ns = S.w + S.w2 + 1, nfam = ns * ns + 1;
        const int nseg = VC_RECYCLE_SEGMENTS, rps = vc_recycle_rows_per_segment(P);
        std::vector<int64_t> row_tot((int64_t)nfam * P, 0), piece_size((size_t)nfam * nseg, 0), piece_base((size_t)nfam * nseg, 0),
            hole_lo(VC_RECYCLE_MAX_HOLES), hole_hi(VC_RECYCLE_MAX_HOLES);
        for (int y = 0; y < S.w + S.w2; y++)
            for (int to = 0; to < P; to++) {
                std::vector<int64_t> carry(ns, 0);
                for (int id = 0; id < P; id++) {
                    int st[2] = {0, 0};
                    const int64_t v = vc_region_slot_size(S, T, y, to, id, nullptr, st);
                    if (!v) continue;
                    const int kd = vc_next_hop(S, st[0], st[1], y);
                    if (kd < 0 || vc_slot_time(S, kd) <= vc_slot_time(S, y)) return -101;
                    slot_off[((int64_t)y * P + to) * P + id] = carry[kd];
                    carry[kd] += v;
                }
                for (int kd = 0; kd < ns; kd++) row_tot[(int64_t)(y * ns + kd) * P + to] = carry[kd];
            }
        if (S.coalesce)
            for (int to = 0; to < P; to++) {
                std::vector<int64_t> run_base(S.G);
                int64_t acc = 0;
                for (int g = 0; g < S.G; g++) { run_base[g] = acc; acc += vc_org_run_size(S, T, to, g); }
                for (int id = 0; id < P; id++)
                    slot_off[((int64_t)S.w * P + to) * P + id] = run_base[id / S.n] + vc_org_slot_rel(S, T, to, id);
                row_tot[(int64_t)(ns * ns) * P + to] = acc;
            }
        // a sub-region is placed in pieces: the rows of rps consecutive receivers each
        for (int f = 0; f < nfam; f++) {
            int64_t acc = 0;
            for (int to = 0; to < P; to++) {
                row_base[(int64_t)f * P + to] = acc;
                piece_size[(size_t)f * nseg + to / rps] += row_tot[(int64_t)f * P + to];
                acc += row_tot[(int64_t)f * P + to];
            }
        }
        stage_bytes = vc_allocate_staging(S, piece_size.data(), piece_base.data(), hole_lo.data(), hole_hi.data());
        for (int f = 0; f < nfam; f++) {
            int64_t start = 0;
            for (int g = 0; g < nseg; g++) {
                const size_t u = (size_t)f * nseg + g;
                if (piece_size[u] > 0 && piece_base[u] + piece_size[u] > stage_bytes) return -102;
                for (int to = g * rps; to < P && to < (g + 1) * rps; to++)
                    if (piece_size[u] > 0) row_base[(int64_t)f * P + to] += piece_base[u] - start;
                start += piece_size[u];
            }
        }
    }
    for (int x = 0; x < S.w + S.w2 && !S.stride && !S.recycle; x++) {
        for (int to = 0; to < P; to++) {
            row_base[(int64_t)x * P + to] = stage_bytes;
            int64_t acc = 0;
            for (int id = 0; id < P; id++) {
                slot_off[((int64_t)x * P + to) * P + id] = acc;
                acc += vc_region_slot_size(S, T, x, to, id);
            }
            stage_bytes += acc;
        }
    }
    if (S.coalesce && !S.recycle)                         // pass 1b: organized region
        for (int to = 0; to < P; to++) {
            row_base[(int64_t)S.w * P + to] = stage_bytes;
            std::vector<int64_t> run_base(S.G);
            int64_t acc = 0;
            for (int g = 0; g < S.G; g++) { run_base[g] = acc; acc += vc_org_run_size(S, T, to, g); }
            for (int id = 0; id < P; id++)
                slot_off[((int64_t)S.w * P + to) * P + id] = run_base[id / S.n] + vc_org_slot_rel(S, T, to, id);
            stage_bytes += acc;
        }
    std::vector<char> stage((size_t)stage_bytes + 64, (char)0xCD);
    std::vector<char> written((size_t)stage_bytes + 64, 0);
    // forwarded execution is checked against the launch-per-digit execution of the same schedule: that one runs first,
    // into copies of the arenas
    char *const recv_final = recv;
    std::vector<char> recv_steps;
    if (forward) { recv_steps.assign(recv, recv + recv_bytes); recv = recv_steps.data(); }

    int64_t errors = 0, moved = 0, items = 0;
    const int nl = (int)L.size();
    for (int k = 0; k < nl; k++) {
        std::vector<VcDesc> descs;
        std::vector<Range> dst_ranges, src_ranges;
        const int nent = vc_entries_per_rank(S, L[k]);
        for (int to = 0; to < P; to++)
            for (int id = 0; id < nent; id++) {
                VcEntry e;
                if (!vc_entry_block(S, L[k], to, id, e)) continue;
                const VcDesc whole = vc_entry_desc(S, T, slot_off.data(), row_base.data(), e, to);
                const int phase = vc_entry_phase(S, T, e);
                const int dst_lo = (int)(whole.dst >> VC_SPACE_SHIFT) == 1 ? recv_lo : 0;
                if (whole.len > 0 && (int)(((whole.dst & VC_OFFSET_MASK) + dst_lo) & (VC_LINE - 1)) != phase) errors++;
                const int cut = vc_entry_cut(S, T, e);
                if ((cut & (VC_LINE - 1)) != phase) errors++;
                const int64_t nchunks = vc_chunk_count(whole.len, phase, cut);
                int64_t covered = 0;
                items += nchunks;
                for (int64_t c = 0; c < nchunks; c++) {
                const VcDesc d = vc_chunk_of(whole, c, phase, cut);
                // the copy kernel's window: VC_CHUNK bytes from the cache-line boundary at or below the destination
                if (d.len + (((d.dst & VC_OFFSET_MASK) + dst_lo) & (VC_LINE - 1)) > VC_CHUNK) errors++;
                if (d.len <= 0 || d.len > VC_CHUNK || d.src - whole.src != covered || d.dst - whole.dst != covered) { errors++; continue; }
                // only the first piece may start off a cache-line boundary of the destination
                if (c > 0 && (((d.dst & VC_OFFSET_MASK) + dst_lo) & (VC_LINE - 1)) != 0) errors++;
                // ... and, in recvbuf, on a 4 KiB boundary
                if (c > 0 && (int)(whole.dst >> VC_SPACE_SHIFT) == 1 && (((d.dst & VC_OFFSET_MASK) + dst_lo) & (VC_PIECE - 1)) != 0) errors++;
                covered += d.len;
                const int sspace = (int)(d.src >> VC_SPACE_SHIFT), dspace = (int)(d.dst >> VC_SPACE_SHIFT);
                const int64_t so = d.src & VC_OFFSET_MASK, dof = d.dst & VC_OFFSET_MASK;
                const int64_t slim = sspace == 0 ? send_bytes : (sspace == 2 ? stage_bytes : -1);
                const int64_t dlim = dspace == 1 ? recv_bytes : (dspace == 2 ? stage_bytes : -1);
                if (so < 0 || so + d.len > slim || dof < 0 || dof + d.len > dlim) { errors++; continue; }
                if (d.from < 0 || d.from >= P || d.to != to) errors++;
                if (sspace == 2)                          // every staged byte is read exactly once: by the block's next hop
                    for (int64_t b = 0; b < d.len; b++) { errors += !written[so + b]; written[so + b] = 0; }
                descs.push_back(d);
                dst_ranges.push_back({dof, dof + d.len, dspace});
                src_ranges.push_back({so, so + d.len, sspace});
                if (traffic_out && k < max_launches) traffic_out[((int64_t)k * P + d.from) * P + d.to] += d.len;
                }
                if (covered != whole.len) errors++;
            }
        errors += count_overlaps(dst_ranges, src_ranges);
        for (const VcDesc &d : descs) {
            const int sspace = (int)(d.src >> VC_SPACE_SHIFT), dspace = (int)(d.dst >> VC_SPACE_SHIFT);
            const char *from = (sspace == 0 ? send : stage.data()) + (d.src & VC_OFFSET_MASK);
            char *to = (dspace == 1 ? recv : stage.data()) + (d.dst & VC_OFFSET_MASK);
            memcpy(to, from, (size_t)d.len);
            if (dspace == 2) {                            // ... and nothing lands on bytes that are still waiting for theirs
                char *wr = written.data() + (d.dst & VC_OFFSET_MASK);
                for (int64_t b = 0; b < d.len; b++) { errors += wr[b] != 0; wr[b] = 1; }
            }
            moved += d.len;
        }
    }
    for (int64_t b = 0; b < stage_bytes; b++) errors += written[b] != 0;          // every staged block has moved on
    if (forward) {
        const int nslots = vc_hop_slots(S), stride = VC_CHAIN_HEAD + nslots;
        if (nslots > VC_MAX_HOP_SLOTS) errors++;
        std::vector<int64_t> hop_src(PP, -1), hop_dst((size_t)nslots * PP, -1);
        for (int k = 0; k < nl; k++) {                    // vc_chain_hops
            const int nent = vc_entries_per_rank(S, L[k]);
            for (int to = 0; to < P; to++)
                for (int id = 0; id < nent; id++) {
                    VcEntry e;
                    if (!vc_entry_block(S, L[k], to, id, e)) continue;
                    if (e.nblk != 1) { errors++; continue; }
                    const VcDesc d = vc_entry_desc(S, T, slot_off.data(), row_base.data(), e, to);
                    const int64_t key = (int64_t)e.t * P + e.s;
                    int64_t &cell = hop_dst[(int64_t)vc_hop_slot(S, L[k], e) * PP + key];
                    if (cell != -1) errors++;             // a block moves at most once per hop slot
                    cell = d.dst;
                    if (e.xprev < 0) { if (hop_src[key] != -1) errors++; hop_src[key] = d.src; }
                }
        }
        std::vector<char> stage2((size_t)stage_bytes + 64, (char)0xCD);
        std::vector<Range> dst_ranges, none;
        std::vector<int64_t> item(stride);
        int64_t chain_items = 0, chain_moved = 0;
        for (int t = 0; t < P; t++)                       // vc_chain_emit + vc_copy_chains_kernel
            for (int s0 = 0; s0 < P; s0++) {
                const int64_t len = (int64_t)T.sc[(int64_t)s0 * P + t] * esz;
                const int64_t cnt = vc_chain_count(S, T, s0, t);
                if ((len > 0) != (cnt > 0)) errors++;
                if (len > 0 && hop_src[(int64_t)t * P + s0] < 0) { errors++; continue; }
                int64_t covered = 0;
                // the closed-form route of the block against what the launches' entries say, hop slot by hop slot
                const int64_t key0 = (int64_t)t * P + s0;
                for (int k = 0; k < nslots; k++) {
                    int64_t d;
                    const bool moves = vc_block_hop(S, T, slot_off.data(), row_base.data(), s0, t, k, d);
                    const int64_t cell = hop_dst[(int64_t)k * PP + key0];
                    if (moves ? cell != d : cell != -1) errors++;
                }
                if (hop_src[key0] != (VC_SPACE_SEND | vc_send_offset(S, T, s0, t))) errors++;
                for (int64_t c = 0; c < cnt; c++) {
                    vc_chain_item(S, T, slot_off.data(), row_base.data(), s0, t, c, item.data());
                    const int64_t src = item[VC_CHAIN_SRC], plen = item[VC_CHAIN_LEN], nhop = item[VC_CHAIN_NHOP];
                    chain_items++;
                    if ((int)(src >> VC_SPACE_SHIFT) != 0 || plen <= 0 || nhop < 1) { errors++; continue; }
                    const int64_t so = src & VC_OFFSET_MASK;
                    if (so + plen > send_bytes) { errors++; continue; }
                    if (so - (hop_src[(int64_t)t * P + s0] & VC_OFFSET_MASK) != covered) errors++;
                    int line = -1;
                    bool reaches_recv = false;
                    for (int64_t k = 0; k < nhop; k++) {
                        const int64_t d = item[VC_CHAIN_HEAD + k];
                        const int dspace = (int)(d >> VC_SPACE_SHIFT);
                        const int64_t dof = d & VC_OFFSET_MASK;
                        const int64_t dlim = dspace == 1 ? recv_bytes : (dspace == 2 ? stage_bytes : -1);
                        if (dof < 0 || dof + plen > dlim) { errors++; continue; }
                        const int ph = (int)((dof + (dspace == 1 ? recv_lo : 0)) & (VC_LINE - 1));
                        if (line >= 0 && ph != line) errors++;        // one lane mapping serves every hop
                        line = ph;
                        if (plen + ph > VC_CHUNK) errors++;
                        if (c > 0 && ph != 0) errors++;
                        dst_ranges.push_back({dof, dof + plen, dspace});
                        memcpy((dspace == 1 ? recv_final : stage2.data()) + dof, send + so, (size_t)plen);
                        chain_moved += plen;
                        reaches_recv |= dspace == 1;
                    }
                    if (!reaches_recv) errors++;
                    covered += plen;
                }
                if (covered != len) errors++;
            }
        errors += count_overlaps(dst_ranges, none);
        // same memory as after the launch-per-digit execution
        if (chain_moved != moved) errors++;
        if (memcmp(stage.data(), stage2.data(), (size_t)stage_bytes) != 0) errors++;
        if (memcmp(recv_steps.data(), recv_final, (size_t)recv_bytes) != 0) errors++;
        items = chain_items;
    }
    stats_out[0] = nl; stats_out[1] = stage_bytes; stats_out[2] = moved; stats_out[3] = errors; stats_out[4] = items;
    return 0;
}

// The staging allocator of the planning kernel on its own: sizes per piece of every (arrival, departure) family in
// (VC_RECYCLE_SEGMENTS pieces per family), bases out.
extern "C" int64_t staging_allocate(int w, int w2, int msd, int coalesce, const int64_t *size, int64_t *base) {
    VcSched S;
    memset(&S, 0, sizeof S);
    S.w = w; S.w2 = w2; S.msd = msd; S.coalesce = coalesce; S.recycle = 1;
    std::vector<int64_t> lo(VC_RECYCLE_MAX_HOLES), hi(VC_RECYCLE_MAX_HOLES);
    return vc_allocate_staging(S, size, base, lo.data(), hi.data());
}


// The library's choice of kernel (csrc/vc_dispatch.h) for a call of function `func` on P ranks whose last forwarded call
// left the hint (valid, items, payload, max_pieces, max_len).  out: lanes, stride, stride_lanes, guard.max_pieces,
// guard.max_items, guard.max_average, guard.max_len.  Returns the schedule's error code.
extern "C" int dispatch_decision(int func, int P, int n, int r, int mode, int call_kind, int valid, int64_t items, int64_t payload,
                                 int64_t max_pieces, int64_t max_len, int64_t *out) {
    VcSched S;
    std::vector<VcLaunchInfo> L;
    const int code = vc_make_schedule((VcFunc)func, P, n, r, 0, 1, 0, S, L, 0, true);
    if (code) return code;
    const VcHint h = {valid, items, payload, max_pieces, max_len};
    const VcDispatch d = vc_dispatch(mode, call_kind, h, S);
    out[0] = d.lanes; out[1] = d.stride; out[2] = d.stride_lanes; out[3] = d.guard.max_pieces; out[4] = d.guard.max_items;
    out[5] = d.guard.max_average; out[6] = d.guard.max_len;
    return 0;
}

extern "C" int recycle_segments() { return VC_RECYCLE_SEGMENTS; }

extern "C" int lanes_for_items(int64_t bytes, int64_t items) { return vc_lanes_for_items(bytes, items); }

// vc_div / vc_mod (csrc/vc_common.h) against the hardware division for every divisor in [d_lo, d_hi]: numerators around every
// multiple of the divisor along a geometric walk up to 2^31 - 1, the ends of the range, and `samples` pseudo-random ones.
// Returns the number of numerators whose quotient or remainder differs.
extern "C" int64_t division_mismatches(int d_lo, int d_hi, int samples) {
    int64_t wrong = 0;
    uint64_t state = 0x9E3779B97F4A7C15ull;
    for (int64_t d = d_lo; d <= d_hi; d++) {
        const VcDivisor v = vc_make_divisor((int)d);
        auto check = [&](int64_t x) {
            if (x < 0 || x > 0x7FFFFFFF) return;
            wrong += vc_div((int)x, v) != (int)(x / d) || vc_mod((int)x, v) != (int)(x % d);
        };
        for (int64_t q = 0; q * d <= 0x7FFFFFFF; q = q < 16 ? q + 1 : q + q / 3) {
            check(q * d - 1); check(q * d); check(q * d + 1); check(q * d + d - 1);
        }
        const int64_t top = 0x7FFFFFFF / d;
        check(top * d - 1); check(top * d); check(0x7FFFFFFF); check(0x7FFFFFFE);
        for (int i = 0; i < samples; i++) {
            state ^= state << 13; state ^= state >> 7; state ^= state << 17;
            check((int64_t)(state >> 33));
        }
    }
    return wrong;
}
