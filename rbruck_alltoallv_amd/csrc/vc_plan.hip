// vc_plan.hip — turns the count tables into the work items of every launch.
//
// The reference learns the size of each incoming block from a metadata
// MPI_Sendrecv before every data round ("two-phase", src/twophase_tunable_rbruckv.cpp:110).
// With all P ranks' tables in one address space the size of a block is simply
// sendcounts[s][t] of the (s, t) it belongs to, and which (s, t) sits in a slot
// follows from the residency invariant (vc_plan_math.h).  Staging offsets (the
// reference's fixed-stride extra_buffer, :59) become exclusive prefix sums over
// the blocks that arrive in a rank's staging area in a digit phase, so the
// staging arena is compact; a second family of prefix sums numbers the work
// items (block pieces of at most VC_CHUNK bytes) so that every launch gets a
// dense list with no empty entries.
#include <cstring>

#include "vc_common.h"
#include "vc_scan.h"

#include "vc_plan_math.h"

// ---- pass 1: row-wise prefix sums ----
// Launch-per-digit execution: grid (P, regions + nl).  Rows y < regions = w + w2: staging sizes of region y,
// slot_off[(y*P + to)*P + id] = offset of the slot inside the row.  Later rows: work-item count and moved bytes of launch
// y - regions; the first of them also sums the payload and counts negative table entries.
// Forwarded execution (chain_row_tot != null, nl = 0): grid (P, regions + 1).  The region rows also sum the bytes of the
// blocks themselves (every staged block is one hop), and the last row counts the chain items of the blocks that end on
// the rank, the most pieces of any of them, the payload and the negative table entries.
// row_bytes rows: [launch or region][P], then [payload][P], then [negative entries][P], then (forwarded) [longest block][P].
__global__ __launch_bounds__(VC_THREADS) void vc_plan_rows(VcSched S, VcLaunchPack pack, const VcLaunchInfo *__restrict__ launches, int nl, VcTables T,
                                                           int64_t *__restrict__ slot_off, int64_t *__restrict__ row_tot,
                                                           int64_t *__restrict__ item_row_tot, int64_t *__restrict__ row_bytes,
                                                           int64_t *__restrict__ chain_row_tot) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int to = blockIdx.x, P = S.P;
    const int nreg = S.w + S.w2;                          // the organized region is laid out by vc_plan_org_rows
    const bool forward = chain_row_tot != nullptr;
    const int nsum = forward ? nreg : nl;                 // rows of row_bytes before the payload row
    if ((int)blockIdx.y < nreg && S.recycle) {
        // reused staging: the slots of the region in one prefix sum per hop slot in which their blocks leave again
        __shared__ int64_t family_carry[VC_RECYCLE_MAX_SLOTS];
        const int y = blockIdx.y, ns = nreg + 1, t_arrive = vc_slot_time(S, y);
        if (threadIdx.x < VC_RECYCLE_MAX_SLOTS) family_carry[threadIdx.x] = 0;
        __syncthreads();
        for (int base = 0; base < P; base += VC_THREADS) {
            const int id = base + threadIdx.x;
            int st[2] = {0, 0};
            const int64_t v = (id < P) ? vc_region_slot_size(S, T, y, to, id, nullptr, st) : 0;
            const int leaves = v ? vc_next_hop(S, st[0], st[1], y) : -1;
            for (int time = t_arrive + 1; time < ns; time++) {
                const int kd = vc_slot_time(S, time);
                int64_t total;
                const int64_t ex = vc_block_exclusive_scan(leaves == kd ? v : 0, lds, total);
                if (leaves == kd) slot_off[((int64_t)y * P + to) * P + id] = family_carry[kd] + ex;
                __syncthreads();
                if (threadIdx.x == 0) family_carry[kd] += total;
                __syncthreads();
            }
            if (id < P && !v) slot_off[((int64_t)y * P + to) * P + id] = 0;
        }
        if ((int)threadIdx.x < ns) row_tot[(int64_t)(y * ns + threadIdx.x) * P + to] = vc_slot_time(S, threadIdx.x) > t_arrive ? family_carry[threadIdx.x] : 0;
        return;
    }
    if ((int)blockIdx.y < nreg) {
        const int y = blockIdx.y;
        int64_t carry = 0, data = 0;
        for (int base0 = 0; base0 < P; base0 += 4 * VC_THREADS) {       // four chunks at a time: their table reads travel together
            int64_t v[4], len[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int id = base0 + u * VC_THREADS + threadIdx.x;
                len[u] = 0;
                v[u] = (id < P) ? vc_region_slot_size(S, T, y, to, id, &len[u]) : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int id = base0 + u * VC_THREADS + threadIdx.x;
                if (base0 + u * VC_THREADS >= P) break;
                int64_t total;
                const int64_t ex = vc_block_exclusive_scan(v[u], lds, total);
                if (id < P) slot_off[((int64_t)y * P + to) * P + id] = carry + ex;
                carry += total;
                data += len[u];
            }
        }
        if (forward) data = vc_block_sum(data, lds);
        if (threadIdx.x == 0) {
            row_tot[(int64_t)y * P + to] = carry;
            if (forward) row_bytes[(int64_t)y * P + to] = data;
        }
        return;
    }
    int64_t items = 0, bytes = 0, payload = 0, most = 0, longest = 0;
    int64_t bad = 0;                                      // entries of this rank's rows no rank could have passed
    const int L = blockIdx.y - nreg;
    if (forward) {
        // sources in chunks of VC_THREADS; the items of every tile of VC_TILE_RANKS sources (half a wavefront) are left for
        // vc_plan_bases, which turns them into the first item of every (receiver, tile) in the list's tiled order.
        // Four chunks at a time, so that the table reads of all of them travel together before the first sum needs them;
        // the checks of this rank's own rows (the loop over ids below, for launch-per-digit execution) ride along.
        const int nchunk = (P + VC_THREADS - 1) / VC_THREADS, ntile = VC_TILES(P);
        int64_t before = 0;
        for (int chunk0 = 0; chunk0 < nchunk; chunk0 += 4) {
            int64_t cnt[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int s = (chunk0 + u) * VC_THREADS + threadIdx.x;
                cnt[u] = 0;
                if (chunk0 + u >= nchunk || s >= P) continue;
                cnt[u] = vc_chain_count(S, T, s, to);
                const int expected = T.rc[(int64_t)to * P + s], sent = T.sc[(int64_t)s * P + to];
                bad += vc_pair_bad_entries(S, T, s, to);
                payload += (int64_t)expected * S.esz;
                most = cnt[u] > most ? cnt[u] : most;
                const int64_t len = (int64_t)sent * S.esz;
                longest = len > longest ? len : longest;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (chunk0 + u >= nchunk) break;
                int64_t tile = cnt[u];
#pragma unroll
                for (int o = VC_TILE_RANKS / 2; o > 0; o >>= 1) tile += __shfl_xor(tile, o, VC_TILE_RANKS);
                const int s = (chunk0 + u) * VC_THREADS + threadIdx.x;
                if (threadIdx.x % VC_TILE_RANKS == 0 && s < P) chain_row_tot[2 * (int64_t)P + (int64_t)to * ntile + s / VC_TILE_RANKS] = tile;
                before += vc_block_sum(cnt[u], lds);
            }
        }
        items = threadIdx.x == 0 ? before : 0;            // vc_block_sum below adds the lanes up
    } else {
        const VcLaunchInfo info = launches ? launches[L] : pack.info[L];     // a short launch table travels as a kernel argument
        const int nent = vc_entries_per_rank(S, info);
        for (int id = threadIdx.x; id < nent; id += VC_THREADS) {
            VcEntry e;
            if (vc_entry_block(S, info, to, id, e)) {
                const int64_t len = vc_entry_len(S, T, e);
                items += vc_chunk_count(len, vc_entry_phase(S, T, e), vc_entry_cut(S, T, e));
                bytes += len;
            }
        }
    }
    if (L == 0 && !forward)                               // forwarded execution has done this above
        for (int id = threadIdx.x; id < P; id += VC_THREADS) {
            payload += (int64_t)T.rc[(int64_t)to * P + id] * S.esz;
            bad += vc_pair_bad_entries(S, T, id, to);
        }
    items = vc_block_sum(items, lds);
    if (forward) { most = vc_block_max(most, lds); longest = vc_block_max(longest, lds); } else bytes = vc_block_sum(bytes, lds);
    if (L == 0) {
        payload = vc_block_sum(payload, lds);
        bad = vc_block_sum(bad, lds);
        // the packed receive layout is an int prefix sum of the rank's receive counts, like the reference's displacements
        if (S.packed_recv && payload > (int64_t)0x7FFFFFFF * S.esz) bad += VC_BAD_OVERFLOW;
    }
    if (threadIdx.x == 0) {
        if (forward) { chain_row_tot[to] = items; chain_row_tot[P + to] = most; row_bytes[(int64_t)(nsum + 2) * P + to] = longest; }
        else { item_row_tot[(int64_t)L * P + to] = items; row_bytes[(int64_t)L * P + to] = bytes; }
        if (L == 0) { row_bytes[(int64_t)nsum * P + to] = payload; row_bytes[(int64_t)(nsum + 1) * P + to] = bad; }
    }
}

// ---- pass 1b (S.coalesce): layout of the organized region, one workgroup per rank ----
// Scan of the run sizes over the groups, then slot_off[(w*P + to)*P + id] for every slot; row_tot[w*P + to].
__global__ __launch_bounds__(VC_THREADS) void vc_plan_org_rows(VcSched S, VcTables T, int64_t *__restrict__ slot_off,
                                                               int64_t *__restrict__ row_tot, int64_t *__restrict__ org_run_base) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int to = blockIdx.x, P = S.P, G = S.G;
    int64_t carry = 0;
    for (int base = 0; base < G; base += VC_THREADS) {
        const int g = base + threadIdx.x;
        int64_t total;
        const int64_t v = (g < G) ? vc_org_run_size(S, T, to, g) : 0;
        const int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (g < G) org_run_base[(int64_t)to * G + g] = carry + ex;
        carry += total;
    }
    const int ns = S.w + S.w2 + 1;
    if (threadIdx.x == 0) row_tot[(int64_t)(S.recycle ? ns * ns : S.w) * P + to] = carry;
    __syncthreads();                                      // org_run_base of this rank is complete (same workgroup wrote it)
    for (int id = threadIdx.x; id < P; id += VC_THREADS)
        slot_off[((int64_t)S.w * P + to) * P + id] = org_run_base[(int64_t)to * G + vc_div(id, S.dn)] + vc_org_slot_rel(S, T, to, id);
}

// ---- pass 2: prefix sums over the rows ----
// (A kernel of its own although a boundary between two kernels of one stream costs as much as the pass itself: folding it
// into pass 1 — every workgroup counts itself when its rows are written, the last one does the prefix sums — needs a
// device-wide release fence per workgroup, which on this chip writes the XCD's L2 back; measured, calls on 160 - 512 ranks
// took twice as long that way.)
// Launch-per-digit execution: grid (nl + 1).  Workgroup L < nl: item bases of launch L's rows (relative to the launch's
// first item), its item count and moved bytes.  Workgroup nl: staging row bases, staging bytes, payload bytes, negative
// table entries.  Forwarded execution (chain_row_tot != null, nl = 0): grid (2 + tile rows).  Workgroup 0 as workgroup nl above,
// and the moved bytes = payload + bytes of the staged blocks as those of launch 0; workgroup 1: chain items per receiver summed up
// (their total, the most pieces, the longest block); workgroup 2 + k: first item of every (receiver, tile of sources) of tile row k.
__global__ __launch_bounds__(VC_THREADS) void vc_plan_bases(VcSched S, int P, int w, int nreg, int nl, const int64_t *__restrict__ row_tot,
                                                            int64_t *__restrict__ row_base, const int64_t *__restrict__ item_row_tot,
                                                            int64_t *__restrict__ item_row_base, const int64_t *__restrict__ row_bytes,
                                                            int64_t *chain_row_tot, int64_t *__restrict__ chain_row_base,
                                                            int64_t *__restrict__ header, int64_t *__restrict__ header_host) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int L = blockIdx.x;
    const bool forward = chain_row_tot != nullptr, recycle = S.recycle != 0;
    const int nsum = forward ? nreg : nl;                 // rows of row_bytes before the payload row
    int64_t carry = 0, bytes = 0;
    if (forward && L >= 2) {
        // tile row L - 2: the receivers [t0, t1).  The list holds, tile row after tile row, the tiles of sources in turn and
        // inside a tile the receivers in turn: an exclusive scan over (tile of sources, receiver) of the counts vc_plan_rows
        // left, in place, started at the items of all receivers before t0.
        const int ntile = VC_TILES(P), t0 = (L - 2) * VC_TILE_RANKS, rows = (t0 + VC_TILE_RANKS < P ? t0 + VC_TILE_RANKS : P) - t0;
        int64_t *tile = chain_row_tot + 2 * (int64_t)P;
        int64_t earlier = 0;
        for (int i = threadIdx.x; i < t0; i += VC_THREADS) earlier += chain_row_tot[i];
        carry = vc_block_sum(earlier, lds);
        const int per = VC_THREADS / VC_TILE_RANKS;       // tiles of sources per pass
        for (int sb0 = 0; sb0 < ntile; sb0 += per) {
            const int sb = sb0 + threadIdx.x / VC_TILE_RANKS, row = threadIdx.x % VC_TILE_RANKS;
            const bool inside = sb < ntile && row < rows;
            int64_t total;
            const int64_t ex = vc_block_exclusive_scan(inside ? tile[(int64_t)(t0 + row) * ntile + sb] : 0, lds, total);
            if (inside) tile[(int64_t)(t0 + row) * ntile + sb] = carry + ex;
            carry += total;
        }
        return;
    }
    if (forward && L == 1) {                              // first chain item of every final receiver
        int64_t most = 0, longest = 0;
        for (int b0 = 0; b0 < P; b0 += VC_THREADS) {
            const int i = b0 + threadIdx.x;
            int64_t total;
            const int64_t ex = vc_block_exclusive_scan((i < P) ? chain_row_tot[i] : 0, lds, total);
            if (i < P) {
                chain_row_base[i] = carry + ex;
                most = chain_row_tot[P + i] > most ? chain_row_tot[P + i] : most;
                const int64_t len = row_bytes[(int64_t)(nsum + 2) * P + i];
                longest = len > longest ? len : longest;
            }
            carry += total;
        }
        most = vc_block_max(most, lds);
        longest = vc_block_max(longest, lds);
        if (threadIdx.x == 0) {
            header[2] = carry; header[VC_HEADER_MAX_PIECES] = most; header[VC_HEADER_MAX_LEN] = longest;
            if (header_host) { header_host[2] = carry; header_host[VC_HEADER_MAX_PIECES] = most; header_host[VC_HEADER_MAX_LEN] = longest; }
        }
        return;
    }
    if (L == nl && recycle) {
        // reused staging: row offsets inside every sub-region, the sizes of the sub-regions' pieces (the rows of
        // vc_recycle_rows_per_segment(P) consecutive receivers each), their places in the arena
        __shared__ int64_t piece_size[VC_RECYCLE_MAX_PAIRS * VC_RECYCLE_SEGMENTS], piece_base[VC_RECYCLE_MAX_PAIRS * VC_RECYCLE_SEGMENTS],
            hole_lo[VC_RECYCLE_MAX_HOLES], hole_hi[VC_RECYCLE_MAX_HOLES];
        const int ns = nreg + 1, nfam = ns * ns + 1, nseg = VC_RECYCLE_SEGMENTS, rps = vc_recycle_rows_per_segment(P);
        for (int f = 0; f < nfam; f++) {
            const int ka = f / ns, kd = f % ns;
            const bool used = f == ns * ns ? w > nreg : (ka < nreg && vc_slot_time(S, kd) > vc_slot_time(S, ka));
            int64_t fam_carry = 0;
            if (used)
                for (int b0 = 0; b0 < P; b0 += VC_THREADS) {
                    const int i = b0 + threadIdx.x;
                    int64_t total;
                    const int64_t ex = vc_block_exclusive_scan((i < P) ? row_tot[(int64_t)f * P + i] : 0, lds, total);
                    if (i < P) {
                        row_base[(int64_t)f * P + i] = fam_carry + ex;
                        if (i % rps == 0) piece_base[f * nseg + i / rps] = fam_carry + ex;      // where the piece starts (for now)
                    }
                    fam_carry += total;
                }
            __syncthreads();
            if ((int)threadIdx.x < nseg) {
                const int g = threadIdx.x;
                const bool has = used && g * rps < P, more = g + 1 < nseg && (g + 1) * rps < P;
                piece_size[f * nseg + g] = has ? (more ? piece_base[f * nseg + g + 1] : fam_carry) - piece_base[f * nseg + g] : 0;
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) carry = vc_allocate_staging(S, piece_size, piece_base, hole_lo, hole_hi);
        __syncthreads();
        for (int64_t i = threadIdx.x; i < (int64_t)nfam * P; i += VC_THREADS) {
            const int f = (int)(i / P), g = (int)(i % P) / rps;
            int64_t start = 0;                            // offset of the piece's first row inside the sub-region
            for (int k = 0; k < g; k++) start += piece_size[f * nseg + k];
            if (piece_size[f * nseg + g] > 0) row_base[i] += piece_base[f * nseg + g] - start;
        }
        int64_t bad = 0;
        for (int i = threadIdx.x; i < P; i += VC_THREADS) { bytes += row_bytes[(int64_t)nsum * P + i]; bad += row_bytes[(int64_t)(nsum + 1) * P + i]; }
        bytes = vc_block_sum(bytes, lds);
        bad = vc_block_sum(bad, lds);
        if (threadIdx.x == 0) {
            header[0] = carry; header[1] = bytes; header[VC_HEADER_BAD] = bad;
            if (header_host) { header_host[0] = carry; header_host[1] = bytes; header_host[VC_HEADER_BAD] = bad; }
        }
        return;
    }
    if (L == nl) {
        const int64_t nrows = (int64_t)w * P;                 // w = number of staging regions
        for (int64_t b0 = 0; b0 < nrows; b0 += VC_THREADS) {
            const int64_t i = b0 + threadIdx.x;
            int64_t total;
            const int64_t v = (i < nrows) ? row_tot[i] : 0;
            const int64_t ex = vc_block_exclusive_scan(v, lds, total);
            if (i < nrows) row_base[i] = carry + ex;
            carry += total;
        }
        int64_t bad = 0, staged = 0;
        for (int i = threadIdx.x; i < P; i += VC_THREADS) { bytes += row_bytes[(int64_t)nsum * P + i]; bad += row_bytes[(int64_t)(nsum + 1) * P + i]; }
        if (forward)
            for (int64_t i = threadIdx.x; i < (int64_t)nreg * P; i += VC_THREADS) staged += row_bytes[i];
        bytes = vc_block_sum(bytes, lds);
        bad = vc_block_sum(bad, lds);
        if (forward) staged = vc_block_sum(staged, lds);
        if (threadIdx.x == 0) {
            header[0] = carry; header[1] = bytes; header[VC_HEADER_BAD] = bad;
            if (header_host) { header_host[0] = carry; header_host[1] = bytes; header_host[VC_HEADER_BAD] = bad; }
            if (forward) {                                // every staged block is one hop, every block's last hop ends in recvbuf
                header[VC_HEADER_FIXED] = bytes + staged;
                if (header_host) header_host[VC_HEADER_FIXED] = bytes + staged;
            }
        }
        return;
    }
    for (int b0 = 0; b0 < P; b0 += VC_THREADS) {
        const int i = b0 + threadIdx.x;
        int64_t total;
        const int64_t v = (i < P) ? item_row_tot[(int64_t)L * P + i] : 0;
        const int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (i < P) item_row_base[(int64_t)L * P + i] = carry + ex;
        carry += total;
        bytes += (i < P) ? row_bytes[(int64_t)L * P + i] : 0;
    }
    bytes = vc_block_sum(bytes, lds);
    if (threadIdx.x == 0) {
        header[VC_HEADER_FIXED + L] = bytes; header[VC_HEADER_FIXED + nl + L] = carry;
        if (header_host) { header_host[VC_HEADER_FIXED + L] = bytes; header_host[VC_HEADER_FIXED + nl + L] = carry; }      // pinned host memory: no copy back
    }
}

// ---- pass 3: the work items ----
// grid (P, nl, Z).  Repeats the row scan of pass 1 to place every block's pieces; Z workgroups share a receiver's entries
// when there are few ranks (their blocks are then huge and have many pieces).
__global__ __launch_bounds__(VC_THREADS) void vc_plan_emit(VcSched S, VcLaunchPack pack, const VcLaunchInfo *__restrict__ launches, VcTables T,
                                                           const int64_t *__restrict__ slot_off, const int64_t *__restrict__ row_base,
                                                           const int64_t *__restrict__ item_row_base, const int64_t *__restrict__ header,
                                                           int nl, VcDesc *__restrict__ items) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int to = blockIdx.x, L = blockIdx.y, P = S.P;
    const VcLaunchInfo info = launches ? launches[L] : pack.info[L];
    int64_t first = 0;                                    // items of the launches before this one
    for (int k = threadIdx.x; k < L; k += VC_THREADS) first += header[VC_HEADER_FIXED + nl + k];
    first = vc_block_sum(first, lds);
    int64_t carry = first + item_row_base[(int64_t)L * P + to];
    // copies of many pieces are written by the whole workgroup: their pieces are numbered by a second prefix sum and
    // every lane takes every 256th piece, finding the copy it belongs to by bisection
    __shared__ VcDesc big_whole[VC_THREADS];
    __shared__ int64_t big_at[VC_THREADS], big_pre[VC_THREADS];
    __shared__ int big_phase[VC_THREADS], big_cut[VC_THREADS];
    const int nent_all = vc_entries_per_rank(S, info);
    // workgroup (to, L, z) writes the z-th slice of the receiver's entries; the items of the slices before it come first
    const int per = (nent_all + (int)gridDim.z - 1) / (int)gridDim.z;
    const int e_lo = (int)blockIdx.z * per < nent_all ? (int)blockIdx.z * per : nent_all;
    const int nent = e_lo + per < nent_all ? e_lo + per : nent_all;
    int64_t before = 0;
    for (int id = threadIdx.x; id < e_lo; id += VC_THREADS) {
        VcEntry e;
        if (vc_entry_block(S, info, to, id, e))
            before += vc_chunk_count(vc_entry_len(S, T, e), vc_entry_phase(S, T, e), vc_entry_cut(S, T, e));
    }
    carry += vc_block_sum(before, lds);
    for (int base = e_lo; base < nent; base += VC_THREADS) {
        const int id = base + threadIdx.x;
        VcEntry e;
        const bool active = id < nent && vc_entry_block(S, info, to, id, e);
        const int64_t len = active ? vc_entry_len(S, T, e) : 0;
        const int phase = active ? vc_entry_phase(S, T, e) : 0, cut = active ? vc_entry_cut(S, T, e) : 0;
        const int64_t cnt = vc_chunk_count(len, phase, cut);
        int64_t total;
        const int64_t at = carry + vc_block_exclusive_scan(cnt, lds, total);
        const bool big = cnt > 4;
        if (cnt) {
            const VcDesc whole = vc_entry_desc(S, T, slot_off, row_base, e, to);
            if (!big)
                for (int64_t c = 0; c < cnt; c++) items[at + c] = vc_chunk_of(whole, c, phase, cut);
            else { big_whole[threadIdx.x] = whole; big_at[threadIdx.x] = at; big_phase[threadIdx.x] = phase; big_cut[threadIdx.x] = cut; }
        }
        if (__syncthreads_or(big)) {
            int64_t btotal;
            big_pre[threadIdx.x] = vc_block_exclusive_scan(big ? cnt : 0, lds, btotal);
            __syncthreads();
            for (int64_t q = threadIdx.x; q < btotal; q += VC_THREADS) {
                int lo = 0, hi = VC_THREADS - 1;              // last lane whose pieces start at or before q
                while (lo < hi) {
                    const int mid = (lo + hi + 1) >> 1;
                    if (big_pre[mid] <= q) lo = mid; else hi = mid - 1;
                }
                const int64_t c = q - big_pre[lo];
                items[big_at[lo] + c] = vc_chunk_of(big_whole[lo], c, big_phase[lo], big_cut[lo]);
            }
            __syncthreads();                              // the lists are reused by the next round
        }
        carry += total;
    }
}

// Workgroups that share one receiver's entries when items are emitted: one per ~2048 items of an average row, so that
// a few ranks with huge blocks (many pieces each) still fill the chip, and small problems stay one workgroup per row.
static int vc_emit_slices(int64_t nitems, int64_t rows) {
    const int64_t per_row = nitems / (rows > 0 ? rows : 1);
    const int64_t z = (per_row + 2047) / 2048;
    return (int)(z < 1 ? 1 : (z > 16 ? 16 : z));
}

static VcLaunchPack vc_pack_launches(const VcLaunchInfo *host, int nl) {
    VcLaunchPack pack;
    memset(&pack, 0, sizeof pack);
    for (int k = 0; k < nl && k < VC_LAUNCH_PACK; k++) pack.info[k] = host[k];
    return pack;
}

hipError_t vc_launch_plan_sizes(const VcSched &S, const VcLaunchInfo *launches_host, const VcLaunchInfo *launches_dev, int nlaunch,
                                VcTables T, int64_t *slot_off,
                                int64_t *row_tot, int64_t *row_base, int64_t *org_run_base, int64_t *item_row_tot,
                                int64_t *item_row_base, int64_t *row_bytes, int64_t *chain_row_tot, int64_t *chain_row_base,
                                int64_t *header, int64_t *header_host, hipStream_t st) {
    const bool forward = chain_row_tot != nullptr;
    const int nl = forward ? 0 : nlaunch;                 // forwarded execution has no use for the per-launch rows
    const int nreg = S.w + S.w2;
    hipLaunchKernelGGL(vc_plan_rows, dim3(S.P, nreg + (forward ? 1 : nl)), dim3(VC_THREADS), 0, st, S,
                       vc_pack_launches(launches_host, nl), nl <= VC_LAUNCH_PACK ? nullptr : launches_dev, nl, T, slot_off,
                       row_tot, item_row_tot, row_bytes, chain_row_tot);
    if (S.coalesce)
        hipLaunchKernelGGL(vc_plan_org_rows, dim3(S.P), dim3(VC_THREADS), 0, st, S, T, slot_off, row_tot, org_run_base);
    hipLaunchKernelGGL(vc_plan_bases, dim3(forward ? 2 + VC_TILES(S.P) : nl + 1), dim3(VC_THREADS), 0, st, S, S.P, vc_regions(S), nreg, nl, row_tot, row_base,
                       item_row_tot, item_row_base, row_bytes, chain_row_tot, chain_row_base, header, header_host);
    return hipGetLastError();
}

hipError_t vc_launch_plan_emit(const VcSched &S, const VcLaunchInfo *launches_host, const VcLaunchInfo *launches_dev, int nlaunch,
                               VcTables T, const int64_t *slot_off,
                               const int64_t *row_base, const int64_t *item_row_base, const int64_t *header, VcDesc *items,
                               int64_t nitems, hipStream_t st) {
    const int slices = vc_emit_slices(nitems, (int64_t)S.P * nlaunch);
    hipLaunchKernelGGL(vc_plan_emit, dim3(S.P, nlaunch, slices), dim3(VC_THREADS), 0, st, S, vc_pack_launches(launches_host, nlaunch),
                       nlaunch <= VC_LAUNCH_PACK ? nullptr : launches_dev, T, slot_off, row_base, item_row_base, header, nlaunch, items);
    return hipGetLastError();
}

// ---- forwarded execution ----
// grid (P, chunks x Z): the chain items of the blocks that end on rank t.  The list is ordered in tiles of VC_TILE_RANKS
// receivers x VC_TILE_RANKS sources, receiver by receiver inside a tile (vc_plan_bases has left the first item of every
// (receiver, tile of sources)); the sources come in chunks of VC_THREADS, and Z workgroups share a chunk (each a whole number
// of tiles) when there are few ranks, which would otherwise leave most of the chip idle: the kernel is a chain of dependent
// table reads per workgroup, and one workgroup per compute unit hides none of them.  Big blocks are written by the whole
// workgroup as in vc_plan_emit.
__global__ __launch_bounds__(VC_THREADS) void vc_chain_emit(VcSched S, VcTables T, const int64_t *__restrict__ slot_off,
                                                            const int64_t *__restrict__ row_base,
                                                            const int64_t *__restrict__ chain_tile_base, int slices,
                                                            int64_t *__restrict__ items, const int64_t *__restrict__ header,
                                                            int64_t cap_items) {
    // a launch that was enqueued before the host had seen the plan: nothing is written unless the tables are in order
    // (their entries could point anywhere) and the list has room for every item
    if (header && (header[VC_HEADER_BAD] != 0 || header[2] > cap_items)) return;
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    __shared__ int64_t big_at[VC_THREADS], big_pre[VC_THREADS];
    // a block of many pieces keeps its route here while the whole workgroup writes its items (routes of more hops than
    // fit are evaluated again for every piece)
    const int VC_ROUTE_CACHE = 6;
    __shared__ int64_t big_dst[VC_THREADS][VC_ROUTE_CACHE];
    __shared__ int big_nhop[VC_THREADS];
    const int t = blockIdx.x, P = S.P;
    const int stride = VC_CHAIN_HEAD + vc_hop_slots(S);
    const bool cached = vc_hop_slots(S) <= VC_ROUTE_CACHE;
    const int chunk = (int)blockIdx.y / slices, z = (int)blockIdx.y % slices;
    const int c_lo = chunk * VC_THREADS, c_hi = c_lo + VC_THREADS < P ? c_lo + VC_THREADS : P;
    const int per = ((c_hi - c_lo + slices - 1) / slices + VC_TILE_RANKS - 1) / VC_TILE_RANKS * VC_TILE_RANKS;      // whole tiles
    const int s_lo = c_lo + z * per < c_hi ? c_lo + z * per : c_hi, s_hi = s_lo + per < c_hi ? s_lo + per : c_hi;
    const int s = s_lo + threadIdx.x;                     // one source per lane: a slice has at most VC_THREADS of them
    const int64_t cnt = s < s_hi ? vc_chain_count(S, T, s, t) : 0;
    // the block's first item: the first item of its (receiver, tile of sources) + the items of the tile's earlier sources
    int64_t upto = cnt;
#pragma unroll
    for (int o = 1; o < VC_TILE_RANKS; o <<= 1) {
        const int64_t below = __shfl_up(upto, o, VC_TILE_RANKS);
        if ((int)(threadIdx.x % VC_TILE_RANKS) >= o) upto += below;
    }
    const int64_t at = (s < s_hi ? chain_tile_base[(int64_t)t * VC_TILES(P) + s / VC_TILE_RANKS] : 0) + upto - cnt;
    const bool big = cnt > 4;
    if (cached && cnt > 0) {
        // the block's route once, in registers (hop slot k in d[k], statically indexed; its table reads go out together); the
        // pieces of a block of few pieces are then arithmetic and stores only — evaluating the route again for every piece
        // was a chain of dependent reads per item
        int64_t d[VC_ROUTE_CACHE];
        unsigned moves = 0;
        const int nslots = vc_hop_slots(S);
#pragma unroll
        for (int k = 0; k < VC_ROUTE_CACHE; k++) {
            d[k] = 0;
            if (k < nslots && vc_block_hop(S, T, slot_off, row_base, s, t, k, d[k])) moves |= 1u << k;
        }
        const int nhop = __popc(moves);
        if (!big) {
            const int64_t src = VC_SPACE_SEND | vc_send_offset(S, T, s, t), len = (int64_t)T.sc[(int64_t)s * P + t] * S.esz;
            const int phase = vc_phase(S, T, s, t), cut = vc_chain_cut(S, T, s, t);
            for (int64_t c = 0; c < cnt; c++) {
                int64_t lo, hi;
                vc_piece_range(len, phase, cut, c, lo, hi);
                int64_t *item = items + (at + c) * stride;
                item[VC_CHAIN_SRC] = src + lo;
                item[VC_CHAIN_LEN] = hi - lo;
                item[VC_CHAIN_NHOP] = nhop;
                int n = 0;
#pragma unroll
                for (int k = 0; k < VC_ROUTE_CACHE; k++)
                    if (moves >> k & 1) item[VC_CHAIN_HEAD + n++] = d[k] + lo;
            }
        } else {
            big_at[threadIdx.x] = at;
            big_nhop[threadIdx.x] = nhop;
            int n = 0;
#pragma unroll
            for (int k = 0; k < VC_ROUTE_CACHE; k++)
                if (moves >> k & 1) big_dst[threadIdx.x][n++] = d[k];
        }
    } else if (!big) {
        for (int64_t c = 0; c < cnt; c++) vc_chain_item(S, T, slot_off, row_base, s, t, c, items + (at + c) * stride);
    } else {
        big_at[threadIdx.x] = at;
    }
    if (__syncthreads_or(big)) {
        int64_t btotal;
        big_pre[threadIdx.x] = vc_block_exclusive_scan(big ? cnt : 0, lds, btotal);
        __syncthreads();
        for (int64_t q = threadIdx.x; q < btotal; q += VC_THREADS) {
            int lo = 0, hi = VC_THREADS - 1;              // last lane whose pieces start at or before q
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (big_pre[mid] <= q) lo = mid; else hi = mid - 1;
            }
            const int64_t c = q - big_pre[lo];
            const int sb = s_lo + lo;
            if (cached)
                vc_chain_piece(VC_SPACE_SEND | vc_send_offset(S, T, sb, t), (int64_t)T.sc[(int64_t)sb * P + t] * S.esz, vc_phase(S, T, sb, t),
                               vc_chain_cut(S, T, sb, t), c, big_dst[lo], big_nhop[lo], items + (big_at[lo] + c) * stride);
            else
                vc_chain_item(S, T, slot_off, row_base, sb, t, c, items + (big_at[lo] + c) * stride);
        }
    }
}

hipError_t vc_launch_chain_plan(const VcSched &S, VcTables T, const int64_t *slot_off, const int64_t *row_base,
                                const int64_t *chain_tile_base, int64_t *items, int64_t nitems, hipStream_t st, const int64_t *header,
                                int64_t cap_items) {
    const int nchunk = (S.P + VC_THREADS - 1) / VC_THREADS;
    // at least ~1024 workgroups (four per compute unit), each a whole number of tiles of sources
    int slices = nchunk > 1 ? 1 : vc_emit_slices(nitems, S.P);
    if (nchunk == 1)
        while (slices < 8 && (int64_t)S.P * slices < 1024 && S.P / (slices * 2) >= VC_TILE_RANKS) slices *= 2;
    hipLaunchKernelGGL(vc_chain_emit, dim3(S.P, nchunk * slices), dim3(VC_THREADS), 0, st, S, T, slot_off, row_base, chain_tile_base,
                       slices, items, header, cap_items);
    return hipGetLastError();
}

// ---- route inspection: bytes sent from every rank to every rank in one launch ----
__global__ __launch_bounds__(VC_THREADS) void vc_traffic_kernel(const VcDesc *__restrict__ desc, int64_t ndesc, int64_t *__restrict__ matrix, int P) {
    int64_t i = (int64_t)blockIdx.x * VC_THREADS + threadIdx.x;
    if (i >= ndesc) return;
    VcDesc d = desc[i];
    if (d.len > 0 && d.from >= 0)
        atomicAdd((unsigned long long *)&matrix[(int64_t)d.from * P + d.to], (unsigned long long)d.len);
}

hipError_t vc_launch_traffic(const VcDesc *desc, int64_t ndesc, int64_t *matrix, int P, hipStream_t st) {
    // a dispatch counts its grid in work-items in 32 bits: at most 2^24 - 1 workgroups of VC_THREADS per launch
    const int64_t step = (((int64_t)1 << 24) - 1) * VC_THREADS;
    for (int64_t done = 0; done < ndesc; done += step) {
        const int64_t now = ndesc - done < step ? ndesc - done : step;
        hipLaunchKernelGGL(vc_traffic_kernel, dim3((unsigned)((now + VC_THREADS - 1) / VC_THREADS)), dim3(VC_THREADS), 0, st, desc + done,
                           now, matrix, P);
    }
    return hipGetLastError();
}
