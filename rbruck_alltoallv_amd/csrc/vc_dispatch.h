// vc_dispatch.h — which kernel a call gets: every threshold and the one function that applies them.
//
// Host code only, no device state: the library calls vc_dispatch() from every entry point (blocking calls, the _async
// twins, the entry point that allocates nothing), and the CPU tests compile this header to pin the decision table.
//
// The choices, measured on MI355X with blocking calls (microseconds per call unless noted):
//  * through the work-item list (lanes = 0): a planning kernel writes one item per block piece after the host has learnt
//    how many there are.  Right for long blocks; the list and the wait for its size cost more than they save below.
//  * without the list, a quarter of a wavefront per pair of ranks: blocks of a few hundred bytes, any number of ranks.
//    Average piece below 768 B: 26 - 30 at 64 ranks (through the list 42), 42 - 73 at 256 (51 - 88), 300 - 900 at 1024
//    (330 - 990); at 1 KiB the two ways are even.  On at most 128 ranks the alternative is a workgroup per pair, and the
//    quarter wins only further down: never up to 32 ranks (1024 pairs leave room for as many workgroups: 26 either way,
//    the workgroup up to 1.3 x faster on KiB blocks), below 1.75 KiB up to 90 ranks (64 ranks: 27 - 33 against 34 - 38),
//    below 3 KiB above (128 ranks: 30 - 70 against 64 - 84).
//  * ... a batch of 16 - 64 pairs per wavefront when the blocks are so short that working out the routes costs more than
//    moving the bytes: on 192 - 2048 ranks 5 - 40 % faster than the quarter up to an average block of 256 bytes, even at
//    512, 3 - 16 % slower beyond.  Not on at most 128 ranks, where batches would leave most of the chip without a wavefront.
//  * ... a wavefront (average piece below 3 KiB) or a workgroup per pair: at most 128 ranks and 32768 pieces (26 - 42
//    against 40 - 57 through the list at 16 and 64 ranks with blocks up to 8 KB, 31 - 77 against 48 - 92 up to 32 KB; a few
//    per cent at 128 ranks; at 256 ranks the list wins).
//  * never without the list after a call with a block of more than 8 (quarter, batch) / 16 (wavefront, workgroup) pieces:
//    one group of lanes moves the pieces of a block in turn.
//  * on fixed-stride staging in ONE launch (stride > 0): the reference's own staging layout, every slot as long as the
//    longest block (src/twophase_tunable_rbruckv.cpp:59), makes slot addresses closed forms, so the call needs no planner
//    at all.  64 ranks with blocks of 0 - 4 KiB 41 -> 24.6; 128 ranks, 0 - 512 B: 41 -> 25.6; 160 ranks: 31 - 42 -> 26 - 34;
//    192 ranks: 31 - 50 -> 30 - 42; but 256 ranks 34 - 68 -> 44 - 68 and 384 ranks 2 x slower (the atomics of the totals
//    and the arena grow with the square of the ranks): only up to 192 ranks and 256 MiB of arena.
#pragma once

#include "vc_common.h"
#include "vc_plan_math.h"
#include "vc_scan.h"

#define VC_LISTLESS_MAX_PAIRS 16384           // "small communicator": at most 128 ranks
#define VC_LISTLESS_MAX_ITEMS 32768           // pieces of a call for a wavefront or a workgroup per pair
#define VC_LISTLESS_MAX_PIECES 8              // pieces of one block: quarter of a wavefront per pair, batches
#define VC_LISTLESS_WG_MAX_PIECES 16          // pieces of one block: wavefront or workgroup per pair
#define VC_LISTLESS_QUARTER_BELOW 768         // average piece below which pairs get a quarter of a wavefront, more than 128 ranks
#define VC_LISTLESS_BATCH_BELOW 384           // average piece below which a wavefront takes a batch of pairs
#define VC_LISTLESS_WAVE_BELOW 3072           // average piece below which a pair gets a wavefront instead of a workgroup
#define VC_LISTLESS_MAX_AVERAGE 4096          // a call the short-block kernels were chosen for must stay below this average
#define VC_STRIDED_MAX_BYTES ((int64_t)256 << 20)
#define VC_STRIDED_MAX_PAIRS 36864            // 192 ranks
// list-driven copy kernels: lanes per work item by the average piece of the launch
#define VC_ITEM_QUARTER_BELOW 448
#define VC_ITEM_WAVE_BELOW 3072

// What the last forwarded call on a communicator looked like: the guess about the next one.
struct VcHint {
    int valid;
    int64_t items;        // block pieces
    int64_t payload;      // bytes
    int64_t max_pieces;   // most pieces of one block
    int64_t max_len;      // longest block, bytes
};

// Who asks.  A blocking call may go through the list (it can wait for the list's size in mid-call); the _async twins and
// the entry point that allocates nothing enqueue everything at once and always run without it.
#define VC_CALL_BLOCKING 0
#define VC_CALL_LISTLESS_ONLY 1

struct VcDispatch {
    int lanes;               // 0: through the work-item list; else lanes per pair of ranks of the listless copy kernel:
                             // VC_THREADS, VC_WAVE, VC_QUARTER, or VC_BATCHED (a batch of pairs per wavefront)
    int stride;              // > 0: first try one launch on fixed-stride staging with slots of this many bytes ...
    int stride_lanes;        // ... with this many lanes per pair (the batches come without the totals: a quarter of a wavefront)
    VcListlessGuard guard;   // what the call must look like for the listless kernel to move anything, checked on the device
                             // against the plan (the hint is only a guess); stage_cap is the caller's to fill in
};

VC_HD int64_t vc_small_quarter_below(int64_t pairs) { return pairs <= 1024 ? 0 : (pairs < 8192 ? 1792 : 3072); }

// mode: vc_comm_set_forwarding (0 launch per digit, 1 the library's choice, 2 the list, 3 / 4 / 5 listless with a workgroup / a
// quarter of a wavefront per pair / batches).  S: the call's schedule (ranks, digits, whether it has an organized region).
inline VcDispatch vc_dispatch(int mode, int call_kind, const VcHint &h, const VcSched &S) {
    VcDispatch d = {0, 0, 0, {0, 0, 0, 0, 0}};
    if (mode == 3) { d.lanes = VC_THREADS; return d; }
    if (mode == 4) { d.lanes = VC_QUARTER; return d; }
    if (mode == 5) { d.lanes = VC_BATCHED; return d; }
    const bool listless_only = call_kind == VC_CALL_LISTLESS_ONLY;
    if (!listless_only && mode != 1) return d;            // per digit, or the list was asked for
    const int64_t pairs = (int64_t)S.P * S.P;
    const bool small_comm = pairs <= VC_LISTLESS_MAX_PAIRS;
    const int64_t average = h.payload / (h.items > 0 ? h.items : 1);
    const bool short_blocks = h.valid && h.max_pieces <= VC_LISTLESS_MAX_PIECES &&
                              average < (small_comm ? vc_small_quarter_below(pairs) : VC_LISTLESS_QUARTER_BELOW);
    if (short_blocks)
        d.lanes = !small_comm && average < VC_LISTLESS_BATCH_BELOW ? VC_BATCHED : VC_QUARTER;
    else if (listless_only)
        d.lanes = VC_THREADS;
    else if (h.valid && small_comm && h.max_pieces <= VC_LISTLESS_WG_MAX_PIECES && h.items <= VC_LISTLESS_MAX_ITEMS)
        d.lanes = average < VC_LISTLESS_WAVE_BELOW ? VC_WAVE : VC_THREADS;
    else
        return d;                                         // no hint yet, or long blocks: the list
    if (listless_only) return d;                          // nothing to fall back to: whatever the call turns out to be, it runs
    // the hint may be wrong about this call: the kernel leaves a call of another kind alone and the host takes the list
    const bool quarter = d.lanes == VC_QUARTER || d.lanes == VC_BATCHED;
    d.guard.max_pieces = quarter ? VC_LISTLESS_MAX_PIECES : VC_LISTLESS_WG_MAX_PIECES;
    d.guard.max_items = quarter ? 0 : VC_LISTLESS_MAX_ITEMS;
    d.guard.max_average = quarter ? VC_LISTLESS_MAX_AVERAGE : 0;
    // one launch on fixed-stride staging: the stride from the last call's longest block, at any cache-line phase
    if (!S.coalesce && vc_hop_slots(S) <= VC_MAX_HOP_SLOTS && pairs <= VC_STRIDED_MAX_PAIRS) {
        const int64_t stride = (h.max_len + 2 * VC_LINE - 1) & ~(int64_t)(VC_LINE - 1);
        VcSched strided = S;
        strided.stride = (int)stride;
        if (stride <= 0x7FFFFF80 && vc_strided_stage_bytes(strided) <= VC_STRIDED_MAX_BYTES) {
            d.stride = (int)stride;
            d.stride_lanes = d.lanes == VC_BATCHED ? VC_QUARTER : d.lanes;
            d.guard.max_len = stride - VC_LINE + 1;
        }
    }
    return d;
}

// Lanes per work item of the list-driven copy kernels, from the average piece of the launch.  Short pieces leave most of a
// workgroup idle, and what bounds the launch is then the number of items in flight: a wavefront per item keeps four times as
// many as a workgroup, a quarter of a wavefront sixteen times.  Measured on 1 Mi items (1024 ranks, times of the copy kernel,
// workgroup / wavefront / quarter): pieces uniform in 0..16 B 830 / 269 / 67 us, 0..256 B 882 / 351 / 189, 0..1 KiB
// 926 / 455 / 431, 0..2 KiB 1105 / 693 / 770, 0..4 KiB 1449 / 1311 / 1462; around 4 KiB and above the workgroup is 5 - 8 %
// faster than the wavefront.
VC_HD int vc_lanes_for_items(int64_t bytes, int64_t items) {
    if (items <= 0) return VC_THREADS;
    const int64_t average = bytes / items;
    return average < VC_ITEM_QUARTER_BELOW ? VC_QUARTER : (average < VC_ITEM_WAVE_BELOW ? VC_WAVE : VC_THREADS);
}

// Pairs per wavefront of the batched listless kernel, and groups of four items in a row per wavefront of the quarter kernels:
// as many as leave every SIMD of the chip a few wavefronts.
VC_HD int vc_batch_pairs(int64_t pairs) { return pairs >= ((int64_t)1 << 19) ? 64 : (pairs >= ((int64_t)1 << 17) ? 32 : 16); }
VC_HD int vc_quarter_rounds(int64_t items) { return items >= ((int64_t)1 << 19) ? 4 : (items >= ((int64_t)1 << 17) ? 2 : 1); }
