// vc_copy_variants.hip — A/B measurements behind the shape of the forwarded copy kernel (vc_copy_chains_kernel<256>).
//
// The program builds the chain items of benchmark configuration 4 on the host (TTPL_BT_alltoallv, 1024 ranks, 32 per
// node, r = 32, 1-byte elements, counts ~ Normal(4096, 1024): one read from sendbuf, one write into the staging slot of the
// intermediate holder, one write into recvbuf; src/twophase_twolayer_rbruck.cpp:334-343,368-377 are the pack / unpack
// memcpys this replaces) in the order the library's planner writes them (tiles of VC_TILE_RANKS receivers x VC_TILE_RANKS
// sources), runs the library's own kernel on them (this file includes csrc/vc_copy.hip, so the first row IS the product
// kernel), then every variant that was tried against it, other orders of the list among them, and the contiguous copies
// that bound them.  Every variant's receive and staging arenas are compared with the product kernel's, vector by vector.
//
//   vc_copy_variants [reps]        (default 7; the best of `reps` launches is printed)
//
// Under rocprofv3 every variant is a kernel of its own name (a template instance), so one --kernel-trace / --pmc pass
// gives the per-variant rows.
#include "../csrc/vc_copy.hip"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#define CK(x)                                                                              \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) {                                                            \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
            fflush(stdout);                                                                \
            exit(1);                                                                       \
        }                                                                                  \
    } while (0)

// items of this program: VC_CHAIN_HEAD words + two hop slots
#define ITEM_WORDS (VC_CHAIN_HEAD + 2)

__device__ __forceinline__ vc_u32x4 load16_aligned(const char *p) { return __builtin_nontemporal_load(reinterpret_cast<const vc_u32x4 *>(p)); }

// What a lane holds of one piece between its loads and its stores (the window of vc_forward_piece<256>).
struct PieceRegs {
    vc_u32x4 v[2];
    bool has[2];
    int64_t edge, w;
    char edge_byte;
};

// ALIGNED = false: the library's loads (16 bytes from any byte address).  ALIGNED = true: every lane loads the 16-byte
// aligned vector at or below its source address, takes the next aligned vector from the lane above it (DPP wave_shl:1; lane
// 63 loads it), and shifts the two into place with v_alignbyte_b32: no load the L1 has to split.
template <bool ALIGNED>
__device__ __forceinline__ void piece_load(const char *src, int64_t len, const char *dst, PieceRegs &R) {
    const int t = threadIdx.x;
    const int64_t w = (int64_t)((uintptr_t)dst & (VC_LINE - 1));
    R.w = w;
    const int64_t first_full = (w + 15) >> 4, end_full = (w + len) >> 4;
    const char *sw = src - w;
    if (!ALIGNED) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int64_t j = t + i * VC_THREADS;
            R.has[i] = (i > 0 || j >= first_full) && j < end_full;
            if (R.has[i]) R.v[i] = vc_load16(sw + (j << 4));
        }
    } else {
        const unsigned delta = (unsigned)((uintptr_t)sw & 15);
        const char *sa = sw - delta;
        const unsigned q = delta >> 2, s = delta & 3;
        const int lane = t & (VC_WAVE - 1);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int64_t j = t + i * VC_THREADS;
            R.has[i] = (i > 0 || j >= first_full) && j < end_full;
            const bool has_prev = j - 1 >= first_full && j - 1 < end_full;
            vc_u32x4 a = {0, 0, 0, 0};
            if (R.has[i] || (delta != 0 && has_prev)) a = load16_aligned(sa + (j << 4));
            vc_u32x4 b;
            b.x = __builtin_amdgcn_update_dpp(0u, a.x, 0x130, 0xf, 0xf, false);      // wave_shl:1: lane l reads lane l + 1
            b.y = __builtin_amdgcn_update_dpp(0u, a.y, 0x130, 0xf, 0xf, false);
            b.z = __builtin_amdgcn_update_dpp(0u, a.z, 0x130, 0xf, 0xf, false);
            b.w = __builtin_amdgcn_update_dpp(0u, a.w, 0x130, 0xf, 0xf, false);
            if (lane == VC_WAVE - 1 && delta != 0 && R.has[i]) b = load16_aligned(sa + ((j + 1) << 4));
            const unsigned x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            vc_u32x4 o;
            switch (q) {
            case 0: o.x = __builtin_amdgcn_alignbyte(x[1], x[0], s); o.y = __builtin_amdgcn_alignbyte(x[2], x[1], s);
                    o.z = __builtin_amdgcn_alignbyte(x[3], x[2], s); o.w = __builtin_amdgcn_alignbyte(x[4], x[3], s); break;
            case 1: o.x = __builtin_amdgcn_alignbyte(x[2], x[1], s); o.y = __builtin_amdgcn_alignbyte(x[3], x[2], s);
                    o.z = __builtin_amdgcn_alignbyte(x[4], x[3], s); o.w = __builtin_amdgcn_alignbyte(x[5], x[4], s); break;
            case 2: o.x = __builtin_amdgcn_alignbyte(x[3], x[2], s); o.y = __builtin_amdgcn_alignbyte(x[4], x[3], s);
                    o.z = __builtin_amdgcn_alignbyte(x[5], x[4], s); o.w = __builtin_amdgcn_alignbyte(x[6], x[5], s); break;
            default: o.x = __builtin_amdgcn_alignbyte(x[4], x[3], s); o.y = __builtin_amdgcn_alignbyte(x[5], x[4], s);
                     o.z = __builtin_amdgcn_alignbyte(x[6], x[5], s); o.w = __builtin_amdgcn_alignbyte(x[7], x[6], s); break;
            }
            R.v[i] = o;
        }
    }
    int64_t head = (first_full << 4) - w;
    if (head > len) head = len;
    int64_t done = (end_full << 4) - w;
    if (done < head) done = head;
    R.edge = t < 16 ? (t < head ? t : -1) : (t < 32 && done + (t - 16) < len ? done + (t - 16) : -1);
    R.edge_byte = 0;
    if (R.edge >= 0) R.edge_byte = src[R.edge];
}

__device__ __forceinline__ void piece_store(char *dst, const PieceRegs &R) {
    const int t = threadIdx.x;
    char *dw = dst - R.w;
    if (R.edge >= 0) dst[R.edge] = R.edge_byte;
#pragma unroll
    for (int i = 0; i < 2; i++)
        if (R.has[i]) vc_store16(dw + ((int64_t)(t + i * VC_THREADS) << 4), R.v[i]);
}

// M      items in a row per workgroup (1: the library's shape)
// PIPE   M > 1: the loads of item m + 1 go out before the stores of item m (two register sets); else all loads first
// ALIGNED see piece_load
// AHEAD  > 0: lane 0 of every workgroup touches the item AHEAD workgroups further down its XCD's range, so that the
//        item's cache line is in the L2 when that workgroup starts (the value is looked at after the stores only)
// WHOLE  M = 1: all five words of the item are fetched in one scalar round trip before anything is decided from them
//        (the library's kernel fetches length and hop count first, then the addresses, then one destination per hop)
// ORDER  only names the instance: the same kernel on another order of the item list, or with fewer workgroups resident
template <int M, bool PIPE, bool ALIGNED, int AHEAD, bool WHOLE, int ORDER>
__global__ __launch_bounds__(VC_THREADS) void variant_kernel(const int64_t *__restrict__ items, unsigned nitems, unsigned per,
                                                             const char *__restrict__ sendbuf, char *__restrict__ recvbuf,
                                                             char *__restrict__ stage) {
    const unsigned group = (blockIdx.x % VC_XCDS) * per + blockIdx.x / VC_XCDS;
    const unsigned first = group * M;
    if (first >= nitems) return;
    unsigned touched = 0;
    if (AHEAD > 0) {
        const unsigned ahead = blockIdx.x / VC_XCDS + AHEAD;
        if (threadIdx.x == 0 && ahead < per) {
            unsigned off = 0;
            asm("" : "+v"(off));      // keeps this a vector load: a scalar one would be waited for together with the item's
            touched = *reinterpret_cast<const unsigned *>(
                reinterpret_cast<const char *>(items + (int64_t)((blockIdx.x % VC_XCDS) * per + ahead) * M * ITEM_WORDS) + off);
        }
    }
    const int64_t *it = items + (int64_t)first * ITEM_WORDS;
    if (WHOLE && M == 1) {
        int64_t w0 = it[0], w1 = it[1], w2 = it[2], w3 = it[3], w4 = it[4];
        asm("" : "+s"(w0), "+s"(w1), "+s"(w2), "+s"(w3), "+s"(w4));
        const int nh = (int)w2;
        if (w1 > 0 && nh > 0) {
            PieceRegs R;
            piece_load<ALIGNED>(vc_resolve(w0, sendbuf, recvbuf, stage), w1, vc_resolve(w3, sendbuf, recvbuf, stage), R);
            piece_store(vc_resolve(w3, sendbuf, recvbuf, stage), R);
            if (nh > 1) piece_store(vc_resolve(w4, sendbuf, recvbuf, stage), R);
        }
    } else if (!PIPE) {
        PieceRegs R[M];
        int64_t len[M];
        int nhop[M];
#pragma unroll
        for (int m = 0; m < M; m++) {
            len[m] = first + m < nitems ? it[m * ITEM_WORDS + VC_CHAIN_LEN] : 0;
            nhop[m] = (int)it[m * ITEM_WORDS + VC_CHAIN_NHOP];
            if (len[m] > 0 && nhop[m] > 0)
                piece_load<ALIGNED>(vc_resolve(it[m * ITEM_WORDS + VC_CHAIN_SRC], sendbuf, recvbuf, stage), len[m],
                                    vc_resolve(it[m * ITEM_WORDS + VC_CHAIN_HEAD], sendbuf, recvbuf, stage), R[m]);
        }
#pragma unroll
        for (int m = 0; m < M; m++)
            if (len[m] > 0 && nhop[m] > 0)
                for (int k = 0; k < nhop[m]; k++) piece_store(vc_resolve(it[m * ITEM_WORDS + VC_CHAIN_HEAD + k], sendbuf, recvbuf, stage), R[m]);
    } else {
        PieceRegs R[2];
        int64_t len[M];
        int nhop[M];
#pragma unroll
        for (int m = 0; m < M; m++) {
            len[m] = first + m < nitems ? it[m * ITEM_WORDS + VC_CHAIN_LEN] : 0;
            nhop[m] = (int)it[m * ITEM_WORDS + VC_CHAIN_NHOP];
        }
        if (len[0] > 0 && nhop[0] > 0)
            piece_load<ALIGNED>(vc_resolve(it[VC_CHAIN_SRC], sendbuf, recvbuf, stage), len[0], vc_resolve(it[VC_CHAIN_HEAD], sendbuf, recvbuf, stage), R[0]);
#pragma unroll
        for (int m = 0; m < M; m++) {
            if (m + 1 < M && len[m + 1] > 0 && nhop[m + 1] > 0)
                piece_load<ALIGNED>(vc_resolve(it[(m + 1) * ITEM_WORDS + VC_CHAIN_SRC], sendbuf, recvbuf, stage), len[m + 1],
                                    vc_resolve(it[(m + 1) * ITEM_WORDS + VC_CHAIN_HEAD], sendbuf, recvbuf, stage), R[(m + 1) & 1]);
            if (len[m] > 0 && nhop[m] > 0)
                for (int k = 0; k < nhop[m]; k++) piece_store(vc_resolve(it[m * ITEM_WORDS + VC_CHAIN_HEAD + k], sendbuf, recvbuf, stage), R[m & 1]);
        }
    }
    if (AHEAD > 0) asm volatile("" ::"v"(touched));      // the touched word's only use, after the stores
}

// Contiguous copies of known size, the access pattern of the block movers without their scatter: WRITES stores per load,
// VECS 16-byte vectors per lane, non-temporal on both sides.
template <int WRITES, int VECS>
__global__ __launch_bounds__(VC_THREADS) void contiguous_copy_kernel(const vc_u32x4 *__restrict__ src, vc_u32x4 *__restrict__ d0,
                                                                     vc_u32x4 *__restrict__ d1, int64_t nvec) {
    const int64_t base = (int64_t)blockIdx.x * VC_THREADS * VECS + threadIdx.x;
    vc_u32x4 v[VECS];
#pragma unroll
    for (int i = 0; i < VECS; i++)
        if (base + i * VC_THREADS < nvec) v[i] = __builtin_nontemporal_load(&src[base + i * VC_THREADS]);
#pragma unroll
    for (int i = 0; i < VECS; i++)
        if (base + i * VC_THREADS < nvec) {
            __builtin_nontemporal_store(v[i], &d0[base + i * VC_THREADS]);
            if (WRITES == 2) __builtin_nontemporal_store(v[i], &d1[base + i * VC_THREADS]);
        }
}

__global__ void compare_kernel(const vc_u32x4 *a, const vc_u32x4 *b, int64_t nvec, unsigned long long *bad) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    unsigned long long n = 0;
    for (; i < nvec; i += step) {
        const vc_u32x4 x = a[i], y = b[i];
        n += (x.x != y.x) | (x.y != y.y) | (x.z != y.z) | (x.w != y.w);
    }
    if (n) atomicAdd(bad, n);
}

template <class F>
static float best_ms(F launch, int reps) {
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    launch();
    CK(hipDeviceSynchronize());
    float best = 1e30f;
    for (int i = 0; i < reps; i++) {
        CK(hipEventRecord(a));
        launch();
        CK(hipEventRecord(b));
        CK(hipEventSynchronize(b));
        float ms;
        CK(hipEventElapsedTime(&ms, a, b));
        best = std::min(best, ms);
    }
    CK(hipEventDestroy(a));
    CK(hipEventDestroy(b));
    return best;
}

int main(int argc, char **argv) {
    const int reps = argc > 1 ? std::max(1, atoi(argv[1])) : 7;
    const int P = 1024, n = 32, G = P / n;
    const int64_t N = (int64_t)P * P;
    std::mt19937_64 rng(1);
    std::normal_distribution<double> normal(4096, 1024);
    std::vector<int> count(N);
    int64_t payload = 0;
    for (auto &c : count) {     // (a block of more than 8 KiB minus its phase would be cut into pieces: 4 sigma away, left out here)
        c = (int)std::min(8000.0, std::max(0.0, std::round(normal(rng))));
        payload += c;
    }
    // send arena: the blocks of rank s back to back in destination order; receive arena: the blocks of rank t back to back in
    // source order (the packed layout of TTPL_BT_alltoallv)
    std::vector<int64_t> send_off(N), recv_off(N), stage_off(N, -1);
    int64_t at = 0;
    for (int s = 0; s < P; s++)
        for (int t = 0; t < P; t++) { send_off[(int64_t)s * P + t] = at; at += count[(int64_t)s * P + t]; }
    at = 0;
    for (int t = 0; t < P; t++)
        for (int s = 0; s < P; s++) { recv_off[(int64_t)s * P + t] = at; at += count[(int64_t)s * P + t]; }
    // staging: rank (gs, lt) holds the blocks (s, t) with ls != lt that leave the node, by destination node, then local offset;
    // a slot starts on a cache line plus the line phase of the block's place in recvbuf (the library's compact layout)
    int64_t stage_bytes = 0, moved = 0;
    for (int h = 0; h < P; h++) {
        const int gh = h / n, lh = h % n;
        for (int gt = 0; gt < G; gt++)
            for (int j = 1; j < n; j++) {
                if (gt == gh) continue;
                const int s = gh * n + (lh + j) % n, t = gt * n + lh;
                const int64_t k = (int64_t)s * P + t, phase = recv_off[k] & (VC_LINE - 1);
                stage_off[k] = stage_bytes + phase;
                stage_bytes += (count[k] + phase + VC_LINE - 1) & ~(int64_t)(VC_LINE - 1);
            }
    }
    std::vector<int64_t> items(N * ITEM_WORDS);      // by receiver, then source; reordered below
    for (int t = 0; t < P; t++)
        for (int s = 0; s < P; s++) {
            const int64_t k = (int64_t)s * P + t;
            int64_t *it = &items[((int64_t)t * P + s) * ITEM_WORDS];
            it[VC_CHAIN_SRC] = VC_SPACE_SEND | send_off[k];
            it[VC_CHAIN_LEN] = count[k];
            if (stage_off[k] >= 0) {
                it[VC_CHAIN_NHOP] = 2;
                it[VC_CHAIN_HEAD] = VC_SPACE_STAGE | stage_off[k];
                it[VC_CHAIN_HEAD + 1] = VC_SPACE_RECV | recv_off[k];
                moved += 2 * (int64_t)count[k];
            } else {
                it[VC_CHAIN_NHOP] = 1;
                it[VC_CHAIN_HEAD] = VC_SPACE_RECV | recv_off[k];
                it[VC_CHAIN_HEAD + 1] = 0;
                moved += count[k];
            }
        }
    const int64_t cap = (std::max(payload, stage_bytes) + 65536 + 4095) & ~(int64_t)4095;
    char *sendbuf, *stage, *recvbuf, *want_stage, *want_recv;
    int64_t *items_dev;
    unsigned long long *bad_dev;
    CK(hipMalloc(&sendbuf, cap));
    CK(hipMalloc(&stage, cap));
    CK(hipMalloc(&recvbuf, cap));
    CK(hipMalloc(&want_stage, cap));
    CK(hipMalloc(&want_recv, cap));
    CK(hipMalloc(&items_dev, sizeof(int64_t) * items.size()));
    CK(hipMalloc(&bad_dev, 8));
    {
        std::vector<uint64_t> bytes(cap / 8);
        uint64_t x = 88172645463325252ull;
        for (auto &w : bytes) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; w = x; }
        CK(hipMemcpy(sendbuf, bytes.data(), cap, hipMemcpyHostToDevice));
    }
    // the list in tiles of TT receivers x TS sources, receiver by receiver inside a tile; vc_chain_emit writes tiles of
    // VC_TILE_RANKS x VC_TILE_RANKS, which is the order every kernel below runs on unless its row says otherwise
    auto in_tiles = [&](int TT, int TS) {
        std::vector<int64_t> tiled(items.size());
        int64_t o = 0;
        for (int tb = 0; tb < P; tb += TT)
            for (int sb = 0; sb < P; sb += TS)
                for (int t = tb; t < tb + TT; t++)
                    for (int s = sb; s < sb + TS; s++) {
                        std::copy(&items[((int64_t)t * P + s) * ITEM_WORDS], &items[((int64_t)t * P + s) * ITEM_WORDS] + ITEM_WORDS, &tiled[o]);
                        o += ITEM_WORDS;
                    }
        return tiled;
    };
    const std::vector<int64_t> library_order = in_tiles(VC_TILE_RANKS, VC_TILE_RANKS);
    CK(hipMemcpy(items_dev, library_order.data(), sizeof(int64_t) * library_order.size(), hipMemcpyHostToDevice));
    const double physical = (double)payload + (double)moved;      // one read, one write per hop
    printf("configuration 4 as chain items: payload %.3f GB, staging %.3f GB, bytes the launch must move %.3f GB, %lld items, best of %d launches\n",
           payload / 1e9, stage_bytes / 1e9, physical / 1e9, (long long)N, reps);

    auto differing = [&]() {
        CK(hipMemset(bad_dev, 0, 8));
        hipLaunchKernelGGL(compare_kernel, dim3(4096), dim3(256), 0, 0, (const vc_u32x4 *)recvbuf, (const vc_u32x4 *)want_recv, cap / 16, bad_dev);
        hipLaunchKernelGGL(compare_kernel, dim3(4096), dim3(256), 0, 0, (const vc_u32x4 *)stage, (const vc_u32x4 *)want_stage, cap / 16, bad_dev);
        unsigned long long bad;
        CK(hipMemcpy(&bad, bad_dev, 8, hipMemcpyDeviceToHost));
        return bad;
    };
    float base_ms = 0.f;
    auto row = [&](const char *name, auto launch) {
        CK(hipMemset(recvbuf, 0xEE, cap));
        CK(hipMemset(stage, 0xEE, cap));
        const float ms = best_ms(launch, reps);
        const unsigned long long bad = differing();
        if (base_ms == 0.f) base_ms = ms;
        printf("%-72s %7.3f ms  %7.1f GB/s  %+6.1f %%  %s\n", name, ms, physical / ms / 1e6, (ms / base_ms - 1) * 100,
               bad ? "RESULT DIFFERS" : "same bytes");
        fflush(stdout);
        return bad;
    };
    const auto product = [&] { CK(vc_launch_copy_chains(items_dev, ITEM_WORDS, N, VC_THREADS, sendbuf, recvbuf, stage, nullptr)); };
    // the product kernel's own result is what every variant is compared with; it is checked against the definition first
    CK(hipMemset(recvbuf, 0xEE, cap));
    CK(hipMemset(stage, 0xEE, cap));
    product();
    CK(hipDeviceSynchronize());
    CK(hipMemcpy(want_recv, recvbuf, cap, hipMemcpyDeviceToDevice));
    CK(hipMemcpy(want_stage, stage, cap, hipMemcpyDeviceToDevice));
    {
        std::vector<char> hs(cap), hr(cap), hg(cap);
        CK(hipMemcpy(hs.data(), sendbuf, cap, hipMemcpyDeviceToHost));
        CK(hipMemcpy(hr.data(), want_recv, cap, hipMemcpyDeviceToHost));
        CK(hipMemcpy(hg.data(), want_stage, cap, hipMemcpyDeviceToHost));
        int64_t wrong = 0;
        for (int64_t k = 0; k < N; k++)
            for (int b = 0; b < count[k]; b += 61) {
                wrong += hs[send_off[k] + b] != hr[recv_off[k] + b];
                if (stage_off[k] >= 0) wrong += hs[send_off[k] + b] != hg[stage_off[k] + b];
            }
        printf("product kernel against the definition (every 61st byte of every block, receive and staging arenas): %lld wrong\n", (long long)wrong);
        if (wrong) return 1;
    }
    unsigned long long failures = 0;
    failures += row("vc_copy_chains_kernel<256> (the library's kernel)", product);
#define VARIANT(label, M, PIPE, ALIGNED, AHEAD, WHOLE)                                                                              \
    failures += row(label, [&] {                                                                                                    \
        hipLaunchKernelGGL((variant_kernel<M, PIPE, ALIGNED, AHEAD, WHOLE, 0>), dim3((unsigned)(N / M)), dim3(VC_THREADS), 0, 0, items_dev, \
                           (unsigned)N, (unsigned)(N / M / VC_XCDS), sendbuf, recvbuf, stage);                                      \
    })
    VARIANT("the same kernel restated in this file", 1, false, false, 0, false);
    VARIANT("item fetched in one scalar round trip", 1, false, false, 0, true);
    VARIANT("item's cache line touched 256 workgroups ahead", 1, false, false, 256, false);
    VARIANT("item's cache line touched 1024 workgroups ahead", 1, false, false, 1024, false);
    VARIANT("one round trip + touched 1024 ahead", 1, false, false, 1024, true);
    VARIANT("2 items per workgroup, all loads first", 2, false, false, 0, false);
    VARIANT("4 items per workgroup, all loads first", 4, false, false, 0, false);
    VARIANT("2 items per workgroup, loads one item ahead of the stores", 2, true, false, 0, false);
    VARIANT("4 items per workgroup, loads one item ahead of the stores", 4, true, false, 0, false);
    VARIANT("8 items per workgroup, loads one item ahead of the stores", 8, true, false, 0, false);
    VARIANT("aligned loads, realigned in registers (DPP wave_shl + v_alignbyte)", 1, false, true, 0, false);
    VARIANT("aligned loads + one round trip + touched 1024 ahead", 1, false, true, 1024, true);
    {   // other orders of the item list
        const int shapes[][2] = {{1, 1024}, {64, 64}, {128, 128}, {32, 1024}};
        for (int v = 0; v < 4; v++) {
            const int TT = shapes[v][0], TS = shapes[v][1];
            const std::vector<int64_t> tiled = in_tiles(TT, TS);
            CK(hipMemcpy(items_dev, tiled.data(), sizeof(int64_t) * tiled.size(), hipMemcpyHostToDevice));
            char name[128];
            if (TT == 1) snprintf(name, sizeof name, "item list receiver after receiver, all sources of a receiver in a row");
            else snprintf(name, sizeof name, "item list in tiles of %d receivers x %d sources", TT, TS);
            const auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3((unsigned)N), dim3(VC_THREADS), 0, 0, items_dev, (unsigned)N, (unsigned)(N / VC_XCDS), sendbuf, recvbuf, stage); };
            if (v == 0) failures += row(name, [&] { launch(variant_kernel<1, false, false, 0, false, 1>); });
            if (v == 1) failures += row(name, [&] { launch(variant_kernel<1, false, false, 0, false, 2>); });
            if (v == 2) failures += row(name, [&] { launch(variant_kernel<1, false, false, 0, false, 3>); });
            if (v == 3) failures += row(name, [&] { launch(variant_kernel<1, false, false, 0, false, 4>); });
        }
        CK(hipMemcpy(items_dev, library_order.data(), sizeof(int64_t) * library_order.size(), hipMemcpyHostToDevice));
    }
    {   // fewer workgroups resident per compute unit (the kernel itself fits 8): dynamic LDS that it never touches takes the room
        const auto launch = [&](auto kernel, unsigned lds_kib) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)N), dim3(VC_THREADS), lds_kib << 10, 0, items_dev, (unsigned)N, (unsigned)(N / VC_XCDS), sendbuf, recvbuf, stage);
        };
        failures += row("restated kernel + 26 KiB of unused LDS per workgroup (fewer resident)", [&] { launch(variant_kernel<1, false, false, 0, false, 26>, 26); });
        failures += row("restated kernel + 40 KiB of unused LDS per workgroup", [&] { launch(variant_kernel<1, false, false, 0, false, 40>, 40); });
        failures += row("restated kernel + 53 KiB of unused LDS per workgroup", [&] { launch(variant_kernel<1, false, false, 0, false, 53>, 53); });
    }
    failures += row("vc_copy_chains_kernel<256> once more", product);
    // what contiguous copies of the payload sustain in the same process
    const int64_t nvec = payload / 16;
    auto ceiling = [&](const char *name, double bytes, auto launch) {
        const float ms = best_ms(launch, reps);
        printf("%-72s %7.3f ms  %7.1f GB/s\n", name, ms, bytes / ms / 1e6);
        fflush(stdout);
    };
#define CONTIGUOUS(label, WRITES, VECS)                                                                                             \
    ceiling(label, (1.0 + WRITES) * nvec * 16, [&] {                                                                                \
        hipLaunchKernelGGL((contiguous_copy_kernel<WRITES, VECS>), dim3((unsigned)((nvec + VC_THREADS * VECS - 1) / (VC_THREADS * VECS))), \
                           dim3(VC_THREADS), 0, 0, (const vc_u32x4 *)sendbuf, (vc_u32x4 *)recvbuf, (vc_u32x4 *)stage, nvec);        \
    })
    CONTIGUOUS("contiguous copy, one read + one write, 1 vector per lane", 1, 1);
    CONTIGUOUS("contiguous copy, one read + one write, 2 vectors per lane", 1, 2);
    CONTIGUOUS("contiguous copy, one read + two writes, 1 vector per lane", 2, 1);
    CONTIGUOUS("contiguous copy, one read + two writes, 2 vectors per lane", 2, 2);
    CONTIGUOUS("contiguous copy, one read + two writes, 4 vectors per lane", 2, 4);
    if (failures) printf("FAILED: a variant's result differs\n");
    return failures ? 1 : 0;
}
