// vc_meta.hip — the caller-side metadata steps of the reference drivers as kernels
// (count-matrix exchange, displacement prefix sums, global maximum), plus the
// payload fill and the exact receiver-side check used by the harness.
#include <climits>

#include "vc_common.h"
#include "vc_scan.h"

// ---------------------------------------------------------------------------
// MPI_Alltoall of one int per pair (examples/rbruckv_example.cpp:76) is the
// transpose of the P x P count matrix.  32 x 32 tiles staged through LDS with a
// one-word pad so that both the row-wise load and the column-wise read are
// bank-conflict free; 256 threads move one tile (each 4 rows).
// ---------------------------------------------------------------------------
#define VC_TILE 32

__global__ __launch_bounds__(VC_THREADS) void vc_transpose_kernel(const int *__restrict__ in, int *__restrict__ out, int P) {
    __shared__ int tile[VC_TILE][VC_TILE + 1];
    const int tx = threadIdx.x % VC_TILE, ty = threadIdx.x / VC_TILE;   // ty in [0, 8)
    const int c0 = blockIdx.x * VC_TILE, r0 = blockIdx.y * VC_TILE;
#pragma unroll
    for (int k = 0; k < VC_TILE; k += VC_THREADS / VC_TILE) {
        int r = r0 + ty + k, c = c0 + tx;
        if (r < P && c < P) tile[ty + k][tx] = in[(int64_t)r * P + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < VC_TILE; k += VC_THREADS / VC_TILE) {
        int r = c0 + ty + k, c = r0 + tx;                                // transposed coordinates
        if (r < P && c < P) out[(int64_t)r * P + c] = tile[tx][ty + k];
    }
}

hipError_t vc_launch_transpose(const int *in, int *out, int P, hipStream_t st) {
    int t = (P + VC_TILE - 1) / VC_TILE;
    hipLaunchKernelGGL(vc_transpose_kernel, dim3(t, t), dim3(VC_THREADS), 0, st, in, out, P);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Displacement prefix sums (examples/rbruckv_example.cpp:69-72,77-82): one
// workgroup per rank, wavefront scans combined through LDS, a running carry for
// rows longer than the workgroup.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(VC_THREADS) void vc_row_scan_kernel(const int *__restrict__ counts, int *__restrict__ displs,
                                                                 int64_t *__restrict__ extent, int *__restrict__ flags, int P) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int p = blockIdx.x;
    int64_t carry = 0;
    for (int base = 0; base < P; base += VC_THREADS) {
        int i = base + threadIdx.x;
        int64_t v = (i < P) ? counts[(int64_t)p * P + i] : 0, total;
        int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (i < P) displs[(int64_t)p * P + i] = (int)(carry + ex);
        if (flags && v < 0) flags[1] = 1;                 // a negative count
        carry += total;
    }
    if (extent && threadIdx.x == 0) extent[p] = carry;
    // the last displacement is the largest when no count is negative
    if (flags && threadIdx.x == 0 && carry > 0x7FFFFFFFll) flags[0] = 1;
}

hipError_t vc_launch_row_scan(const int *counts, int *displs, int64_t *extent, int *flags, int P, hipStream_t st) {
    hipLaunchKernelGGL(vc_row_scan_kernel, dim3(P), dim3(VC_THREADS), 0, st, counts, displs, extent, flags, P);
    return hipGetLastError();
}

// base[p] = sum_{q<p} roundup(extent[q]*esz, align); one workgroup.
__global__ __launch_bounds__(VC_THREADS) void vc_bases_kernel(const int64_t *__restrict__ extent, int esz, int64_t align,
                                                              int64_t *__restrict__ base, int64_t *__restrict__ total_out, int P) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    int64_t carry = 0;
    for (int b0 = 0; b0 < P; b0 += VC_THREADS) {
        int i = b0 + threadIdx.x;
        int64_t v = 0, total;
        if (i < P) v = (extent[i] * esz + align - 1) / align * align;
        int64_t ex = vc_block_exclusive_scan(v, lds, total);
        if (i < P) base[i] = carry + ex;
        carry += total;
    }
    if (total_out && threadIdx.x == 0) *total_out = carry;
}

hipError_t vc_launch_bases(const int64_t *extent, int esz, int64_t align, int64_t *base, int64_t *total, int P, hipStream_t st) {
    hipLaunchKernelGGL(vc_bases_kernel, dim3(1), dim3(VC_THREADS), 0, st, extent, esz, align, base, total, P);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// MPI_Allreduce(MAX) of the block length (src/twophase_tunable_rbruckv.cpp:40-44).
// ---------------------------------------------------------------------------
// One atomic per workgroup (the wavefronts' maxima meet in LDS first): 256 atomics on the one word instead of one per
// wavefront, which is what the call waited for at 1024 ranks.
__global__ __launch_bounds__(VC_THREADS) void vc_max_kernel(const int *__restrict__ counts, int *__restrict__ out, int64_t n) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    int m = INT_MIN;
    for (int64_t i = (int64_t)blockIdx.x * VC_THREADS + threadIdx.x; i < n; i += (int64_t)gridDim.x * VC_THREADS) m = max(m, counts[i]);
    const int64_t all = vc_block_max(m, lds);
    if (threadIdx.x == 0) atomicMax(out, (int)all);
}

__global__ void vc_lowest_int_kernel(int *p) { *p = INT_MIN; }

hipError_t vc_launch_max(const int *counts, int *out, int64_t nelem, hipStream_t st) {
    hipLaunchKernelGGL(vc_lowest_int_kernel, dim3(1), dim3(1), 0, st, out);
    int64_t blocks = (nelem + 4 * VC_THREADS - 1) / (4 * VC_THREADS);
    if (blocks > 256) blocks = 256;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(vc_max_kernel, dim3((unsigned)blocks), dim3(VC_THREADS), 0, st, counts, out, nelem);
    return hipGetLastError();
}

// Equal-block tables implied by the uniform_* functions: counts = count, displs[p][i] = i*count.
__global__ void vc_uniform_tables_kernel(int *counts, int *displs, int count, int P) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (int64_t)P * P) {
        counts[i] = count;
        displs[i] = (int)(i % P) * count;
    }
}

hipError_t vc_launch_uniform_tables(int *counts, int *displs, int count, int P, hipStream_t st) {
    int64_t nb = ((int64_t)P * P + VC_THREADS - 1) / VC_THREADS;
    hipLaunchKernelGGL(vc_uniform_tables_kernel, dim3((unsigned)nb), dim3(VC_THREADS), 0, st, counts, displs, count, P);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Payload.  The reference drivers fill `i + rank*10` (examples/rbruckv_example.cpp:88-92);
// here every byte depends on source, destination and position.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t vc_splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

__device__ __forceinline__ uint64_t vc_hash4(uint64_t seed, uint64_t a, uint64_t b, uint64_t c) {
    uint64_t h = vc_splitmix64(seed + a);
    h = vc_splitmix64(h + b);
    return vc_splitmix64(h + c);
}

// gridDim.z workgroups per (source, destination) pair, each on its own slice of the block; a thread writes 8 bytes at
// a time.
static unsigned vc_slices_per_block(int P) {
    const int64_t z = (4ll << 20) / ((int64_t)P * P);      // about 4 Mi workgroups at most; many slices when P is small
    return (unsigned)(z < 1 ? 1 : (z > 64 ? 64 : z));
}

__global__ __launch_bounds__(VC_THREADS) void vc_fill_kernel(int mode, uint64_t seed, char *__restrict__ sendbuf,
                                                             const int *__restrict__ sc, const int *__restrict__ sd,
                                                             const int64_t *__restrict__ sbase, int esz, int P) {
    const int s = blockIdx.y, d = blockIdx.x;
    const int64_t len = (int64_t)sc[(int64_t)s * P + d] * esz;
    unsigned char *at = (unsigned char *)sendbuf + sbase[s] + (int64_t)sd[(int64_t)s * P + d] * esz;
    const int64_t nwords = (len + 7) >> 3;
    const int64_t per = (nwords + gridDim.z - 1) / gridDim.z;
    const int64_t kend = (blockIdx.z + 1) * per < nwords ? (blockIdx.z + 1) * per : nwords;
    for (int64_t k = blockIdx.z * per + threadIdx.x; k < kend; k += VC_THREADS) {
        uint64_t word;
        if (mode == 1) {
            uint64_t lo = ((uint64_t)s << 20) + ((uint64_t)d << 10) + (uint64_t)(2 * k);
            uint64_t hi = ((uint64_t)s << 20) + ((uint64_t)d << 10) + (uint64_t)(2 * k + 1);
            word = (lo & 0xFFFFFFFFull) | (hi << 32);
        } else {
            word = vc_hash4(seed, (uint64_t)s, (uint64_t)d, (uint64_t)k);
        }
        int64_t b0 = k << 3;
        int nb = (len - b0) < 8 ? (int)(len - b0) : 8;
        for (int q = 0; q < nb; q++) at[b0 + q] = (unsigned char)(word >> (8 * q));
    }
}

hipError_t vc_launch_fill_payload(int mode, uint64_t seed, char *sendbuf, const int *sc, const int *sd, const int64_t *sbase,
                                  int esz, int P, hipStream_t st) {
    hipLaunchKernelGGL(vc_fill_kernel, dim3(P, P, vc_slices_per_block(P)), dim3(VC_THREADS), 0, st, mode, seed, sendbuf, sc, sd, sbase, esz, P);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Exact check of the textbook definition recv_t[rdispls_t[s] + k] = send_s[sdispls_s[t] + k]
// (the reference's check, src/utils.cpp:31-46, only looks at a residue of each word).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(VC_THREADS) void vc_verify_kernel(const char *__restrict__ sendbuf, const char *__restrict__ recvbuf,
                                                               VcTables T, int esz, int P, int packed,
                                                               unsigned long long *__restrict__ mismatch) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int t = blockIdx.y, s = blockIdx.x;
    const int64_t len = (int64_t)T.sc[(int64_t)s * P + t] * esz;
    int64_t bad = 0;
    if (blockIdx.z == 0 && threadIdx.x == 0 && (int64_t)T.rc[(int64_t)t * P + s] * esz != len) bad = 1;     // the count exchange itself is wrong
    const int *rd = packed ? T.rd_packed : T.rd;
    const unsigned char *a = (const unsigned char *)sendbuf + T.sbase[s] + (int64_t)T.sd[(int64_t)s * P + t] * esz;
    const unsigned char *b = (const unsigned char *)recvbuf + T.rbase[t] + (int64_t)rd[(int64_t)t * P + s] * esz;
    const int64_t per = (len + gridDim.z - 1) / gridDim.z;
    const int64_t kend = (blockIdx.z + 1) * per < len ? (blockIdx.z + 1) * per : len;
    for (int64_t k = blockIdx.z * per + threadIdx.x; k < kend; k += VC_THREADS) bad += a[k] != b[k];
    bad = vc_block_sum(bad, lds);
    if (threadIdx.x == 0 && bad) atomicAdd(mismatch, (unsigned long long)bad);
}

hipError_t vc_launch_verify(const char *sendbuf, const char *recvbuf, VcTables t, int esz, int P, int packed,
                            unsigned long long *mismatch, hipStream_t st) {
    hipLaunchKernelGGL(vc_verify_kernel, dim3(P, P, vc_slices_per_block(P)), dim3(VC_THREADS), 0, st, sendbuf, recvbuf, t, esz, P, packed, mismatch);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Traffic model for choosing the radix.  For radix r = cand[c]: moved[c] = sum over all blocks of hops_r(s, t) *
// bytes(s, t) and moved[ncand + 1 + c] = sum of hops_r(s, t) * pieces(s, t), where hops = non-zero base-r digits of the
// (local) offset, plus one if the node differs, and 1 for a rank's block to itself; pieces = the 4 KiB work items a
// block is cut into.  moved[ncand] and moved[2 ncand + 1] receive the payload and the pieces of all blocks (one hop
// each).  grid (P, ncand + 1); the last row of workgroups adds up the radix-independent totals.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(VC_THREADS) void vc_hop_bytes_kernel(const int *__restrict__ sc, int esz, int P, int n, int ncand,
                                                                  const int *__restrict__ cand, unsigned long long *__restrict__ moved) {
    __shared__ int64_t lds[VC_WAVES_PER_BLOCK];
    const int s = blockIdx.x, c = blockIdx.y;
    const int r = c < ncand ? cand[c] : 0;                // r = 0: every block counts once
    int64_t acc = 0, items = 0;
    for (int t = threadIdx.x; t < P; t += VC_THREADS) {
        int hops = 1;
        if (r && s != t) {
            hops = (s / n != t / n) ? 1 : 0;
            for (int j = (s % n - t % n + n) % n; j; j /= r) hops += (j % r) != 0;
        }
        const int64_t len = (int64_t)sc[(int64_t)s * P + t] * esz;
        acc += hops * len;
        items += hops * (len <= VC_CHUNK ? (len > 0) : (len + VC_PIECE - 1) / VC_PIECE);
    }
    acc = vc_block_sum(acc, lds);
    items = vc_block_sum(items, lds);
    if (threadIdx.x == 0 && acc) atomicAdd(&moved[c], (unsigned long long)acc);
    if (threadIdx.x == 0 && items) atomicAdd(&moved[ncand + 1 + c], (unsigned long long)items);
}

hipError_t vc_launch_hop_bytes(const int *sc, int esz, int P, int n, const int *cand_dev, int ncand, unsigned long long *moved_dev,
                               hipStream_t st) {
    hipLaunchKernelGGL(vc_hop_bytes_kernel, dim3(P, ncand + 1), dim3(VC_THREADS), 0, st, sc, esz, P, n, ncand, cand_dev, moved_dev);
    return hipGetLastError();
}

// A kernel that does nothing: what one launch costs is measured with a row of these.
__global__ void vc_empty_kernel() {}

hipError_t vc_launch_empty(hipStream_t st) {
    hipLaunchKernelGGL(vc_empty_kernel, dim3(1), dim3(VC_WAVE), 0, st);
    return hipGetLastError();
}
