// vc_copy.hip — the data movers.  A Bruck round on P virtual ranks is a set of
// independent block copies inside HBM: the reference's pack (memcpy into
// temp_send_buffer), MPI_Sendrecv and unpack (memcpy out of temp_recv_buffer)
// (src/twophase_tunable_rbruckv.cpp:90-100,119,126-139) collapse into one read of
// the block where the sender holds it and one write where the receiver wants it.
#include "vc_common.h"

struct __attribute__((packed, aligned(1))) VcU128 { uint32_t a, b, c, d; };

__device__ __forceinline__ uint4 vc_load16_unaligned(const char *p) {
    VcU128 v = *reinterpret_cast<const VcU128 *>(p);
    return make_uint4(v.a, v.b, v.c, v.d);
}

__device__ __forceinline__ char *vc_resolve(int64_t loc, const char *sendbuf, char *recvbuf, char *stage) {
    const int64_t off = loc & VC_OFFSET_MASK;
    const int space = (int)(loc >> VC_SPACE_SHIFT);
    char *base = space == 0 ? const_cast<char *>(sendbuf) : (space == 1 ? recvbuf : stage);
    return base + off;
}

// Copies len bytes with a whole workgroup: byte stores up to the first 16-byte
// boundary of dst, then aligned 16-byte stores fed by (possibly unaligned)
// 16-byte loads, then the tail.
__device__ __forceinline__ void vc_copy_block(char *__restrict__ dst, const char *__restrict__ src, int64_t len) {
    int64_t head = (16 - ((uintptr_t)dst & 15)) & 15;
    if (head > len) head = len;
    if ((int64_t)threadIdx.x < head) dst[threadIdx.x] = src[threadIdx.x];
    const int64_t nvec = (len - head) >> 4;
    const char *s2 = src + head;
    char *d2 = dst + head;
    for (int64_t i = threadIdx.x; i < nvec; i += VC_THREADS)
        *reinterpret_cast<uint4 *>(d2 + (i << 4)) = vc_load16_unaligned(s2 + (i << 4));
    const int64_t done = head + (nvec << 4);
    const int64_t tail = len - done;
    if ((int64_t)threadIdx.x < tail) dst[done + threadIdx.x] = src[done + threadIdx.x];
}

// One workgroup per descriptor; empty descriptors return at once.
__global__ __launch_bounds__(VC_THREADS) void vc_copy_dense_kernel(const VcDesc *__restrict__ desc, const char *__restrict__ sendbuf,
                                                                   char *__restrict__ recvbuf, char *__restrict__ stage) {
    const VcDesc d = desc[blockIdx.x];
    if (d.len <= 0) return;
    vc_copy_block(vc_resolve(d.dst, sendbuf, recvbuf, stage), vc_resolve(d.src, sendbuf, recvbuf, stage), d.len);
}

hipError_t vc_launch_copy_dense(const VcDesc *desc, int64_t ndesc, const char *sendbuf, char *recvbuf, char *stage, hipStream_t st) {
    if (ndesc <= 0) return hipSuccess;
    hipLaunchKernelGGL(vc_copy_dense_kernel, dim3((unsigned)ndesc), dim3(VC_THREADS), 0, st, desc, sendbuf, recvbuf, stage);
    return hipGetLastError();
}
