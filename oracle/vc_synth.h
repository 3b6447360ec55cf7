/*
 * vc_synth.h — counter-based synthetic payload shared by the CPU oracle, the
 * MPI driver around the reference build and (restated in HIP / numpy) the GPU
 * harness.  TEST INFRASTRUCTURE: nothing in the product library includes it.
 *
 * Every side can generate the payload of block (src, dst) without talking to
 * anybody else, the way the reference drivers fill `i + rank*10`
 * (examples/rbruckv_example.cpp:88-92) — but with a value that pins source,
 * destination AND position inside the block, which the reference's residue
 * check (src/utils.cpp:31-46) cannot see.
 */
#ifndef VC_SYNTH_H_
#define VC_SYNTH_H_

#include <stdint.h>

static inline uint64_t vc_splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ULL;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    return x ^ (x >> 31);
}

/* H(seed, a, b, c): three chained splitmix64 rounds. */
static inline uint64_t vc_hash4(uint64_t seed, uint64_t a, uint64_t b, uint64_t c) {
    uint64_t h = vc_splitmix64(seed + a);
    h = vc_splitmix64(h + b);
    return vc_splitmix64(h + c);
}

/* payload modes */
#define VC_PAYLOAD_HASH 0     /* byte k of block (s,d) = byte (k & 7) of H(seed, s, d, k >> 3) */
#define VC_PAYLOAD_SELFDESC32 1 /* int32 word idx of block (s,d) = s*2^20 + d*2^10 + idx (elem size 4) */

static inline unsigned char vc_payload_byte(int mode, uint64_t seed, int src, int dst, int64_t k) {
    if (mode == VC_PAYLOAD_SELFDESC32) {
        uint32_t word = ((uint32_t)src << 20) + ((uint32_t)dst << 10) + (uint32_t)(k >> 2);
        return (unsigned char)(word >> (8 * (k & 3)));
    }
    return (unsigned char)(vc_hash4(seed, (uint64_t)src, (uint64_t)dst, (uint64_t)(k >> 3)) >> (8 * (k & 7)));
}

/* Fill nbytes of one block. */
static inline void vc_fill_block(int mode, uint64_t seed, int src, int dst, unsigned char *out, int64_t nbytes) {
    for (int64_t k = 0; k < nbytes; k++) out[k] = vc_payload_byte(mode, seed, src, dst, k);
}

/* FNV-1a 64 over a byte range (used for per-rank digests of recvbuf). */
static inline uint64_t vc_fnv1a64(const unsigned char *p, int64_t n, uint64_t h) {
    for (int64_t i = 0; i < n; i++) { h ^= p[i]; h *= 0x100000001B3ULL; }
    return h;
}
#define VC_FNV_OFFSET 0xCBF29CE484222325ULL

#endif /* VC_SYNTH_H_ */
