"""Synthetic alltoallv workloads: count matrices, displacement layouts, payload.

The reference's drivers synthesise their inputs per rank from clock-seeded
generators (examples/rbruckv_example.cpp:57-66, examples/other_distributions.cpp:69-108,
examples/FFT_distribution.cpp:61-90) and exchange the counts with MPI_Alltoall
(examples/rbruckv_example.cpp:76).  Here the whole P x P matrix is derived from a
counter-based hash so that every side (GPU harness, CPU oracle, the MPI driver
around the reference build) can regenerate identical inputs from a seed.

Host-side numpy only; nothing here touches the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(x: np.ndarray) -> np.ndarray:
    """One splitmix64 round on uint64 arrays (wrap-around arithmetic)."""
    with np.errstate(over="ignore"):
        x = (np.asarray(x, dtype=np.uint64) + np.uint64(0x9E3779B97F4A7C15)) & _M64
        x = ((x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        x = ((x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return x ^ (x >> np.uint64(31))


def hash4(seed, a, b, c) -> np.ndarray:
    """H(seed, a, b, c): three chained splitmix64 rounds; broadcasts over a, b, c."""
    with np.errstate(over="ignore"):
        h = splitmix64(np.uint64(seed) + np.asarray(a, dtype=np.uint64))
        h = splitmix64(h + np.asarray(b, dtype=np.uint64))
        return splitmix64(h + np.asarray(c, dtype=np.uint64))


PAYLOAD_HASH = 0
PAYLOAD_SELFDESC32 = 1


def block_payload(mode: int, seed: int, src: int, dst: int, nbytes: int) -> np.ndarray:
    """Bytes of block (src, dst): byte k = byte (k & 7) of H(seed, src, dst, k >> 3), or, in the
    self-describing mode, little-endian int32 words src*2^20 + dst*2^10 + idx."""
    if nbytes == 0:
        return np.zeros(0, dtype=np.uint8)
    if mode == PAYLOAD_SELFDESC32:
        nwords = (nbytes + 3) // 4
        words = (np.uint32(src) << np.uint32(20)) + (np.uint32(dst) << np.uint32(10)) + np.arange(nwords, dtype=np.uint32)
        return words.astype("<u4").view(np.uint8)[:nbytes]
    nwords = (nbytes + 7) // 8
    words = hash4(seed, src, dst, np.arange(nwords, dtype=np.uint64))
    return words.astype("<u8").view(np.uint8)[:nbytes]


# ----------------------------------------------------------------- count matrices

def counts_uniform_random(P: int, hi: int, seed: int = 0) -> np.ndarray:
    """counts[s][d] = H(seed, s, d, 0) % (hi + 1)."""
    s, d = np.meshgrid(np.arange(P, dtype=np.uint64), np.arange(P, dtype=np.uint64), indexing="ij")
    return (hash4(seed, s, d, 0) % np.uint64(hi + 1)).astype(np.int32)


def counts_zipf(P: int, max_count: int = 65536, exponent: float = 1.2, zero_percent: int = 5, seed: int = 0) -> np.ndarray:
    """Heavy-tailed rows: a per-source Fisher-Yates permutation pi_s of the destinations,
    count = clip(round(max_count / (pi_s(d) + 1)^exponent), 1, max_count), then zero_percent %
    of the pairs forced to zero."""
    perm = np.tile(np.arange(P, dtype=np.int64), (P, 1))
    rows = np.arange(P)
    for i in range(P - 1, 0, -1):
        j = (hash4(seed, rows, i, 7) % np.uint64(i + 1)).astype(np.int64)
        pi, pj = perm[rows, i].copy(), perm[rows, j].copy()
        perm[rows, i], perm[rows, j] = pj, pi
    counts = np.clip(np.rint(max_count / np.power(perm + 1.0, exponent)), 1, max_count).astype(np.int32)
    s, d = np.meshgrid(np.arange(P, dtype=np.uint64), np.arange(P, dtype=np.uint64), indexing="ij")
    zero = (hash4(seed + 1, s, d, 0) % np.uint64(100)) < np.uint64(zero_percent)
    counts[zero] = 0
    return counts


def counts_normal(P: int, mean: float = 4096.0, sd: float = 1024.0, lo: int = 0, hi: int = 16384, seed: int = 0) -> np.ndarray:
    """Box-Muller on two hashed uniforms, clipped."""
    s, d = np.meshgrid(np.arange(P, dtype=np.uint64), np.arange(P, dtype=np.uint64), indexing="ij")
    u1 = ((hash4(seed, s, d, 1) >> np.uint64(11)).astype(np.float64) + 1.0) / 9007199254740992.0
    u2 = (hash4(seed, s, d, 2) >> np.uint64(11)).astype(np.float64) / 9007199254740992.0
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return np.clip(np.rint(mean + sd * z), lo, hi).astype(np.int32)


def counts_fft_rows(P: int, row_len: int, count: int) -> np.ndarray:
    """Pencil transpose: ranks form a (P/row_len) x row_len grid; a rank sends `count` elements to every
    rank of its own grid row (itself included) and nothing elsewhere."""
    row = np.arange(P) // row_len
    return np.where(row[:, None] == row[None, :], count, 0).astype(np.int32)


def _row_shuffle(rows: np.ndarray, seed: int) -> np.ndarray:
    """Every row shuffled on its own (the reference's drivers std::shuffle each rank's sendcounts with a time seed;
    here the order comes from the hash)."""
    P = rows.shape[0]
    s, d = np.meshgrid(np.arange(P, dtype=np.uint64), np.arange(rows.shape[1], dtype=np.uint64), indexing="ij")
    order = np.argsort(hash4(seed, s, d, 7), axis=1, kind="stable")
    return np.take_along_axis(rows, order, axis=1)


def counts_truncated_normal_rows(P: int, mean: float, deviation: float, max_value: int, seed: int = 0) -> np.ndarray:
    """examples/other_distributions.cpp:70-88 (dist 0): every rank draws P counts from Normal(mean, deviation), redrawing
    values outside [0, max_value], then shuffles them."""
    s, d = np.meshgrid(np.arange(P, dtype=np.uint64), np.arange(P, dtype=np.uint64), indexing="ij")
    out = np.full((P, P), -1.0)
    for attempt in range(64):
        todo = (out < 0) | (out > max_value)
        if not todo.any():
            break
        u1 = ((hash4(seed + 2 * attempt, s, d, 1) >> np.uint64(11)).astype(np.float64) + 1.0) / 9007199254740992.0
        u2 = (hash4(seed + 2 * attempt + 1, s, d, 2) >> np.uint64(11)).astype(np.float64) / 9007199254740992.0
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out = np.where(todo, mean + deviation * z, out)
    out = np.clip(out, 0, max_value)
    return _row_shuffle(out.astype(np.int32), seed)


def counts_power_law_rows(P: int, x: float, max_value: int, seed: int = 0) -> np.ndarray:
    """examples/other_distributions.cpp:91-103 (dist 1): counts max_value * x^k, k = 0 .. P-1, shuffled per rank."""
    row = (max_value * np.power(float(x), np.arange(P))).astype(np.int32)
    return _row_shuffle(np.tile(row, (P, 1)), seed)


def counts_sparse_blocks(P: int, xzero: float, yzero: float, number: int, last: int = 0) -> np.ndarray:
    """examples/FFT_distribution.cpp:68-87: the first ranks send `number` elements to the first destinations, a share
    xzero of the destinations and yzero of the ranks stays empty; with last > 0 every rank sends `number` to all but
    the last destination, which gets `last`."""
    counts = np.zeros((P, P), dtype=np.int32)
    if last == 0:
        number_count = P - int(np.ceil(P * xzero))
        rank_count = P - int(np.ceil(P * yzero))
        counts[:rank_count, :number_count] = number
    else:
        counts[:, :P - 1] = number
        counts[:, P - 1] = last
    return counts


def counts_from_text(path: str) -> np.ndarray:
    """Whitespace-separated P x P matrix, row = sender (the layout of the reference's
    inputs/<P>proc/global_comm_pattern_<P>proc.txt, read by examples/MLinputs_example.cpp:119-145)."""
    m = np.loadtxt(path, dtype=np.int64)
    assert m.ndim == 2 and m.shape[0] == m.shape[1]
    return m


def counts_from_npz(path: str, divide: int = 1) -> np.ndarray:
    """A P x P byte-count matrix stored as the array `counts` of an .npz file (the binary form of the reference's
    inputs/<P>proc matrices); `divide` > 1 scales the counts down for parity-test sizes."""
    with np.load(path, allow_pickle=False) as z:
        m = z["counts"].astype(np.int64)
    assert m.ndim == 2 and m.shape[0] == m.shape[1]
    return (m // divide).astype(np.int32)


# ------------------------------------------------------------------ displacements

def layout_displs(counts_rows: np.ndarray, layout: int) -> tuple[np.ndarray, np.ndarray]:
    """Displacements (elements) for every rank's row of counts, and each rank's extent (elements).

    layout 0: packed, ascending peer order (examples/rbruckv_example.cpp:69-72).
    layout 1: peers placed in descending order, block i of rank p preceded by a gap of (i + p) % 3
              elements — displacements neither sorted nor contiguous.
    """
    P = counts_rows.shape[0]
    c = counts_rows.astype(np.int64)
    if layout == 0:
        displs = np.cumsum(c, axis=1) - c
        extent = c.sum(axis=1)
    elif layout == 1:
        gaps = (np.arange(P)[None, :] + np.arange(P)[:, None]) % 3
        padded = (c + gaps)[:, ::-1]
        ends = np.cumsum(padded, axis=1)[:, ::-1]       # end offset (exclusive) of block i
        displs = ends - c
        extent = ends[:, 0]
    else:
        raise ValueError("layout must be 0 or 1")
    assert extent.max(initial=0) < 2**31, "per-rank displacements must fit int32 like the reference's"
    return displs.astype(np.int32), extent.astype(np.int64)


def aligned_bases(extent_bytes: np.ndarray, align: int = 256) -> tuple[np.ndarray, int]:
    """Byte offset of every rank's buffer inside one arena: exclusive scan of the extents, each rank's
    start rounded up to `align` (what separate per-rank allocations would give)."""
    padded = (extent_bytes.astype(np.int64) + align - 1) // align * align
    bases = np.cumsum(padded) - padded
    return bases.astype(np.int64), int(padded.sum())


@dataclass
class Problem:
    """Everything the P virtual ranks would pass to one alltoallv call, in rank-major tables."""
    P: int
    esz: int
    sendcounts: np.ndarray   # [P][P] int32, row s = what rank s sends to each peer
    sdispls: np.ndarray      # [P][P] int32, elements
    recvcounts: np.ndarray   # [P][P] int32, row t = what rank t receives from each peer
    rdispls: np.ndarray      # [P][P] int32
    sbase: np.ndarray        # [P] int64 bytes
    rbase: np.ndarray        # [P] int64 bytes
    send_bytes: int          # arena sizes
    recv_bytes: int

    @property
    def payload_bytes(self) -> int:
        return int(self.sendcounts.astype(np.int64).sum()) * self.esz


def make_problem(counts: np.ndarray, esz: int, send_layout: int = 0, recv_layout: int = 0, align: int = 256) -> Problem:
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    P = counts.shape[0]
    recvcounts = np.ascontiguousarray(counts.T)          # the MPI_Alltoall of the counts
    sdispls, sext = layout_displs(counts, send_layout)
    rdispls, rext = layout_displs(recvcounts, recv_layout)
    sbase, stot = aligned_bases(sext * esz, align)
    rbase, rtot = aligned_bases(rext * esz, align)
    return Problem(P, esz, counts, np.ascontiguousarray(sdispls), recvcounts, np.ascontiguousarray(rdispls),
                   sbase, rbase, max(stot, 1), max(rtot, 1))


def make_uniform_problem(P: int, count: int, esz: int, align: int = 256) -> Problem:
    return make_problem(np.full((P, P), count, dtype=np.int32), esz, 0, 0, align)


def fill_send_arena(prob: Problem, mode: int, seed: int) -> np.ndarray:
    """Host-side payload (the GPU harness has its own fill kernel for big problems): block (s, d) holds
    block_payload(mode, seed, s, d, nbytes).  One vectorised pass per source rank."""
    arena = np.zeros(prob.send_bytes, dtype=np.uint8)
    P, esz = prob.P, prob.esz
    unit = 4 if mode == PAYLOAD_SELFDESC32 else 8
    ranks = np.arange(P)
    lane = np.arange(unit, dtype=np.int64)[None, :]
    for s in range(P):
        nb = prob.sendcounts[s].astype(np.int64) * esz
        nw = (nb + unit - 1) // unit
        tot = int(nw.sum())
        if tot == 0:
            continue
        d_idx = np.repeat(ranks, nw)
        k_idx = np.arange(tot, dtype=np.int64) - np.repeat(np.cumsum(nw) - nw, nw)
        if mode == PAYLOAD_SELFDESC32:
            words = ((np.uint32(s) << np.uint32(20)) + (d_idx.astype(np.uint32) << np.uint32(10)) + k_idx.astype(np.uint32)).astype("<u4")
        else:
            words = hash4(seed, s, d_idx.astype(np.uint64), k_idx.astype(np.uint64)).astype("<u8")
        data = words.view(np.uint8).reshape(tot, unit)
        pos = k_idx[:, None] * unit + lane                       # byte position inside the block
        valid = pos < nb[d_idx][:, None]
        dest = (int(prob.sbase[s]) + prob.sdispls[s].astype(np.int64)[d_idx] * esz)[:, None] + pos
        arena[dest[valid]] = data[valid]
    return arena


def expected_recv_arena(prob: Problem, send_arena: np.ndarray, fill: int = 0xEE, packed_recv: bool = False) -> np.ndarray:
    """The textbook definition of MPI_Alltoallv: recv_t[rdispls_t[s] + k] = send_s[sdispls_s[t] + k]."""
    out = np.full(prob.recv_bytes, fill, dtype=np.uint8)
    for t in range(prob.P):
        for s in range(prob.P):
            nb = int(prob.sendcounts[s, t]) * prob.esz
            if nb:
                src = int(prob.sbase[s]) + int(prob.sdispls[s, t]) * prob.esz
                dst = int(prob.rbase[t]) + int(prob.rdispls[t, s]) * prob.esz
                out[dst:dst + nb] = send_arena[src:src + nb]
    return out


# ----------------------------------------------------------------- benchmark configurations

def config_counts(name: str, seed: int = 0, scale: int = 1) -> tuple[np.ndarray, int, dict]:
    """Count matrix, element size and tunables of one of the five benchmark configurations.
    `scale` > 1 divides the counts (parity-test sized versions of the same shape)."""
    if name == "C1":
        return counts_uniform_random(8, 64, 0), 4, {"r": 2}
    if name == "C2":
        return counts_uniform_random(64, 4096 // scale, seed), 1, {"r": 2}
    if name == "C3":
        return counts_zipf(256, 65536 // scale, 1.2, 5, seed), 4, {"r": 16}
    if name == "C4":
        return counts_normal(1024, 4096.0 / scale, 1024.0 / scale, 0, 16384 // scale, seed), 1, {"n": 32, "r": 32}
    if name == "C5":
        return counts_fft_rows(512, 32, 131072 // scale), 8, {"r": 32}
    raise ValueError(name)


# -------------------------------------------------------------- traffic model

def radix_params(P: int, r: int) -> tuple[int, int, int, int]:
    """(w, nlpow, d, K) in integer arithmetic (src/tuna.cpp:28-31)."""
    w, top = 0, P - 1
    while top:
        w += 1
        top //= r
    nlpow = r ** max(w - 1, 0)
    d = (nlpow * r - P) // nlpow
    return w, nlpow, d, w * (r - 1) - d


def _nonzero_digits(j: np.ndarray, r: int) -> np.ndarray:
    h = np.zeros_like(j)
    while j.any():
        h += (j % r) != 0
        j = j // r
    return h


def hops_flat(P: int, r: int) -> np.ndarray:
    """hops[s][t] of radix-r Bruck: non-zero base-r digits of (s - t) mod P, 1 for the self block."""
    s, t = np.meshgrid(np.arange(P), np.arange(P), indexing="ij")
    h = _nonzero_digits((s - t) % P, r)
    h[s == t] = 1
    return h


def hops_twolayer(P: int, n: int, r: int) -> np.ndarray:
    """Two-layer: non-zero base-r digits of the local offset, plus one if the node differs."""
    s, t = np.meshgrid(np.arange(P), np.arange(P), indexing="ij")
    h = _nonzero_digits((s % n - t % n) % n, min(r, n)) + ((s // n) != (t // n))
    h[s == t] = 1
    return h


def hops_twolayer_bruck(P: int, n: int, r: int) -> np.ndarray:
    """Two-layer with a Bruck over the nodes as well: non-zero base-r digits of the local offset plus those of the
    group offset (r clamped to n, src/twophase_twolayer_rbruck.cpp:26)."""
    s, t = np.meshgrid(np.arange(P), np.arange(P), indexing="ij")
    reff = max(min(r, n), 2)
    h = _nonzero_digits((s % n - t % n) % n, reff) + _nonzero_digits((s // n - t // n) % (P // n), reff)
    h[s == t] = 1
    return h


def algorithmic_bytes(counts: np.ndarray, esz: int, hops: np.ndarray) -> int:
    """A = 2 * sum hops(s,t) * bytes(s,t): one read and one write per hop."""
    return int(2 * (hops.astype(np.int64) * counts.astype(np.int64)).sum() * esz)
