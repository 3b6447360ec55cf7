/*
 * bruck_oracle.c — CPU oracle: the reference's per-rank Bruck alltoallv
 * algorithms restated for P virtual ranks inside one process.
 *
 * TEST INFRASTRUCTURE ONLY (see bruck_oracle.h).  Nothing here is shipped or
 * timed as the product; the product library is the HIP one.
 *
 * How a collective round is simulated: the reference runs the same code on
 * every rank and meets in MPI_Sendrecv.  Here each round is three sweeps over
 * the ranks — every rank packs its outgoing message into its mailbox, then
 * every rank picks up the mailbox of the rank it receives from, then unpacks.
 * Private per-rank state (current block sizes, moved flags, the fixed-stride
 * staging slots) is kept exactly as the reference keeps it, so that the
 * oracle follows the same route block by block and not just the same result.
 */
#include "bruck_oracle.h"
#include "vc_synth.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ trace */

static ora_trace_rec *g_trace = NULL;
static int64_t g_trace_n = 0, g_trace_cap = 0;
static int g_trace_on = 0;

void ora_trace_begin(void) { g_trace_n = 0; g_trace_on = 1; }
void ora_trace_end(void) { g_trace_on = 0; }
int64_t ora_trace_count(void) { return g_trace_n; }
const ora_trace_rec *ora_trace_data(void) { return g_trace; }

static void trace_msg(int kind, int digit, int z, int from, int to, int nblocks, int64_t bytes) {
    if (!g_trace_on) return;
    if (g_trace_n == g_trace_cap) {
        g_trace_cap = g_trace_cap ? 2 * g_trace_cap : 4096;
        g_trace = (ora_trace_rec *)realloc(g_trace, (size_t)g_trace_cap * sizeof(ora_trace_rec));
    }
    ora_trace_rec *t = &g_trace[g_trace_n++];
    t->kind = kind; t->digit = digit; t->z = z; t->from = from; t->to = to;
    t->nblocks = nblocks; t->bytes = bytes;
}

/* ------------------------------------------------------------ small helpers */

/* src/utils.cpp:9-16 computes x^p by recursive squaring; same value, iterative. */
int ora_pow(int x, unsigned int p) {
    int acc = 1;
    while (p) {
        if (p & 1u) acc *= x;
        p >>= 1;
        if (p) x *= x;
    }
    return acc;
}

/* src/twophase_tunable_rbruckv.cpp:30-32: w from a double log divided by a
 * float log (kept, because on exact powers it can come out one too large). */
void ora_radix_params_float(int P, int r, int *w, int *nlpow, int *d) {
    float lr = (float)log((double)r);
    int ww = (int)ceil(log((double)P) / lr);
    int np = ora_pow(r, (unsigned)(ww - 1));
    *w = ww; *nlpow = np; *d = (ora_pow(r, (unsigned)ww) - P) / np;
}

/* src/tuna.cpp:28-31: digits of P-1 in base r by repeated division. */
void ora_radix_params_int(int P, int r, int *w, int *nlpow, int *d, int *K) {
    int ww = 0, np = 1, top = P - 1;
    while (top) { ww++; top /= r; }
    for (int i = 0; i < ww - 1; i++) np *= r;
    *w = ww; *nlpow = np; *d = (np * r - P) / np;
    if (K) *K = ww * (r - 1) - *d;
}

typedef struct {
    int P, esz;
    char *sarena; const int64_t *sbase;
    char *rarena; const int64_t *rbase;
    const int *sc, *sd, *rc, *rd;
} ora_ctx;

static inline char *sbuf(const ora_ctx *c, int p) { return c->sarena + c->sbase[p]; }
static inline char *rbuf(const ora_ctx *c, int p) { return c->rarena + c->rbase[p]; }
#define SC(c, p, i) ((c)->sc[(int64_t)(p) * (c)->P + (i)])
#define SD(c, p, i) ((c)->sd[(int64_t)(p) * (c)->P + (i)])
#define RC(c, p, i) ((c)->rc[(int64_t)(p) * (c)->P + (i)])
#define RD(c, p, i) ((c)->rd[(int64_t)(p) * (c)->P + (i)])

static int global_max_count(const ora_ctx *c) {
    /* local maximum per rank, then MPI_Allreduce(MAX): the maximum of the whole matrix
     * (src/twophase_tunable_rbruckv.cpp:40-44) */
    int m = 0;
    for (int64_t i = 0; i < (int64_t)c->P * c->P; i++) if (c->sc[i] > m) m = c->sc[i];
    return m;
}

/* the block rank p sends to itself (src/twophase_tunable_rbruckv.cpp:63) */
static void self_copies(const ora_ctx *c) {
    for (int p = 0; p < c->P; p++) {
        int64_t nb = (int64_t)RC(c, p, p) * c->esz;
        memcpy(rbuf(c, p) + (int64_t)RD(c, p, p) * c->esz, sbuf(c, p) + (int64_t)SD(c, p, p) * c->esz, (size_t)nb);
        trace_msg(4, -1, 0, p, p, 1, nb);
    }
}

/* Offsets j in [0, span) whose base-r digit at weight `dist` equals z, ascending
 * (src/twophase_tunable_rbruckv.cpp:78-84).  Returns how many. */
static int digit_offsets(int span, int dist, int r, int z, int *out) {
    int n = 0;
    int64_t step = (int64_t)dist * r;
    for (int64_t i = (int64_t)z * dist; i < span; i += step)
        for (int64_t j = i; j < i + dist && j < span; j++) out[n++] = (int)j;
    return n;
}

typedef struct { int nblk; int *sizes; int64_t nbytes; char *bytes; } ora_msg;

static void msg_reserve(ora_msg *m, int nblk, int64_t nbytes) {
    m->nblk = nblk; m->nbytes = nbytes;
    m->sizes = (int *)malloc(sizeof(int) * (size_t)(nblk > 0 ? nblk : 1));
    m->bytes = (char *)malloc((size_t)(nbytes > 0 ? nbytes : 1));
}
static void msg_release(ora_msg *m) { free(m->sizes); free(m->bytes); m->sizes = NULL; m->bytes = NULL; }

static ora_ctx make_ctx(char *sa, const int64_t *sb, const int *sc, const int *sd, int esz, char *ra,
                        const int64_t *rb, const int *rc, const int *rd, int P) {
    ora_ctx c; c.P = P; c.esz = esz; c.sarena = sa; c.sbase = sb; c.rarena = ra; c.rbase = rb;
    c.sc = sc; c.sd = sd; c.rc = rc; c.rd = rd; return c;
}

/* --------------------------------- 1. two-phase radix-r Bruck, MSD first ---
 * src/twophase_tunable_rbruckv.cpp:13-152.  Every block that has moved sits in
 * slot `id = (j + rank) % P` of a P-slot staging area with stride
 * max_send_count*typesize (:59); `cur` is sendNcopy, `moved` is pos_status. */
int ora_twophase_rbruck_alltoallv(int r, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                  const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                                  const int *recvcounts, const int *rdispls, int P) {
    if (r < 2) return -1;                       /* :16 */
    if (r > P) r = P;                           /* :22 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    int w, nlpow, d;
    ora_radix_params_float(P, r, &w, &nlpow, &d);
    int64_t stride = (int64_t)global_max_count(&c) * esz;

    int *cur = (int *)malloc(sizeof(int) * (size_t)P * P);
    char *moved = (char *)calloc((size_t)P * P, 1);
    char **extra = (char **)malloc(sizeof(char *) * (size_t)P);
    ora_msg *box = (ora_msg *)calloc((size_t)P, sizeof(ora_msg));
    int *offs = (int *)malloc(sizeof(int) * (size_t)(nlpow > 0 ? nlpow : 1));
    memcpy(cur, sendcounts, sizeof(int) * (size_t)P * P);                       /* :45 */
    for (int p = 0; p < P; p++) extra[p] = (char *)malloc((size_t)(stride * P + 1));
    self_copies(&c);

    int dist = nlpow;
    for (int x = w - 1; x >= 0; x--) {
        int ze = (x == w - 1) ? r - d : r;      /* :71 */
        int64_t ndist = (int64_t)dist * r;
        for (int z = ze - 1; z > 0; z--) {
            int hop = z * dist;
            int nb = digit_offsets(P, dist, r, z, offs);
            /* pack (:90-100) */
            for (int p = 0; p < P; p++) {
                int64_t tot = 0;
                for (int i = 0; i < nb; i++) {
                    int slot = (offs[i] + p) % P;
                    int key = (2 * p - slot + P) % P;               /* rotate_index_array[slot], :53 */
                    tot += (int64_t)cur[(int64_t)p * P + key] * esz;
                }
                msg_reserve(&box[p], nb, tot);
                int64_t off = 0;
                for (int i = 0; i < nb; i++) {
                    int slot = (offs[i] + p) % P;
                    int key = (2 * p - slot + P) % P;
                    int cnt = cur[(int64_t)p * P + key];
                    const char *from = moved[(int64_t)p * P + key]
                                           ? extra[p] + (int64_t)slot * stride
                                           : sbuf(&c, p) + (int64_t)SD(&c, p, key) * esz;
                    box[p].sizes[i] = cnt;
                    memcpy(box[p].bytes + off, from, (size_t)((int64_t)cnt * esz));
                    off += (int64_t)cnt * esz;
                }
            }
            /* exchange + replace (:106-139): rank p receives what rank p+hop sent */
            for (int p = 0; p < P; p++) {
                int from_rank = (p + hop) % P;
                const ora_msg *m = &box[from_rank];
                trace_msg(0, x, z, from_rank, p, nb, m->nbytes);
                int64_t off = 0;
                for (int i = 0; i < nb; i++) {
                    int slot = (offs[i] + p) % P;
                    int key = (2 * p - slot + P) % P;
                    int64_t nbytes = (int64_t)m->sizes[i] * esz;
                    int origin = (slot - p + P) % P;
                    if (origin % ndist == (from_rank - p + P) % P)                       /* :131 */
                        memcpy(rbuf(&c, p) + (int64_t)RD(&c, p, slot) * esz, m->bytes + off, (size_t)nbytes);
                    else
                        memcpy(extra[p] + (int64_t)slot * stride, m->bytes + off, (size_t)nbytes);
                    off += nbytes;
                    moved[(int64_t)p * P + key] = 1;
                    cur[(int64_t)p * P + key] = m->sizes[i];
                }
            }
            for (int p = 0; p < P; p++) msg_release(&box[p]);
        }
        dist /= r;
    }
    for (int p = 0; p < P; p++) free(extra[p]);
    free(extra); free(box); free(offs); free(cur); free(moved);
    return 0;
}

/* index of slot j in the compact staging area, evaluated the way the reference
 * does, through float logs (src/tuna.cpp:93-97, src/twophase_tunable_rbruckv-om.cpp:80-84) */
static int compact_slot_float(int j, int r) {
    int dx = (int)(log((double)j) / (float)log((double)r));
    int low = ora_pow(r, (unsigned)dx);
    int dz = (int)(j / (float)low);
    return j - r - (dx - 1) * (r - 1) - dz;
}

/* Shared body of the LSD-first, compact-staging variants.  `direct_if_single`
 * selects how a round is recognised as a single-block round: by the length of
 * the enumerated list (om, :70) or by the closed-form ns (tuna.cpp:75-80). */
static int lsd_compact_bruck(ora_ctx *c, int r, int w, int nlpow, int d, int K, int batch, int use_ns_formula) {
    int P = c->P, esz = c->esz;
    int nstage = P - K - 1;
    int64_t stride = 0;
    int *stage_cnt = NULL;
    char **stage = (char **)calloc((size_t)P, sizeof(char *));
    if (nstage > 0) {
        stride = (int64_t)global_max_count(c) * esz;
        stage_cnt = (int *)calloc((size_t)P * nstage, sizeof(int));
        for (int p = 0; p < P; p++) stage[p] = (char *)malloc((size_t)(stride * nstage + 1));
    }
    self_copies(c);

    ora_msg *box = (ora_msg *)calloc((size_t)P, sizeof(ora_msg));
    int *offs = (int *)malloc(sizeof(int) * (size_t)(nlpow > 0 ? nlpow : 1));
    int *cid = (int *)malloc(sizeof(int) * (size_t)(nlpow > 0 ? nlpow : 1));
    int dist = 1;
    for (int x = 0; x < w; x++) {
        int ze = (x == w - 1) ? r - d : r;
        int64_t ndist = (int64_t)dist * r;
        for (int z0 = 1; z0 < ze; z0 += batch) {
            int in_batch = ze - z0 < batch ? ze - z0 : batch;
            for (int bi = 0; bi < in_batch; bi++) {
                int z = z0 + bi;
                int hop = z * dist;
                int nb;
                if (use_ns_formula) {
                    int nc = (int)(P / ndist) * dist, rem = (int)(P % ndist) - hop;       /* tuna.cpp:75-77 */
                    if (rem < 0) rem = 0;
                    nb = rem > dist ? nc + dist : nc + rem;
                } else {
                    nb = digit_offsets(P, dist, r, z, offs);
                }
                if (nb == 1) {
                    /* one block, straight from the sender's sendbuf into the receiver's recvbuf
                     * (om :70-75, tuna.cpp:80-86) */
                    for (int p = 0; p < P; p++) {
                        int from_rank = (p + hop) % P;
                        int64_t nbytes = (int64_t)SC(c, from_rank, p) * esz;
                        memcpy(rbuf(c, p) + (int64_t)RD(c, p, from_rank) * esz,
                               sbuf(c, from_rank) + (int64_t)SD(c, from_rank, p) * esz, (size_t)nbytes);
                        trace_msg(1, x, z, from_rank, p, 1, nbytes);
                    }
                    continue;
                }
                nb = digit_offsets(P, dist, r, z, offs);
                for (int i = 0; i < nb; i++) cid[i] = compact_slot_float(offs[i], r);
                for (int p = 0; p < P; p++) {
                    int64_t tot = 0;
                    for (int i = 0; i < nb; i++) {
                        int slot = (offs[i] + p) % P;
                        int key = (2 * p - slot + P) % P;
                        int cnt = (i % dist == 0) ? SC(c, p, key) : stage_cnt[(int64_t)p * nstage + cid[i]];
                        tot += (int64_t)cnt * esz;
                    }
                    msg_reserve(&box[p], nb, tot);
                    int64_t off = 0;
                    for (int i = 0; i < nb; i++) {
                        int slot = (offs[i] + p) % P;
                        int key = (2 * p - slot + P) % P;
                        int cnt; const char *from;
                        if (i % dist == 0) {                    /* never moved: still in sendbuf */
                            cnt = SC(c, p, key);
                            from = sbuf(c, p) + (int64_t)SD(c, p, key) * esz;
                        } else {
                            cnt = stage_cnt[(int64_t)p * nstage + cid[i]];
                            from = stage[p] + (int64_t)cid[i] * stride;
                        }
                        box[p].sizes[i] = cnt;
                        memcpy(box[p].bytes + off, from, (size_t)((int64_t)cnt * esz));
                        off += (int64_t)cnt * esz;
                    }
                }
                for (int p = 0; p < P; p++) {
                    int from_rank = (p + hop) % P;
                    const ora_msg *m = &box[from_rank];
                    trace_msg(0, x, z, from_rank, p, nb, m->nbytes);
                    int64_t off = 0;
                    for (int i = 0; i < nb; i++) {
                        int slot = (offs[i] + p) % P;
                        int64_t nbytes = (int64_t)m->sizes[i] * esz;
                        if (i < dist) {                         /* no higher digit left: final */
                            memcpy(rbuf(c, p) + (int64_t)RD(c, p, slot) * esz, m->bytes + off, (size_t)nbytes);
                        } else {
                            memcpy(stage[p] + (int64_t)cid[i] * stride, m->bytes + off, (size_t)nbytes);
                            stage_cnt[(int64_t)p * nstage + cid[i]] = m->sizes[i];
                        }
                        off += nbytes;
                    }
                }
                for (int p = 0; p < P; p++) msg_release(&box[p]);
            }
            /* MPI_Waitall of the batch (tuna.cpp:165): nothing left to do in lockstep */
        }
        dist *= r;
    }
    for (int p = 0; p < P; p++) free(stage[p]);
    free(stage); free(stage_cnt); free(box); free(offs); free(cid);
    return 0;
}

/* -------------------------- 2. memory-optimised two-phase Bruck, LSD first */
int ora_twophase_rbruck_alltoallv_om(int r, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                     const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                                     const int *recvcounts, const int *rdispls, int P) {
    if (r < 2) return -1;                       /* -om.cpp:13 */
    if (r > P) r = P;                           /* :19 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    int w, nlpow, d;
    ora_radix_params_float(P, r, &w, &nlpow, &d);       /* :27-29 */
    int K = w * (r - 1) - d;                            /* :30 */
    return lsd_compact_bruck(&c, r, w, nlpow, d, K, 1, 0);
}

/* ------------------------------------------------------------------ 3. TuNA */
int ora_tuna_algorithm(int r, int b, char *sendarena, const int64_t *sbase, const int *sendcounts,
                       const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                       const int *recvcounts, const int *rdispls, int P) {
    if (P < 3) return -3;                       /* tuna.cpp:20,28 would loop forever */
    if (r < 2) r = 2;                           /* :13 */
    if (r > P - 1) r = P - 1;                   /* :20 */
    if (b <= 0 || b > P) b = P;                 /* :21 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    int w, nlpow, d, K;
    ora_radix_params_int(P, r, &w, &nlpow, &d, &K);
    return lsd_compact_bruck(&c, r, w, nlpow, d, K, b, 1);
}

/* ----------------------------------------------------------------- 3b. TuNA2
 * src/tuna2.cpp:10-239: TuNA's rounds, but the data of all rounds of a digit is received into one buffer and
 * unpacked only after the digit's last batch (:202-223); the compact staging index comes from a table (:63-73).
 * The reference packs every round of a batch into ONE temp_send_buffer while earlier MPI_Isends from it may still
 * be in flight (:175-185), which corrupts messages for b > 1; a correct run is what is restated here (each round
 * keeps its own message), so for b > 1 the pin is the alltoallv definition and not a reference run. */
int ora_tuna2_algorithm(int r, int b, char *sendarena, const int64_t *sbase, const int *sendcounts,
                        const int *sdispls, int esz, char *recvarena, const int64_t *rbase,
                        const int *recvcounts, const int *rdispls, int P) {
    if (P < 3) return -3;                       /* :19, :27 would loop forever */
    if (r < 2) r = 2;                           /* :13 */
    if (r > P - 1) r = P - 1;                   /* :20 */
    if (b <= 0 || b > P) b = P;                 /* :21 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    int w, nlpow, d, K;
    ora_radix_params_int(P, r, &w, &nlpow, &d, &K);
    int nstage = P - K - 1;
    int64_t stride = 0;
    int *stage_cnt = NULL, *table = NULL;
    char **stage = (char **)calloc((size_t)P, sizeof(char *));
    if (K < P - 1) {
        stride = (int64_t)global_max_count(&c) * esz;
        stage_cnt = (int *)calloc((size_t)P * nstage, sizeof(int));
        for (int p = 0; p < P; p++) stage[p] = (char *)malloc((size_t)(stride * nstage + 1));
        /* table of compact indices: offsets with at least two non-zero digits, numbered in ascending order (:63-73) */
        table = (int *)malloc(sizeof(int) * (size_t)P);
        for (int i = 0; i < P; i++) table[i] = -1;
        int di = 0, dist = 1;
        for (int x = 0; x < w; x++) {
            for (int z = 1; z < r; z++) {
                int sp = z * dist;
                if (sp > P) break;
                int end = sp + dist > P ? P : sp + dist;
                for (int i = sp + 1; i < end; i++) table[i] = di++;
            }
            dist *= r;
        }
    }
    self_copies(&c);

    int *offs = (int *)malloc(sizeof(int) * (size_t)(nlpow > 0 ? nlpow : 1));
    ora_msg **inbox = (ora_msg **)calloc((size_t)r, sizeof(ora_msg *));     /* [z][rank]: what rank received in round z */
    int *nbs = (int *)calloc((size_t)r, sizeof(int));
    for (int z = 0; z < r; z++) inbox[z] = (ora_msg *)calloc((size_t)P, sizeof(ora_msg));
    int dist = 1;
    for (int x = 0; x < w; x++) {
        int ze = (x == w - 1) ? r - d : r;
        int64_t ndist = (int64_t)dist * r;
        for (int k = 1; k < ze; k += b) {
            int ss = ze - k < b ? ze - k : b;
            for (int si = 0; si < ss; si++) {
                int z = k + si, hop = z * dist;
                int nc = (int)(P / ndist) * dist, rem = (int)(P % ndist) - hop;           /* :127-129 */
                if (rem < 0) rem = 0;
                int ns = rem > dist ? nc + dist : nc + rem;
                nbs[z] = ns;
                if (ns == 1) {                                                      /* :136-141 */
                    for (int p = 0; p < P; p++) {
                        int from_rank = (p + hop) % P;
                        int64_t nbytes = (int64_t)SC(&c, from_rank, p) * esz;
                        memcpy(rbuf(&c, p) + (int64_t)RD(&c, p, from_rank) * esz,
                               sbuf(&c, from_rank) + (int64_t)SD(&c, from_rank, p) * esz, (size_t)nbytes);
                        trace_msg(1, x, z, from_rank, p, 1, nbytes);
                    }
                    continue;
                }
                int nb = digit_offsets(P, dist, r, z, offs);
                /* every rank packs (:150-185); rank p's message goes to p - hop, i.e. inbox[z][p - hop] */
                for (int p = 0; p < P; p++) {
                    int to = (p - hop + P) % P;
                    ora_msg *m = &inbox[z][to];
                    int64_t tot = 0;
                    for (int i = 0; i < nb; i++) {
                        int key = (p - offs[i] + P) % P;
                        tot += (int64_t)((i % dist == 0) ? SC(&c, p, key) : stage_cnt[(int64_t)p * nstage + table[offs[i]]]) * esz;
                    }
                    msg_reserve(m, nb, tot);
                    int64_t off = 0;
                    for (int i = 0; i < nb; i++) {
                        int key = (p - offs[i] + P) % P;
                        int cnt; const char *from;
                        if (i % dist == 0) { cnt = SC(&c, p, key); from = sbuf(&c, p) + (int64_t)SD(&c, p, key) * esz; }
                        else { int ci = table[offs[i]]; cnt = stage_cnt[(int64_t)p * nstage + ci]; from = stage[p] + (int64_t)ci * stride; }
                        m->sizes[i] = cnt;
                        memcpy(m->bytes + off, from, (size_t)((int64_t)cnt * esz));
                        off += (int64_t)cnt * esz;
                    }
                    trace_msg(0, x, z, p, to, nb, tot);
                }
            }
            /* MPI_Waitall of the batch (:190) */
        }
        /* deferred unpack of the whole digit (:202-223) */
        for (int z = 1; z < ze; z++) {
            if (nbs[z] <= 1) continue;
            int nb = digit_offsets(P, dist, r, z, offs);
            for (int p = 0; p < P; p++) {
                ora_msg *m = &inbox[z][p];
                int64_t off = 0;
                for (int i = 0; i < nb; i++) {
                    int slot = (offs[i] + p) % P;
                    int64_t nbytes = (int64_t)m->sizes[i] * esz;
                    if (i < dist) {
                        memcpy(rbuf(&c, p) + (int64_t)RD(&c, p, slot) * esz, m->bytes + off, (size_t)nbytes);
                    } else {
                        int ci = table[offs[i]];
                        memcpy(stage[p] + (int64_t)ci * stride, m->bytes + off, (size_t)nbytes);
                        stage_cnt[(int64_t)p * nstage + ci] = m->sizes[i];
                    }
                    off += nbytes;
                }
                msg_release(m);
            }
        }
        dist *= r;
    }
    for (int z = 0; z < r; z++) free(inbox[z]);
    for (int p = 0; p < P; p++) free(stage[p]);
    free(inbox); free(nbs); free(offs); free(stage); free(stage_cnt); free(table);
    return 0;
}

/* compact staging index of offset j (>= 2 non-zero digits), float form of tuna.cpp:93-97; exported for tests */
int ora_compact_slot_float(int j, int r) { return compact_slot_float(j, r); }

/* ----------------------------- 4/5. two-phase two-layer, non-uniform (TTPL) */

typedef struct {
    int n, ngroup, sw, r;
    int64_t stride;
    int *cur;       /* [P][P] updated_sentcouts */
    char *moved;    /* [P][P] pos_status */
    char **extra;   /* [P] P slots each */
} ttpl_state;

/* Intra-node Bruck over local offsets, LSD first, carrying one sub-list per
 * destination group (src/twophase_twolayer_rbruck.cpp:311-384 and :541-619).
 * `finals_to_recvbuf` is the staggered variant's unpack rule (:603-609). */
static void ttpl_intra(ora_ctx *c, ttpl_state *st, int finals_to_recvbuf) {
    int P = c->P, esz = c->esz, n = st->n, ngroup = st->ngroup, r = st->r;
    int *loc = (int *)malloc(sizeof(int) * (size_t)n);
    ora_msg *box = (ora_msg *)calloc((size_t)P, sizeof(ora_msg));
    int dist = 1;
    for (int x = 0; x < st->sw; x++) {
        int64_t ndist = (int64_t)dist * r;
        for (int z = 1; z < r; z++) {
            int hop = z * dist;
            if (hop > n - 1) break;                                 /* :314 */
            int nl = digit_offsets(n, dist, r, z, loc);
            int nb = nl * ngroup;
            for (int p = 0; p < P; p++) {
                int grank = p % n;
                int64_t tot = 0;
                for (int g = 0; g < ngroup; g++)
                    for (int i = 0; i < nl; i++) {
                        int slot = g * n + (loc[i] + grank) % n;
                        int key = g * n + (2 * grank - slot % n + n) % n;       /* rotate_index_array, :290-295 */
                        tot += (int64_t)st->cur[(int64_t)p * P + key] * esz;
                    }
                msg_reserve(&box[p], nb, tot);
                int64_t off = 0; int k = 0;
                for (int g = 0; g < ngroup; g++)
                    for (int i = 0; i < nl; i++, k++) {
                        int slot = g * n + (loc[i] + grank) % n;
                        int key = g * n + (2 * grank - slot % n + n) % n;
                        int cnt = st->cur[(int64_t)p * P + key];
                        const char *from = st->moved[(int64_t)p * P + key]
                                               ? st->extra[p] + (int64_t)slot * st->stride
                                               : sbuf(c, p) + (int64_t)SD(c, p, key) * esz;
                        box[p].sizes[k] = cnt;
                        memcpy(box[p].bytes + off, from, (size_t)((int64_t)cnt * esz));
                        off += (int64_t)cnt * esz;
                    }
            }
            for (int p = 0; p < P; p++) {
                int grank = p % n, gid = p / n;
                int from_rank = gid * n + (grank + hop) % n;         /* :345 */
                const ora_msg *m = &box[from_rank];
                trace_msg(0, x, z, from_rank, p, nb, m->nbytes);
                int64_t off = 0; int k = 0;
                for (int g = 0; g < ngroup; g++)
                    for (int i = 0; i < nl; i++, k++) {
                        int slot = g * n + (loc[i] + grank) % n;
                        int key = g * n + (2 * grank - slot % n + n) % n;
                        int64_t nbytes = (int64_t)m->sizes[k] * esz;
                        int origin = (slot % n - grank + n) % n;
                        if (finals_to_recvbuf && slot / n == gid && origin < ndist)     /* :603-605 */
                            memcpy(rbuf(c, p) + (int64_t)RD(c, p, slot) * esz, m->bytes + off, (size_t)nbytes);
                        else
                            memcpy(st->extra[p] + (int64_t)slot * st->stride, m->bytes + off, (size_t)nbytes);
                        off += nbytes;
                        st->moved[(int64_t)p * P + key] = 1;
                        st->cur[(int64_t)p * P + key] = m->sizes[k];
                    }
            }
            for (int p = 0; p < P; p++) msg_release(&box[p]);
        }
        dist *= r;
    }
    free(loc); free(box);
}

static int ttpl_setup(ora_ctx *c, ttpl_state *st, int n, int r) {
    int P = c->P;
    if (n < 1 || P % n != 0) return -2;         /* the reference truncates P/n and hangs (:260) */
    if (r > n) r = n;                           /* :248 */
    st->n = n; st->ngroup = P / n; st->r = r;
    st->sw = (n > 1) ? (int)ceil(log((double)n) / (float)log((double)r)) : 0;   /* :263 */
    st->stride = (int64_t)global_max_count(c) * c->esz;
    st->cur = (int *)malloc(sizeof(int) * (size_t)P * P);
    memcpy(st->cur, c->sc, sizeof(int) * (size_t)P * P);                        /* :298 */
    st->moved = (char *)calloc((size_t)P * P, 1);
    st->extra = (char **)malloc(sizeof(char *) * (size_t)P);
    for (int p = 0; p < P; p++) st->extra[p] = (char *)malloc((size_t)(st->stride * P + 1));
    return 0;
}

static void ttpl_teardown(ora_ctx *c, ttpl_state *st) {
    for (int p = 0; p < c->P; p++) free(st->extra[p]);
    free(st->extra); free(st->cur); free(st->moved);
}

int ora_TTPL_BT_alltoallv(int n, int r, int bblock, char *sendarena, const int64_t *sbase,
                          const int *sendcounts, const int *sdispls, int esz, char *recvarena,
                          const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    if (r < 2) return -1;                       /* :242 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    ttpl_state st;
    int rc = ttpl_setup(&c, &st, n, r);
    if (rc) return rc;
    int ngroup = st.ngroup;
    ttpl_intra(&c, &st, 0);

    /* organize (:388-398): all P slots of a rank back to back, slot order; then per-group
     * totals and byte displacements on both sides (:406-418) */
    char **org = (char **)malloc(sizeof(char *) * (size_t)P);
    int64_t *nsend = (int64_t *)malloc(sizeof(int64_t) * (size_t)P * ngroup);
    int64_t *nsdisp = (int64_t *)malloc(sizeof(int64_t) * (size_t)P * ngroup);
    int64_t *nrecv = (int64_t *)malloc(sizeof(int64_t) * (size_t)P * ngroup);
    int64_t *nrdisp = (int64_t *)malloc(sizeof(int64_t) * (size_t)P * ngroup);
    for (int p = 0; p < P; p++) {
        int grank = p % n;
        int64_t tot = 0;
        for (int i = 0; i < P; i++) {
            int key = (i / n) * n + (2 * grank - i % n + n) % n;
            tot += (int64_t)st.cur[(int64_t)p * P + key] * esz;
        }
        org[p] = (char *)malloc((size_t)(tot + 1));
        int64_t off = 0;
        for (int i = 0; i < P; i++) {
            int key = (i / n) * n + (2 * grank - i % n + n) % n;
            int64_t nbytes = (int64_t)st.cur[(int64_t)p * P + key] * esz;
            const char *from = (grank == i % n) ? sbuf(&c, p) + (int64_t)SD(&c, p, i) * esz
                                                : st.extra[p] + (int64_t)i * st.stride;
            memcpy(org[p] + off, from, (size_t)nbytes);
            off += nbytes;
        }
        int64_t so = 0, ro = 0;
        for (int g = 0; g < ngroup; g++) {
            int64_t ns = 0, nr = 0;
            for (int j = 0; j < n; j++) {
                int id = g * n + j;
                int key = g * n + (2 * grank - j + n) % n;
                ns += st.cur[(int64_t)p * P + key];
                nr += RC(&c, p, id);
            }
            nsend[(int64_t)p * ngroup + g] = ns * esz; nrecv[(int64_t)p * ngroup + g] = nr * esz;
            nsdisp[(int64_t)p * ngroup + g] = so; nrdisp[(int64_t)p * ngroup + g] = ro;
            so += ns * esz; ro += nr * esz;
        }
    }
    /* inter-node: bblock groups at a time (:420-453).  The receive side is the packed,
     * source-rank-ordered layout; rdispls is never read. */
    if (bblock <= 0 || bblock > ngroup) bblock = ngroup;
    for (int ii = 0; ii < ngroup; ii += bblock) {
        int ss = ngroup - ii < bblock ? ngroup - ii : bblock;
        for (int p = 0; p < P; p++) {
            int grank = p % n, gid = p / n;
            for (int i = 0; i < ss; i++) {
                int ndst = (gid - i - ii + 2 * ngroup) % ngroup;
                int dst = ndst * n + grank;
                int64_t nbytes = nsend[(int64_t)p * ngroup + ndst];
                memcpy(rbuf(&c, dst) + nrdisp[(int64_t)dst * ngroup + gid],
                       org[p] + nsdisp[(int64_t)p * ngroup + ndst], (size_t)nbytes);
                trace_msg(2, -1, i + ii, p, dst, n, nbytes);
            }
        }
    }
    for (int p = 0; p < P; p++) free(org[p]);
    free(org); free(nsend); free(nsdisp); free(nrecv); free(nrdisp);
    ttpl_teardown(&c, &st);
    return 0;
}

int ora_TTPL_BT_alltoallv_s1(int n, int r, int bblock, char *sendarena, const int64_t *sbase,
                             const int *sendcounts, const int *sdispls, int esz, char *recvarena,
                             const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    if (r < 2) return -1;                       /* :472 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    ttpl_state st;
    int rc = ttpl_setup(&c, &st, n, r);
    if (rc) return rc;
    int ngroup = st.ngroup;
    self_copies(&c);                            /* :535 */
    ttpl_intra(&c, &st, 1);

    /* inter-node, one message per block, bblock (group distance, local index) pairs at a
     * time, own group skipped (:623-671) */
    if (bblock <= 0 || bblock > P) bblock = P;
    for (int ii = 0; ii < P; ii += bblock) {
        int ss = P - ii < bblock ? P - ii : bblock;
        for (int p = 0; p < P; p++) {
            int grank = p % n, gid = p / n;
            for (int i = 0; i < ss; i++) {
                int gi = (ii + i) / n, gr = (ii + i) % n;
                int ndst = (gid - gi + ngroup) % ngroup;
                if (ndst == gid) continue;
                int dst = ndst * n + grank;
                int id = ndst * n + gr;
                int key = ndst * n + (2 * grank - gr + n) % n;
                int64_t nbytes = (int64_t)st.cur[(int64_t)p * P + key] * esz;
                const char *from = (gr == grank) ? sbuf(&c, p) + (int64_t)SD(&c, p, id) * esz
                                                 : st.extra[p] + (int64_t)id * st.stride;
                /* the receiver posted Irecv(recvbuf + rdispls[gid*n + gr], src = p, tag = gr) (:647) */
                memcpy(rbuf(&c, dst) + (int64_t)RD(&c, dst, gid * n + gr) * esz, from, (size_t)nbytes);
                trace_msg(3, -1, gi, p, dst, 1, nbytes);
            }
        }
    }
    ttpl_teardown(&c, &st);
    return 0;
}

/* src/twophase_twolayer_rbruck.cpp:15-235: the intra-node phase is the staggered variant's (:88-168: finals of the own
 * node go to recvbuf, :151-152); then a Bruck over the nodes, least significant digit of the group offset first,
 * between ranks of equal local index: in round (x, z) a rank sends to the rank z*r^x nodes below (:211) the n blocks
 * of every group slot whose offset has digit x equal to z (:186-207).  The reference frees its buffers right after
 * the exchange (:222-231); the unpack below is what its intra-node phase does at :147-161, applied to group offsets:
 * a block whose offset has no higher non-zero digit is final, every other one waits in a slot. */
int ora_TTPL_rbruck_alltoallv(int n, int r, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                              int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    if (r < 2) return -1;                       /* :20 */
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    ttpl_state st;
    int rc = ttpl_setup(&c, &st, n, r);         /* :26 clamps r to n */
    if (rc) return rc;
    int ngroup = st.ngroup;
    r = st.r < 2 ? 2 : st.r;                    /* n == 1 would leave radix 1 (:26), which has no digits */
    self_copies(&c);                            /* :86 */
    ttpl_intra(&c, &st, 1);

    /* slot (jg, jj) of a rank: the block of group offset jg and source local index jj while it travels */
    char **xbuf = (char **)malloc(sizeof(char *) * (size_t)P);
    int *xcnt = (int *)calloc((size_t)P * P, sizeof(int));
    for (int p = 0; p < P; p++) xbuf[p] = (char *)malloc((size_t)(st.stride * P + 1));
    int *loc = (int *)malloc(sizeof(int) * (size_t)(ngroup > 0 ? ngroup : 1));
    ora_msg *box = (ora_msg *)calloc((size_t)P, sizeof(ora_msg));
    int gw = 0;
    for (int top = ngroup - 1; top; top /= r) gw++;                 /* = ceil(log(ngroup)/log(r)) of :45 */
    int dist = 1;
    for (int x = 0; x < gw; x++) {
        int64_t ndist = (int64_t)dist * r;
        for (int z = 1; z < r; z++) {
            int hop = z * dist;
            if (hop > ngroup - 1) break;                            /* :183 */
            int nl = digit_offsets(ngroup, dist, r, z, loc);        /* :187-193 */
            for (int p = 0; p < P; p++) {
                int grank = p % n, gid = p / n;
                int64_t tot = 0;
                for (int pass = 0; pass < 2; pass++) {
                    if (pass) msg_reserve(&box[p], nl * n, tot);
                    int64_t off = 0; int k = 0;
                    for (int i = 0; i < nl; i++)
                        for (int jj = 0; jj < n; jj++, k++) {
                            int jg = loc[i], cnt;
                            const char *from;
                            if (jg % dist == 0) {                   /* first hop between nodes: where the intra phase left it */
                                int gt = (gid - jg + ngroup) % ngroup;          /* inter_rotate, :171-174 */
                                int ci = gt * n + jj;
                                int key = gt * n + (2 * grank - jj + n) % n;
                                cnt = st.cur[(int64_t)p * P + key];
                                from = (jj == grank) ? sbuf(&c, p) + (int64_t)SD(&c, p, ci) * esz       /* :202-205 */
                                                     : st.extra[p] + (int64_t)ci * st.stride;
                            } else {
                                cnt = xcnt[(int64_t)p * P + jg * n + jj];
                                from = xbuf[p] + (int64_t)(jg * n + jj) * st.stride;
                            }
                            if (!pass) { tot += (int64_t)cnt * esz; continue; }
                            box[p].sizes[k] = cnt;
                            memcpy(box[p].bytes + off, from, (size_t)((int64_t)cnt * esz));
                            off += (int64_t)cnt * esz;
                        }
                }
            }
            for (int p = 0; p < P; p++) {
                int grank = p % n, gid = p / n;
                int from_rank = ((gid + hop) % ngroup) * n + grank;  /* :210 */
                const ora_msg *m = &box[from_rank];
                trace_msg(6, x, z, from_rank, p, nl * n, m->nbytes);
                int64_t off = 0; int k = 0;
                for (int i = 0; i < nl; i++)
                    for (int jj = 0; jj < n; jj++, k++) {
                        int jg = loc[i];
                        int64_t nbytes = (int64_t)m->sizes[k] * esz;
                        if (jg < ndist) {                            /* no higher digit: this rank is the destination */
                            int src = ((gid + jg) % ngroup) * n + jj;
                            memcpy(rbuf(&c, p) + (int64_t)RD(&c, p, src) * esz, m->bytes + off, (size_t)nbytes);
                        } else {
                            memcpy(xbuf[p] + (int64_t)(jg * n + jj) * st.stride, m->bytes + off, (size_t)nbytes);
                            xcnt[(int64_t)p * P + jg * n + jj] = m->sizes[k];
                        }
                        off += nbytes;
                    }
            }
            for (int p = 0; p < P; p++) msg_release(&box[p]);
        }
        dist *= r;
    }
    for (int p = 0; p < P; p++) free(xbuf[p]);
    free(xbuf); free(xcnt); free(loc); free(box);
    ttpl_teardown(&c, &st);
    return 0;
}

/* ------------------------------------------------ 6/7. two-layer, uniform */

/* In-place local rotation of every group's n blocks: block id swaps with
 * gsp + (2*grank - j) mod n (src/twolayer_rbruck.cpp:51-63).  The reference
 * marks visited blocks in recvbuf[0..P); a private array is equivalent as
 * long as recvbuf held no '1' bytes there on entry. */
static void uniform_rotate(char *buf, int P, int n, int grank, int64_t unit, char *tmp) {
    char *seen = (char *)calloc((size_t)P, 1);
    for (int g = 0; g < P / n; g++)
        for (int j = 0; j < n; j++) {
            int id = g * n + j, rid = g * n + (2 * grank - j + n) % n;
            if (rid == id || seen[id]) continue;
            memcpy(tmp, buf + id * unit, (size_t)unit);
            memcpy(buf + id * unit, buf + rid * unit, (size_t)unit);
            memcpy(buf + rid * unit, tmp, (size_t)unit);
            seen[id] = seen[rid] = 1;
        }
    free(seen);
}

/* Intra-node Bruck, MSD first, equal blocks, staged in sendbuf itself
 * (src/twolayer_rbruck.cpp:66-104 and :195-231). */
static void uniform_intra(ora_ctx *c, int n, int r, int64_t unit) {
    int P = c->P, ngroup = P / n;
    int sw = (int)ceil(log((double)n) / (float)log((double)r));
    int sd = (ora_pow(r, (unsigned)sw) - n) / ora_pow(r, (unsigned)(sw - 1));
    int *loc = (int *)malloc(sizeof(int) * (size_t)n);
    char **box = (char **)malloc(sizeof(char *) * (size_t)P);
    int dist = ora_pow(r, (unsigned)(sw - 1));
    for (int x = sw - 1; x >= 0; x--) {
        int ze = (x == sw - 1) ? r - 1 - sd : r - 1;
        for (int z = ze; z > 0; z--) {
            int hop = z * dist;
            int nl = digit_offsets(n, dist, r, z, loc);
            int64_t nb = (int64_t)nl * ngroup;
            for (int p = 0; p < P; p++) {
                int grank = p % n; int64_t k = 0;
                box[p] = (char *)malloc((size_t)(nb * unit + 1));
                for (int g = 0; g < ngroup; g++)
                    for (int i = 0; i < nl; i++, k++)
                        memcpy(box[p] + k * unit, sbuf(c, p) + (int64_t)(g * n + (loc[i] + grank) % n) * unit, (size_t)unit);
            }
            for (int p = 0; p < P; p++) {
                int grank = p % n, gid = p / n; int64_t k = 0;
                int from_rank = gid * n + (grank + hop) % n;
                trace_msg(0, x, z, from_rank, p, (int)nb, nb * unit);
                for (int g = 0; g < ngroup; g++)
                    for (int i = 0; i < nl; i++, k++)
                        memcpy(sbuf(c, p) + (int64_t)(g * n + (loc[i] + grank) % n) * unit, box[from_rank] + k * unit, (size_t)unit);
            }
            for (int p = 0; p < P; p++) free(box[p]);
        }
        dist /= r;
    }
    free(loc); free(box);
}

int ora_uniform_spreadout_twolayer(int n, int r, char *sendarena, const int64_t *sbase, int sendcount,
                                   int esz, char *recvarena, const int64_t *rbase, int P) {
    if (r < 2) return -1;                                   /* :12 */
    if (n < 2 || n >= P || P % n != 0) return -2;           /* :18-22 aborts (and misses n ∤ P) */
    ora_ctx c = make_ctx(sendarena, sbase, NULL, NULL, esz, recvarena, rbase, NULL, NULL, P);
    int64_t unit = (int64_t)sendcount * esz;
    int ngroup = P / n;
    if (r > n) r = n;
    char *tmp = (char *)malloc((size_t)(unit + 1));
    for (int p = 0; p < P; p++) uniform_rotate(sbuf(&c, p), P, n, p % n, unit, tmp);
    free(tmp);
    uniform_intra(&c, n, r, unit);
    /* spread-out of n-block chunks between ranks with the same local index (:106-128) */
    int64_t chunk = unit * n;
    for (int p = 0; p < P; p++) {
        int grank = p % n, gid = p / n;
        for (int i = 0; i < ngroup; i++) {
            int ndst = (gid - i + ngroup) % ngroup;
            int dst = ndst * n + grank;
            memcpy(rbuf(&c, dst) + gid * chunk, sbuf(&c, p) + ndst * chunk, (size_t)chunk);
            trace_msg(2, -1, i, p, dst, n, chunk);
        }
    }
    return 0;
}

int ora_uniform_inverse_isplit_r_bruck(int n, int r1, int r2, char *sendarena, const int64_t *sbase,
                                       int sendcount, int esz, char *recvarena, const int64_t *rbase, int P) {
    (void)r2;
    if (r1 < 2) r1 = 2;                                     /* :143 */
    if (n < 2 || n >= P || P % n != 0) return -2;           /* :145-149 aborts */
    ora_ctx c = make_ctx(sendarena, sbase, NULL, NULL, esz, recvarena, rbase, NULL, NULL, P);
    int64_t unit = (int64_t)sendcount * esz;
    int ngroup = P / n;
    int rg = ngroup;                                        /* r2 is overwritten, :158 */
    if (r1 > n) r1 = n;
    int gw = (int)ceil(log((double)ngroup) / (float)log((double)rg));
    int glpow = ora_pow(rg, (unsigned)(gw - 1));
    int gd = (ora_pow(rg, (unsigned)gw) - ngroup) / glpow;

    char *tmp = (char *)malloc((size_t)(unit + 1));
    for (int p = 0; p < P; p++) uniform_rotate(sbuf(&c, p), P, n, p % n, unit, tmp);
    free(tmp);
    uniform_intra(&c, n, r1, unit);

    /* group-level rotation into recvbuf (:233-240) */
    int64_t chunk = unit * n;
    for (int p = 0; p < P; p++) {
        int gid = p / n;
        for (int i = 0; i < ngroup; i++) {
            int index = (2 * gid - i + ngroup) % ngroup;
            memcpy(rbuf(&c, p) + index * chunk, sbuf(&c, p) + i * chunk, (size_t)chunk);
        }
    }
    /* group-level Bruck, MSD first, staged in recvbuf (:242-274) */
    int *goff = (int *)malloc(sizeof(int) * (size_t)ngroup);
    char **box = (char **)malloc(sizeof(char *) * (size_t)P);
    int dist = glpow;
    for (int x = gw - 1; x >= 0; x--) {
        int ze = (x == gw - 1) ? rg - 1 - gd : rg - 1;
        for (int z = ze; z > 0; z--) {
            int hop = z * dist;
            int nb = digit_offsets(ngroup, dist, rg, z, goff);
            for (int p = 0; p < P; p++) {
                int gid = p / n;
                box[p] = (char *)malloc((size_t)(nb * chunk + 1));
                for (int i = 0; i < nb; i++)
                    memcpy(box[p] + i * chunk, rbuf(&c, p) + (int64_t)((goff[i] + gid) % ngroup) * chunk, (size_t)chunk);
            }
            for (int p = 0; p < P; p++) {
                int gid = p / n;
                int from_rank = (int)(((int64_t)p + (int64_t)hop * n) % P);      /* :258 */
                trace_msg(2, x, z, from_rank, p, nb * n, nb * chunk);
                for (int i = 0; i < nb; i++)
                    memcpy(rbuf(&c, p) + (int64_t)((goff[i] + gid) % ngroup) * chunk, box[from_rank] + i * chunk, (size_t)chunk);
            }
            for (int p = 0; p < P; p++) free(box[p]);
        }
        dist /= rg;
    }
    free(goff); free(box);
    return 0;
}

/* ------------------------------------------------ linear comparators -------
 * One message per (source, destination) pair, straight between the user buffers.
 * They differ only in the order and batching of the messages and in which empty
 * messages are skipped. */

static void direct_message(const ora_ctx *c, int from, int to, int step) {
    int64_t nbytes = (int64_t)SC(c, from, to) * c->esz;
    memcpy(rbuf(c, to) + (int64_t)RD(c, to, from) * c->esz, sbuf(c, from) + (int64_t)SD(c, from, to) * c->esz, (size_t)nbytes);
    trace_msg(5, -1, step, from, to, 1, nbytes);
}

/* benchmarks/common.cpp:10-37: rank p receives from p+i and sends to p-i for i = 0..P-1, one Waitall. */
int ora_spreadout_alltoallv(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls, int esz,
                            char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    for (int p = 0; p < P; p++)
        for (int i = 0; i < P; i++) direct_message(&c, p, (p - i + P) % P, i);
    return 0;
}

/* src/MPICH_scattered.cpp:31-70: the same pairs, bblock at a time, empty messages not posted. */
int ora_MPICH_intra_scattered(int bblock, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                              int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    if (bblock <= 0 || bblock > P) bblock = P;                        /* :31 */
    for (int ii = 0; ii < P; ii += bblock) {
        int ss = P - ii < bblock ? P - ii : bblock;
        for (int p = 0; p < P; p++)
            for (int i = 0; i < ss; i++) {
                int dst = (p - i - ii + 2 * P) % P;                   /* :56 */
                if (SC(&c, p, dst)) direct_message(&c, p, dst, i + ii);
            }
    }
    return 0;
}

/* src/OpenMPI_basic_linear.cpp:10-77: memcpy to self, then all receives and all sends of non-empty messages. */
int ora_ompi_alltoallv_intra_basic_linear(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                          int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                          const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    self_copies(&c);                                                   /* :28-30 */
    for (int p = 0; p < P; p++) if (SC(&c, p, p) < 0) return -1;       /* :32 */
    for (int p = 0; p < P; p++)
        for (int i = 0; i < P; i++)
            if (i != p && SC(&c, p, i) > 0) direct_message(&c, p, i, (p - i + P) % P);
    return 0;
}

/* src/OpenMPI_pairwise.cpp:32-58: step = 0..P-1, send to rank+step, receive from rank-step. */
int ora_ompi_alltoallv_intra_pairwise(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                      int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                      const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    for (int step = 0; step < P; step++)
        for (int p = 0; p < P; p++) {
            int to = (p + step) % P;
            if (SC(&c, p, to) > 0) direct_message(&c, p, to, step);
        }
    return 0;
}

/* src/exclusive_or_alltoallv.cpp:12-51: partner = rank XOR step; only for P a power of two (:31). */
int ora_exclisive_or_alltoallv(char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls, int esz,
                               char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    int w = (int)ceil(log((double)P) / (float)log(2.0));              /* :25 */
    if (P != ora_pow(2, (unsigned)w)) return -1;                       /* :31 */
    for (int step = 0; step < P; step++)
        for (int p = 0; p < P; p++) direct_message(&c, p, p ^ step, step);
    return 0;
}

/* src/twolayer_communicator_linear.cpp:13-88 and :92-192: MPICH_intra_scattered on the ranks of the own node (bblock1
 * at a time, 0 = all), then the messages between nodes: all posted before one Waitall (plain), or bblock2 at a time
 * over ii = 1 .. P-1 with gi = ii / n the group distance and gr = ii % n the source's local index on the receiving
 * side (_s2; the sender posts the same message in batch gi * n + destination's local index, so on a real network it
 * completes in the later of the two). */
static int twolayer_linear(int n, int bblock1, int bblock2, int batched_inter, ora_ctx *c) {
    int P = c->P;
    if (n < 1 || n >= P || P % n != 0) return -2;                        /* :24-28 aborts (and misses n that does not divide P) */
    int ngroup = P / n;
    if (bblock1 <= 0 || bblock1 > n) bblock1 = n;                        /* MPICH_scattered.cpp:31 on the node communicator */
    for (int ii = 0; ii < n; ii += bblock1) {
        int ss = n - ii < bblock1 ? n - ii : bblock1;
        for (int p = 0; p < P; p++)
            for (int i = 0; i < ss; i++) {
                int dst = p / n * n + (p % n - i - ii + 2 * n) % n;
                if (SC(c, p, dst)) direct_message(c, p, dst, i + ii);
            }
    }
    if (!batched_inter) {
        for (int p = 0; p < P; p++)
            for (int i = 1; i < ngroup; i++)                              /* :55-83 */
                for (int j = 0; j < n; j++) direct_message(c, p, ((p / n + i) % ngroup) * n + j, i);
        return 0;
    }
    if (bblock2 <= 0 || bblock2 > P) bblock2 = P;                        /* :132-133 */
    for (int ii = 1; ii < P; ii += bblock2) {
        int ss = P - ii < bblock2 ? P - ii : bblock2;
        for (int p = 0; p < P; p++)
            for (int i = 0; i < ss; i++) {
                int gi = (ii + i) / n, gr = (ii + i) % n;
                int nsrc = (p / n - gi + ngroup) % ngroup;                /* :152; a message is attributed to the batch */
                if (nsrc == p / n) continue;                              /* in which its receive is posted            */
                direct_message(c, nsrc * n + gr, p, ii + i);
            }
    }
    return 0;
}

int ora_twolayer_communicator_linear(int n, char *sendarena, const int64_t *sbase, const int *sendcounts, const int *sdispls,
                                     int esz, char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    return twolayer_linear(n, 0, 0, 0, &c);
}

int ora_twolayer_communicator_linear_s2(int n, int bblock1, int bblock2, char *sendarena, const int64_t *sbase, const int *sendcounts,
                                        const int *sdispls, int esz, char *recvarena, const int64_t *rbase, const int *recvcounts,
                                        const int *rdispls, int P) {
    ora_ctx c = make_ctx(sendarena, sbase, sendcounts, sdispls, esz, recvarena, rbase, recvcounts, rdispls, P);
    return twolayer_linear(n, bblock1, bblock2, 1, &c);
}

/* ------------------------------------------------------- payload + digests */

void ora_fill_payload(int mode, uint64_t seed, char *sendarena, const int64_t *sbase, const int *sendcounts,
                      const int *sdispls, int esz, int P) {
    for (int s = 0; s < P; s++)
        for (int t = 0; t < P; t++) {
            int64_t nbytes = (int64_t)sendcounts[(int64_t)s * P + t] * esz;
            unsigned char *at = (unsigned char *)sendarena + sbase[s] + (int64_t)sdispls[(int64_t)s * P + t] * esz;
            vc_fill_block(mode, seed, s, t, at, nbytes);
        }
}

void ora_digest_recv(const char *recvarena, const int64_t *rbase, const int *recvcounts, const int *rdispls,
                     int esz, int P, uint64_t *digest_out) {
    for (int t = 0; t < P; t++) {
        uint64_t h = VC_FNV_OFFSET;
        for (int s = 0; s < P; s++) {
            const unsigned char *at = (const unsigned char *)recvarena + rbase[t] + (int64_t)rdispls[(int64_t)t * P + s] * esz;
            h = vc_fnv1a64(at, (int64_t)recvcounts[(int64_t)t * P + s] * esz, h);
        }
        digest_out[t] = h;
    }
}
