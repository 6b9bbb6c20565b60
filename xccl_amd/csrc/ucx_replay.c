/*
 * ucx_replay.c -- libxccl_ucx_replay.so (see include/xccl_rocm_ucx_replay.h).
 *
 * Structure:
 *   1. loopback transport: tag-less FIFO matching per (sender, receiver) pair,
 *      one memcpy_async per matched pair on a transport stream, completion
 *      by sequence number against pooled mem-component events;
 *   2. k-nomial geometry and scatter-reduce segment arithmetic;
 *   3. four per-rank state machines (phase switch, re-entered until done);
 *   4. the driver that sweeps over the ranks.
 *
 * Every reduction goes through the dispatcher entry points of
 * include/xccl_rocm_mem_component.h, with the operands the reference call
 * sites pass (cited at each call).
 */
#include "xccl_rocm_ucx_replay.h"
#include "xccl_rocm_mem_component.h"

#include <hip/hip_runtime_api.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define MT          UCS_MEMORY_TYPE_ROCM
#define MAX_RADIX   17 /* 2*(radix-1) requests <= MAX_REQS = 32, reference xccl_ucx_lib.h:65 */
#define MAX_REQS    (2 * MAX_RADIX + 2)
#define MAX_MARKS   32 /* transport completion marks in flight: with one reduction event per rank
                          (<= 17) this stays inside the component's pool of 64 events */
#define WALL_LIMIT_S 120.0

enum { ROLE_BASE = 0, ROLE_PROXY = 1, ROLE_EXTRA = 2 };

/* ------------------------------------------------------------------------ */
/* 1. loopback transport                                                      */
/* ------------------------------------------------------------------------ */

typedef struct lb_req {
    int      active;
    int      is_send;
    int      from, to; /* sender rank, receiver rank */
    char    *buf;
    size_t   len;
    uint64_t seq;      /* 0 = not matched yet; else done once transport.done_seq >= seq */
    uint64_t stamp;    /* post order, for first-posted-first-matched */
} lb_req_t;

typedef struct lb_mark {
    uint64_t         seq;
    xccl_mc_event_t *ev;
} lb_mark_t;

typedef struct transport {
    hipStream_t   stream;
    xccl_stream_t xs;
    uint64_t      next_seq, done_seq, marked_seq, next_stamp;
    lb_mark_t     marks[MAX_MARKS];
    int           mark_head, mark_count;
    lb_req_t     *reqs; /* team_size * MAX_REQS slots; rank r owns [r*MAX_REQS, (r+1)*MAX_REQS) */
    int           team_size;
    xccl_replay_stats_t *stats;
} transport_t;

static xccl_status_t tr_init(transport_t *t, int team_size, xccl_replay_stats_t *stats)
{
    memset(t, 0, sizeof(*t));
    if (hipStreamCreateWithFlags(&t->stream, hipStreamNonBlocking) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    t->xs.type   = XCCL_STREAM_TYPE_ROCM;
    t->xs.stream = &t->stream;
    t->team_size = team_size;
    t->stats     = stats;
    t->reqs      = (lb_req_t *)calloc((size_t)team_size * MAX_REQS, sizeof(lb_req_t));
    return t->reqs ? XCCL_OK : XCCL_ERR_NO_MEMORY;
}

static void tr_destroy(transport_t *t)
{
    int i;
    if (t->stream) {
        (void)hipStreamSynchronize(t->stream);
    }
    for (i = 0; i < t->mark_count; i++) {
        xccl_mc_event_free(t->marks[(t->mark_head + i) % MAX_MARKS].ev);
    }
    if (t->stream) {
        (void)hipStreamDestroy(t->stream);
    }
    free(t->reqs);
    memset(t, 0, sizeof(*t));
}

/* Retire completion marks in stream order. */
static xccl_status_t tr_progress(transport_t *t)
{
    while (t->mark_count > 0) {
        lb_mark_t    *m  = &t->marks[t->mark_head];
        xccl_status_t st = xccl_mc_event_query(m->ev);
        if (st == XCCL_INPROGRESS) {
            return XCCL_OK;
        }
        if (st != XCCL_OK) {
            return st;
        }
        t->done_seq = m->seq;
        xccl_mc_event_free(m->ev);
        t->mark_head = (t->mark_head + 1) % MAX_MARKS;
        t->mark_count--;
    }
    if (t->done_seq < t->next_seq && t->marked_seq < t->next_seq) {
        /* copies were enqueued past the last mark (the event pool was empty) */
        if (hipStreamSynchronize(t->stream) != hipSuccess) {
            return XCCL_ERR_NO_MESSAGE;
        }
        t->done_seq = t->marked_seq = t->next_seq;
    }
    return XCCL_OK;
}

/* One enqueued copy; returns its sequence number through *seq. */
static xccl_status_t tr_copy(transport_t *t, const void *src, void *dst, size_t len, uint64_t *seq)
{
    xccl_mc_event_t *ev = NULL;
    xccl_status_t    st;

    st = xccl_mem_component_memcpy_async((void *)src, dst, len, &t->xs);
    if (st != XCCL_OK) {
        return st;
    }
    *seq = ++t->next_seq;
    t->stats->messages++;
    t->stats->bytes_moved += len;
    if (t->mark_count < MAX_MARKS && xccl_mc_event_record(&t->xs, &ev) == XCCL_OK) {
        lb_mark_t *m = &t->marks[(t->mark_head + t->mark_count) % MAX_MARKS];
        m->seq       = *seq;
        m->ev        = ev;
        t->mark_count++;
        t->marked_seq = *seq;
    }
    return XCCL_OK;
}

/* Posts a send (me -> peer) or a receive (peer -> me) and pairs it with the
 * oldest unmatched counterpart, as tag matching does for one (pair, tag). */
static xccl_status_t tr_post(transport_t *t, int is_send, int me, int peer, void *buf, size_t len, lb_req_t **out)
{
    lb_req_t *mine = NULL, *other = NULL, *slots;
    int       i, from = is_send ? me : peer, to = is_send ? peer : me;

    slots = &t->reqs[(size_t)me * MAX_REQS];
    for (i = 0; i < MAX_REQS; i++) {
        if (!slots[i].active) {
            mine = &slots[i];
            break;
        }
    }
    if (mine == NULL || peer < 0 || peer >= t->team_size) {
        return XCCL_ERR_NO_RESOURCE;
    }
    mine->active  = 1;
    mine->is_send = is_send;
    mine->from    = from;
    mine->to      = to;
    mine->buf     = (char *)buf;
    mine->len     = len;
    mine->seq     = 0;
    mine->stamp   = ++t->next_stamp;
    *out          = mine;

    slots = &t->reqs[(size_t)peer * MAX_REQS];
    for (i = 0; i < MAX_REQS; i++) {
        lb_req_t *r = &slots[i];
        if (r->active && r->seq == 0 && r->is_send != is_send && r->from == from && r->to == to) {
            if (other == NULL || r->stamp < other->stamp) {
                other = r;
            }
        }
    }
    if (other != NULL) {
        lb_req_t *snd = is_send ? mine : other, *rcv = is_send ? other : mine;
        uint64_t  seq;
        xccl_status_t st;
        if (snd->len > rcv->len) {
            return XCCL_ERR_MESSAGE_TRUNCATED;
        }
        st = tr_copy(t, snd->buf, rcv->buf, snd->len, &seq);
        if (st != XCCL_OK) {
            return st;
        }
        snd->seq = rcv->seq = seq;
    }
    return XCCL_OK;
}

static int tr_req_done(const transport_t *t, const lb_req_t *r)
{
    return r->seq != 0 && r->seq <= t->done_seq;
}

/* ------------------------------------------------------------------------ */
/* 2. geometry                                                                */
/* ------------------------------------------------------------------------ */

/* allreduce_knomial.h:10-34 */
void xccl_replay_knomial_geometry(int radix, int rank, int team_size, int *rounds, int *full_size, int *role)
{
    int levels = 1, reach = radix, tree, nsub, full;

    while (reach < team_size) {
        levels++;
        reach *= radix;
    }
    tree = (reach != team_size) ? reach / radix : reach; /* largest complete subtree */
    if (reach != team_size && team_size / tree == 1) {
        levels--; /* a single complete subtree: no round between subtrees */
    }
    nsub = team_size / tree;
    full = nsub * tree;
    if (rounds) {
        *rounds = levels;
    }
    if (full_size) {
        *full_size = full;
    }
    if (role) {
        *role = rank >= full ? ROLE_EXTRA : (team_size > full && rank < team_size - full) ? ROLE_PROXY : ROLE_BASE;
    }
}

/* Peer k (1 <= k < radix) of `rank` in the round whose groups span radix_pow*radix ranks
 * (allreduce_knomial.c:91-93, allreduce_sra.c:14-17). */
static int kn_peer(int rank, int k, int radix_pow, int radix)
{
    const int span = radix_pow * radix;
    return (rank + k * radix_pow) % span + (rank - rank % span);
}

/* Segment arithmetic of the scatter-reduce, allreduce_sra.c:35-74: a block of
 * `block` elements is cut into `parts` segments, the first block % parts of
 * them one element longer. */
static size_t seg_index(int rank, int radix_pow, int radix)
{
    return (size_t)((rank % (radix_pow * radix)) / radix_pow);
}

static size_t seg_size(size_t block, size_t parts, size_t i)
{
    return block / parts + (i < block % parts ? 1 : 0);
}

static size_t seg_offset(size_t block, size_t parts, size_t i)
{
    const size_t rem = block % parts;
    return (block / parts) * i + (i < rem ? i : rem);
}

/* Size of the block `rank` works on in round `step` (allreduce_sra.c:62-75;
 * cuts by the full radix: every round below the top one has complete groups). */
static size_t block_count_at(size_t count, int radix, int rank, int step)
{
    size_t block = count;
    int    i, kpow = 1;

    for (i = 0; i < step; i++) {
        block = seg_size(block, (size_t)radix, seg_index(rank, kpow, radix));
        kpow *= radix;
    }
    return block;
}

static int step_radix_of(int rank, int radix_pow, int radix, int full_size)
{
    int k, n = 1;
    for (k = 1; k < radix; k++) {
        if (kn_peer(rank, k, radix_pow, radix) < full_size) {
            n++;
        }
    }
    return n;
}

/* allreduce_sra.c:77-127 */
void xccl_replay_sra_segment(size_t count, int rank, int radix, int team_size, size_t *offset, size_t *length)
{
    int    rounds, full, role, step, radix_pow = 1, parts = 1;
    size_t block = count, off = 0, si = 0;

    xccl_replay_knomial_geometry(radix, rank, team_size, &rounds, &full, &role);
    if (role == ROLE_EXTRA) {
        if (offset) {
            *offset = 0;
        }
        if (length) {
            *length = count;
        }
        return;
    }
    for (step = 0; step < rounds; step++) {
        parts = step_radix_of(rank, radix_pow, radix, full);
        si    = seg_index(rank, radix_pow, radix);
        off += seg_offset(block, (size_t)parts, si);
        if (step < rounds - 1) {
            block = seg_size(block, (size_t)parts, si);
            radix_pow *= radix;
        }
    }
    if (offset) {
        *offset = off;
    }
    if (length) {
        *length = seg_size(block, (size_t)parts, si);
    }
}

/* ------------------------------------------------------------------------ */
/* 3. per-rank state machines                                                 */
/* ------------------------------------------------------------------------ */

typedef struct ctx {
    const xccl_replay_params_t *p;
    xccl_replay_stats_t        *stats;
    transport_t                 tr;
    size_t                      esize, len; /* element bytes, vector bytes */
    int                         radix;
} ctx_t;

typedef struct rank_state {
    int   rank, phase, done;
    char *src, *dst, *scratch;
    int   scratch_owned;
    lb_req_t        *reqs[MAX_REQS];
    int              nreqs;
    xccl_mc_event_t *reduce_ev;
    uint64_t         copy_seq;
    /* k-nomial exchange */
    int rounds, full_size, role, iter, radix_pow, npeers;
    /* scatter-reduce / allgather */
    char  *cur_src, *recv_base, *ag_src;
    size_t block, local_cnt, local_off;
    /* rooted reduce */
    int   dist, max_dist, level_kind, next;
    char *data_buf, *rdst;
} rank_state_t;

static xccl_status_t post(ctx_t *c, rank_state_t *s, int is_send, int peer, void *buf, size_t len)
{
    lb_req_t     *req = NULL;
    xccl_status_t st;

    if (s->nreqs >= MAX_REQS) {
        return XCCL_ERR_NO_RESOURCE;
    }
    st = tr_post(&c->tr, is_send, s->rank, peer, buf, len, &req);
    if (req != NULL) {
        s->reqs[s->nreqs++] = req; /* tracked even if its copy failed, so that the slot is released */
    }
    return st;
}

/* XCCL_OK when every posted request of the rank has completed (they are
 * released then), XCCL_INPROGRESS otherwise -- xccl_ucx_testall. */
static xccl_status_t wait_all(ctx_t *c, rank_state_t *s)
{
    xccl_status_t st = tr_progress(&c->tr);
    int           i;

    if (st != XCCL_OK) {
        return st;
    }
    for (i = 0; i < s->nreqs; i++) {
        if (!tr_req_done(&c->tr, s->reqs[i])) {
            return XCCL_INPROGRESS;
        }
    }
    for (i = 0; i < s->nreqs; i++) {
        s->reqs[i]->active = 0;
    }
    s->nreqs = 0;
    return XCCL_OK;
}

static xccl_status_t scratch_alloc(ctx_t *c, rank_state_t *s, size_t bytes)
{
    void         *p  = NULL;
    xccl_status_t st = xccl_mem_component_alloc(&p, bytes, MT);
    if (st == XCCL_OK) {
        s->scratch       = (char *)p;
        s->scratch_owned = 1;
        c->stats->scratch_allocs++;
    }
    return st;
}

static void scratch_free(rank_state_t *s)
{
    if (s->scratch_owned) {
        xccl_mem_component_free(s->scratch, MT);
        s->scratch_owned = 0;
    }
    s->scratch = NULL;
}

/* Issues one reduction in the configured mode.  n2 == 0 means the 2-source
 * `reduce` entry; otherwise reduce_multi with n2 vectors at `stride`. */
static xccl_status_t issue_reduce(ctx_t *c, rank_state_t *s, void *s1, void *s2, void *out, size_t n2, size_t count,
                                  size_t stride)
{
    const xccl_replay_params_t *p = c->p;

    if (n2 == 0) {
        c->stats->reduce_calls++;
    } else {
        c->stats->reduce_multi_calls++;
        if (n2 > c->stats->max_multi_vectors) {
            c->stats->max_multi_vectors = n2;
        }
    }
    if (out == s1) {
        c->stats->inplace_sbuf1++;
    } else if (out == s2) {
        c->stats->inplace_sbuf2++;
    }
    s->reduce_ev = NULL;
    if (p->reduce_mode == XCCL_REPLAY_REDUCE_BLOCKING) {
        return n2 == 0 ? xccl_mem_component_reduce(s1, s2, out, count, p->dtype, p->op, MT)
                       : xccl_mem_component_reduce_multi(s1, s2, out, n2, count, stride, p->dtype, p->op, MT);
    }
    /* As the patched call sites do (allreduce_knomial.c:74-80,129-135 and the
     * other three files with integration/xccl-rocm.patch applied): one call,
     * status ignored beyond passing it on; the dispatcher leaves the event
     * NULL when the reduction is complete on return -- empty, or run through
     * the blocking entry because the component's event pool was empty (other
     * collectives hold it). */
    return n2 == 0 ? xccl_mem_component_reduce_nb(s1, s2, out, count, p->dtype, p->op, MT, NULL, &s->reduce_ev)
                   : xccl_mem_component_reduce_multi_nb(s1, s2, out, n2, count, stride, p->dtype, p->op, MT, NULL,
                                                        &s->reduce_ev);
}

/* The "reduce in flight" phase: XCCL_OK once the result may be read. */
static xccl_status_t reduce_finished(ctx_t *c, rank_state_t *s)
{
    xccl_status_t st;

    if (s->reduce_ev == NULL) {
        return XCCL_OK;
    }
    st = xccl_mc_event_query(s->reduce_ev);
    if (st == XCCL_INPROGRESS) {
        c->stats->reduce_inflight_returns++;
        return XCCL_INPROGRESS;
    }
    xccl_mc_event_free(s->reduce_ev);
    s->reduce_ev = NULL;
    return st;
}

#define TRY(expr)                      \
    do {                               \
        xccl_status_t try_st_ = (expr); \
        if (try_st_ != XCCL_OK) {      \
            return try_st_;            \
        }                              \
    } while (0)

/* Runs `expr`; XCCL_INPROGRESS leaves the progress function (to be re-entered
 * in the same phase), an error propagates, XCCL_OK falls through. */
#define AWAIT(expr) TRY(expr)

/* ---- allreduce, recursive k-nomial: allreduce_knomial.c:24-188 ------------- */
enum { KN_START, KN_EXTRA_WAIT, KN_PROXY_WAIT, KN_PROXY_REDUCE, KN_ROUND_POST, KN_ROUND_WAIT, KN_ROUND_REDUCE, KN_TAIL,
       KN_TAIL_WAIT };

static xccl_status_t progress_allreduce_knomial(ctx_t *c, rank_state_t *s)
{
    const int radix = c->radix;
    char     *round_src;
    int       k, peer;

    for (;;) {
        switch (s->phase) {
        case KN_START:
            xccl_replay_knomial_geometry(radix, s->rank, c->p->team_size, &s->rounds, &s->full_size, &s->role);
            TRY(scratch_alloc(c, s, (size_t)(radix - 1) * c->len)); /* :181-183 */
            s->iter      = 0;
            s->radix_pow = 1;
            if (s->role == ROLE_EXTRA) { /* :48-57 */
                TRY(post(c, s, 1, s->rank - s->full_size, s->src, c->len));
                TRY(post(c, s, 0, s->rank - s->full_size, s->dst, c->len));
                s->phase = KN_EXTRA_WAIT;
            } else if (s->role == ROLE_PROXY) { /* :59-64 */
                TRY(post(c, s, 0, s->rank + s->full_size, s->scratch, c->len));
                s->phase = KN_PROXY_WAIT;
            } else {
                s->phase = KN_ROUND_POST;
            }
            break;
        case KN_EXTRA_WAIT:
            AWAIT(wait_all(c, s));
            scratch_free(s);
            s->done = 1;
            return XCCL_OK;
        case KN_PROXY_WAIT:
            AWAIT(wait_all(c, s));
            /* :74-80  reduce(src, scratch, dst, count) */
            TRY(issue_reduce(c, s, s->src, s->scratch, s->dst, 0, c->p->count, 0));
            s->phase = KN_PROXY_REDUCE;
            break;
        case KN_PROXY_REDUCE:
            AWAIT(reduce_finished(c, s));
            s->phase = KN_ROUND_POST;
            break;
        case KN_ROUND_POST:
            if (s->iter >= s->rounds) {
                s->phase = KN_TAIL;
                break;
            }
            round_src = (s->iter == 0 && s->role == ROLE_BASE) ? s->src : s->dst; /* :85-91 */
            s->npeers = 0;
            for (k = 1; k < radix; k++) {
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer < s->full_size) {
                    TRY(post(c, s, 1, peer, round_src, c->len));
                }
            }
            for (k = 1; k < radix; k++) { /* :104-114: arrivals packed into scratch in peer order */
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer < s->full_size) {
                    TRY(post(c, s, 0, peer, s->scratch + (size_t)s->npeers * c->len, c->len));
                    s->npeers++;
                }
            }
            s->radix_pow *= radix;
            s->phase = s->npeers ? KN_ROUND_WAIT : KN_ROUND_REDUCE;
            break;
        case KN_ROUND_WAIT:
            AWAIT(wait_all(c, s));
            round_src = (s->iter == 0 && s->role == ROLE_BASE) ? s->src : s->dst;
            /* :129-135  reduce_multi(src_or_dst, scratch, dst, active_reqs/2, count, stride = len) */
            TRY(issue_reduce(c, s, round_src, s->scratch, s->dst, (size_t)s->npeers, c->p->count, c->len));
            s->phase = KN_ROUND_REDUCE;
            break;
        case KN_ROUND_REDUCE:
            AWAIT(reduce_finished(c, s)); /* the next round sends dst: it must be complete */
            s->iter++;
            s->phase = KN_ROUND_POST;
            break;
        case KN_TAIL:
            if (s->role == ROLE_PROXY) { /* :138-145 */
                TRY(post(c, s, 1, s->rank + s->full_size, s->dst, c->len));
                s->phase = KN_TAIL_WAIT;
                break;
            }
            scratch_free(s);
            s->done = 1;
            return XCCL_OK;
        case KN_TAIL_WAIT:
            AWAIT(wait_all(c, s));
            scratch_free(s);
            s->done = 1;
            return XCCL_OK;
        default:
            return XCCL_ERR_INVALID_PARAM;
        }
    }
}

/* ---- allreduce, scatter-reduce + allgather: allreduce_sra.c:149-501 ------- */
enum { SRA_START, SRA_EXTRA_WAIT, SRA_PROXY_WAIT, SRA_PROXY_REDUCE, SRA_ROUND_POST, SRA_ROUND_WAIT, SRA_ROUND_REDUCE,
       SRA_FINAL, SRA_FINAL_WAIT, AG_START, AG_EXTRA_WAIT, AG_ROUND_POST, AG_ROUND_WAIT, AG_TAIL, AG_TAIL_WAIT };

static xccl_status_t progress_allreduce_sra(ctx_t *c, rank_state_t *s)
{
    const int    radix = c->radix;
    const size_t es    = c->esize;
    char        *from, *base;
    size_t       parts, si, psi, seglen, segoff, off, cnt;
    int          k, peer;

    for (;;) {
        switch (s->phase) {
        case SRA_START:
            xccl_replay_knomial_geometry(radix, s->rank, c->p->team_size, &s->rounds, &s->full_size, &s->role);
            s->iter      = 0;
            s->radix_pow = 1;
            s->cur_src   = s->src;
            s->scratch   = s->dst; /* :316 the destination doubles as work space ... */
            if (s->src == s->dst || s->role == ROLE_PROXY) {
                TRY(scratch_alloc(c, s, c->len)); /* :178-186 ... unless it still holds live input */
            }
            if (s->role == ROLE_EXTRA) { /* :188-194 */
                TRY(post(c, s, 1, s->rank - s->full_size, s->src, c->len));
                s->phase = SRA_EXTRA_WAIT;
            } else if (s->role == ROLE_PROXY) { /* :196-201 */
                TRY(post(c, s, 0, s->rank + s->full_size, s->scratch, c->len));
                s->phase = SRA_PROXY_WAIT;
            } else {
                s->phase = SRA_ROUND_POST;
            }
            break;
        case SRA_EXTRA_WAIT:
            AWAIT(wait_all(c, s));
            if (s->scratch_owned) {
                scratch_free(s);
            }
            s->phase = AG_START;
            break;
        case SRA_PROXY_WAIT:
            AWAIT(wait_all(c, s));
            /* :212-218  reduce(src, scratch, dst, count) */
            TRY(issue_reduce(c, s, s->src, s->scratch, s->dst, 0, c->p->count, 0));
            s->phase = SRA_PROXY_REDUCE;
            break;
        case SRA_PROXY_REDUCE:
            AWAIT(reduce_finished(c, s));
            s->cur_src = s->dst; /* :219 */
            s->phase   = SRA_ROUND_POST;
            break;
        case SRA_ROUND_POST:
            if (s->iter >= s->rounds) {
                s->phase = SRA_FINAL;
                break;
            }
            parts    = (size_t)step_radix_of(s->rank, s->radix_pow, radix, s->full_size);
            s->block = block_count_at(c->p->count, radix, s->rank, s->iter);
            from     = s->iter == 0 ? s->cur_src : s->scratch; /* :229-230 */
            for (k = 1; k < radix; k++) {                       /* :232-244 each peer gets ITS segment of my block */
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer >= s->full_size) {
                    continue;
                }
                psi = seg_index(peer, s->radix_pow, radix);
                TRY(post(c, s, 1, peer, from + seg_offset(s->block, parts, psi) * es,
                         seg_size(s->block, parts, psi) * es));
            }
            si           = seg_index(s->rank, s->radix_pow, radix);
            s->local_cnt = seg_size(s->block, parts, si);
            s->local_off = seg_offset(s->block, parts, si);
            /* :249-263 the peers' copies of MY segment land back to back: at the start of the
             * work space in round 0, right behind my current block afterwards */
            s->recv_base = s->iter == 0 ? s->scratch : s->scratch + s->block * es;
            s->npeers    = 0;
            for (k = 1; k < radix; k++) {
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer >= s->full_size) {
                    continue;
                }
                TRY(post(c, s, 0, peer, s->recv_base + (size_t)s->npeers * s->local_cnt * es, s->local_cnt * es));
                s->npeers++;
            }
            if (s->npeers) {
                s->phase = SRA_ROUND_WAIT;
            } else {
                s->iter++; /* nobody to exchange with at this level (:264 guards the whole step) */
            }
            break;
        case SRA_ROUND_WAIT:
            AWAIT(wait_all(c, s));
            from = s->iter == 0 ? s->cur_src : s->scratch;
            /* :281-284  reduce_multi(local_data, dst_buffer, scratch, active_reqs/2, local_seg_count,
             *                        stride = local_seg_count*dt_size): the result goes to the START of
             *           the work space (== sbuf2 in round 0; == sbuf1 later when my segment is the first) */
            TRY(issue_reduce(c, s, from + s->local_off * es, s->recv_base, s->scratch, (size_t)s->npeers, s->local_cnt,
                             s->local_cnt * es));
            s->phase = SRA_ROUND_REDUCE;
            break;
        case SRA_ROUND_REDUCE:
            AWAIT(reduce_finished(c, s));
            s->radix_pow *= radix;
            s->iter++;
            s->phase = SRA_ROUND_POST;
            break;
        case SRA_FINAL:
            /* :291-297 my finished segment moves from the start of the work space to its place in dst */
            xccl_replay_sra_segment(c->p->count, s->rank, radix, c->p->team_size, &off, &cnt);
            s->ag_src   = s->dst + off * es;
            s->copy_seq = 0;
            if (s->scratch != s->ag_src && cnt > 0) {
                TRY(tr_copy(&c->tr, s->scratch, s->ag_src, cnt * es, &s->copy_seq));
            }
            s->phase = SRA_FINAL_WAIT;
            break;
        case SRA_FINAL_WAIT:
            TRY(tr_progress(&c->tr));
            if (s->copy_seq > c->tr.done_seq) {
                return XCCL_INPROGRESS;
            }
            if (s->scratch_owned) {
                scratch_free(s); /* :299-302 */
            }
            s->iter      = s->rounds - 1; /* :304-305 */
            s->radix_pow = s->radix_pow / radix;
            s->phase     = AG_START;
            break;
        case AG_START: /* allreduce_sra.c:344-351 */
            if (s->role == ROLE_EXTRA) {
                TRY(post(c, s, 0, s->rank - s->full_size, s->dst, c->len));
                s->phase = AG_EXTRA_WAIT;
            } else {
                s->phase = AG_ROUND_POST;
            }
            break;
        case AG_EXTRA_WAIT:
            AWAIT(wait_all(c, s));
            s->done = 1;
            return XCCL_OK;
        case AG_ROUND_POST: /* :363-401: rounds in reverse; my block at this level grows around my segment */
            if (s->iter < 0) {
                s->phase = AG_TAIL;
                break;
            }
            parts    = (size_t)step_radix_of(s->rank, s->radix_pow, radix, s->full_size);
            s->block = block_count_at(c->p->count, radix, s->rank, s->iter);
            si       = seg_index(s->rank, s->radix_pow, radix);
            seglen   = seg_size(s->block, parts, si);
            base     = s->ag_src - seg_offset(s->block, parts, si) * es;
            s->npeers = 0;
            for (k = 1; k < radix; k++) {
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer < s->full_size) {
                    TRY(post(c, s, 1, peer, s->ag_src, seglen * es));
                }
            }
            for (k = 1; k < radix; k++) {
                peer = kn_peer(s->rank, k, s->radix_pow, radix);
                if (peer >= s->full_size) {
                    continue;
                }
                psi    = seg_index(peer, s->radix_pow, radix);
                segoff = seg_offset(s->block, parts, psi);
                TRY(post(c, s, 0, peer, base + segoff * es, seg_size(s->block, parts, psi) * es));
                s->npeers++;
            }
            s->ag_src = base;
            s->phase  = AG_ROUND_WAIT;
            break;
        case AG_ROUND_WAIT:
            AWAIT(wait_all(c, s));
            if (s->npeers) {
                s->radix_pow /= radix;
            }
            s->iter--;
            s->phase = AG_ROUND_POST;
            break;
        case AG_TAIL: /* :412-418 */
            if (s->role == ROLE_PROXY) {
                TRY(post(c, s, 1, s->rank + s->full_size, s->dst, c->len));
                s->phase = AG_TAIL_WAIT;
                break;
            }
            s->done = 1;
            return XCCL_OK;
        case AG_TAIL_WAIT:
            AWAIT(wait_all(c, s));
            s->done = 1;
            return XCCL_OK;
        default:
            return XCCL_ERR_INVALID_PARAM;
        }
    }
}

/* ---- rooted reduce, k-nomial tree: reduce_knomial.c:18-122 ------------------ */
enum { RK_START, RK_LEVEL, RK_WAIT, RK_REDUCE };

static xccl_status_t progress_reduce_knomial(ctx_t *c, rank_state_t *s)
{
    const int P = c->p->team_size, root = c->p->root, radix = c->radix;
    const int vrank = (s->rank - root + P) % P;
    int       i, pos, vpeer;

    for (;;) {
        switch (s->phase) {
        case RK_START:
            s->dist     = 1;
            s->max_dist = 1;
            while (s->max_dist * radix < P) { /* :9-14 */
                s->max_dist *= radix;
            }
            s->data_buf = s->src;
            TRY(scratch_alloc(c, s, (size_t)radix * c->len)); /* :120-121 */
            /* :35-36 a non-root rank accumulates in the last slot of its scratch */
            s->rdst  = s->rank == root ? s->dst : s->scratch + (size_t)(radix - 1) * c->len;
            s->phase = RK_LEVEL;
            break;
        case RK_LEVEL:
            if (s->dist > s->max_dist) {
                scratch_free(s);
                s->done = 1;
                return XCCL_OK;
            }
            pos           = (vrank % s->dist == 0) ? (vrank / s->dist) % radix : -1;
            s->level_kind = 0;
            if (pos == 0) { /* :49-60 parent at this level: children arrive into scratch, farthest first */
                for (i = radix - 1; i >= 1; i--) {
                    vpeer = vrank + i * s->dist;
                    if (vpeer < P) {
                        TRY(post(c, s, 0, (vpeer + root) % P, s->scratch + (size_t)s->nreqs * c->len, c->len));
                        s->level_kind = 1;
                    }
                }
            } else if (pos > 0) { /* :61-69 child: hand the partial result up and stop taking part */
                TRY(post(c, s, 1, (vrank - pos * s->dist + root) % P, s->data_buf, c->len));
                s->level_kind = 2;
            }
            s->dist *= radix;
            if (s->nreqs) {
                s->npeers = s->nreqs;
                s->phase  = RK_WAIT;
            }
            break;
        case RK_WAIT:
            AWAIT(wait_all(c, s));
            if (s->level_kind == 1) {
                /* :79-85  reduce_multi(src_buffer, scratch, dst_buffer, active_reqs, count, stride = len);
                 *         from the second level on src_buffer == dst_buffer (:86-88) */
                TRY(issue_reduce(c, s, s->data_buf, s->scratch, s->rdst, (size_t)s->npeers, c->p->count, c->len));
                s->phase = RK_REDUCE;
            } else {
                s->phase = RK_LEVEL;
            }
            break;
        case RK_REDUCE:
            AWAIT(reduce_finished(c, s));
            s->data_buf = s->rdst;
            s->phase    = RK_LEVEL;
            break;
        default:
            return XCCL_ERR_INVALID_PARAM;
        }
    }
}

/* ---- rooted reduce, linear: reduce_linear.c:10-88 ---------------------------- */
enum { RL_START, RL_COPY_WAIT, RL_RECV, RL_WAIT, RL_REDUCE, RL_SEND_WAIT };

static xccl_status_t progress_reduce_linear(ctx_t *c, rank_state_t *s)
{
    const int P = c->p->team_size, root = c->p->root;

    for (;;) {
        switch (s->phase) {
        case RL_START:
            if (s->rank != root) { /* :48-53 */
                TRY(post(c, s, 1, root, s->src, c->len));
                s->phase = RL_SEND_WAIT;
                break;
            }
            TRY(scratch_alloc(c, s, c->len)); /* :76-79 */
            s->copy_seq = 0;
            if (s->src != s->dst) { /* :80-84 the root's own contribution seeds dst */
                TRY(tr_copy(&c->tr, s->src, s->dst, c->len, &s->copy_seq));
            }
            s->next  = (root + 1) % P;
            s->phase = RL_COPY_WAIT;
            break;
        case RL_COPY_WAIT:
            TRY(tr_progress(&c->tr));
            if (s->copy_seq > c->tr.done_seq) {
                return XCCL_INPROGRESS;
            }
            s->phase = RL_RECV;
            break;
        case RL_RECV:
            if (s->next == root) {
                scratch_free(s);
                s->done = 1;
                return XCCL_OK;
            }
            TRY(post(c, s, 0, s->next, s->scratch, c->len)); /* :21-26, :36-41 one peer at a time */
            s->phase = RL_WAIT;
            break;
        case RL_WAIT:
            AWAIT(wait_all(c, s));
            /* :28-34  reduce(scratch, dst, dst): the target aliases sbuf2 */
            TRY(issue_reduce(c, s, s->scratch, s->dst, s->dst, 0, c->p->count, 0));
            s->phase = RL_REDUCE;
            break;
        case RL_REDUCE:
            AWAIT(reduce_finished(c, s));
            s->next  = (s->next + 1) % P;
            s->phase = RL_RECV;
            break;
        case RL_SEND_WAIT:
            AWAIT(wait_all(c, s));
            s->done = 1;
            return XCCL_OK;
        default:
            return XCCL_ERR_INVALID_PARAM;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* 4. driver                                                                  */
/* ------------------------------------------------------------------------ */

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

xccl_status_t xccl_replay_run(const xccl_replay_params_t *p, xccl_replay_stats_t *stats, uint64_t max_sweeps)
{
    xccl_status_t (*progress)(ctx_t *, rank_state_t *);
    xccl_replay_stats_t local_stats;
    rank_state_t       *ranks;
    ctx_t               c;
    xccl_status_t       st = XCCL_OK;
    uint64_t            sweep;
    double              t0;
    int                 r, remaining;

    if (p == NULL || p->team_size < 2 || p->src == NULL || p->dst == NULL || xccl_dt_size(p->dtype) == 0 ||
        p->root < 0 || p->root >= p->team_size || p->radix < 2) {
        return XCCL_ERR_INVALID_PARAM;
    }
    if (stats == NULL) {
        stats = &local_stats;
    }
    memset(stats, 0, sizeof(*stats));
    memset(&c, 0, sizeof(c));
    c.p     = p;
    c.stats = stats;
    c.esize = xccl_dt_size(p->dtype);
    c.len   = p->count * c.esize;
    c.radix = p->radix > p->team_size ? p->team_size : p->radix; /* allreduce_knomial.c:170-173 */
    if (c.radix > MAX_RADIX) {
        return XCCL_ERR_INVALID_PARAM;
    }
    switch (p->alg) {
    case XCCL_REPLAY_ALLREDUCE_KNOMIAL:
        progress = progress_allreduce_knomial;
        break;
    case XCCL_REPLAY_ALLREDUCE_SRA:
        /* allreduce_sra.c:496-500: too little room in dst for radix-1 incoming segments -> radix 2 */
        if (((p->count + (size_t)c.radix - 1) / (size_t)c.radix) * (size_t)(c.radix - 1) > p->count ||
            (size_t)(c.radix - 1) > p->count) {
            c.radix = 2;
        }
        progress = progress_allreduce_sra;
        break;
    case XCCL_REPLAY_REDUCE_KNOMIAL:
        progress = progress_reduce_knomial;
        break;
    case XCCL_REPLAY_REDUCE_LINEAR:
        progress = progress_reduce_linear;
        break;
    default:
        return XCCL_ERR_INVALID_PARAM;
    }

    ranks = (rank_state_t *)calloc((size_t)p->team_size, sizeof(rank_state_t));
    if (ranks == NULL) {
        return XCCL_ERR_NO_MEMORY;
    }
    st = tr_init(&c.tr, p->team_size, stats);
    if (st != XCCL_OK) {
        free(ranks);
        return st;
    }
    for (r = 0; r < p->team_size; r++) {
        ranks[r].rank = r;
        ranks[r].src  = (char *)p->src[r];
        ranks[r].dst  = (char *)p->dst[r];
    }

    if (max_sweeps == 0) {
        max_sweeps = (uint64_t)1 << 34;
    }
    remaining = p->team_size;
    t0        = now_s();
    for (sweep = 0; remaining > 0 && st == XCCL_OK; sweep++) {
        if (sweep >= max_sweeps || ((sweep & 0x3ff) == 0x3ff && now_s() - t0 > WALL_LIMIT_S)) {
            st = XCCL_ERR_NO_PROGRESS;
            break;
        }
        for (r = 0; r < p->team_size; r++) {
            xccl_status_t rs;
            if (ranks[r].done) {
                continue;
            }
            stats->progress_calls++;
            rs = progress(&c, &ranks[r]);
            if (rs == XCCL_INPROGRESS) {
                continue;
            }
            if (rs != XCCL_OK) {
                st = rs;
                break;
            }
            if (ranks[r].done) {
                remaining--;
            }
        }
    }

    /* nothing may stay in flight or allocated behind an error */
    for (r = 0; r < p->team_size; r++) {
        if (ranks[r].reduce_ev != NULL) {
            xccl_mc_event_wait(ranks[r].reduce_ev);
            xccl_mc_event_free(ranks[r].reduce_ev);
        }
    }
    tr_destroy(&c.tr);
    for (r = 0; r < p->team_size; r++) {
        if (ranks[r].scratch_owned) {
            xccl_mem_component_free(ranks[r].scratch, MT);
        }
    }
    free(ranks);
    return st;
}
