/*
 * mrb_oracle.c — CPU restatement of the reference's replay-buffer path.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker that the HIP library is
 * compared against; only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may load it. The product never links or calls it.
 *
 * What it restates. The reference's buffer classes are wrappers around
 * MindSpore primitives:
 *   mindspore_rl/core/uniform_replay_buffer.py:82-89   BufferAppend / BufferGetItem / BufferSample
 *   mindspore_rl/core/priority_replay_buffer.py:62-76  PriorityReplayBufferCreate/Push/Sample/Update/Destroy
 * The arithmetic behind those primitives lives in the third-party module
 * `mindspore` (2.2 for mindspore_rl 0.8, mindspore_rl/__init__.py:52-63), which
 * is not part of the reference tree. This file restates the published
 * algorithm (Schaul et al., "Prioritized Experience Replay", proportional
 * variant with a sum tree and a min tree; a FIFO ring for the rows) as one
 * sequential, single-threaded implementation, in the order the reference's CPU
 * path is specified to work: per-item leaf write followed by a leaf-to-root walk.
 *
 * PARITY STATUS. The reference's own tests for this path are disabled and hold
 * no numeric vectors (tests/st/test_priority_replay_buffer.py:26 skipped,
 * tests/st/test_uniform_replay_buffer.py:58 never collected). What those tests
 * assert (indices < size, gathered row == row written at that index, a
 * minimised priority is not drawn again, successive samples differ) is checked
 * in tests/. Functions whose tie-breaks no reference file can pin are marked
 * "parity unpinned" below: they follow the decisions listed next to them.
 *
 *   orc_powf        parity unpinned vs the reference's libm powf: own
 *                   deterministic algorithm, checked against libm pow() to 1 ulp.
 *   orc_per_sample  descent tie-break (mass <= left goes left) and the IS
 *                   weight expression: parity unpinned; pinned only by
 *                   brute-force prefix-sum search and the float64 closed form.
 *   orc_rng_*       the reference's generator (engine + distribution) is
 *                   unspecified by its sources: parity unpinned; draws are
 *                   normally supplied by the caller.
 *   orc_res_*       reservoir policy (draw range, which stream): parity unpinned;
 *                   pinned by the reservoir's defining property (every row kept
 *                   with probability capacity / rows seen) and the reference
 *                   test's row-consistency invariant.
 *   ring / gather / tree build / update: pinned by closed forms, brute force
 *                   and numpy library routines in tests/test_oracle_*.py.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_FIELDS 16

/* ------------------------------------------------------------------------
 * Deterministic powf: double arithmetic only (+ - * / floor, no fused ops),
 * so that an implementation on another IEEE-754 machine performing the same
 * operations in the same order returns the same bits.
 *   log(m)  = 2s (1 + z/3 + ... + z^11/23),  s = (m-1)/(m+1), z = s*s, m in (sqrt.5, sqrt2]
 *   2^y     = 2^n * exp(r ln2), n = floor(y + .5), Taylor to degree 14
 * ---------------------------------------------------------------------- */
static double orc_u64_as_double(uint64_t u) {
    double d;
    memcpy(&d, &u, 8);
    return d;
}
static uint64_t orc_double_as_u64(double d) {
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
}

float orc_powf(float x, float a) {
    if (a == 0.0f) return 1.0f;
    if (x == 0.0f) return a < 0.0f ? INFINITY : 0.0f; /* as pow(): 0^-b is +inf, so a zero minimum priority gives weights 0, not inf */
    if (a == 1.0f) return x;
    if (x == 1.0f) return 1.0f;
    uint64_t bits = orc_double_as_u64((double)x);
    int e = (int)((bits >> 52) & 0x7ff) - 1023;
    double m = orc_u64_as_double((bits & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL);
    if (m > 1.4142135623730951) {
        m = m * 0.5;
        e = e + 1;
    }
    double f = m - 1.0;
    double s = f / (2.0 + f);
    double z = s * s;
    double p = 1.0 / 23.0;
    p = p * z + 1.0 / 21.0;
    p = p * z + 1.0 / 19.0;
    p = p * z + 1.0 / 17.0;
    p = p * z + 1.0 / 15.0;
    p = p * z + 1.0 / 13.0;
    p = p * z + 1.0 / 11.0;
    p = p * z + 1.0 / 9.0;
    p = p * z + 1.0 / 7.0;
    p = p * z + 1.0 / 5.0;
    p = p * z + 1.0 / 3.0;
    p = p * z + 1.0;
    double lm = 2.0 * s * p;
    double log2x = (double)e + lm * 1.4426950408889634;
    double y = (double)a * log2x;
    if (y > 200.0) y = 200.0;
    if (y < -200.0) y = -200.0;
    double n = floor(y + 0.5);
    double t = (y - n) * 0.6931471805599453;
    double q = 1.0 / 87178291200.0; /* 1/14! */
    q = q * t + 1.0 / 6227020800.0;
    q = q * t + 1.0 / 479001600.0;
    q = q * t + 1.0 / 39916800.0;
    q = q * t + 1.0 / 3628800.0;
    q = q * t + 1.0 / 362880.0;
    q = q * t + 1.0 / 40320.0;
    q = q * t + 1.0 / 5040.0;
    q = q * t + 1.0 / 720.0;
    q = q * t + 1.0 / 120.0;
    q = q * t + 1.0 / 24.0;
    q = q * t + 1.0 / 6.0;
    q = q * t + 0.5;
    q = q * t + 1.0;
    q = q * t + 1.0;
    double scale = orc_u64_as_double((uint64_t)((int64_t)n + 1023) << 52);
    return (float)(q * scale);
}

void orc_powf_n(const float *x, float a, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_powf(x[i], a);
}

/* Counter-based generator: one 64-bit mix of (seed, call counter, lane). */
uint64_t orc_rng_u64(uint64_t seed, uint64_t counter, uint64_t k) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ULL * ((counter << 32) + k + 1ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}
float orc_rng_uniform(uint64_t seed, uint64_t counter, uint64_t k) {
    return (float)(orc_rng_u64(seed, counter, k) >> 40) * 5.9604644775390625e-8f; /* 2^-24 */
}
int64_t orc_rng_below(uint64_t seed, uint64_t counter, uint64_t k, int64_t bound) {
    return (int64_t)(((unsigned __int128)orc_rng_u64(seed, counter, k) * (unsigned __int128)(uint64_t)bound) >> 64);
}

/* Threads used for the row copies of orc_per_sample / orc_urb_gather (1 = the
 * sequential restatement; more only for the "all host cores" timing baseline). */
static int orc_threads = 1;
void orc_set_threads(int n) { orc_threads = n < 1 ? 1 : n; }

/* ------------------------------------------------------------------------
 * Row storage: structure of arrays, field i = [capacity, bytes_i]
 * (mindspore_rl/core/uniform_replay_buffer.py:26-47).
 * ---------------------------------------------------------------------- */
typedef struct {
    int64_t capacity;
    int nfields;
    int64_t bytes[ORC_MAX_FIELDS];
    unsigned char *data[ORC_MAX_FIELDS];
} orc_rows;

static int rows_init(orc_rows *r, int64_t capacity, int nfields, const int64_t *bytes) {
    if (capacity <= 0 || nfields <= 0 || nfields > ORC_MAX_FIELDS) return 1;
    r->capacity = capacity;
    r->nfields = nfields;
    for (int i = 0; i < nfields; ++i) {
        if (bytes[i] <= 0) return 1;
        r->bytes[i] = bytes[i];
        r->data[i] = (unsigned char *)calloc((size_t)capacity, (size_t)bytes[i]);
        if (!r->data[i]) return 1;
    }
    return 0;
}
static void rows_free(orc_rows *r) {
    for (int i = 0; i < r->nfields; ++i) free(r->data[i]);
}
static void rows_put(orc_rows *r, int64_t slot, const void *const *src, int64_t src_row) {
    for (int i = 0; i < r->nfields; ++i)
        memcpy(r->data[i] + slot * r->bytes[i], (const unsigned char *)src[i] + src_row * r->bytes[i],
               (size_t)r->bytes[i]);
}
static void rows_get(const orc_rows *r, int64_t slot, void *const *dst, int64_t dst_row) {
    for (int i = 0; i < r->nfields; ++i)
        memcpy((unsigned char *)dst[i] + dst_row * r->bytes[i], r->data[i] + slot * r->bytes[i],
               (size_t)r->bytes[i]);
}

/* ------------------------------------------------------------------------
 * Uniform FIFO buffer (uniform_replay_buffer.py:75-172).
 * ---------------------------------------------------------------------- */
typedef struct {
    orc_rows rows;
    int64_t count, head;
    uint64_t seed, calls;
} orc_urb;

orc_urb *orc_urb_create(int64_t capacity, int nfields, const int64_t *bytes) {
    orc_urb *b = (orc_urb *)calloc(1, sizeof(orc_urb));
    if (!b) return NULL;
    if (rows_init(&b->rows, capacity, nfields, bytes)) {
        free(b);
        return NULL;
    }
    return b;
}
void orc_urb_destroy(orc_urb *b) {
    if (!b) return;
    rows_free(&b->rows);
    free(b);
}
void orc_urb_seed(orc_urb *b, uint64_t seed) {
    b->seed = seed;
    b->calls = 0;
}

/* insert(): uniform_replay_buffer.py:101-115. The write position is chosen
 * once per call: `count` while the buffer has never been full (count <
 * capacity and head == 0), otherwise `head` (the oldest row). Rows then go to
 * consecutive slots modulo capacity, later rows overwriting earlier ones. */
int orc_urb_append(orc_urb *b, const void *const *src, int64_t nrows) {
    if (nrows <= 0) return 1;
    int64_t cap = b->rows.capacity;
    int growing = b->count < cap && b->head == 0;
    int64_t w = growing ? b->count : b->head;
    for (int64_t j = 0; j < nrows; ++j) rows_put(&b->rows, (w + j) % cap, src, j);
    if (growing) {
        if (b->count + nrows <= cap) {
            b->count += nrows;
        } else {
            b->head = (b->count + nrows) % cap; /* wrapped: the slot after the newest row holds the oldest */
            b->count = cap;
        }
    } else {
        b->head = (b->head + nrows) % cap;
        b->count = b->count + nrows < cap ? b->count + nrows : cap;
    }
    return 0;
}

/* get_item(): uniform_replay_buffer.py:117-128; logical index with 0 = oldest
 * (caller: mindspore_rl/utils/n_step_buffer.py:85-92 passes count - td + m). */
int orc_urb_get_item(const orc_urb *b, int64_t index, void *const *dst) {
    if (index < 0) index += b->count;
    if (index < 0 || index >= b->count) return 1;
    int64_t t = b->count - b->head;
    int64_t slot = index < t ? index + b->head : index - t;
    rows_get(&b->rows, slot, dst, 0);
    return 0;
}

/* Gather half of sample(): uniform_replay_buffer.py:130-139. */
int orc_urb_gather(const orc_urb *b, const int64_t *indices, int64_t n, void *const *dst) {
    for (int64_t k = 0; k < n; ++k)
        if (indices[k] < 0 || indices[k] >= b->count) return 1;
#pragma omp parallel for num_threads(orc_threads) schedule(static) if (orc_threads > 1)
    for (int64_t k = 0; k < n; ++k) rows_get(&b->rows, indices[k], dst, k);
    return 0;
}

int orc_urb_sample(orc_urb *b, int64_t n, int64_t *out_indices, void *const *dst) {
    if (n <= 0 || n > b->count) return 1;
    for (int64_t k = 0; k < n; ++k) {
        int64_t idx = orc_rng_below(b->seed, b->calls, (uint64_t)k, b->count);
        if (out_indices) out_indices[k] = idx;
        rows_get(&b->rows, idx, dst, k);
    }
    b->calls += 1;
    return 0;
}
void orc_urb_reset(orc_urb *b) { b->count = 0; } /* uniform_replay_buffer.py:149: head untouched */
int64_t orc_urb_count(const orc_urb *b) { return b->count; }
int64_t orc_urb_head(const orc_urb *b) { return b->head; }
const void *orc_urb_field(const orc_urb *b, int i) { return b->rows.data[i]; }
/* Checkpoint counterpart (the reference persists no buffers; the state is what continuing
 * identically needs): {count, head, seed, calls}. Row storage is reached through orc_urb_field. */
void orc_urb_get_state(const orc_urb *b, int64_t *out4) {
    out4[0] = b->count, out4[1] = b->head, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
}
int orc_urb_set_state(orc_urb *b, const int64_t *in4) {
    if (in4[0] < 0 || in4[0] > b->rows.capacity || in4[1] < 0 || in4[1] >= b->rows.capacity) return 1;
    b->count = in4[0], b->head = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    return 0;
}

/* ------------------------------------------------------------------------
 * Discounted return (mindspore_rl/utils/discounted_return.py:84-92, the
 * reference's own non-fused loop): walking the time axis backwards,
 *   last = reward[t] + (1 - done[t]) * gamma * last;  out[t] = last
 * with reward [T, B, inner], done [T, B], last_state_value [B, inner], all
 * float32, each operation rounded once, left to right as written there.
 * Pinned by the reference's known-answer vectors
 * (tests/st/test_discounted_return.py:39-53).
 * ---------------------------------------------------------------------- */
void orc_discounted_return(const float *reward, const unsigned char *done, const float *last_value, float *out,
                           int64_t timesteps, int64_t batch, int64_t inner, float gamma) {
    for (int64_t b = 0; b < batch; ++b)
        for (int64_t i = 0; i < inner; ++i) {
            float last = last_value[b * inner + i];
            for (int64_t t = timesteps - 1; t >= 0; --t) {
                float keep = 1.0f - (done[t * batch + b] ? 1.0f : 0.0f);
                float scaled = keep * gamma;
                last = reward[(t * batch + b) * inner + i] + scaled * last;
                out[(t * batch + b) * inner + i] = last;
            }
        }
}

/* ------------------------------------------------------------------------
 * Reservoir buffer (mindspore_rl/core/reservoir_replay_buffer.py:61-100):
 * Vitter's Algorithm R. The first `capacity` rows fill the slots in order; row
 * number t (0-based) after that draws r uniformly in [0, t] and replaces slot r
 * if r < capacity, so every row seen so far is retained with probability
 * capacity / (t + 1). sample() draws slots uniformly in [0, size) with
 * replacement (the reference's own test samples 256 rows from 100,
 * tests/st/test_reservoir_replay_buffer.py:33-49).
 * Parity unpinned: the reference's generator and draw order are not in its
 * sources; draw t of the push stream is orc_rng_below(seed, 0, t, t + 1), call
 * c of sample() uses stream counter c + 1.
 * ---------------------------------------------------------------------- */
typedef struct {
    orc_rows rows;
    int64_t size, total;
    uint64_t seed, calls;
} orc_res;

orc_res *orc_res_create(int64_t capacity, int nfields, const int64_t *bytes, uint64_t seed) {
    orc_res *b = (orc_res *)calloc(1, sizeof(orc_res));
    if (!b) return NULL;
    if (rows_init(&b->rows, capacity, nfields, bytes)) {
        free(b);
        return NULL;
    }
    b->seed = seed;
    return b;
}
void orc_res_destroy(orc_res *b) {
    if (!b) return;
    rows_free(&b->rows);
    free(b);
}
int orc_res_push(orc_res *b, const void *const *src, int64_t nrows) {
    if (nrows <= 0) return 1;
    for (int64_t j = 0; j < nrows; ++j) {
        int64_t t = b->total;
        if (t < b->rows.capacity) {
            rows_put(&b->rows, t, src, j);
            b->size += 1;
        } else {
            int64_t r = orc_rng_below(b->seed, 0, (uint64_t)t, t + 1);
            if (r < b->rows.capacity) rows_put(&b->rows, r, src, j);
        }
        b->total += 1;
    }
    return 0;
}
int orc_res_sample(orc_res *b, int64_t n, int64_t *out_indices, void *const *dst) {
    if (n <= 0 || b->size <= 0) return 1;
    for (int64_t k = 0; k < n; ++k) {
        int64_t idx = orc_rng_below(b->seed, b->calls + 1, (uint64_t)k, b->size);
        if (out_indices) out_indices[k] = idx;
        rows_get(&b->rows, idx, dst, k);
    }
    b->calls += 1;
    return 0;
}
int64_t orc_res_size(const orc_res *b) { return b->size; }
int64_t orc_res_total(const orc_res *b) { return b->total; }
const void *orc_res_field(const orc_res *b, int i) { return b->rows.data[i]; }
/* {size, total, seed, calls} */
void orc_res_get_state(const orc_res *b, int64_t *out4) {
    out4[0] = b->size, out4[1] = b->total, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
}
int orc_res_set_state(orc_res *b, const int64_t *in4) {
    int64_t want = in4[1] < b->rows.capacity ? in4[1] : b->rows.capacity;
    if (in4[1] < 0 || in4[0] != want) return 1;
    b->size = in4[0], b->total = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    return 0;
}

/* ------------------------------------------------------------------------
 * Prioritized buffer (priority_replay_buffer.py:60-138): FIFO rows + a sum
 * tree and a min tree over next_pow2(capacity) leaves, heap order, root 1.
 * ---------------------------------------------------------------------- */
typedef struct {
    orc_rows rows;
    int64_t leaves, size, pushes;
    float alpha, max_priority;
    float *sum, *mn;
    uint64_t seed, calls;
} orc_per;

static int64_t next_pow2(int64_t v) {
    int64_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

orc_per *orc_per_create(int64_t capacity, float alpha, int nfields, const int64_t *bytes, uint64_t seed) {
    orc_per *b = (orc_per *)calloc(1, sizeof(orc_per));
    if (!b) return NULL;
    if (rows_init(&b->rows, capacity, nfields, bytes)) {
        free(b);
        return NULL;
    }
    b->leaves = next_pow2(capacity);
    b->alpha = alpha;
    b->max_priority = 1.0f;
    b->seed = seed;
    b->sum = (float *)calloc((size_t)(2 * b->leaves), sizeof(float));
    b->mn = (float *)malloc((size_t)(2 * b->leaves) * sizeof(float));
    for (int64_t i = 0; i < 2 * b->leaves; ++i) b->mn[i] = FLT_MAX;
    return b;
}
void orc_per_destroy(orc_per *b) {
    if (!b) return;
    rows_free(&b->rows);
    free(b->sum);
    free(b->mn);
    free(b);
}

/* Write one leaf and recompute its ancestors, leaf to root, each from its two children. */
static void tree_set(orc_per *b, int64_t slot, float v) {
    int64_t i = b->leaves + slot;
    b->sum[i] = v;
    b->mn[i] = v;
    for (i >>= 1; i >= 1; i >>= 1) {
        b->sum[i] = b->sum[2 * i] + b->sum[2 * i + 1];
        b->mn[i] = fminf(b->mn[2 * i], b->mn[2 * i + 1]);
    }
}

/* update_priorities(): priority_replay_buffer.py:108-120. In batch order, so
 * a later duplicate index overwrites an earlier one. */
int orc_per_update(orc_per *b, const int64_t *indices, const float *priorities, int64_t n) {
    for (int64_t j = 0; j < n; ++j) {
        if (indices[j] < 0 || indices[j] >= b->rows.capacity) return 1;
        if (!(priorities[j] >= 0.0f) || isinf(priorities[j])) return 2;
    }
    for (int64_t j = 0; j < n; ++j) {
        float q = orc_powf(priorities[j], b->alpha);
        tree_set(b, indices[j], q);
        if (q > b->max_priority) b->max_priority = q;
    }
    return 0;
}

/* insert()/push: priority_replay_buffer.py:78-90. Row goes to the next ring
 * slot with the running max priority; optional explicit priorities are applied
 * as an update of the new slots afterwards. */
int orc_per_push(orc_per *b, const void *const *src, int64_t nrows, const float *opt_priorities) {
    if (nrows <= 0) return 1;
    int64_t cap = b->rows.capacity;
    int64_t first = b->pushes;
    for (int64_t j = 0; j < nrows; ++j) {
        int64_t slot = b->pushes % cap;
        rows_put(&b->rows, slot, src, j);
        b->pushes += 1;
        if (b->size < cap) b->size += 1;
        tree_set(b, slot, b->max_priority);
    }
    if (opt_priorities) {
        for (int64_t j = 0; j < nrows; ++j) {
            int64_t slot = (first + j) % cap;
            int rc = orc_per_update(b, &slot, &opt_priorities[j], 1);
            if (rc) return rc;
        }
    }
    return 0;
}

/* sample(beta): priority_replay_buffer.py:92-106. Stratified: segment k of
 * the total mass gets one draw; the sum tree is descended from the root,
 * going left when the remaining mass is <= the left child's sum. */
int orc_per_sample(orc_per *b, int64_t batch, float beta, const float *uniforms, int64_t *out_indices,
                   float *out_weights, void *const *out_fields) {
    if (batch <= 0 || b->size <= 0) return 1;
    float total = b->sum[1];
    float pmin = b->mn[1];
    if (!(total > 0.0f) || isinf(total)) return 2;
    float seg = total / (float)batch;
    float fsize = (float)b->size;
    float max_w = orc_powf(pmin / total * fsize, -beta);
    for (int64_t k = 0; k < batch; ++k) {
        float u = uniforms ? uniforms[k] : orc_rng_uniform(b->seed, b->calls, (uint64_t)k);
        float mass = (u + (float)k) * seg;
        int64_t i = 1;
        while (i < b->leaves) {
            float left = b->sum[2 * i];
            if (mass <= left) {
                i = 2 * i;
            } else {
                mass -= left;
                i = 2 * i + 1;
            }
        }
        int64_t idx = i - b->leaves;
        float p = b->sum[i];
        out_indices[k] = idx;
        out_weights[k] = orc_powf(p / total * fsize, -beta) / max_w;
        /* No clamp on the index: rounding in the last stratum can carry the
         * descent onto an unfilled leaf, and that index is returned as it is.
         * Only the row copy is kept inside the storage. */
        if (out_fields && orc_threads <= 1)
            rows_get(&b->rows, idx < b->rows.capacity ? idx : b->rows.capacity - 1, out_fields, k);
    }
    if (out_fields && orc_threads > 1) {
        /* the all-cores baseline: the descent stays sequential, the row copies are shared out */
#pragma omp parallel for num_threads(orc_threads) schedule(static)
        for (int64_t k = 0; k < batch; ++k) {
            int64_t idx = out_indices[k];
            rows_get(&b->rows, idx < b->rows.capacity ? idx : b->rows.capacity - 1, out_fields, k);
        }
    }
    if (!uniforms) b->calls += 1;
    return 0;
}

void orc_per_export_tree(const orc_per *b, float *sum_heap, float *min_heap) {
    if (sum_heap) memcpy(sum_heap, b->sum, (size_t)(2 * b->leaves) * sizeof(float));
    if (min_heap) memcpy(min_heap, b->mn, (size_t)(2 * b->leaves) * sizeof(float));
}
int64_t orc_per_leaves(const orc_per *b) { return b->leaves; }
int64_t orc_per_size(const orc_per *b) { return b->size; }
int64_t orc_per_head(const orc_per *b) { return b->pushes % b->rows.capacity; }
float orc_per_max_priority(const orc_per *b) { return b->max_priority; }
const void *orc_per_field(const orc_per *b, int i) { return b->rows.data[i]; }
/* {size, pushes, seed, calls} */
void orc_per_get_state(const orc_per *b, int64_t *out4) {
    out4[0] = b->size, out4[1] = b->pushes, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
}
/* Loads a saved state: counters, running max and the stored leaves of slots [0, n) (values as
 * stored, i.e. already raised to alpha); every other leaf becomes empty and every internal node is
 * recomputed from its two children, bottom-up - the value a leaf-to-root walk after the last write
 * leaves there. */
int orc_per_load_state(orc_per *b, const int64_t *in4, const float *leaves, int64_t n, float max_priority) {
    int64_t cap = b->rows.capacity;
    int64_t want = in4[1] < cap ? in4[1] : cap;
    if (in4[1] < 0 || in4[0] != want || n < 0 || n > cap) return 1;
    b->size = in4[0], b->pushes = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    b->max_priority = max_priority;
    for (int64_t i = 0; i < b->leaves; ++i) {
        b->sum[b->leaves + i] = i < n ? leaves[i] : 0.0f;
        b->mn[b->leaves + i] = i < n ? leaves[i] : FLT_MAX;
    }
    for (int64_t i = b->leaves - 1; i >= 1; --i) {
        b->sum[i] = b->sum[2 * i] + b->sum[2 * i + 1];
        b->mn[i] = fminf(b->mn[2 * i], b->mn[2 * i + 1]);
    }
    return 0;
}
