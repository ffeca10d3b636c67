/*
 * mni_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded restatement of the pure-Rust CPU backend of
 * mni-ml/framework for the fp32 matmul path: tensor store, autograd tape and
 * the handful of ops the path and its callers touch.  It exists only so that
 * the tests, the smoke check and the cpu_baseline leg of the benchmark have
 * something to compare the HIP backend against.  Nothing in the shipped
 * library links, loads or calls this file.
 *
 * Build: gcc -O3 -ffp-contract=off -fno-fast-math (no -march=native) so every
 * sum is the same sequence of separately rounded f32 multiplies and adds the
 * reference's release build performs (Rust never contracts a*b+c to an FMA;
 * src/native/Cargo.toml:30-32 sets opt-level 3 on the x86-64 baseline target).
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  What pins each function is listed next to it as
 * "pinned by": reference-held test vectors (the test suites under test/), closed forms and
 * brute force in tests/test_oracle_*.py.  Transcendentals (expf, logf, tanhf,
 * sqrtf, powf) come from glibc, not Rust's libm: they may differ by an ulp or
 * two from the reference, which is far inside the parity tolerance.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_DIMS 8
#define ORC_BAD UINT32_MAX

typedef struct {
    int live;
    float *data;            /* raw buffer, `size` floats                     */
    size_t shape[ORC_MAX_DIMS];
    size_t strides[ORC_MAX_DIMS]; /* in elements                             */
    int ndim;
    size_t size;
    int requires_grad;
    long grad;              /* tensor id of .grad, or -1                     */
    float *adam_m, *adam_v; /* lazily created by adamw_step                  */
} orc_tensor;

/* tensor.rs:96-100 TensorStore{tensors, free_ids, alloc} */
typedef struct {
    orc_tensor *t;
    size_t len, cap;
    size_t *free_ids;
    size_t nfree, capfree;
} orc_store;

enum orc_op { /* subset of autograd.rs:28-62 BackwardOp */
    OP_ADD, OP_MUL, OP_SUB, OP_NEG, OP_MULSCALAR, OP_MATMUL, OP_GELU, OP_RELU,
    OP_SUM, OP_MEAN, OP_VIEW, OP_PERMUTE, OP_CONTIGUOUS, OP_CROSSENTROPY,
    OP_SOFTMAX, OP_FLASHATTENTION, OP_BIASGELU,
    OP_EXP, OP_LOG, OP_DIV, OP_SIGMOID, OP_POW, OP_MAX, OP_LAYERNORM,
    OP_EMBEDDING, OP_DROPOUT, OP_RESIDUALLAYERNORM
};

/* autograd.rs:65-70 TapeEntry + the SavedContext variants the subset needs */
typedef struct {
    int op;
    size_t output_id;
    size_t input_ids[4];
    int n_inputs;
    size_t saved_ids[4];          /* Tensor / Tensors / TensorsAndShape ids  */
    size_t saved_shape[ORC_MAX_DIMS]; /* Shape / TensorAndShape / Permutation orig */
    int saved_ndim;
    size_t saved_perm[ORC_MAX_DIMS];
    float saved_scalar;
    size_t *targets;              /* Indices(targets, n, v, sm_id)           */
    size_t ce_n, ce_v, ce_sm;
    size_t fa_out, fa_lse;        /* FlashAttention{q,k,v,out,lse,scale,s,d,causal} */
    int fa_causal;
    size_t emb_batch, emb_seq;    /* Indices(indices, batch, seq_len, weight) */
    size_t drop_mask;             /* DropoutMask(mask_id, rate): rate in saved_scalar */
} orc_entry;

typedef struct {
    orc_entry *e;
    size_t len, cap;
    int enabled;
} orc_tape;

static orc_store g_store;
static orc_tape g_tape = {0, 0, 0, 1};
static char g_err[512];

static uint32_t fail(const char *msg) {
    snprintf(g_err, sizeof g_err, "%s", msg);
    return ORC_BAD;
}
const char *orc_last_error(void) { return g_err; }

/* ---- shape helpers ------------------------------------------------------ */

/* tensor.rs:7-17 compute_strides */
static void compute_strides(const size_t *shape, int ndim, size_t *strides) {
    if (ndim == 0) return;
    strides[ndim - 1] = 1;
    for (int i = ndim - 2; i >= 0; --i) strides[i] = strides[i + 1] * shape[i + 1];
}

/* tensor.rs:19-21 shape_size: product, at least 1 */
static size_t shape_size(const size_t *shape, int ndim) {
    size_t p = 1;
    for (int i = 0; i < ndim; ++i) p *= shape[i];
    return p < 1 ? 1 : p;
}

/* tensor.rs:41-53 is_contiguous: every dim checked, size-1 dims included */
static int is_contiguous(const orc_tensor *t) {
    if (t->ndim == 0) return 1;
    size_t expected = 1;
    for (int i = t->ndim - 1; i >= 0; --i) {
        if (t->strides[i] != expected) return 0;
        expected *= t->shape[i];
    }
    return 1;
}

/* utils.rs:3-20 broadcast_shape; returns -1 where the reference panics */
static int broadcast_shape(const size_t *a, int na, const size_t *b, int nb, size_t *out) {
    int n = na > nb ? na : nb;
    for (int i = 0; i < n; ++i) {
        size_t da = i < n - na ? 1 : a[i - (n - na)];
        size_t db = i < n - nb ? 1 : b[i - (n - nb)];
        if (da == db) out[i] = da;
        else if (da == 1) out[i] = db;
        else if (db == 1) out[i] = da;
        else return -1;
    }
    return n;
}

static int same_shape(const size_t *a, int na, const size_t *b, int nb) {
    if (na != nb) return 0;
    for (int i = 0; i < na; ++i) if (a[i] != b[i]) return 0;
    return 1;
}

/* utils.rs:39-66 unbroadcast: sum a grad of grad_shape down to orig_shape,
 * visiting grad elements in flat order (so each output receives its terms in
 * increasing flat index). */
static float *unbroadcast(const float *g, const size_t *gshape, int gnd,
                          const size_t *oshape, int ond) {
    size_t osz = shape_size(oshape, ond);
    if (same_shape(gshape, gnd, oshape, ond)) {
        float *out = (float *)malloc(osz * sizeof(float));
        memcpy(out, g, osz * sizeof(float));
        return out;
    }
    float *out = (float *)calloc(osz, sizeof(float));
    size_t gstr[ORC_MAX_DIMS], ostr[ORC_MAX_DIMS];
    compute_strides(gshape, gnd, gstr);
    compute_strides(oshape, ond, ostr);
    int offset = gnd - ond;
    size_t gsz = shape_size(gshape, gnd);
    for (size_t i = 0; i < gsz; ++i) {
        size_t rem = i, out_idx = 0;
        for (int d = 0; d < gnd; ++d) {
            size_t c = rem / gstr[d];
            rem %= gstr[d];
            if (d >= offset) {
                int od = d - offset;
                out_idx += (oshape[od] == 1 ? 0 : c) * ostr[od];
            }
        }
        out[out_idx] += g[i];
    }
    return out;
}

/* ---- store -------------------------------------------------------------- */

/* tensor.rs:104-113 insert: pop the most recently freed id, else append */
static size_t store_insert(float *data, const size_t *shape, const size_t *strides, int ndim, size_t size) {
    size_t id;
    if (g_store.nfree) {
        id = g_store.free_ids[--g_store.nfree];
    } else {
        if (g_store.len == g_store.cap) {
            g_store.cap = g_store.cap ? g_store.cap * 2 : 64;
            g_store.t = (orc_tensor *)realloc(g_store.t, g_store.cap * sizeof(orc_tensor));
        }
        id = g_store.len++;
    }
    orc_tensor *t = &g_store.t[id];
    memset(t, 0, sizeof *t);
    t->live = 1;
    t->data = data;
    t->ndim = ndim;
    for (int i = 0; i < ndim; ++i) { t->shape[i] = shape[i]; t->strides[i] = strides[i]; }
    t->size = size;
    t->grad = -1;
    return id;
}

/* tensor.rs:263-270 from_vec (takes ownership of data) */
static size_t from_vec(float *data, const size_t *shape, int ndim) {
    size_t strides[ORC_MAX_DIMS];
    compute_strides(shape, ndim, strides);
    return store_insert(data, shape, strides, ndim, shape_size(shape, ndim));
}

/* tensor.rs:115-117 get: "tensor already freed" panic -> NULL */
static orc_tensor *get(size_t id) {
    if (id >= g_store.len || !g_store.t[id].live) return NULL;
    return &g_store.t[id];
}

/* tensor.rs:169-174 free */
static void store_free(size_t id) {
    if (id >= g_store.len || !g_store.t[id].live) return;
    orc_tensor *t = &g_store.t[id];
    free(t->data); free(t->adam_m); free(t->adam_v);
    t->live = 0; t->data = NULL; t->adam_m = t->adam_v = NULL;
    if (g_store.nfree == g_store.capfree) {
        g_store.capfree = g_store.capfree ? g_store.capfree * 2 : 64;
        g_store.free_ids = (size_t *)realloc(g_store.free_ids, g_store.capfree * sizeof(size_t));
    }
    g_store.free_ids[g_store.nfree++] = id;
}

/* tensor.rs:292-309 make_contiguous_data: gather by strides in flat order */
static float *make_contiguous_data(const orc_tensor *t) {
    float *out = (float *)calloc(t->size ? t->size : 1, sizeof(float));
    size_t ostr[ORC_MAX_DIMS];
    compute_strides(t->shape, t->ndim, ostr);
    for (size_t i = 0; i < t->size; ++i) {
        size_t src = 0, rem = i;
        for (int d = 0; d < t->ndim; ++d) {
            size_t c = rem / ostr[d];
            rem %= ostr[d];
            src += c * t->strides[d];
        }
        out[i] = t->data[src];
    }
    return out;
}

/* tensor.rs:184-191 to_host: always a fresh copy */
static float *to_host(const orc_tensor *t) {
    if (is_contiguous(t)) {
        float *out = (float *)malloc((t->size ? t->size : 1) * sizeof(float));
        memcpy(out, t->data, t->size * sizeof(float));
        return out;
    }
    return make_contiguous_data(t);
}

/* tensor.rs:311-318 ensure_contiguous: same id when already contiguous */
static size_t ensure_contiguous(size_t id) {
    orc_tensor *t = get(id);
    if (is_contiguous(t)) return id;
    float *d = make_contiguous_data(t);
    size_t shape[ORC_MAX_DIMS]; int nd = t->ndim;
    memcpy(shape, t->shape, sizeof shape);
    return from_vec(d, shape, nd);
}

/* tensor.rs:207-215 zeros / :217-226 ones */
static size_t zeros(const size_t *shape, int ndim) {
    size_t n = shape_size(shape, ndim);
    return from_vec((float *)calloc(n, sizeof(float)), shape, ndim);
}
static size_t ones(const size_t *shape, int ndim) {
    size_t n = shape_size(shape, ndim);
    float *d = (float *)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; ++i) d[i] = 1.0f;
    return from_vec(d, shape, ndim);
}

/* tensor.rs:144-152 ensure_grad */
static size_t ensure_grad(size_t id) {
    orc_tensor *t = get(id);
    if (t->grad >= 0) return (size_t)t->grad;
    size_t shape[ORC_MAX_DIMS]; int nd = t->ndim;
    memcpy(shape, t->shape, sizeof shape);
    size_t g = zeros(shape, nd);
    get(id)->grad = (long)g;
    return g;
}

/* tensor.rs:272-280 accumulate_grad: raw-buffer order, src.size elements */
static void accumulate_grad(size_t dst, size_t src) {
    size_t gid = ensure_grad(dst);
    orc_tensor *s = get(src), *g = get(gid);
    for (size_t i = 0; i < s->size; ++i) g->data[i] += s->data[i];
}

/* tensor.rs:283-290 add_inplace */
static void add_inplace(size_t dst, size_t src) {
    orc_tensor *s = get(src), *d = get(dst);
    for (size_t i = 0; i < s->size; ++i) d->data[i] += s->data[i];
}

/* ---- tape --------------------------------------------------------------- */

/* autograd.rs:90-94 record */
static orc_entry *tape_record(orc_tape *tp, int op, size_t out, int n_in, size_t in0, size_t in1) {
    static orc_entry dummy;
    if (!tp->enabled) { memset(&dummy, 0, sizeof dummy); return &dummy; }
    if (tp->len == tp->cap) {
        tp->cap = tp->cap ? tp->cap * 2 : 64;
        tp->e = (orc_entry *)realloc(tp->e, tp->cap * sizeof(orc_entry));
    }
    orc_entry *e = &tp->e[tp->len++];
    memset(e, 0, sizeof *e);
    e->op = op; e->output_id = out; e->n_inputs = n_in;
    e->input_ids[0] = in0; e->input_ids[1] = in1;
    e->saved_ids[0] = in0; e->saved_ids[1] = in1;
    return e;
}

static void tape_clear(orc_tape *tp) {
    for (size_t i = 0; i < tp->len; ++i) free(tp->e[i].targets);
    free(tp->e);
    tp->e = NULL; tp->len = tp->cap = 0; tp->enabled = 1;
}

/* ---- matmul (the path) -------------------------------------------------- */

/* ops/matmul.rs:18-78 matmul, cpu arm.  Both operands are materialised
 * contiguous (:20-21) and cloned (:45-46); the batch index of an operand is
 * `batch % operand_batch_size` (:55-56); the hot loop is i-k-j with an f32
 * accumulator that starts at +0.0 (:62-69).
 * pinned by: test/tensor.test.ts:222-240 vectors, f64 brute force, A*I=A,
 * ones*ones=K, integer-exact cases (tests/test_oracle_matmul.py). */
static uint32_t matmul_impl(size_t a, size_t b, orc_tape *tp) {
    if (!get(a) || !get(b)) return fail("tensor already freed");
    size_t a_id = ensure_contiguous(a);
    size_t b_id = ensure_contiguous(b);
    orc_tensor *A = get(a_id), *B = get(b_id);
    if (A->ndim < 2 || B->ndim < 2) return fail("matmul requires at least 2D tensors");
    size_t m = A->shape[A->ndim - 2], k = A->shape[A->ndim - 1];
    size_t k2 = B->shape[B->ndim - 2], n = B->shape[B->ndim - 1];
    if (k != k2) return fail("matmul inner dimensions must match");

    size_t out_shape[ORC_MAX_DIMS];
    int nb = broadcast_shape(A->shape, A->ndim - 2, B->shape, B->ndim - 2, out_shape);
    if (nb < 0) return fail("shapes are not broadcastable");
    if (nb + 2 > ORC_MAX_DIMS) return fail("too many dims");
    size_t batch_size = shape_size(out_shape, nb);
    out_shape[nb] = m; out_shape[nb + 1] = n;
    size_t a_bs = shape_size(A->shape, A->ndim - 2);
    size_t b_bs = shape_size(B->shape, B->ndim - 2);

    float *a_data = to_host(A);
    float *b_data = to_host(B);
    size_t out_size = shape_size(out_shape, nb + 2);
    float *out = (float *)calloc(out_size, sizeof(float));
    size_t a_mat = m * k, b_mat = k * n, c_mat = m * n;

    for (size_t batch = 0; batch < batch_size; ++batch) {
        size_t a_bi = a_bs == 1 ? 0 : batch % a_bs;
        size_t b_bi = b_bs == 1 ? 0 : batch % b_bs;
        const float *ap = a_data + a_bi * a_mat;
        const float *bp = b_data + b_bi * b_mat;
        float *cp = out + batch * c_mat;
        for (size_t i = 0; i < m; ++i) {
            for (size_t kk = 0; kk < k; ++kk) {
                float a_val = ap[i * k + kk];
                const float *brow = bp + kk * n;
                float *crow = cp + i * n;
                for (size_t j = 0; j < n; ++j) crow[j] += a_val * brow[j];
            }
        }
    }
    free(a_data); free(b_data);
    size_t out_id = from_vec(out, out_shape, nb + 2);
    tape_record(tp, OP_MATMUL, out_id, 2, a, b); /* original ids, :73-76 */
    return (uint32_t)out_id;
}

/* ops/matmul.rs:329-333 matmul_no_grad: a throwaway disabled tape */
static uint32_t matmul_no_grad(size_t a, size_t b) {
    orc_tape dummy = {0, 0, 0, 0};
    return matmul_impl(a, b, &dummy);
}

/* ops/matmul.rs:258-284 transpose_last2, cpu arm
 * pinned by: (A*B)^T = B^T*A^T and numpy transpose in tests. */
static size_t transpose_last2(size_t a) {
    orc_tensor *t = get(a);
    size_t shape[ORC_MAX_DIMS]; int nd = t->ndim;
    memcpy(shape, t->shape, sizeof shape);
    size_t a_id = ensure_contiguous(a);
    float *data = to_host(get(a_id));
    size_t m = shape[nd - 2], n = shape[nd - 1];
    size_t bs = 1;
    for (int i = 0; i < nd - 2; ++i) bs *= shape[i];
    if (bs < 1) bs = 1;
    size_t total = get(a_id)->size;
    float *out = (float *)calloc(total ? total : 1, sizeof(float));
    size_t mat = m * n;
    for (size_t b = 0; b < bs; ++b) {
        size_t off = b * mat;
        for (size_t i = 0; i < m; ++i)
            for (size_t j = 0; j < n; ++j) out[off + j * m + i] = data[off + i * n + j];
    }
    free(data);
    shape[nd - 2] = n; shape[nd - 1] = m;
    return from_vec(out, shape, nd);
}

/* ops/matmul.rs:199-222 matmul_backward, cpu arm: both grads always.
 * pinned by: dX/dY of test/autograd.test.ts:42-46 in closed form, f64 central
 * differences on small cases, broadcast-batch sums vs numpy. */
static int matmul_backward(size_t grad, const orc_entry *e, long *out) {
    size_t a = e->saved_ids[0], b = e->saved_ids[1];
    if (!get(a) || !get(b) || !get(grad)) { fail("tensor already freed"); return -1; }
    size_t a_shape[ORC_MAX_DIMS], b_shape[ORC_MAX_DIMS];
    int a_nd = get(a)->ndim, b_nd = get(b)->ndim;
    memcpy(a_shape, get(a)->shape, sizeof a_shape);
    memcpy(b_shape, get(b)->shape, sizeof b_shape);

    size_t b_t = transpose_last2(b);
    uint32_t grad_a = matmul_no_grad(grad, b_t);
    if (grad_a == ORC_BAD) return -1;
    float *gad = to_host(get(grad_a));
    float *ga = unbroadcast(gad, get(grad_a)->shape, get(grad_a)->ndim, a_shape, a_nd);
    free(gad);
    out[0] = (long)from_vec(ga, a_shape, a_nd);

    size_t a_t = transpose_last2(a);
    uint32_t grad_b = matmul_no_grad(a_t, grad);
    if (grad_b == ORC_BAD) return -1;
    float *gbd = to_host(get(grad_b));
    float *gb = unbroadcast(gbd, get(grad_b)->shape, get(grad_b)->ndim, b_shape, b_nd);
    free(gbd);
    out[1] = (long)from_vec(gb, b_shape, b_nd);
    return 0;
}

/* ---- elementwise -------------------------------------------------------- */

/* ops/elementwise.rs:20-56 broadcast_binary; op: 0 add, 1 sub, 2 mul, 3 div,
 * 4 lt, 5 eq, 6 gt (1.0 / 0.0, :1099-1216), 7 is_close with tolerance `tol` (:1258-1288)
 * pinned by: test/tensor.test.ts:248-256 broadcast values, numpy broadcasting. */
static float g_binary_tol;
static uint32_t broadcast_binary(size_t a, size_t b, int op, size_t *out_shape, int *out_nd) {
    orc_tensor *A = get(a), *B = get(b);
    if (!A || !B) return fail("tensor already freed");
    int nd = broadcast_shape(A->shape, A->ndim, B->shape, B->ndim, out_shape);
    if (nd < 0) return fail("shapes are not broadcastable");
    size_t out_size = shape_size(out_shape, nd);
    size_t ostr[ORC_MAX_DIMS], astr[ORC_MAX_DIMS], bstr[ORC_MAX_DIMS];
    compute_strides(out_shape, nd, ostr);
    compute_strides(A->shape, A->ndim, astr);
    compute_strides(B->shape, B->ndim, bstr);
    float *ad = to_host(A), *bd = to_host(B);
    float *out = (float *)calloc(out_size, sizeof(float));
    int a_off = nd - A->ndim, b_off = nd - B->ndim;
    for (size_t i = 0; i < out_size; ++i) {
        size_t coord[ORC_MAX_DIMS], rem = i;
        for (int d = 0; d < nd; ++d) { coord[d] = rem / ostr[d]; rem %= ostr[d]; }
        size_t ai = 0, bi = 0;
        for (int d = 0; d < A->ndim; ++d) ai += (A->shape[d] == 1 ? 0 : coord[d + a_off]) * astr[d];
        for (int d = 0; d < B->ndim; ++d) bi += (B->shape[d] == 1 ? 0 : coord[d + b_off]) * bstr[d];
        float x = ad[ai], y = bd[bi];
        out[i] = op == 0 ? x + y : op == 1 ? x - y : op == 2 ? x * y : op == 3 ? x / y
               : op == 4 ? (x < y ? 1.0f : 0.0f) : op == 5 ? (x == y ? 1.0f : 0.0f) : op == 6 ? (x > y ? 1.0f : 0.0f)
               : (fabsf(x - y) < g_binary_tol ? 1.0f : 0.0f);
    }
    free(ad); free(bd);
    *out_nd = nd;
    return (uint32_t)from_vec(out, out_shape, nd);
}

/* ops/elementwise.rs:62-73 add, :237-248 mul, :474-485 sub */
static uint32_t binary_op(size_t a, size_t b, int op) {
    size_t shape[ORC_MAX_DIMS]; int nd;
    uint32_t out = broadcast_binary(a, b, op, shape, &nd);
    if (out == ORC_BAD) return out;
    orc_entry *e = tape_record(&g_tape, op == 0 ? OP_ADD : op == 1 ? OP_SUB : OP_MUL, out, 2, a, b);
    memcpy(e->saved_shape, shape, sizeof shape);
    e->saved_ndim = nd;
    return out;
}

/* ops/elementwise.rs:199-211 add_backward, :558-571 sub_backward */
static int addsub_backward(size_t grad, const orc_entry *e, long *out, int is_sub) {
    orc_tensor *A = get(e->saved_ids[0]), *B = get(e->saved_ids[1]), *G = get(grad);
    if (!A || !B || !G) { fail("tensor already freed"); return -1; }
    size_t a_shape[ORC_MAX_DIMS], b_shape[ORC_MAX_DIMS], g_shape[ORC_MAX_DIMS];
    int a_nd = A->ndim, b_nd = B->ndim, g_nd = G->ndim;
    memcpy(a_shape, A->shape, sizeof a_shape);
    memcpy(b_shape, B->shape, sizeof b_shape);
    memcpy(g_shape, G->shape, sizeof g_shape);
    size_t gsz = G->size;
    float *gd = to_host(G);
    float *ga = unbroadcast(gd, g_shape, g_nd, a_shape, a_nd);
    if (is_sub) for (size_t i = 0; i < gsz; ++i) gd[i] = -gd[i];
    float *gb = unbroadcast(gd, g_shape, g_nd, b_shape, b_nd);
    free(gd);
    out[0] = (long)from_vec(ga, a_shape, a_nd);
    out[1] = (long)from_vec(gb, b_shape, b_nd);
    return 0;
}

/* ops/elementwise.rs:348-390 mul_backward */
static int mul_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *A = get(e->saved_ids[0]), *B = get(e->saved_ids[1]), *G = get(grad);
    if (!A || !B || !G) { fail("tensor already freed"); return -1; }
    size_t a_shape[ORC_MAX_DIMS], b_shape[ORC_MAX_DIMS], g_shape[ORC_MAX_DIMS];
    int a_nd = A->ndim, b_nd = B->ndim, nd = G->ndim;
    memcpy(a_shape, A->shape, sizeof a_shape);
    memcpy(b_shape, B->shape, sizeof b_shape);
    memcpy(g_shape, G->shape, sizeof g_shape);
    float *ad = to_host(A), *bd = to_host(B), *gd = to_host(G);
    size_t gsz = shape_size(g_shape, nd);
    size_t ostr[ORC_MAX_DIMS], astr[ORC_MAX_DIMS], bstr[ORC_MAX_DIMS];
    compute_strides(g_shape, nd, ostr);
    compute_strides(a_shape, a_nd, astr);
    compute_strides(b_shape, b_nd, bstr);
    float *ga_full = (float *)calloc(gsz, sizeof(float));
    float *gb_full = (float *)calloc(gsz, sizeof(float));
    int a_off = nd - a_nd, b_off = nd - b_nd;
    for (size_t i = 0; i < gsz; ++i) {
        size_t coord[ORC_MAX_DIMS], rem = i;
        for (int d = 0; d < nd; ++d) { coord[d] = rem / ostr[d]; rem %= ostr[d]; }
        size_t ai = 0, bi = 0;
        for (int d = 0; d < a_nd; ++d) ai += (a_shape[d] == 1 ? 0 : coord[d + a_off]) * astr[d];
        for (int d = 0; d < b_nd; ++d) bi += (b_shape[d] == 1 ? 0 : coord[d + b_off]) * bstr[d];
        ga_full[i] = gd[i] * bd[bi];
        gb_full[i] = gd[i] * ad[ai];
    }
    float *ga = unbroadcast(ga_full, g_shape, nd, a_shape, a_nd);
    float *gb = unbroadcast(gb_full, g_shape, nd, b_shape, b_nd);
    free(ad); free(bd); free(gd); free(ga_full); free(gb_full);
    out[0] = (long)from_vec(ga, a_shape, a_nd);
    out[1] = (long)from_vec(gb, b_shape, b_nd);
    return 0;
}

/* ops/elementwise.rs:918-928 div; comparisons record nothing on the tape */
static uint32_t div_op(size_t a, size_t b) {
    size_t shape[ORC_MAX_DIMS]; int nd;
    uint32_t out = broadcast_binary(a, b, 3, shape, &nd);
    if (out == ORC_BAD) return out;
    tape_record(&g_tape, OP_DIV, out, 2, a, b);
    return out;
}
static uint32_t compare_op(size_t a, size_t b, int op, float tol) {
    size_t shape[ORC_MAX_DIMS]; int nd;
    g_binary_tol = tol;
    return broadcast_binary(a, b, op, shape, &nd);
}
/* ops/elementwise.rs:991-1029 div_backward: da = g / b, db = -g * a / (b * b), unbroadcast.
 * pinned by: float64 closed form with and without broadcasting. */
static int div_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *A = get(e->saved_ids[0]), *B = get(e->saved_ids[1]), *G = get(grad);
    if (!A || !B || !G) { fail("tensor already freed"); return -1; }
    size_t a_shape[ORC_MAX_DIMS], b_shape[ORC_MAX_DIMS], g_shape[ORC_MAX_DIMS];
    int a_nd = A->ndim, b_nd = B->ndim, nd = G->ndim;
    memcpy(a_shape, A->shape, sizeof a_shape);
    memcpy(b_shape, B->shape, sizeof b_shape);
    memcpy(g_shape, G->shape, sizeof g_shape);
    float *ad = to_host(A), *bd = to_host(B), *gd = to_host(G);
    size_t gsz = shape_size(g_shape, nd);
    size_t ostr[ORC_MAX_DIMS], astr[ORC_MAX_DIMS], bstr[ORC_MAX_DIMS];
    compute_strides(g_shape, nd, ostr);
    compute_strides(a_shape, a_nd, astr);
    compute_strides(b_shape, b_nd, bstr);
    float *ga_full = (float *)calloc(gsz ? gsz : 1, sizeof(float));
    float *gb_full = (float *)calloc(gsz ? gsz : 1, sizeof(float));
    int a_off = nd - a_nd, b_off = nd - b_nd;
    for (size_t i = 0; i < gsz; ++i) {
        size_t coord[ORC_MAX_DIMS], rem = i;
        for (int d = 0; d < nd; ++d) { coord[d] = rem / ostr[d]; rem %= ostr[d]; }
        size_t ai = 0, bi = 0;
        for (int d = 0; d < a_nd; ++d) ai += (a_shape[d] == 1 ? 0 : coord[d + a_off]) * astr[d];
        for (int d = 0; d < b_nd; ++d) bi += (b_shape[d] == 1 ? 0 : coord[d + b_off]) * bstr[d];
        ga_full[i] = gd[i] / bd[bi];
        gb_full[i] = -gd[i] * ad[ai] / (bd[bi] * bd[bi]);
    }
    float *ga = unbroadcast(ga_full, g_shape, nd, a_shape, a_nd);
    float *gb = unbroadcast(gb_full, g_shape, nd, b_shape, b_nd);
    free(ad); free(bd); free(gd); free(ga_full); free(gb_full);
    out[0] = (long)from_vec(ga, a_shape, a_nd);
    out[1] = (long)from_vec(gb, b_shape, b_nd);
    return 0;
}

/* ops/elementwise.rs:760-770 exp, :839-849 log, :1341-1351 pow (powf);
 * ops/activation.rs:194-204 sigmoid.  kind: 0 exp, 1 log, 2 sigmoid, 3 pow.
 * Saved: exp and sigmoid keep their OUTPUT, log and pow their input.
 * pinned by: float64 closed forms; derivative identities. */
static uint32_t unary2_op(size_t a, int kind, float s) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    float *d = to_host(A);
    for (size_t i = 0; i < A->size; ++i) {
        float x = d[i];
        d[i] = kind == 0 ? expf(x) : kind == 1 ? logf(x) : kind == 2 ? 1.0f / (1.0f + expf(-x)) : powf(x, s);
    }
    size_t shape[ORC_MAX_DIMS]; int nd = A->ndim;
    memcpy(shape, A->shape, sizeof shape);
    size_t out = from_vec(d, shape, nd);
    static const int ops[4] = {OP_EXP, OP_LOG, OP_SIGMOID, OP_POW};
    orc_entry *e = tape_record(&g_tape, ops[kind], out, 1, a, 0);
    e->saved_scalar = s;
    e->saved_ids[0] = (kind == 0 || kind == 2) ? out : a;
    return (uint32_t)out;
}
/* ops/elementwise.rs:800-809 exp_backward (g * out), :879-888 log_backward (g / x),
 * :1375-1386 pow_backward (g * e * x^(e-1)); ops/activation.rs:231-241 sigmoid_backward (g * o * (1 - o)) */
static int unary2_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *G = get(grad), *S = get(e->saved_ids[0]);
    if (!G || !S) { fail("tensor already freed"); return -1; }
    float *gd = to_host(G), *sd = to_host(S);
    size_t shape[ORC_MAX_DIMS]; int nd = G->ndim; size_t n = G->size;
    memcpy(shape, G->shape, sizeof shape);
    for (size_t i = 0; i < n; ++i) {
        float g = gd[i], v = sd[i];
        gd[i] = e->op == OP_EXP ? g * v : e->op == OP_LOG ? g / v : e->op == OP_SIGMOID ? g * v * (1.0f - v)
              : g * e->saved_scalar * powf(v, e->saved_scalar - 1.0f);
    }
    free(sd);
    out[0] = (long)from_vec(gd, shape, nd);
    return 0;
}

/* ---- unary ops ---------------------------------------------------------- */

/* ops/activation.rs:15-18 gelu_scalar (tanh approximation) */
static float gelu_scalar(float x) {
    float s = sqrtf(2.0f / 3.14159265358979323846f);
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}
/* ops/activation.rs:20-28 gelu_grad_scalar */
static float gelu_grad_scalar(float x) {
    float s = sqrtf(2.0f / 3.14159265358979323846f);
    float inner = s * (x + 0.044715f * x * x * x);
    float th = tanhf(inner);
    float sech2 = 1.0f - th * th;
    float d_inner = s * (1.0f + 3.0f * 0.044715f * x * x);
    return 0.5f * (1.0f + th) + 0.5f * x * sech2 * d_inner;
}

/* ops/activation.rs:34-44 gelu_forward, :114-124 relu_forward;
 * ops/elementwise.rs neg / mul_scalar (same map-over-to_host shape).
 * kind: 0 relu, 1 gelu, 2 neg, 3 mul_scalar
 * pinned by: test/nn.test.ts:17-27 relu/gelu anchors, f64 closed forms. */
static uint32_t unary_op(size_t a, int kind, float s) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    float *d = to_host(A);
    for (size_t i = 0; i < A->size; ++i) {
        float x = d[i];
        d[i] = kind == 0 ? (x > 0.0f ? x : 0.0f) /* f32::max(x, 0.0) */
             : kind == 1 ? gelu_scalar(x)
             : kind == 2 ? -x : x * s;
    }
    size_t shape[ORC_MAX_DIMS]; int nd = A->ndim;
    memcpy(shape, A->shape, sizeof shape);
    size_t out = from_vec(d, shape, nd);
    static const int ops[4] = {OP_RELU, OP_GELU, OP_NEG, OP_MULSCALAR};
    orc_entry *e = tape_record(&g_tape, ops[kind], out, 1, a, 0);
    e->saved_scalar = s;
    return (uint32_t)out;
}

/* ops/activation.rs:74-84 gelu_backward, :154-164 relu_backward; neg and
 * mul_scalar backward scale the grad. */
static int unary_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *G = get(grad);
    if (!G) { fail("tensor already freed"); return -1; }
    float *gd = to_host(G);
    size_t shape[ORC_MAX_DIMS]; int nd = G->ndim; size_t n = G->size;
    memcpy(shape, G->shape, sizeof shape);
    if (e->op == OP_RELU || e->op == OP_GELU) {
        orc_tensor *X = get(e->saved_ids[0]);
        if (!X) { free(gd); fail("tensor already freed"); return -1; }
        float *xd = to_host(X);
        for (size_t i = 0; i < n; ++i)
            gd[i] = e->op == OP_RELU ? (xd[i] > 0.0f ? gd[i] : 0.0f) : gd[i] * gelu_grad_scalar(xd[i]);
        free(xd);
    } else if (e->op == OP_NEG) {
        for (size_t i = 0; i < n; ++i) gd[i] = -gd[i];
    } else {
        for (size_t i = 0; i < n; ++i) gd[i] = gd[i] * e->saved_scalar;
    }
    out[0] = (long)from_vec(gd, shape, nd);
    return 0;
}

/* ---- reductions --------------------------------------------------------- */

/* ops/reduce.rs:5-7 resolve_dim */
static int resolve_dim(int dim, int ndim) { return dim < 0 ? ndim + dim : dim; }

/* ops/reduce.rs:13-46 sum along dim (kept as size 1), flat-order accumulation */
static uint32_t sum_impl(size_t a, int dim, orc_tape *tp) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    int nd = A->ndim;
    int d = resolve_dim(dim, nd);
    if (d < 0 || d >= nd) return fail("reduce dim out of range");
    size_t a_shape[ORC_MAX_DIMS], out_shape[ORC_MAX_DIMS];
    memcpy(a_shape, A->shape, sizeof a_shape);
    memcpy(out_shape, A->shape, sizeof out_shape);
    out_shape[d] = 1;
    float *ad = to_host(A);
    size_t out_size = shape_size(out_shape, nd);
    float *out = (float *)calloc(out_size, sizeof(float));
    size_t astr[ORC_MAX_DIMS], ostr[ORC_MAX_DIMS];
    compute_strides(a_shape, nd, astr);
    compute_strides(out_shape, nd, ostr);
    size_t total = shape_size(a_shape, nd);
    for (size_t i = 0; i < total; ++i) {
        size_t oi = 0, rem = i;
        for (int dd = 0; dd < nd; ++dd) {
            size_t c = rem / astr[dd];
            rem %= astr[dd];
            oi += (dd == d ? 0 : c) * ostr[dd];
        }
        out[oi] += ad[i];
    }
    free(ad);
    size_t out_id = from_vec(out, out_shape, nd);
    orc_entry *e = tape_record(tp, OP_SUM, out_id, 1, a, 0);
    memcpy(e->saved_shape, a_shape, sizeof a_shape);
    e->saved_ndim = nd;
    return (uint32_t)out_id;
}

/* ops/reduce.rs:169-184 mean = sum (recorded) then divide (recorded as Mean
 * with the same input) */
static uint32_t mean_impl(size_t a, int dim) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    int nd = A->ndim;
    int d = resolve_dim(dim, nd);
    if (d < 0 || d >= nd) return fail("reduce dim out of range");
    size_t a_shape[ORC_MAX_DIMS];
    memcpy(a_shape, A->shape, sizeof a_shape);
    float count = (float)a_shape[d];
    uint32_t s = sum_impl(a, dim, &g_tape);
    if (s == ORC_BAD) return s;
    orc_tensor *S = get(s);
    float *sd = to_host(S);
    for (size_t i = 0; i < S->size; ++i) sd[i] = sd[i] / count;
    size_t shape[ORC_MAX_DIMS]; int snd = S->ndim;
    memcpy(shape, S->shape, sizeof shape);
    size_t out = from_vec(sd, shape, snd);
    orc_entry *e = tape_record(&g_tape, OP_MEAN, out, 1, a, 0);
    memcpy(e->saved_shape, a_shape, sizeof a_shape);
    e->saved_ndim = nd;
    return (uint32_t)out;
}

/* ops/reduce.rs:94-118 sum_backward; :232-263 mean_backward (divisor = the
 * LAST dim with grad 1 and orig > 1, else 1) */
static int reduce_backward(size_t grad, const orc_entry *e, long *out, int is_mean) {
    orc_tensor *G = get(grad);
    if (!G) { fail("tensor already freed"); return -1; }
    int nd = e->saved_ndim;
    const size_t *orig = e->saved_shape;
    size_t gshape[ORC_MAX_DIMS];
    memcpy(gshape, G->shape, sizeof gshape);
    float *gd = to_host(G);
    size_t osz = shape_size(orig, nd);
    size_t gstr[ORC_MAX_DIMS], ostr[ORC_MAX_DIMS];
    compute_strides(gshape, G->ndim, gstr);
    compute_strides(orig, nd, ostr);
    float div = 1.0f;
    if (is_mean)
        for (int d = 0; d < nd; ++d)
            if (gshape[d] == 1 && orig[d] > 1) div = (float)orig[d];
    float *o = (float *)calloc(osz, sizeof(float));
    for (size_t i = 0; i < osz; ++i) {
        size_t gi = 0, rem = i;
        for (int d = 0; d < nd; ++d) {
            size_t c = rem / ostr[d];
            rem %= ostr[d];
            gi += (gshape[d] == 1 ? 0 : c) * gstr[d];
        }
        o[i] = is_mean ? gd[gi] / div : gd[gi];
    }
    free(gd);
    out[0] = (long)from_vec(o, orig, nd);
    return 0;
}

/* ---- layout ------------------------------------------------------------- */

/* ops/layout.rs:66-77 view (always a copy) */
static uint32_t view_impl(size_t a, const size_t *new_shape, int nd) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    size_t orig[ORC_MAX_DIMS]; int ond = A->ndim;
    memcpy(orig, A->shape, sizeof orig);
    size_t a_id = ensure_contiguous(a);
    float *d = to_host(get(a_id));
    size_t out = from_vec(d, new_shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_VIEW, out, 1, a, 0);
    memcpy(e->saved_shape, orig, sizeof orig);
    e->saved_ndim = ond;
    return (uint32_t)out;
}

/* ops/layout.rs:112-134 permute: cloned raw buffer + permuted shape/strides */
static uint32_t permute_impl(size_t a, const size_t *dims, int nd) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    if (nd != A->ndim) return fail("permute dims length mismatch");
    size_t ns[ORC_MAX_DIMS], nst[ORC_MAX_DIMS], a_shape[ORC_MAX_DIMS];
    memcpy(a_shape, A->shape, sizeof a_shape);
    for (int i = 0; i < nd; ++i) {
        if (dims[i] >= (size_t)nd) return fail("permute dim out of range");
        ns[i] = A->shape[dims[i]];
        nst[i] = A->strides[dims[i]];
    }
    size_t size = A->size;
    float *d = (float *)malloc((size ? size : 1) * sizeof(float));
    memcpy(d, A->data, size * sizeof(float));
    size_t out = store_insert(d, ns, nst, nd, size);
    orc_entry *e = tape_record(&g_tape, OP_PERMUTE, out, 1, a, 0);
    memcpy(e->saved_shape, a_shape, sizeof a_shape);
    e->saved_ndim = nd;
    for (int i = 0; i < nd; ++i) e->saved_perm[i] = dims[i];
    return (uint32_t)out;
}

/* ops/layout.rs:162-195 permute_backward: inverse-permutation scatter */
static int permute_backward(size_t grad, const orc_entry *e, long *out) {
    if (!get(grad)) { fail("tensor already freed"); return -1; }
    int nd = e->saved_ndim;
    size_t inv[ORC_MAX_DIMS];
    for (int i = 0; i < nd; ++i) inv[e->saved_perm[i]] = (size_t)i;
    size_t gc = ensure_contiguous(grad);
    orc_tensor *G = get(gc);
    float *d = to_host(G);
    size_t sstr[ORC_MAX_DIMS], ostr[ORC_MAX_DIMS];
    compute_strides(G->shape, nd, sstr);
    compute_strides(e->saved_shape, nd, ostr);
    size_t size = shape_size(G->shape, nd);
    float *o = (float *)calloc(size, sizeof(float));
    for (size_t i = 0; i < size; ++i) {
        size_t coord[ORC_MAX_DIMS], rem = i;
        for (int dd = 0; dd < nd; ++dd) { coord[dd] = rem / sstr[dd]; rem %= sstr[dd]; }
        size_t oi = 0;
        for (int dd = 0; dd < nd; ++dd) oi += coord[inv[dd]] * ostr[dd];
        o[oi] = d[i];
    }
    free(d);
    out[0] = (long)from_vec(o, e->saved_shape, nd);
    return 0;
}

/* ops/layout.rs:92-97 view_backward */
static int view_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *G = get(grad);
    if (!G) { fail("tensor already freed"); return -1; }
    float *d = to_host(G);
    out[0] = (long)from_vec(d, e->saved_shape, e->saved_ndim);
    return 0;
}

/* ---- loss --------------------------------------------------------------- */

/* ops/loss.rs:24-67 cross_entropy, cpu arm (-ln p, no epsilon)
 * pinned by: f64 log-softmax closed form; test/nn.test.ts:70-76 ordering. */
static uint32_t cross_entropy_impl(size_t logits, const int64_t *targets, size_t nt) {
    orc_tensor *L = get(logits);
    if (!L) return fail("tensor already freed");
    int nd = L->ndim;
    if (nd < 1) return fail("cross_entropy needs at least 1 dim");
    size_t shape[ORC_MAX_DIMS];
    memcpy(shape, L->shape, sizeof shape);
    size_t v = shape[nd - 1];
    size_t n = shape_size(shape, nd) / v;
    if (nt < n) return fail("index out of bounds: targets shorter than rows");
    float *data = to_host(L);
    float *sm = (float *)calloc((n * v) > 0 ? n * v : 1, sizeof(float));
    float loss_sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        size_t off = i * v;
        float mx = -INFINITY;
        for (size_t j = 0; j < v; ++j) mx = data[off + j] > mx ? data[off + j] : mx;
        float sum = 0.0f;
        for (size_t j = 0; j < v; ++j) {
            float ex = expf(data[off + j] - mx);
            sm[off + j] = ex;
            sum += ex;
        }
        for (size_t j = 0; j < v; ++j) sm[off + j] /= sum;
        if (targets[i] < 0 || (size_t)targets[i] >= v) {
            free(data); free(sm);
            return fail("index out of bounds: target class");
        }
        loss_sum += -logf(sm[off + (size_t)targets[i]]);
    }
    free(data);
    float *lv = (float *)malloc(sizeof(float));
    lv[0] = loss_sum / (float)n;
    size_t one = 1;
    size_t loss_id = from_vec(lv, &one, 1);
    size_t sm_id = from_vec(sm, shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_CROSSENTROPY, loss_id, 1, logits, 0);
    if (g_tape.enabled) {
        e->targets = (size_t *)malloc((n ? n : 1) * sizeof(size_t));
        for (size_t i = 0; i < n; ++i) e->targets[i] = (size_t)targets[i];
    }
    e->ce_n = n; e->ce_v = v; e->ce_sm = sm_id;
    return (uint32_t)loss_id;
}

/* ops/loss.rs:131-149 cross_entropy_backward */
static int cross_entropy_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *G = get(grad), *S = get(e->ce_sm);
    if (!G || !S) { fail("tensor already freed"); return -1; }
    float grad_val = G->data[0];
    float *dl = to_host(S);
    size_t shape[ORC_MAX_DIMS]; int nd = S->ndim;
    memcpy(shape, S->shape, sizeof shape);
    for (size_t i = 0; i < e->ce_n; ++i) {
        size_t off = i * e->ce_v;
        dl[off + e->targets[i]] -= 1.0f;
        float scale = grad_val / (float)e->ce_n;
        for (size_t j = 0; j < e->ce_v; ++j) dl[off + j] *= scale;
    }
    out[0] = (long)from_vec(dl, shape, nd);
    return 0;
}

/* ops/reduce.rs:333-368 max along dim (kept as size 1): strict `>` against a
 * running maximum that starts at -inf, in flat order.
 * pinned by: numpy max; ties; backward mask. */
static uint32_t max_impl(size_t a, int dim) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    int nd = A->ndim;
    int d = resolve_dim(dim, nd);
    if (d < 0 || d >= nd) return fail("index out of bounds: max dim");
    size_t shape[ORC_MAX_DIMS], oshape[ORC_MAX_DIMS], astr[ORC_MAX_DIMS], ostr[ORC_MAX_DIMS];
    memcpy(shape, A->shape, sizeof shape);
    memcpy(oshape, shape, sizeof oshape);
    oshape[d] = 1;
    compute_strides(shape, nd, astr);
    compute_strides(oshape, nd, ostr);
    size_t total = shape_size(shape, nd), osz = shape_size(oshape, nd);
    float *ad = to_host(A);
    float *out = (float *)malloc((osz ? osz : 1) * sizeof(float));
    for (size_t i = 0; i < osz; ++i) out[i] = -INFINITY;
    for (size_t i = 0; i < total; ++i) {
        size_t oi = 0, rem = i;
        for (int dd = 0; dd < nd; ++dd) {
            size_t coord = rem / astr[dd];
            rem %= astr[dd];
            oi += (dd == d ? 0 : coord) * ostr[dd];
        }
        if (ad[i] > out[oi]) out[oi] = ad[i];
    }
    free(ad);
    size_t out_id = from_vec(out, oshape, nd);
    orc_entry *e = tape_record(&g_tape, OP_MAX, out_id, 1, a, 0);
    e->saved_ids[1] = out_id;
    return (uint32_t)out_id;
}
/* ops/reduce.rs:416-447 max_backward: the grad goes to every element within
 * 1e-6 of the maximum (ties all receive it). */
static int max_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *X = get(e->saved_ids[0]), *M = get(e->saved_ids[1]), *G = get(grad);
    if (!X || !M || !G) { fail("tensor already freed"); return -1; }
    int nd = X->ndim;
    size_t shape[ORC_MAX_DIMS], mshape[ORC_MAX_DIMS], xstr[ORC_MAX_DIMS], mstr[ORC_MAX_DIMS];
    memcpy(shape, X->shape, sizeof shape);
    memcpy(mshape, M->shape, sizeof mshape);
    compute_strides(shape, nd, xstr);
    compute_strides(mshape, nd, mstr);
    float *xd = to_host(X), *md = to_host(M), *gd = to_host(G);
    size_t total = shape_size(shape, nd);
    float *o = (float *)calloc(total ? total : 1, sizeof(float));
    for (size_t i = 0; i < total; ++i) {
        size_t mi = 0, rem = i;
        for (int dd = 0; dd < nd; ++dd) {
            size_t coord = rem / xstr[dd];
            rem %= xstr[dd];
            mi += (mshape[dd] == 1 ? 0 : coord) * mstr[dd];
        }
        if (fabsf(xd[i] - md[mi]) < 1e-6f) o[i] = gd[mi];
    }
    free(xd); free(md); free(gd);
    out[0] = (long)from_vec(o, shape, nd);
    return 0;
}

/* ops/norm.rs:167-215 layernorm over the last extent: mean, biased variance
 * (two passes, f32, index order), rstd = 1 / sqrt(var / c + eps).
 * pinned by: float64 closed form; normalised rows have mean 0, variance 1 when
 * gamma = 1, beta = 0; finite differences of the backward. */
static uint32_t layernorm_impl(size_t x, size_t gamma, size_t beta, float eps) {
    orc_tensor *X = get(x), *Gm = get(gamma), *Bt = get(beta);
    if (!X || !Gm || !Bt) return fail("tensor already freed");
    int nd = X->ndim;
    if (nd < 1) return fail("index out of bounds: layernorm of a scalar");
    size_t shape[ORC_MAX_DIMS];
    memcpy(shape, X->shape, sizeof shape);
    size_t c = shape[nd - 1];
    size_t n = c ? shape_size(shape, nd) / c : 0;
    if (Gm->size < c || Bt->size < c) return fail("index out of bounds: gamma/beta shorter than the last extent");
    float *xd = to_host(X), *gd = to_host(Gm), *bd = to_host(Bt);
    float *mean = (float *)calloc(n ? n : 1, sizeof(float)), *rstd = (float *)calloc(n ? n : 1, sizeof(float));
    float *out = (float *)calloc((n * c) > 0 ? n * c : 1, sizeof(float));
    for (size_t row = 0; row < n; ++row) {
        size_t off = row * c;
        float sum = 0.0f;
        for (size_t j = 0; j < c; ++j) sum += xd[off + j];
        float m = sum / (float)c;
        mean[row] = m;
        float var = 0.0f;
        for (size_t j = 0; j < c; ++j) { float d = xd[off + j] - m; var += d * d; }
        float r = 1.0f / sqrtf(var / (float)c + eps);
        rstd[row] = r;
        for (size_t j = 0; j < c; ++j) out[off + j] = (xd[off + j] - m) * r * gd[j] + bd[j];
    }
    free(xd); free(gd); free(bd);
    size_t mean_id = from_vec(mean, &n, 1), rstd_id = from_vec(rstd, &n, 1);
    size_t out_id = from_vec(out, shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_LAYERNORM, out_id, 3, x, gamma);
    e->input_ids[2] = beta; e->saved_ids[2] = beta;
    e->fa_out = mean_id; e->fa_lse = rstd_id; /* Tensors[x, gamma, mean, rstd] */
    return (uint32_t)out_id;
}
/* ops/norm.rs:273-322 layernorm_backward */
static int layernorm_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *X = get(e->input_ids[0]), *Gm = get(e->input_ids[1]), *Mn = get(e->fa_out), *Rs = get(e->fa_lse), *G = get(grad);
    if (!X || !Gm || !Mn || !Rs || !G) { fail("tensor already freed"); return -1; }
    int nd = X->ndim, gnd = Gm->ndim;
    size_t shape[ORC_MAX_DIMS], gshape[ORC_MAX_DIMS];
    memcpy(shape, X->shape, sizeof shape);
    memcpy(gshape, Gm->shape, sizeof gshape);
    size_t c = shape[nd - 1], n = c ? shape_size(shape, nd) / c : 0;
    float *xd = to_host(X), *gm = to_host(Gm), *mn = to_host(Mn), *rs = to_host(Rs), *gd = to_host(G);
    float *dx = (float *)calloc((n * c) > 0 ? n * c : 1, sizeof(float));
    float *dgamma = (float *)calloc(Gm->size ? Gm->size : 1, sizeof(float));
    float *dbeta = (float *)calloc(Gm->size ? Gm->size : 1, sizeof(float));
    for (size_t row = 0; row < n; ++row) {
        size_t off = row * c;
        float m = mn[row], r = rs[row];
        float sum_dg = 0.0f, sum_dgx = 0.0f;
        for (size_t j = 0; j < c; ++j) {
            float xhat = (xd[off + j] - m) * r;
            float dg = gd[off + j] * gm[j];
            sum_dg += dg;
            sum_dgx += dg * xhat;
            dgamma[j] += gd[off + j] * xhat;
            dbeta[j] += gd[off + j];
        }
        for (size_t j = 0; j < c; ++j) {
            float xhat = (xd[off + j] - m) * r;
            float dg = gd[off + j] * gm[j];
            dx[off + j] = r * (dg - sum_dg / (float)c - xhat * sum_dgx / (float)c);
        }
    }
    free(xd); free(gm); free(mn); free(rs); free(gd);
    out[0] = (long)from_vec(dx, shape, nd);
    out[1] = (long)from_vec(dgamma, gshape, gnd);
    out[2] = (long)from_vec(dbeta, gshape, gnd);
    return 0;
}

/* ---- fused bias + GELU ---------------------------------------------------- */

/* ops/fused.rs:247-273 bias_gelu, cpu arm: val = x[i] + bias[i % c] with c the
 * last extent of x, GELU with the literal constant 0.7978845608 (:263).
 * pinned by: equality with gelu(add(x, bias)) of this oracle to rounding,
 * float64 closed form, shape assertion of test/native.test.ts:39-43. */
static uint32_t bias_gelu_impl(size_t x, size_t bias) {
    orc_tensor *X = get(x), *B = get(bias);
    if (!X || !B) return fail("tensor already freed");
    if (X->ndim < 1) return fail("called `Option::unwrap()` on a `None` value: bias_gelu of a scalar");
    size_t shape[ORC_MAX_DIMS]; int nd = X->ndim;
    memcpy(shape, X->shape, sizeof shape);
    size_t c = shape[nd - 1], total = shape_size(shape, nd);
    if (B->size < c) return fail("index out of bounds: bias shorter than the last extent");
    float *xd = to_host(X), *bd = to_host(B);
    float *out = (float *)calloc(total ? total : 1, sizeof(float));
    for (size_t i = 0; i < total; ++i) {
        float val = xd[i] + bd[i % c];
        float inner = 0.7978845608f * (val + 0.044715f * val * val * val);
        out[i] = 0.5f * val * (1.0f + tanhf(inner));
    }
    free(xd); free(bd);
    size_t out_id = from_vec(out, shape, nd);
    tape_record(&g_tape, OP_BIASGELU, out_id, 2, x, bias);
    return (uint32_t)out_id;
}

/* ops/fused.rs:316-351 bias_gelu_backward: g = grad * gelu'(x + bias);
 * dx = g, dbias[j] += g in flat index order (i.e. down each column).
 * pinned by: float64 derivative, dbias = column sums of dx, finite differences. */
static int bias_gelu_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *X = get(e->saved_ids[0]), *B = get(e->saved_ids[1]), *G = get(grad);
    if (!X || !B || !G) { fail("tensor already freed"); return -1; }
    size_t shape[ORC_MAX_DIMS], bshape[ORC_MAX_DIMS]; int nd = X->ndim, bnd = B->ndim;
    memcpy(shape, X->shape, sizeof shape);
    memcpy(bshape, B->shape, sizeof bshape);
    size_t c = shape[nd - 1], total = shape_size(shape, nd);
    float *xd = to_host(X), *bd = to_host(B), *gd = to_host(G);
    float *dx = (float *)calloc(total ? total : 1, sizeof(float));
    float *db = (float *)calloc(B->size ? B->size : 1, sizeof(float));
    for (size_t i = 0; i < total; ++i) {
        size_t j = i % c;
        float val = xd[i] + bd[j];
        float inner = 0.7978845608f * (val + 0.044715f * val * val * val);
        float th = tanhf(inner);
        float sech2 = 1.0f - th * th;
        float d_inner = 0.7978845608f * (1.0f + 3.0f * 0.044715f * val * val);
        float dgelu = 0.5f * (1.0f + th) + 0.5f * val * sech2 * d_inner;
        float g = gd[i] * dgelu;
        dx[i] = g;
        db[j] += g;
    }
    free(xd); free(bd); free(gd);
    out[0] = (long)from_vec(dx, shape, nd);
    out[1] = (long)from_vec(db, bshape, bnd);
    return 0;
}

/* ---- softmax ------------------------------------------------------------ */

/* ops/norm.rs:10-50 softmax, cpu arm: per (outer, inner) line -- running max,
 * exp(x - max) stored and summed in index order, then divided by the sum.
 * The tape keeps `dim as f32` exactly as passed (possibly negative), :47.
 * pinned by: test/nn.test.ts:46-54 (rows of [1,2,3] sum to 1, positive,
 * ordered), float64 closed form on random lines, shift invariance. */
static uint32_t softmax_impl(size_t a, int dim) {
    orc_tensor *A = get(a);
    if (!A) return fail("tensor already freed");
    int nd = A->ndim;
    size_t shape[ORC_MAX_DIMS];
    memcpy(shape, A->shape, sizeof shape);
    int d = dim < 0 ? nd + dim : dim; /* :13 */
    if (d < 0 || d >= nd) return fail("index out of bounds: softmax dim");
    float *x = to_host(A);
    size_t total = shape_size(shape, nd), dim_size = shape[d];
    size_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= shape[i];
    if (outer < 1) outer = 1;
    if (inner < 1) inner = 1;
    float *out = (float *)calloc(total ? total : 1, sizeof(float));
    for (size_t o = 0; o < outer; ++o)
        for (size_t i = 0; i < inner; ++i) {
            float mx = -INFINITY;
            for (size_t t = 0; t < dim_size; ++t) {
                float v = x[o * dim_size * inner + t * inner + i];
                mx = v > mx ? v : mx;
            }
            float sum = 0.0f;
            for (size_t t = 0; t < dim_size; ++t) {
                size_t idx = o * dim_size * inner + t * inner + i;
                float e = expf(x[idx] - mx);
                out[idx] = e;
                sum += e;
            }
            for (size_t t = 0; t < dim_size; ++t) out[o * dim_size * inner + t * inner + i] /= sum;
        }
    free(x);
    size_t out_id = from_vec(out, shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_SOFTMAX, out_id, 1, a, 0);
    e->saved_scalar = (float)dim; /* ScalarAndTensor(dim as f32, out_id) */
    e->saved_ids[0] = out_id;
    return (uint32_t)out_id;
}

/* ops/norm.rs:96-123 softmax_backward: dx = sm * (g - sum(g * sm)) along the
 * saved dim.  The dim comes back as `*dim_f as usize`: Rust's float-to-integer
 * cast saturates, so a NEGATIVE saved dim (softmax(x, -1), the TypeScript
 * default, src/nn.ts:77) becomes 0 and the reduction runs along dim 0 --
 * reproduced here as the reference behaves, not as it presumably intends.
 * pinned by: float64 Jacobian-vector product for dim >= 0; for dim = -1 on a
 * 2-D input the result must equal the dim-0 formula (tests/test_oracle_attention.py). */
static int softmax_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *S = get(e->saved_ids[0]), *G = get(grad);
    if (!S || !G) { fail("tensor already freed"); return -1; }
    int nd = S->ndim;
    size_t shape[ORC_MAX_DIMS];
    memcpy(shape, S->shape, sizeof shape);
    size_t d = e->saved_scalar > 0.0f ? (size_t)e->saved_scalar : 0; /* saturating cast */
    if ((int)d >= nd) { fail("index out of bounds: softmax dim"); return -1; }
    float *sm = to_host(S), *g = to_host(G);
    size_t total = shape_size(shape, nd), dim_size = shape[d];
    size_t outer = 1, inner = 1;
    for (size_t i = 0; i < d; ++i) outer *= shape[i];
    for (int i = (int)d + 1; i < nd; ++i) inner *= shape[i];
    if (outer < 1) outer = 1;
    if (inner < 1) inner = 1;
    float *o_ = (float *)calloc(total ? total : 1, sizeof(float));
    for (size_t o = 0; o < outer; ++o)
        for (size_t i = 0; i < inner; ++i) {
            float dot = 0.0f;
            for (size_t t = 0; t < dim_size; ++t) {
                size_t idx = o * dim_size * inner + t * inner + i;
                dot += g[idx] * sm[idx];
            }
            for (size_t t = 0; t < dim_size; ++t) {
                size_t idx = o * dim_size * inner + t * inner + i;
                o_[idx] = sm[idx] * (g[idx] - dot);
            }
        }
    free(sm); free(g);
    out[0] = (long)from_vec(o_, shape, nd);
    return 0;
}

/* ---- attention ---------------------------------------------------------- */

/* ops/attention.rs:14-78 flash_attention, cpu arm.  q, k, v are read as
 * [bh, s, d] from their first three dims (:21-24); per (b, row) an online
 * softmax over col < col_end (row + 1 when causal): running max, running sum
 * and accumulator rescaled by exp(old_max - new_max) (:41-53), then
 * out = acc / sum and lse = max + ln(sum) (:56-60).
 * pinned by: float64 softmax(q k^T scale) v with and without the causal mask,
 * v = ones -> out = ones, causal row 0 = v[0], equal scores -> mean of v,
 * lse against float64 log-sum-exp (tests/test_oracle_attention.py). */
static uint32_t flash_attention_impl(size_t q, size_t k, size_t v, float scale, int causal) {
    orc_tensor *Q = get(q), *K = get(k), *V = get(v);
    if (!Q || !K || !V) return fail("tensor already freed");
    if (Q->ndim < 3) return fail("index out of bounds: flash_attention needs [bh, s, d]");
    size_t bh = Q->shape[0], s = Q->shape[1], d = Q->shape[2];
    if (K->size < bh * s * d || V->size < bh * s * d) return fail("index out of bounds: flash_attention k/v shorter than q");
    float *qd = to_host(Q), *kd = to_host(K), *vd = to_host(V);
    float *out = (float *)calloc((bh * s * d) > 0 ? bh * s * d : 1, sizeof(float));
    float *lse = (float *)calloc((bh * s) > 0 ? bh * s : 1, sizeof(float));
    float *acc = (float *)malloc((d ? d : 1) * sizeof(float));
    for (size_t b = 0; b < bh; ++b)
        for (size_t row = 0; row < s; ++row) {
            size_t col_end = causal ? row + 1 : s;
            float running_max = -INFINITY, running_sum = 0.0f;
            for (size_t dd = 0; dd < d; ++dd) acc[dd] = 0.0f;
            for (size_t col = 0; col < col_end; ++col) {
                float dot = 0.0f;
                for (size_t dd = 0; dd < d; ++dd) dot += qd[b * s * d + row * d + dd] * kd[b * s * d + col * d + dd];
                dot *= scale;
                float old_max = running_max;
                running_max = running_max > dot ? running_max : dot; /* f32::max */
                float exp_diff = expf(old_max - running_max);
                running_sum = running_sum * exp_diff + expf(dot - running_max);
                for (size_t dd = 0; dd < d; ++dd)
                    acc[dd] = acc[dd] * exp_diff + expf(dot - running_max) * vd[b * s * d + col * d + dd];
            }
            float inv_sum = 1.0f / running_sum;
            for (size_t dd = 0; dd < d; ++dd) out[b * s * d + row * d + dd] = acc[dd] * inv_sum;
            lse[b * s + row] = running_max + logf(running_sum);
        }
    free(acc); free(qd); free(kd); free(vd);
    size_t oshape[3] = {bh, s, d}, lshape[2] = {bh, s};
    size_t out_id = from_vec(out, oshape, 3);
    size_t lse_id = from_vec(lse, lshape, 2);
    orc_entry *e = tape_record(&g_tape, OP_FLASHATTENTION, out_id, 3, q, k);
    e->input_ids[2] = v; e->saved_ids[2] = v;
    e->fa_out = out_id; e->fa_lse = lse_id; e->saved_scalar = scale; e->fa_causal = causal;
    return (uint32_t)out_id;
}

/* ops/attention.rs:143-202 flash_attention_backward, cpu arm: di = sum(dO * O)
 * per row, p = exp(dot * scale - lse), dv += p dO, dp = dO . v,
 * ds = p (dp - di) scale, dq += ds k, dk += ds q, all accumulated in f32 in
 * (b, row, col) order.
 * pinned by: float64 central finite differences of sum(w * out) in q, k, v
 * (causal and not), sum over rows of dS = 0 identity through dq for k = const. */
static int flash_attention_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *Q = get(e->input_ids[0]), *K = get(e->input_ids[1]), *V = get(e->input_ids[2]);
    orc_tensor *O = get(e->fa_out), *L = get(e->fa_lse), *G = get(grad);
    if (!Q || !K || !V || !O || !L || !G) { fail("tensor already freed"); return -1; }
    size_t bh = Q->shape[0], s = Q->shape[1], d = Q->shape[2];
    float scale = e->saved_scalar;
    float *qd = to_host(Q), *kd = to_host(K), *vd = to_host(V), *od = to_host(O), *ld = to_host(L), *gd = to_host(G);
    size_t total = bh * s * d;
    float *dq = (float *)calloc(total ? total : 1, sizeof(float));
    float *dk = (float *)calloc(total ? total : 1, sizeof(float));
    float *dv = (float *)calloc(total ? total : 1, sizeof(float));
    for (size_t b = 0; b < bh; ++b)
        for (size_t row = 0; row < s; ++row) {
            size_t col_end = e->fa_causal ? row + 1 : s;
            float lse_val = ld[b * s + row];
            float di = 0.0f;
            for (size_t dd = 0; dd < d; ++dd) di += gd[b * s * d + row * d + dd] * od[b * s * d + row * d + dd];
            for (size_t col = 0; col < col_end; ++col) {
                float dot = 0.0f;
                for (size_t dd = 0; dd < d; ++dd) dot += qd[b * s * d + row * d + dd] * kd[b * s * d + col * d + dd];
                dot *= scale;
                float p = expf(dot - lse_val);
                float dp = 0.0f;
                for (size_t dd = 0; dd < d; ++dd) {
                    dp += gd[b * s * d + row * d + dd] * vd[b * s * d + col * d + dd];
                    dv[b * s * d + col * d + dd] += p * gd[b * s * d + row * d + dd];
                }
                float ds = p * (dp - di) * scale;
                for (size_t dd = 0; dd < d; ++dd) {
                    dq[b * s * d + row * d + dd] += ds * kd[b * s * d + col * d + dd];
                    dk[b * s * d + col * d + dd] += ds * qd[b * s * d + row * d + dd];
                }
            }
        }
    free(qd); free(kd); free(vd); free(od); free(ld); free(gd);
    size_t shape[3] = {bh, s, d};
    out[0] = (long)from_vec(dq, shape, 3);
    out[1] = (long)from_vec(dk, shape, 3);
    out[2] = (long)from_vec(dv, shape, 3);
    return 0;
}

/* ---- token-side ops: random numbers, dropout, datasets, embedding, tile, residual layernorm ---- */

/* Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11), the generator the HIP
 * backend draws rand / randn / dropout masks from.  The reference draws from
 * rand 0.8's unseedable thread RNG (tensor.rs:228-250, dropout.rs:37-44), so
 * no stream can match it; what its consumers rely on is the distribution
 * (uniform on multiples of 2^-24 in [0, 1); standard normal).
 * pinned by: the known-answer vectors published with the generator
 * (Random123 kat_vectors), moments of the outputs. */
static void philox4x32_10(uint64_t counter, uint64_t seed, uint32_t out[4]) {
    uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0, c3 = 0;
    uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
/* the general form (4-word counter, 2-word key) for the published vectors */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
void orc_philox_words(uint64_t seed, uint64_t offset, uint32_t *out, size_t n) {
    for (size_t i = 0; i < n; i += 4) {
        uint32_t w[4];
        philox4x32_10(offset + i / 4, seed, w);
        for (size_t j = 0; j < 4 && i + j < n; ++j) out[i + j] = w[j];
    }
}
static float u01(uint32_t w) { return (float)(w >> 8) * 5.9604644775390625e-8f; }
static uint64_t g_rng_seed = 0, g_rng_offset = 0;
void orc_seed(uint64_t seed) { g_rng_seed = seed; g_rng_offset = 0; }
static uint64_t rng_take(size_t n) {
    uint64_t at = g_rng_offset;
    g_rng_offset += (n + 3) / 4;
    return at;
}
/* mode 0: uniform [0, 1) (tensor.rs:228-238); 1: standard normal by Box-Muller (tensor.rs:240-250) */
static uint32_t random_tensor(const size_t *shape, int nd, int mode) {
    size_t n = shape_size(shape, nd);
    float *d = (float *)malloc((n + 4) * sizeof(float));
    uint64_t at = rng_take(n);
    for (size_t i = 0; i < n; i += 4) {
        uint32_t w[4];
        float v[4];
        philox4x32_10(at + i / 4, g_rng_seed, w);
        if (mode == 0) {
            for (int j = 0; j < 4; ++j) v[j] = u01(w[j]);
        } else {
            for (int j = 0; j < 4; j += 2) {
                float u1 = (float)((w[j] >> 8) + 1u) * 5.9604644775390625e-8f, u2 = u01(w[j + 1]);
                float r = sqrtf(-2.0f * logf(u1)), a = 6.283185307179586f * u2;
                v[j] = r * cosf(a);
                v[j + 1] = r * sinf(a);
            }
        }
        for (size_t j = 0; j < 4 && i + j < n; ++j) d[i + j] = v[j];
    }
    return (uint32_t)from_vec(d, shape, nd);
}

/* ops/dropout.rs:25-58 dropout_forward, cpu arm: the input id itself when not
 * training or rate == 0; else mask = (u >= rate), out = x * mask * scale with
 * scale = 1 / (1 - rate), mask kept as a tensor.
 * pinned by: out is 0 or x / (1 - rate) elementwise, kept fraction ~ 1 - rate,
 * backward equals forward applied to the gradient with the same mask. */
static uint32_t dropout_impl(size_t x, float rate, int training) {
    orc_tensor *X = get(x);
    if (!X) return fail("tensor already freed");
    if (!training || rate == 0.0f) return (uint32_t)x;
    float *xd = to_host(X);
    size_t shape[ORC_MAX_DIMS]; int nd = X->ndim;
    memcpy(shape, X->shape, sizeof shape);
    size_t size = X->size;
    float scale = 1.0f / (1.0f - rate);
    float *mask = (float *)malloc((size + 4) * sizeof(float)), *out = (float *)malloc((size + 4) * sizeof(float));
    uint64_t at = rng_take(size);
    for (size_t i = 0; i < size; i += 4) {
        uint32_t w[4];
        philox4x32_10(at + i / 4, g_rng_seed, w);
        for (size_t j = 0; j < 4 && i + j < size; ++j) {
            mask[i + j] = u01(w[j]) >= rate ? 1.0f : 0.0f;
            out[i + j] = xd[i + j] * mask[i + j] * scale;
        }
    }
    free(xd);
    size_t mask_id = from_vec(mask, shape, nd);
    size_t out_id = from_vec(out, shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_DROPOUT, out_id, 1, x, 0);
    e->drop_mask = mask_id; e->saved_scalar = rate;
    return (uint32_t)out_id;
}
/* ops/dropout.rs:114-126 */
static int dropout_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *G = get(grad), *M = get(e->drop_mask);
    if (!G || !M) { fail("tensor already freed"); return -1; }
    float *gd = to_host(G), *md = to_host(M);
    size_t shape[ORC_MAX_DIMS]; int nd = G->ndim;
    memcpy(shape, G->shape, sizeof shape);
    float scale = 1.0f / (1.0f - e->saved_scalar);
    size_t n = G->size;
    float *o = (float *)malloc((n ? n : 1) * sizeof(float));
    for (size_t i = 0; i < n; ++i) o[i] = gd[i] * md[i] * scale;
    free(gd); free(md);
    out[0] = (long)from_vec(o, shape, nd);
    return 0;
}

/* ops/data.rs:13-56 IntBuffer / IntStore (cpu arm: host vectors, LIFO id recycling) */
typedef struct { int live; int32_t *data; size_t len; } orc_intbuf;
static orc_intbuf *g_int;
static size_t g_int_len, g_int_cap, *g_int_free, g_int_nfree, g_int_capfree;
static size_t int_insert(int32_t *data, size_t len) {
    if (g_int_nfree) {
        size_t id = g_int_free[--g_int_nfree];
        g_int[id].live = 1; g_int[id].data = data; g_int[id].len = len;
        return id;
    }
    if (g_int_len == g_int_cap) {
        g_int_cap = g_int_cap ? g_int_cap * 2 : 16;
        g_int = (orc_intbuf *)realloc(g_int, g_int_cap * sizeof(orc_intbuf));
    }
    g_int[g_int_len].live = 1; g_int[g_int_len].data = data; g_int[g_int_len].len = len;
    return g_int_len++;
}
static orc_intbuf *int_get(size_t id) {
    if (id >= g_int_len || !g_int[id].live) { fail("int buffer already freed"); return NULL; }
    return &g_int[id];
}
static void int_clear(void) {
    for (size_t i = 0; i < g_int_len; ++i) if (g_int[i].live) free(g_int[i].data);
    free(g_int); free(g_int_free);
    g_int = NULL; g_int_free = NULL; g_int_len = g_int_cap = g_int_nfree = g_int_capfree = 0;
}
uint32_t orc_create_dataset(const int32_t *data, size_t len) { /* lib.rs:476-479, data.rs:59-66 */
    int32_t *d = (int32_t *)malloc((len ? len : 1) * sizeof(int32_t));
    memcpy(d, data, len * sizeof(int32_t));
    return (uint32_t)int_insert(d, len);
}
void orc_free_int_buffer(uint32_t id) { /* lib.rs:494-497, data.rs:53-56 */
    if (id >= g_int_len) return;
    if (g_int[id].live) free(g_int[id].data);
    g_int[id].live = 0; g_int[id].data = NULL;
    if (g_int_nfree == g_int_capfree) {
        g_int_capfree = g_int_capfree ? g_int_capfree * 2 : 16;
        g_int_free = (size_t *)realloc(g_int_free, g_int_capfree * sizeof(size_t));
    }
    g_int_free[g_int_nfree++] = id;
}
int64_t orc_int_buffer_len(uint32_t id) { orc_intbuf *b = int_get(id); return b ? (int64_t)b->len : -1; }
int orc_int_buffer_to_host(uint32_t id, int32_t *out, size_t cap) {
    orc_intbuf *b = int_get(id);
    if (!b || cap < b->len) return -1;
    memcpy(out, b->data, b->len * sizeof(int32_t));
    return 0;
}
/* ops/data.rs:79-109 sample_batch, cpu arm, with the window starts supplied by
 * the caller in place of rng.gen_range(0..len - block_size - 1): inputs are
 * data[start + t], targets data[start + t + 1].
 * pinned by: windows of an arange dataset; range of valid starts. */
int orc_sample_batch_at(uint32_t dataset, int64_t block, int64_t batch, const int64_t *starts, uint32_t *out_ids) {
    orc_intbuf *ds = int_get(dataset);
    if (!ds) return -1;
    if (block <= 0 || batch <= 0 || (int64_t)ds->len - block - 1 <= 0) { fail("cannot sample empty range"); return -1; }
    size_t total = (size_t)(batch * block);
    int32_t *inp = (int32_t *)malloc(total * sizeof(int32_t)), *tgt = (int32_t *)malloc(total * sizeof(int32_t));
    for (int64_t b = 0; b < batch; ++b) {
        if (starts[b] < 0 || starts[b] >= (int64_t)ds->len - block - 1) { free(inp); free(tgt); fail("start outside the sampled range"); return -1; }
        for (int64_t t = 0; t < block; ++t) {
            inp[b * block + t] = ds->data[starts[b] + t];
            tgt[b * block + t] = ds->data[starts[b] + t + 1];
        }
    }
    out_ids[0] = (uint32_t)int_insert(inp, total);
    out_ids[1] = (uint32_t)int_insert(tgt, total);
    return 0;
}

/* ops/embedding.rs:25-53 embedding_forward, cpu arm
 * pinned by: numpy fancy indexing; backward against np.add.at and, bitwise,
 * a sequential float32 loop in token order. */
static uint32_t embedding_impl(size_t weight, const size_t *indices, size_t batch, size_t seq_len) {
    orc_tensor *W = get(weight);
    if (!W) return fail("tensor already freed");
    if (W->ndim < 2) return fail("index out of bounds: embedding weight needs 2 dims");
    size_t dim = W->shape[1], rows = W->shape[0];
    float *wd = to_host(W);
    float *out = (float *)calloc((batch * seq_len * dim) > 0 ? batch * seq_len * dim : 1, sizeof(float));
    for (size_t b = 0; b < batch; ++b)
        for (size_t t = 0; t < seq_len; ++t) {
            size_t idx = indices[b * seq_len + t];
            if (idx >= rows) { free(wd); free(out); return fail("index out of bounds: embedding index"); }
            memcpy(out + (b * seq_len + t) * dim, wd + idx * dim, dim * sizeof(float));
        }
    free(wd);
    size_t shape[3] = {batch, seq_len, dim};
    size_t out_id = from_vec(out, shape, 3);
    orc_entry *e = tape_record(&g_tape, OP_EMBEDDING, out_id, 1, weight, 0);
    if (g_tape.enabled) {
        size_t n = batch * seq_len;
        e->targets = (size_t *)malloc((n ? n : 1) * sizeof(size_t));
        memcpy(e->targets, indices, n * sizeof(size_t));
    }
    e->emb_batch = batch; e->emb_seq = seq_len;
    return (uint32_t)out_id;
}
/* ops/embedding.rs:104-128 embedding_backward: dw rows accumulate in token order */
static int embedding_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *W = get(e->input_ids[0]), *G = get(grad);
    if (!W || !G) { fail("tensor already freed"); return -1; }
    size_t wshape[ORC_MAX_DIMS]; int wnd = W->ndim;
    memcpy(wshape, W->shape, sizeof wshape);
    size_t vocab = wshape[0], dim = wshape[1];
    float *gd = to_host(G);
    float *dw = (float *)calloc((vocab * dim) > 0 ? vocab * dim : 1, sizeof(float));
    for (size_t b = 0; b < e->emb_batch; ++b)
        for (size_t t = 0; t < e->emb_seq; ++t) {
            size_t idx = e->targets[b * e->emb_seq + t];
            const float *src = gd + (b * e->emb_seq + t) * dim;
            float *dst = dw + idx * dim;
            for (size_t j = 0; j < dim; ++j) dst[j] += src[j];
        }
    free(gd);
    out[0] = (long)from_vec(dw, wshape, wnd);
    return 0;
}

/* ops/pooling.rs:276-309 tile (nothing recorded on the tape)
 * pinned by: numpy.tile. */
static uint32_t tile_impl(size_t input, const size_t *reps, int nreps) {
    orc_tensor *A = get(input);
    if (!A) return fail("tensor already freed");
    int nd = A->ndim;
    if (nreps != nd) return fail("tile: reps must match tensor dimensions");
    if (nd < 1) return fail("attempt to subtract with overflow: tile of a scalar");
    size_t shape[ORC_MAX_DIMS], out_shape[ORC_MAX_DIMS], in_strides[ORC_MAX_DIMS], out_strides[ORC_MAX_DIMS];
    memcpy(shape, A->shape, sizeof shape);
    float *data = to_host(A);
    for (int i = 0; i < nd; ++i) out_shape[i] = shape[i] * reps[i];
    size_t out_size = shape_size(out_shape, nd);
    int empty = 0;
    for (int i = 0; i < nd; ++i) if (out_shape[i] == 0) empty = 1;
    compute_strides(shape, nd, in_strides);
    compute_strides(out_shape, nd, out_strides);
    float *o = (float *)calloc(out_size ? out_size : 1, sizeof(float));
    for (size_t i = 0; i < out_size && !empty; ++i) {
        size_t src = 0, rem = i;
        for (int d = 0; d < nd; ++d) {
            size_t coord = rem / out_strides[d];
            rem %= out_strides[d];
            src += (coord % shape[d]) * in_strides[d];
        }
        o[i] = data[src];
    }
    free(data);
    return (uint32_t)from_vec(o, out_shape, nd);
}

/* ops/fused.rs:23-78 residual_layernorm, cpu arm: res = x + residual, then the
 * layernorm of norm.rs over the last extent; saves [res, gamma, mean, rstd].
 * pinned by: equality with layernorm(add(x, residual)) of this oracle, bit for
 * bit; float64 closed form. */
static uint32_t residual_layernorm_impl(size_t x, size_t residual, size_t gamma, size_t beta, float eps) {
    orc_tensor *X = get(x), *R = get(residual), *Gm = get(gamma), *Bt = get(beta);
    if (!X || !R || !Gm || !Bt) return fail("tensor already freed");
    int nd = X->ndim;
    if (nd < 1) return fail("called `Option::unwrap()` on a `None` value: residual_layernorm of a scalar");
    size_t shape[ORC_MAX_DIMS];
    memcpy(shape, X->shape, sizeof shape);
    size_t c = shape[nd - 1];
    size_t n = c ? shape_size(shape, nd) / c : 0;
    if (R->size < n * c) return fail("index out of bounds: residual shorter than x");
    if (Gm->size < c || Bt->size < c) return fail("index out of bounds: gamma/beta shorter than the last extent");
    float *xd = to_host(X), *rd = to_host(R), *gd = to_host(Gm), *bd = to_host(Bt);
    float *res = (float *)calloc((n * c) > 0 ? n * c : 1, sizeof(float));
    float *out = (float *)calloc((n * c) > 0 ? n * c : 1, sizeof(float));
    float *mean = (float *)calloc(n ? n : 1, sizeof(float)), *rstd = (float *)calloc(n ? n : 1, sizeof(float));
    for (size_t row = 0; row < n; ++row) {
        size_t off = row * c;
        float sum = 0.0f;
        for (size_t j = 0; j < c; ++j) {
            float val = xd[off + j] + rd[off + j];
            res[off + j] = val;
            sum += val;
        }
        float m = sum / (float)c;
        mean[row] = m;
        float var = 0.0f;
        for (size_t j = 0; j < c; ++j) { float d = res[off + j] - m; var += d * d; }
        float r = 1.0f / sqrtf(var / (float)c + eps);
        rstd[row] = r;
        for (size_t j = 0; j < c; ++j) out[off + j] = (res[off + j] - m) * r * gd[j] + bd[j];
    }
    free(xd); free(rd); free(gd); free(bd);
    size_t res_id = from_vec(res, shape, nd);
    size_t mean_id = from_vec(mean, &n, 1), rstd_id = from_vec(rstd, &n, 1);
    size_t out_id = from_vec(out, shape, nd);
    orc_entry *e = tape_record(&g_tape, OP_RESIDUALLAYERNORM, out_id, 4, x, residual);
    e->input_ids[2] = gamma; e->input_ids[3] = beta;
    e->saved_ids[0] = res_id; e->saved_ids[1] = gamma; e->saved_ids[2] = mean_id; e->saved_ids[3] = rstd_id;
    return (uint32_t)out_id;
}
/* ops/fused.rs:134-186: the layernorm backward on the saved sum; the one dx
 * tensor is returned for x and for the residual. */
static int residual_layernorm_backward(size_t grad, const orc_entry *e, long *out) {
    orc_tensor *S = get(e->saved_ids[0]), *Gm = get(e->saved_ids[1]), *Mn = get(e->saved_ids[2]), *Rs = get(e->saved_ids[3]), *G = get(grad);
    if (!S || !Gm || !Mn || !Rs || !G) { fail("tensor already freed"); return -1; }
    int nd = S->ndim, gnd = Gm->ndim;
    size_t shape[ORC_MAX_DIMS], gshape[ORC_MAX_DIMS];
    memcpy(shape, S->shape, sizeof shape);
    memcpy(gshape, Gm->shape, sizeof gshape);
    size_t c = shape[nd - 1], n = c ? shape_size(shape, nd) / c : 0;
    float *xd = to_host(S), *gm = to_host(Gm), *mn = to_host(Mn), *rs = to_host(Rs), *gd = to_host(G);
    float *dx = (float *)calloc((n * c) > 0 ? n * c : 1, sizeof(float));
    size_t gsz = Gm->size > c ? Gm->size : c;
    float *dgamma = (float *)calloc(gsz ? gsz : 1, sizeof(float));
    float *dbeta = (float *)calloc(gsz ? gsz : 1, sizeof(float));
    for (size_t row = 0; row < n; ++row) {
        size_t off = row * c;
        float m = mn[row], r = rs[row];
        float sum_dg = 0.0f, sum_dgx = 0.0f;
        for (size_t j = 0; j < c; ++j) {
            float xhat = (xd[off + j] - m) * r;
            float dg = gd[off + j] * gm[j];
            sum_dg += dg;
            sum_dgx += dg * xhat;
            dgamma[j] += gd[off + j] * xhat;
            dbeta[j] += gd[off + j];
        }
        for (size_t j = 0; j < c; ++j) {
            float xhat = (xd[off + j] - m) * r;
            float dg = gd[off + j] * gm[j];
            dx[off + j] = r * (dg - sum_dg / (float)c - xhat * sum_dgx / (float)c);
        }
    }
    free(xd); free(gm); free(mn); free(rs); free(gd);
    out[0] = out[1] = (long)from_vec(dx, shape, nd);
    out[2] = (long)from_vec(dgamma, gshape, gnd); /* c sums under gamma's shape, fused.rs:176-185 */
    out[3] = (long)from_vec(dbeta, gshape, gnd);
    return 0;
}

/* ops/mixed_precision.rs:17-32 scale_grads, cpu arm */
int orc_scale_grads(const uint32_t *ids, size_t n, double inv_scale_) {
    float inv_scale = (float)inv_scale_;
    int found = 0;
    for (size_t p = 0; p < n; ++p) {
        orc_tensor *T = get(ids[p]);
        if (!T || T->grad < 0) continue;
        orc_tensor *G = get((size_t)T->grad);
        if (!G) continue;
        for (size_t i = 0; i < G->size; ++i) {
            G->data[i] *= inv_scale;
            if (isinf(G->data[i]) || isnan(G->data[i])) found = 1;
        }
    }
    return found;
}

/* ---- backward ----------------------------------------------------------- */

/* autograd.rs:180-222 dispatch_backward */
static int dispatch_backward(const orc_entry *e, size_t grad, long *out) {
    out[0] = out[1] = out[2] = out[3] = -1;
    switch (e->op) {
    case OP_ADD: return addsub_backward(grad, e, out, 0);
    case OP_SUB: return addsub_backward(grad, e, out, 1);
    case OP_MUL: return mul_backward(grad, e, out);
    case OP_NEG: case OP_MULSCALAR: case OP_RELU: case OP_GELU: return unary_backward(grad, e, out);
    case OP_MATMUL: return matmul_backward(grad, e, out);
    case OP_SUM: return reduce_backward(grad, e, out, 0);
    case OP_MEAN: return reduce_backward(grad, e, out, 1);
    case OP_VIEW: return view_backward(grad, e, out);
    case OP_PERMUTE: return permute_backward(grad, e, out);
    case OP_CONTIGUOUS: out[0] = (long)grad; return 0; /* layout.rs:229-231 */
    case OP_CROSSENTROPY: return cross_entropy_backward(grad, e, out);
    case OP_EXP: case OP_LOG: case OP_SIGMOID: case OP_POW: return unary2_backward(grad, e, out);
    case OP_DIV: return div_backward(grad, e, out);
    case OP_MAX: return max_backward(grad, e, out);
    case OP_LAYERNORM: return layernorm_backward(grad, e, out);
    case OP_BIASGELU: return bias_gelu_backward(grad, e, out);        /* autograd.rs BiasGelu */
    case OP_SOFTMAX: return softmax_backward(grad, e, out);           /* autograd.rs:204 */
    case OP_FLASHATTENTION: return flash_attention_backward(grad, e, out); /* autograd.rs:210 */
    case OP_EMBEDDING: return embedding_backward(grad, e, out);
    case OP_DROPOUT: return dropout_backward(grad, e, out);
    case OP_RESIDUALLAYERNORM: return residual_layernorm_backward(grad, e, out);
    }
    return -1;
}

typedef struct {
    const orc_entry *entries;
    const long *out2entry;
    const unsigned char *relevant;
    unsigned char *visited;
    size_t *order;
    size_t norder;
    size_t nslots;
} dfs_ctx;

/* autograd.rs:120-137 recursive post-order DFS */
static void dfs(dfs_ctx *c, size_t tid) {
    if (tid >= c->nslots || c->visited[tid]) return;
    c->visited[tid] = 1;
    long idx = c->out2entry[tid];
    if (idx >= 0) {
        const orc_entry *e = &c->entries[idx];
        for (int i = 0; i < e->n_inputs; ++i)
            if (e->input_ids[i] < c->nslots && c->relevant[e->input_ids[i]]) dfs(c, e->input_ids[i]);
    }
    c->order[c->norder++] = tid;
}

/* autograd.rs:96-171 Tape::backward.
 * pinned by: gradient values of test/autograd.test.ts:19-46 in closed form,
 * the shared-input case diff.mul(diff) -> 2*diff*g, end-to-end regression of
 * test/module.test.ts:113-130 converging. */
static int tape_backward(orc_tape *tp, size_t loss_id) {
    if (!get(loss_id)) { fail("tensor already freed"); return -1; }
    size_t nslots = g_store.len + 1;
    long *out2entry = (long *)malloc(nslots * sizeof(long));
    for (size_t i = 0; i < nslots; ++i) out2entry[i] = -1;
    for (size_t i = 0; i < tp->len; ++i)
        if (tp->e[i].output_id < nslots) out2entry[tp->e[i].output_id] = (long)i; /* later entry wins */

    unsigned char *relevant = (unsigned char *)calloc(nslots, 1);
    unsigned char *visited = (unsigned char *)calloc(nslots, 1);
    size_t *stack = (size_t *)malloc((2 * tp->len + 2) * sizeof(size_t));
    size_t sp = 0;
    stack[sp++] = loss_id;
    while (sp) {
        size_t tid = stack[--sp];
        if (tid >= nslots || relevant[tid]) continue;
        relevant[tid] = 1;
        long idx = out2entry[tid];
        if (idx >= 0)
            for (int i = 0; i < tp->e[idx].n_inputs; ++i) stack[sp++] = tp->e[idx].input_ids[i];
    }
    free(stack);

    dfs_ctx c = {tp->e, out2entry, relevant, visited, (size_t *)malloc(nslots * sizeof(size_t)), 0, nslots};
    dfs(&c, loss_id);

    /* grads: tensor id -> grad id.  Backward creates tensors, so ids beyond
     * nslots can appear as grad ids but never as keys. */
    long *grads = (long *)malloc(nslots * sizeof(long));
    for (size_t i = 0; i < nslots; ++i) grads[i] = -1;
    {
        orc_tensor *L = get(loss_id);
        size_t shape[ORC_MAX_DIMS]; int nd = L->ndim;
        memcpy(shape, L->shape, sizeof shape);
        grads[loss_id] = (long)ones(shape, nd); /* ones_like for any shape, :143 */
    }
    int rc = 0;
    for (size_t oi = c.norder; oi-- > 0 && rc == 0;) { /* reversed post-order */
        size_t tid = c.order[oi];
        if (grads[tid] < 0) continue;
        long idx = out2entry[tid];
        if (idx < 0) continue;
        orc_entry e = tp->e[idx];
        long ig[4];
        if (dispatch_backward(&e, (size_t)grads[tid], ig) != 0) { rc = -1; break; }
        for (int i = 0; i < e.n_inputs; ++i) {
            if (ig[i] < 0) continue;
            size_t inp = e.input_ids[i];
            orc_tensor *T = get(inp);
            if (!T) { fail("tensor already freed"); rc = -1; break; }
            if (T->requires_grad) accumulate_grad(inp, (size_t)ig[i]);
            if (inp < nslots && grads[inp] >= 0) add_inplace((size_t)grads[inp], (size_t)ig[i]);
            else if (inp < nslots) grads[inp] = ig[i];
        }
    }
    free(out2entry); free(relevant); free(visited); free(c.order); free(grads);
    return rc;
}

/* ---- optimiser ---------------------------------------------------------- */

/* ops/optimizer.rs:126-138 grad_norm: f64 accumulation, f32 sqrt */
static float grad_norm_impl(const uint32_t *ids, size_t n) {
    double sq = 0.0;
    for (size_t p = 0; p < n; ++p) {
        orc_tensor *T = get(ids[p]);
        if (!T || T->grad < 0) continue;
        orc_tensor *G = get((size_t)T->grad);
        for (size_t i = 0; i < G->size; ++i) sq += (double)G->data[i] * (double)G->data[i];
    }
    return sqrtf((float)sq);
}

/* f32::powi: repeated multiplication (llvm.powi); exponentiation by squaring
 * as compiler-rt's __powisf2 does. */
static float powi_f32(float a, int b) {
    int recip = b < 0;
    float r = 1.0f;
    while (1) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0f / r : r;
}

/* ops/optimizer.rs:21-65 adamw_step, cpu arm
 * pinned by: one-step closed form (first Adam step moves by lr*sign(g) up to
 * eps), regression convergence. */
static void adamw_step_impl(const uint32_t *ids, size_t n, float lr, float b1, float b2,
                            float eps, float wd, uint32_t step) {
    float bc1 = 1.0f - powi_f32(b1, (int)step);
    float bc2 = 1.0f - powi_f32(b2, (int)step);
    for (size_t p = 0; p < n; ++p) {
        orc_tensor *T = get(ids[p]);
        if (!T || T->grad < 0) continue;
        size_t size = T->size;
        float *gd = to_host(get((size_t)T->grad));
        if (!T->adam_m) {
            T->adam_m = (float *)calloc(size, sizeof(float));
            T->adam_v = (float *)calloc(size, sizeof(float));
        }
        float *m = T->adam_m, *v = T->adam_v, *data = T->data;
        for (size_t i = 0; i < size; ++i) {
            float g = gd[i];
            if (wd > 0.0f) data[i] *= 1.0f - lr * wd;
            m[i] = b1 * m[i] + (1.0f - b1) * g;
            v[i] = b2 * v[i] + (1.0f - b2) * g * g;
            float m_hat = m[i] / bc1;
            float v_hat = v[i] / bc2;
            data[i] -= lr * m_hat / (sqrtf(v_hat) + eps);
        }
        free(gd);
    }
}

/* ========================================================================= *
 * Exported surface: one function per N-API export of src/native/src/lib.rs
 * that the path's callers use (names follow lib.rs, prefixed orc_).
 * ========================================================================= */

static int conv_shape(const int64_t *shape, int nd, size_t *out) {
    if (nd < 0 || nd > ORC_MAX_DIMS) { fail("too many dims"); return -1; }
    for (int i = 0; i < nd; ++i) out[i] = (size_t)shape[i];
    return 0;
}

/* ---- KV cache --------------------------------------------------------------
 * ops/kv_cache.rs, cpu arm (:20-334, quantisation helpers :336-383): per cache
 * fp32 or int8 (+ per-row f32 scale) storage [bh, max_seq, d]; append writes
 * position `len`; decode_step appends k, v and runs the online-softmax attention
 * of q over positions 0..len (:259-287).
 * pinned by: float64 softmax attention over the appended history, the
 * quantisation bound |x - q * scale| <= scale / 2 and its exact arithmetic on
 * hand-picked rows, the error cases of test/native.test.ts:112-151. */
typedef struct {
    int live, quantized;
    size_t batch, heads, d, max_seq, len;
    float *k32, *v32, *kscale, *vscale;
    signed char *k8, *v8;
} orc_kv;
static orc_kv *g_kv;
static size_t g_kv_cap;
static uint32_t g_kv_next = 1; /* lib.rs:36 */

static orc_kv *kv_get(uint32_t id) {
    if (id == 0 || id >= g_kv_cap || !g_kv[id].live) return NULL;
    return &g_kv[id];
}
static void kv_release(orc_kv *c) {
    free(c->k32); free(c->v32); free(c->kscale); free(c->vscale); free(c->k8); free(c->v8);
    memset(c, 0, sizeof *c);
}
static void kv_clear_storage(orc_kv *c) { /* :73-81 reset */
    size_t cap = c->batch * c->heads * c->max_seq * c->d, sc = c->batch * c->heads * c->max_seq;
    c->len = 0;
    memset(c->k32, 0, cap * sizeof(float)); memset(c->v32, 0, cap * sizeof(float));
    memset(c->k8, 0, cap); memset(c->v8, 0, cap);
    for (size_t i = 0; i < sc; ++i) { c->kscale[i] = 1.0f; c->vscale[i] = 1.0f; }
}
uint32_t orc_kv_cache_create(int64_t batch, int64_t heads, int64_t head_dim, int64_t max_seq, int quantized) { /* lib.rs:586-607 */
    uint32_t id = g_kv_next++;
    if (id >= g_kv_cap) {
        size_t ncap = g_kv_cap ? g_kv_cap * 2 : 16;
        while (ncap <= id) ncap *= 2;
        g_kv = (orc_kv *)realloc(g_kv, ncap * sizeof(orc_kv));
        memset(g_kv + g_kv_cap, 0, (ncap - g_kv_cap) * sizeof(orc_kv));
        g_kv_cap = ncap;
    }
    orc_kv *c = &g_kv[id];
    c->live = 1; c->quantized = quantized != 0;
    c->batch = (size_t)batch; c->heads = (size_t)heads; c->d = (size_t)head_dim; c->max_seq = (size_t)max_seq;
    size_t cap = c->batch * c->heads * c->max_seq * c->d, sc = c->batch * c->heads * c->max_seq;
    c->k32 = (float *)malloc((cap ? cap : 1) * sizeof(float)); c->v32 = (float *)malloc((cap ? cap : 1) * sizeof(float));
    c->k8 = (signed char *)malloc(cap ? cap : 1); c->v8 = (signed char *)malloc(cap ? cap : 1);
    c->kscale = (float *)malloc((sc ? sc : 1) * sizeof(float)); c->vscale = (float *)malloc((sc ? sc : 1) * sizeof(float));
    kv_clear_storage(c);
    return id;
}
int64_t orc_kv_cache_len(uint32_t id) { orc_kv *c = kv_get(id); return c ? (int64_t)c->len : 0; }       /* lib.rs:609-616 */
int orc_kv_cache_quantized(uint32_t id) { orc_kv *c = kv_get(id); return c ? c->quantized : 0; }        /* lib.rs:618-625 */
void orc_kv_cache_reset(uint32_t id) { orc_kv *c = kv_get(id); if (c) kv_clear_storage(c); }             /* lib.rs:627-633 */
void orc_kv_cache_free(uint32_t id) { orc_kv *c = kv_get(id); if (c) kv_release(c); }                    /* lib.rs:635-639 */

/* :336-349 parse_bhsd */
static int kv_parse_bhsd(const orc_tensor *t, size_t *b, size_t *h, size_t *s_, size_t *d, char *err, size_t cap) {
    if (t->ndim == 4) { *b = t->shape[0]; *h = t->shape[1]; *s_ = t->shape[2]; *d = t->shape[3]; return 0; }
    if (t->ndim == 3) { *b = 1; *h = t->shape[0]; *s_ = t->shape[1]; *d = t->shape[2]; return 0; }
    size_t n = (size_t)snprintf(err, cap, "expected [B,H,S,D] or [BH,S,D], got shape [");
    for (int i = 0; i < t->ndim && n < cap; ++i) n += (size_t)snprintf(err + n, cap - n, i ? ", %zu" : "%zu", t->shape[i]);
    if (n < cap) snprintf(err + n, cap - n, "]");
    return -1;
}
/* :83-111 validate_single_step_shape */
static int kv_validate(const orc_kv *c, const orc_tensor *t, const char *op, char *err, size_t cap) {
    size_t b, h, s_, d;
    if (kv_parse_bhsd(t, &b, &h, &s_, &d, err, cap) != 0) return -1;
    if (s_ != 1) { snprintf(err, cap, "kv cache %s expects seq_len=1, got %zu", op, s_); return -1; }
    if (b != c->batch || h != c->heads || d != c->d) {
        snprintf(err, cap, "kv cache %s shape mismatch: expected [B=%zu, H=%zu, S=1, D=%zu], got [B=%zu, H=%zu, S=1, D=%zu]",
                 op, c->batch, c->heads, c->d, b, h, d);
        return -1;
    }
    return 0;
}
/* :357-370 quantize_row_i8: scale = max(max|x| / 127, 1e-8); q = clamp(round(x * (1 / scale)), -127, 127) */
static float kv_quantize_row(const float *in, size_t d, signed char *out) {
    float max_abs = 0.0f;
    for (size_t i = 0; i < d; ++i) { float a = fabsf(in[i]); max_abs = a > max_abs ? a : max_abs; }
    float scale = max_abs / 127.0f;
    if (!(scale > 1e-8f)) scale = 1e-8f;
    float inv = 1.0f / scale;
    for (size_t i = 0; i < d; ++i) {
        float q = roundf(in[i] * inv); /* f32::round: half away from zero */
        q = q < -127.0f ? -127.0f : q > 127.0f ? 127.0f : q;
        out[i] = (signed char)q;
    }
    return scale;
}
/* :113-171 append_inner */
static int kv_append_inner(orc_kv *c, const orc_tensor *K, const orc_tensor *V, char *err, size_t cap) {
    if (c->len >= c->max_seq) { snprintf(err, cap, "kv cache is full (len=%zu, max_seq_len=%zu)", c->len, c->max_seq); return -1; }
    size_t bh = c->batch * c->heads, d = c->d, pos = c->len;
    if (K->size != bh * d || V->size != bh * d) { snprintf(err, cap, "expected %zu elements for single-step tensor, got %zu", bh * d, K->size != bh * d ? K->size : V->size); return -1; }
    float *kd = to_host(K), *vd = to_host(V);
    for (size_t row = 0; row < bh; ++row) {
        size_t src = row * d, dst = (row * c->max_seq + pos) * d;
        if (c->quantized) {
            c->kscale[row * c->max_seq + pos] = kv_quantize_row(kd + src, d, c->k8 + dst);
            c->vscale[row * c->max_seq + pos] = kv_quantize_row(vd + src, d, c->v8 + dst);
        } else {
            memcpy(c->k32 + dst, kd + src, d * sizeof(float));
            memcpy(c->v32 + dst, vd + src, d * sizeof(float));
        }
    }
    free(kd); free(vd);
    c->len += 1;
    return 0;
}
static int same_dims(const orc_tensor *a, const orc_tensor *b) { return same_shape(a->shape, a->ndim, b->shape, b->ndim); }

int orc_kv_cache_append(uint32_t id, uint32_t k, uint32_t v) { /* lib.rs:661-676, kv_cache.rs:173-181 */
    orc_kv *c = kv_get(id);
    if (!c) { snprintf(g_err, sizeof g_err, "invalid kv cache id: %u", id); return -1; }
    orc_tensor *K = get(k), *V = get(v);
    if (!K || !V) { fail("tensor already freed"); return -1; }
    char why[400];
    int rc = 0;
    if (!same_dims(K, V)) { snprintf(why, sizeof why, "k/v shapes must match for kv cache append"); rc = -1; }
    if (rc == 0) rc = kv_validate(c, K, "append", why, sizeof why);
    if (rc == 0) rc = kv_append_inner(c, K, V, why, sizeof why);
    if (rc != 0) snprintf(g_err, sizeof g_err, "kv cache append failed: %s", why);
    return rc;
}
uint32_t orc_kv_cache_decode_step(uint32_t id, uint32_t q, uint32_t k, uint32_t v, double scale_) { /* lib.rs:641-659, kv_cache.rs:183-306 */
    orc_kv *c = kv_get(id);
    if (!c) { snprintf(g_err, sizeof g_err, "invalid kv cache id: %u", id); return ORC_BAD; }
    orc_tensor *Q = get(q), *K = get(k), *V = get(v);
    if (!Q || !K || !V) return fail("tensor already freed");
    char why[400];
    int rc = 0;
    if (!same_dims(Q, K) || !same_dims(Q, V)) { snprintf(why, sizeof why, "q/k/v shapes must match for kv cache decode"); rc = -1; }
    if (rc == 0) rc = kv_validate(c, Q, "decode", why, sizeof why);
    if (rc == 0) rc = kv_append_inner(c, K, V, why, sizeof why);
    if (rc != 0) { snprintf(g_err, sizeof g_err, "kv cache decode failed: %s", why); return ORC_BAD; }
    float scale = (float)scale_;
    size_t bh = c->batch * c->heads, d = c->d, cur = c->len;
    int q_nd = Q->ndim;
    float *qd = to_host(Q);
    float *out = (float *)calloc((bh * d) > 0 ? bh * d : 1, sizeof(float));
    float *acc = (float *)malloc((d ? d : 1) * sizeof(float));
    for (size_t row = 0; row < bh; ++row) {
        float running_max = -INFINITY, running_sum = 0.0f;
        for (size_t dd = 0; dd < d; ++dd) acc[dd] = 0.0f;
        for (size_t col = 0; col < cur; ++col) {
            size_t off = (row * c->max_seq + col) * d;
            float ks = c->kscale[row * c->max_seq + col], vs = c->vscale[row * c->max_seq + col];
            float dot = 0.0f;
            for (size_t dd = 0; dd < d; ++dd) {
                float kv = c->quantized ? (float)c->k8[off + dd] * ks : c->k32[off + dd]; /* :372-383 dequantize */
                dot += qd[row * d + dd] * kv;
            }
            dot *= scale;
            float old_max = running_max;
            running_max = running_max > dot ? running_max : dot;
            float exp_diff = expf(old_max - running_max);
            float w = expf(dot - running_max);
            running_sum = running_sum * exp_diff + w;
            for (size_t dd = 0; dd < d; ++dd) {
                float vv = c->quantized ? (float)c->v8[off + dd] * vs : c->v32[off + dd];
                acc[dd] = acc[dd] * exp_diff + w * vv;
            }
        }
        float inv_sum = running_sum > 0.0f ? 1.0f / running_sum : 0.0f;
        for (size_t dd = 0; dd < d; ++dd) out[row * d + dd] = acc[dd] * inv_sum;
    }
    free(acc); free(qd);
    size_t s4[4] = {c->batch, c->heads, 1, d}, s3[3] = {bh, 1, d};
    return (uint32_t)(q_nd == 4 ? from_vec(out, s4, 4) : from_vec(out, s3, 3));
}

/* ---- public surface ------------------------------------------------------ */
uint32_t orc_zeros(const int64_t *shape, int nd) { /* lib.rs:45-50 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s)) return ORC_BAD;
    return (uint32_t)zeros(s, nd);
}
uint32_t orc_ones(const int64_t *shape, int nd) { /* lib.rs:52-57 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s)) return ORC_BAD;
    return (uint32_t)ones(s, nd);
}
/* lib.rs:73-78 from_float32 -> tensor.rs:252-261 from_slice */
uint32_t orc_from_float32(const float *data, size_t len, const int64_t *shape, int nd) {
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s)) return ORC_BAD;
    size_t n = shape_size(s, nd);
    if (len < n) return fail("range end index out of range for slice");
    float *d = (float *)malloc(n * sizeof(float));
    memcpy(d, data, n * sizeof(float));
    return (uint32_t)from_vec(d, s, nd);
}
int orc_tensor_shape(uint32_t id, int64_t *out, int cap) { /* lib.rs:80-84 */
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    for (int i = 0; i < t->ndim && i < cap; ++i) out[i] = (int64_t)t->shape[i];
    return t->ndim;
}
int64_t orc_tensor_size(uint32_t id) { /* lib.rs:86-90 */
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    return (int64_t)t->size;
}
int orc_to_float32(uint32_t id, float *out, size_t cap) { /* lib.rs:92-97 */
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    if (cap < t->size) { fail("output buffer too small"); return -1; }
    float *d = to_host(t);
    memcpy(out, d, t->size * sizeof(float));
    free(d);
    return 0;
}
int orc_get_scalar(uint32_t id, double *out) { /* lib.rs:99-103 */
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    *out = (double)t->data[0];
    return 0;
}
void orc_free_tensor(uint32_t id) { store_free(id); } /* lib.rs:105-109 */
int orc_set_requires_grad(uint32_t id, int r) { /* lib.rs:115-119 */
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    t->requires_grad = r;
    return 0;
}
/* lib.rs:121-125 get_grad: 1 and *out when a grad exists, 0 when None */
int orc_get_grad(uint32_t id, uint32_t *out) {
    orc_tensor *t = get(id);
    if (!t) { fail("tensor already freed"); return -1; }
    if (t->grad < 0) return 0;
    *out = (uint32_t)t->grad;
    return 1;
}
/* lib.rs:131-137 backward: the tape is swapped for a fresh enabled one */
int orc_backward(uint32_t loss) {
    orc_tape old = g_tape;
    g_tape.e = NULL; g_tape.len = g_tape.cap = 0; g_tape.enabled = 1;
    int rc = tape_backward(&old, loss);
    tape_clear(&old);
    return rc;
}
int orc_zero_grad(const uint32_t *ids, size_t n) { /* lib.rs:139-146, tensor.rs:197-205 */
    for (size_t p = 0; p < n; ++p) {
        orc_tensor *t = get(ids[p]);
        if (!t) { fail("tensor already freed"); return -1; }
        if (t->grad >= 0) {
            orc_tensor *g = get((size_t)t->grad);
            if (!g) { fail("tensor already freed"); return -1; }
            for (size_t i = 0; i < g->size; ++i) g->data[i] = 0.0f;
        }
    }
    return 0;
}
void orc_no_grad_start(void) { g_tape.enabled = 0; } /* lib.rs:148-152 */
void orc_no_grad_end(void) { g_tape.enabled = 1; }   /* lib.rs:154-158 */

uint32_t orc_add(uint32_t a, uint32_t b) { return binary_op(a, b, 0); } /* lib.rs:164-169 */
uint32_t orc_sub(uint32_t a, uint32_t b) { return binary_op(a, b, 1); } /* lib.rs:178-183 */
uint32_t orc_mul(uint32_t a, uint32_t b) { return binary_op(a, b, 2); } /* lib.rs:171-176 */
uint32_t orc_neg(uint32_t a) { return unary_op(a, 2, 0.0f); }            /* lib.rs:185-190 */
uint32_t orc_mul_scalar(uint32_t a, double s) { return unary_op(a, 3, (float)s); } /* lib.rs:192-197 */
uint32_t orc_matmul(uint32_t a, uint32_t b) { return matmul_impl(a, b, &g_tape); } /* lib.rs:199-204 */
uint32_t orc_gelu(uint32_t a) { return unary_op(a, 1, 0.0f); }           /* lib.rs:206-211 */
uint32_t orc_relu(uint32_t a) { return unary_op(a, 0, 0.0f); }           /* lib.rs:213-218 */
uint32_t orc_sum_op(uint32_t a, int64_t dim) { return sum_impl(a, (int)dim, &g_tape); } /* lib.rs:234-239 */
uint32_t orc_mean_op(uint32_t a, int64_t dim) { return mean_impl(a, (int)dim); }         /* lib.rs:241-246 */
uint32_t orc_sum_all(uint32_t a) { /* lib.rs:255-265 */
    orc_tensor *t = get(a);
    if (!t) return fail("tensor already freed");
    uint32_t cur = a;
    for (int d = t->ndim - 1; d >= 0 && cur != ORC_BAD; --d) cur = sum_impl(cur, d, &g_tape);
    return cur;
}
uint32_t orc_mean_all(uint32_t a) { /* lib.rs:267-277 */
    orc_tensor *t = get(a);
    if (!t) return fail("tensor already freed");
    uint32_t cur = a;
    for (int d = t->ndim - 1; d >= 0 && cur != ORC_BAD; --d) cur = mean_impl(cur, d);
    return cur;
}
uint32_t orc_view(uint32_t a, const int64_t *shape, int nd) { /* lib.rs:279-285 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s)) return ORC_BAD;
    return view_impl(a, s, nd);
}
uint32_t orc_permute(uint32_t a, const int64_t *dims, int nd) { /* lib.rs:287-293 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(dims, nd, s)) return ORC_BAD;
    return permute_impl(a, s, nd);
}
uint32_t orc_contiguous(uint32_t a) { /* lib.rs:295-300 -> layout.rs:218-227 */
    if (!get(a)) return fail("tensor already freed");
    size_t out = ensure_contiguous(a);
    if (out != a) tape_record(&g_tape, OP_CONTIGUOUS, out, 1, a, 0);
    return (uint32_t)out;
}
uint32_t orc_exp_op(uint32_t a) { return unary2_op(a, 0, 0.0f); }   /* lib.rs:220-225 */
uint32_t orc_log_op(uint32_t a) { return unary2_op(a, 1, 0.0f); }   /* lib.rs:227-232 */
uint32_t orc_sigmoid(uint32_t a) { return unary2_op(a, 2, 0.0f); }  /* lib.rs:374-379 */
uint32_t orc_pow_op(uint32_t a, double e) { return unary2_op(a, 3, (float)e); } /* lib.rs:381-386 */
uint32_t orc_div(uint32_t a, uint32_t b) { return div_op(a, b); }   /* lib.rs:339-344 */
uint32_t orc_lt(uint32_t a, uint32_t b) { return compare_op(a, b, 4, 0.0f); }    /* lib.rs:346-351 */
uint32_t orc_eq_op(uint32_t a, uint32_t b) { return compare_op(a, b, 5, 0.0f); } /* lib.rs:353-358 */
uint32_t orc_gt(uint32_t a, uint32_t b) { return compare_op(a, b, 6, 0.0f); }    /* lib.rs:360-365 */
uint32_t orc_is_close(uint32_t a, uint32_t b, double tol) { return compare_op(a, b, 7, (float)tol); } /* lib.rs:367-372 */
uint32_t orc_max_op(uint32_t a, int64_t dim) { return max_impl(a, (int)dim); }   /* lib.rs:248-253 */
uint32_t orc_layernorm_op(uint32_t x, uint32_t gamma, uint32_t beta, double eps) { /* lib.rs:309-315 */
    return layernorm_impl(x, gamma, beta, (float)eps);
}
uint32_t orc_bias_gelu(uint32_t x, uint32_t bias) { return bias_gelu_impl(x, bias); } /* lib.rs:526-531 */
uint32_t orc_softmax_op(uint32_t a, int64_t dim) { return softmax_impl(a, (int)dim); } /* lib.rs:302-307 */
uint32_t orc_flash_attention(uint32_t q, uint32_t k, uint32_t v, double scale, int causal) { /* lib.rs:575-584 */
    return flash_attention_impl(q, k, v, (float)scale, causal);
}
uint32_t orc_cross_entropy_loss(uint32_t logits, const int64_t *targets, size_t n) { /* lib.rs:328-336 */
    return cross_entropy_impl(logits, targets, n);
}
void orc_adamw_step(const uint32_t *ids, size_t n, double lr, double b1, double b2, double eps,
                    double wd, int64_t step) { /* lib.rs:400-412 */
    adamw_step_impl(ids, n, (float)lr, (float)b1, (float)b2, (float)eps, (float)wd, (uint32_t)step);
}
double orc_grad_norm(const uint32_t *ids, size_t n) { return (double)grad_norm_impl(ids, n); } /* lib.rs:414-419 */
/* lib.rs:428-442 -> ops/optimizer.rs:224-245 clip_and_step */
double orc_clip_and_step(const uint32_t *ids, size_t n, double lr, double b1, double b2, double eps,
                         double wd, int64_t step, double max_grad_norm) {
    float norm = grad_norm_impl(ids, n);
    float mg = (float)max_grad_norm;
    if (mg > 0.0f && norm > mg) {
        float scale = mg / norm;
        for (size_t p = 0; p < n; ++p) {
            orc_tensor *T = get(ids[p]);
            if (!T || T->grad < 0) continue;
            orc_tensor *G = get((size_t)T->grad);
            for (size_t i = 0; i < G->size; ++i) G->data[i] *= scale;
        }
    }
    adamw_step_impl(ids, n, (float)lr, (float)b1, (float)b2, (float)eps, (float)wd, (uint32_t)step);
    return (double)norm;
}
uint32_t orc_rand_tensor(const int64_t *shape, int nd) { /* lib.rs:60-64 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s) != 0) return ORC_BAD;
    return random_tensor(s, nd, 0);
}
uint32_t orc_randn_tensor(const int64_t *shape, int nd) { /* lib.rs:67-71 */
    size_t s[ORC_MAX_DIMS];
    if (conv_shape(shape, nd, s) != 0) return ORC_BAD;
    return random_tensor(s, nd, 1);
}
uint32_t orc_dropout_op(uint32_t x, double rate, int training) { return dropout_impl(x, (float)rate, training); } /* lib.rs:388-394 */
uint32_t orc_embedding_forward(uint32_t weight, const int64_t *indices, size_t n, int64_t batch, int64_t seq_len) { /* lib.rs:319-326 */
    if (batch < 0 || seq_len < 0 || (size_t)(batch * seq_len) > n) return fail("index out of bounds: fewer indices than batch * seq_len");
    size_t *idx = (size_t *)malloc((n ? n : 1) * sizeof(size_t));
    for (size_t i = 0; i < n; ++i) idx[i] = (size_t)indices[i];
    uint32_t r = embedding_impl(weight, idx, (size_t)batch, (size_t)seq_len);
    free(idx);
    return r;
}
uint32_t orc_embedding_forward_gpu(uint32_t weight, uint32_t int_buf, int64_t batch, int64_t seq_len) { /* lib.rs:501-511, embedding.rs (GpuIndices arm) */
    orc_intbuf *b = int_get(int_buf);
    if (!b) return ORC_BAD;
    if (batch < 0 || seq_len < 0 || (size_t)(batch * seq_len) > b->len) return fail("index out of bounds: fewer indices than batch * seq_len");
    size_t *idx = (size_t *)malloc((b->len ? b->len : 1) * sizeof(size_t));
    for (size_t i = 0; i < b->len; ++i) idx[i] = (size_t)b->data[i];
    uint32_t r = embedding_impl(weight, idx, (size_t)batch, (size_t)seq_len);
    free(idx);
    return r;
}
uint32_t orc_cross_entropy_loss_gpu(uint32_t logits, uint32_t int_buf) { /* lib.rs:679-691 -> loss.rs:190-229 */
    orc_tensor *L = get(logits);
    orc_intbuf *b = int_get(int_buf);
    if (!L || !b) return ORC_BAD;
    if (L->ndim < 1) return fail("index out of bounds: cross_entropy of a scalar");
    size_t v = L->shape[L->ndim - 1];
    if (v == 0) return fail("attempt to divide by zero");
    size_t flat[2] = {L->size / v, v};
    uint32_t f = view_impl(logits, flat, 2);
    if (f == ORC_BAD) return ORC_BAD;
    int64_t *t = (int64_t *)malloc((b->len ? b->len : 1) * sizeof(int64_t));
    for (size_t i = 0; i < b->len; ++i) t[i] = b->data[i];
    uint32_t r = cross_entropy_impl(f, t, b->len);
    free(t);
    return r;
}
uint32_t orc_residual_layernorm(uint32_t x, uint32_t residual, uint32_t gamma, uint32_t beta, double eps) { /* lib.rs:515-523 */
    return residual_layernorm_impl(x, residual, gamma, beta, (float)eps);
}
uint32_t orc_tile(uint32_t input, const int64_t *reps, int n) { /* lib.rs:568-573 */
    size_t r[ORC_MAX_DIMS];
    if (n < 0 || n > ORC_MAX_DIMS) return fail("tile: reps must match tensor dimensions");
    for (int i = 0; i < n; ++i) { if (reps[i] < 0) return fail("negative repeat count"); r[i] = (size_t)reps[i]; }
    return tile_impl(input, r, n);
}
void orc_reset_engine(void) { /* lib.rs:460-468 */
    int_clear();
    for (size_t i = 0; i < g_kv_cap; ++i) if (g_kv[i].live) kv_release(&g_kv[i]);
    g_kv_next = 1;
    for (size_t i = 0; i < g_store.len; ++i)
        if (g_store.t[i].live) { free(g_store.t[i].data); free(g_store.t[i].adam_m); free(g_store.t[i].adam_v); }
    free(g_store.t); free(g_store.free_ids);
    memset(&g_store, 0, sizeof g_store);
    tape_clear(&g_tape);
}
void orc_gc_tensors(const uint32_t *keep, size_t n) { /* lib.rs:693-706 */
    size_t len = g_store.len;
    unsigned char *k = (unsigned char *)calloc(len + 1, 1);
    for (size_t i = 0; i < n; ++i) if (keep[i] < len) k[keep[i]] = 1;
    for (size_t id = 0; id < len; ++id)
        if (!k[id] && g_store.t[id].live) store_free(id);
    free(k);
    tape_clear(&g_tape);
}

/* Raw kernel-level check: C[M,N] = A[M,K] * B[K,N] with the reference's loop
 * order and rounding, no store/tape/clones.  Used to pin the HIP GEMM on
 * shapes where building tensors through the engine would only add copies.
 * Same loop as ops/matmul.rs:62-69. */
void orc_sgemm_ikj(const float *a, const float *b, float *c, size_t m, size_t n, size_t k) {
    memset(c, 0, m * n * sizeof(float));
    for (size_t i = 0; i < m; ++i)
        for (size_t kk = 0; kk < k; ++kk) {
            float a_val = a[i * k + kk];
            const float *brow = b + kk * n;
            float *crow = c + i * n;
            for (size_t j = 0; j < n; ++j) crow[j] += a_val * brow[j];
        }
}
