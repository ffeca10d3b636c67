// Engine level of libmni_rocm.so: a device-resident counterpart of the
// reference's Engine { store, tape } (src/native/src/lib.rs:19-39) for the
// matmul path and its callers.  Tensors are ids into a slot vector with LIFO
// id recycling (src/native/src/tensor.rs:96-113); buffers live in HBM and are
// reference-counted, so permute() is a zero-copy view and a transposed matmul
// operand is only a pair of swapped strides handed to the GEMM.  In-place
// writers (gradient accumulation, zero_grad, clipping, AdamW) copy a shared
// buffer first, which keeps the reference's value semantics (its permute
// clones the buffer, src/native/src/ops/layout.rs:125).
#include <math.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "common.h"
#include "gemm_internal.h"
#include <functional>

namespace mni {
namespace {

struct Buf {
    float *p = nullptr;
    size_t n = 0;  // floats
    ~Buf() { if (p) dev_free(p); }
};
using BufP = std::shared_ptr<Buf>;

static BufP new_buf(size_t n) {
    void *p = nullptr;
    if (dev_alloc(&p, (n ? n : 1) * sizeof(float)) != MNI_OK) return nullptr;
    BufP b = std::make_shared<Buf>();
    b->p = (float *)p;
    b->n = n;
    return b;
}

using Shape = std::vector<int64_t>;

// src/native/src/tensor.rs:27-37 GpuTensor
struct Tensor {
    bool live = false;
    BufP buf;
    Shape shape, strides;
    int64_t size = 0;
    bool requires_grad = false;
    int64_t grad = -1;
    BufP adam_m, adam_v;
    // A gradient that is known to hold only zeros (fresh, or just cleared):
    // the first accumulation into it shares the incoming buffer instead of
    // adding to zeros, and the zeros themselves are only written
    // (zero_filled) when somebody reads the tensor before that: get() does it.
    // Every in-place writer goes through make_unique().
    bool known_zero = false, zero_filled = false;
};

enum Op {  // subset of src/native/src/autograd.rs:28-62 plus the fused Linear
    OP_ADD, OP_MUL, OP_SUB, OP_NEG, OP_MULSCALAR, OP_MATMUL, OP_GELU, OP_RELU,
    OP_SUM, OP_MEAN, OP_VIEW, OP_PERMUTE, OP_CONTIGUOUS, OP_CROSSENTROPY, OP_LINEAR,
    OP_SOFTMAX, OP_FLASHATTENTION, OP_BIASGELU,
    OP_EXP, OP_LOG, OP_DIV, OP_SIGMOID, OP_POW, OP_MAX, OP_LAYERNORM,
    OP_EMBEDDING, OP_DROPOUT, OP_RESIDUALLAYERNORM, OP_MSEROWS
};

// src/native/src/autograd.rs:65-70 TapeEntry
struct Entry {
    int op;
    uint32_t output_id;
    uint32_t inputs[4];
    int n_inputs;
    Shape saved_shape;   // Shape / TensorAndShape / Permutation original shape
    Shape saved_perm;
    float scalar = 0.f;
    int act = 0;         // OP_LINEAR: epilogue
    uint32_t aux = MNI_BAD_ID;  // cross-entropy softmax / linear pre-activation / softmax output / attention output
    uint32_t aux2 = MNI_BAD_ID; // attention log-sum-exp
    uint32_t aux3 = MNI_BAD_ID; // residual + layernorm: the saved sum x + residual
    std::shared_ptr<void> targets;  // device int32 targets / embedding indices
    BufP ce_grad_for_one;           // cross-entropy of a small batch: d loss / d logits, computed with the loss
    BufP mse_grad_for_ones;         // fused mseLoss: d loss / d prediction for an upstream gradient of ones, computed with the loss
    int64_t ce_n = 0, ce_v = 0;
    uint64_t rng_seed = 0, rng_offset = 0;  // dropout: where its mask starts in the random stream
};

struct Tape {
    std::vector<Entry> entries;
    bool enabled = true;
    void record(Entry &&e) { if (enabled) entries.push_back(std::move(e)); }
};

// ops/kv_cache.rs:20-47 KvCacheConfig + KvCache, storage on the device
struct KvCache {
    int64_t batch = 0, heads = 0, d = 0, max_seq = 0, len = 0;
    bool quantized = false;
    std::shared_ptr<void> keys, vals;      // [bh, max_seq, d] float or int8
    std::shared_ptr<void> kscale, vscale;  // [bh, max_seq] float (quantized only)
};

// ops/data.rs:13-27 IntBuffer, on the device.  lo / hi bound the values it can
// hold (a batch sampled from a dataset inherits the dataset's bounds), so an
// index can be checked against a table without reading the device.
struct IntBuf {
    bool live = false;
    std::shared_ptr<void> data;  // int32
    int64_t len = 0;
    int32_t lo = 0, hi = 0;
};

struct Engine {
    std::vector<Tensor> tensors;
    std::vector<uint32_t> free_ids;
    Tape tape;
    std::map<uint32_t, KvCache> kv_caches;  // lib.rs:23-24
    uint32_t next_kv_cache_id = 1;          // lib.rs:36
    std::vector<IntBuf> int_bufs;           // ops/data.rs:24-27 IntStore
    std::vector<uint32_t> int_free;
    // Random numbers: Philox blocks (seed, offset) on the device, a Mersenne
    // twister for the host-side window starts.  Seeded from the system's
    // entropy like the reference's thread_rng unless mni_seed() fixes it.
    bool rng_ready = false;
    uint64_t rng_seed = 0, rng_offset = 0;
    std::mt19937_64 host_rng;
    // While Tape::backward runs: what a fused Linear needs to see of the walk in order to hand the
    // gradient of its input straight through the GELU of the Linear that produced it.
    const Tape *bw_tape = nullptr;
    const std::vector<int64_t> *bw_out2entry = nullptr;  // tensor id -> tape entry that produced it
    const std::vector<int> *bw_consumers = nullptr;      // tensor id -> tape entries that read it
    const std::vector<int64_t> *bw_grads = nullptr;      // tensor id -> gradient gathered so far
    // output id of a GELU Linear -> the strip sums of its bias gradient ([rows, cols]: the gradient is their column
    // sums), when the gradient that reaches it has already been taken through gelu' by the entry that consumed it.
    // That layer's own backward adds the strips up, in the launch of its two products where that launch takes them.
    struct PendingStrips {
        BufP strips;
        int64_t rows, cols;
    };
    std::map<uint32_t, PendingStrips> preact_strips;
    // One float holding 1.0, shared by every scalar loss as the gradient backward() starts from (writers copy
    // a shared buffer before they touch it, so nobody changes it).
    BufP one;
    // The same for the last loss that was not a scalar (the reference's mseLoss leaves one value per row): a buffer of
    // that many ones, refilled only when the size changes.
    BufP ones;
    int64_t ones_n = 0;
};
static Engine &eng() {
    // Never destroyed: releasing device buffers from a static destructor would
    // run after the HIP runtime may already have shut down.
    static Engine *e = new Engine;
    return *e;
}

// ---- shape helpers -----------------------------------------------------------
static Shape compute_strides(const Shape &shape) {  // tensor.rs:7-17
    Shape s(shape.size(), 0);
    if (shape.empty()) return s;
    s.back() = 1;
    for (int i = (int)shape.size() - 2; i >= 0; --i) s[i] = s[i + 1] * shape[i + 1];
    return s;
}
static int64_t shape_size(const Shape &shape) {  // tensor.rs:19-21
    int64_t p = 1;
    for (int64_t d : shape) p *= d;
    return p < 1 ? 1 : p;
}
static int64_t shape_size(const int64_t *s, int n) {
    int64_t p = 1;
    for (int i = 0; i < n; ++i) p *= s[i];
    return p < 1 ? 1 : p;
}
static bool is_contiguous(const Tensor &t) {  // tensor.rs:41-53
    int64_t expected = 1;
    for (int i = (int)t.shape.size() - 1; i >= 0; --i) {
        if (t.strides[i] != expected) return false;
        expected *= t.shape[i];
    }
    return true;
}
static bool broadcast_shape(const Shape &a, const Shape &b, Shape *out) {  // utils.rs:3-20
    const size_t n = a.size() > b.size() ? a.size() : b.size();
    out->assign(n, 0);
    for (size_t i = 0; i < n; ++i) {
        const int64_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
        const int64_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
        if (da == db) (*out)[i] = da;
        else if (da == 1) (*out)[i] = db;
        else if (db == 1) (*out)[i] = da;
        else return false;
    }
    return true;
}

// ---- store ----------------------------------------------------------------------
// The slot as it is: a cleared gradient may not have had its zeros written yet.
static Tensor *peek(uint32_t id) {
    Engine &e = eng();
    if (id >= e.tensors.size() || !e.tensors[id].live) {
        set_error(MNI_ERR_FREED, "tensor already freed (id %u)", id);
        return nullptr;
    }
    return &e.tensors[id];
}
static Tensor *get(uint32_t id) {  // tensor.rs:115-117
    Tensor *t = peek(id);
    if (t && t->known_zero && !t->zero_filled) {
        if (k_fill(t->buf->p, 0.0f, (int64_t)t->buf->n) != MNI_OK) return nullptr;
        t->zero_filled = true;
    }
    return t;
}
// Shapes are taken by value: a caller may pass a reference into the slot
// vector, which emplace_back can reallocate.
static uint32_t insert(BufP buf, Shape shape, Shape strides, int64_t size) {  // tensor.rs:104-113
    Engine &e = eng();
    uint32_t id;
    if (!e.free_ids.empty()) {
        id = e.free_ids.back();
        e.free_ids.pop_back();
    } else {
        id = (uint32_t)e.tensors.size();
        e.tensors.emplace_back();
    }
    Tensor &t = e.tensors[id];
    t = Tensor();
    t.live = true;
    t.buf = std::move(buf);
    t.shape = std::move(shape);
    t.strides = std::move(strides);
    t.size = size;
    return id;
}
static uint32_t insert_contig(BufP buf, Shape shape) {
    Shape strides = compute_strides(shape);
    const int64_t size = shape_size(shape);
    return insert(std::move(buf), std::move(shape), std::move(strides), size);
}
static void free_tensor(uint32_t id) {  // tensor.rs:169-174 (cuda arm :351-356)
    Engine &e = eng();
    if (id >= e.tensors.size() || !e.tensors[id].live) return;
    e.tensors[id] = Tensor();
    e.free_ids.push_back(id);
}

// A contiguous device buffer with the tensor's logical contents: its own
// buffer when already contiguous, else a gathered temporary
// (make_contiguous_data, tensor.rs:292-309, on the device).
static BufP contiguous_buf(const Tensor &t) {
    if (is_contiguous(t)) return t.buf;
    BufP out = new_buf((size_t)t.size);
    if (!out) return nullptr;
    if (k_strided_copy(out->p, t.buf->p, t.shape.data(), t.strides.data(), (int)t.shape.size()) != MNI_OK) return nullptr;
    return out;
}
static BufP clone_buf(const BufP &src, size_t n) {
    BufP out = new_buf(n);
    if (!out) return nullptr;
    if (n && mni_rocm_d2d(out->p, src->p, n * sizeof(float)) != MNI_OK) return nullptr;
    return out;
}
// Copy-on-write before an in-place update.
static int make_unique(Tensor &t) {
    t.known_zero = false;
    if (t.buf.use_count() <= 1) return MNI_OK;
    BufP c = clone_buf(t.buf, t.buf->n);
    if (!c) return MNI_ERR_NOMEM;
    t.buf = std::move(c);
    return MNI_OK;
}
static uint32_t zeros(const Shape &shape) {  // tensor.rs:412-420
    const int64_t n = shape_size(shape);
    BufP b = new_buf((size_t)n);
    if (!b || k_fill(b->p, 0.0f, n) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(b), shape);
}
static uint32_t filled(const Shape &shape, float v) {
    const int64_t n = shape_size(shape);
    BufP b = new_buf((size_t)n);
    if (!b || k_fill(b->p, v, n) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(b), shape);
}
static int64_t ensure_grad(uint32_t id) {  // tensor.rs:144-152
    Tensor *t = get(id);
    if (!t) return -1;
    if (t->grad >= 0) return t->grad;
    const Shape shape = t->shape;
    BufP b = new_buf((size_t)shape_size(shape));
    if (!b) return -1;
    const uint32_t g = insert_contig(std::move(b), shape);
    Tensor *G = peek(g);
    G->known_zero = true;  // zeros on demand
    G->zero_filled = false;
    get(id)->grad = g;
    return g;
}
// tensor.rs:475-491 accumulate_grad / :493-508 add_inplace: raw buffer order,
// src.size elements.
static int add_into(uint32_t dst, uint32_t src) {
    Tensor *s = get(src), *d = peek(dst);
    if (!s || !d) return MNI_ERR_FREED;
    if ((int64_t)d->buf->n < s->size) return set_error(MNI_ERR_INVALID, "add_inplace: destination smaller than source");
    if (d->known_zero && d->buf->n == s->buf->n && s->size == (int64_t)s->buf->n) {
        d->buf = s->buf;  // 0 + x = x: share x (a later in-place writer of either tensor copies first)
        d->known_zero = false;
        return MNI_OK;
    }
    if (!get(dst)) return MNI_ERR_HIP;  // writes the pending zeros
    MNI_TRY(make_unique(*d));
    return k_axpy(d->buf->p, s->buf->p, 1.0f, s->size);
}

static bool to_shape(const int64_t *shape, int nd, Shape *out) {
    if (nd < 0 || nd > MNI_MAX_DIMS || (nd > 0 && !shape)) {
        set_error(MNI_ERR_INVALID, "rank %d out of range (max %d)", nd, MNI_MAX_DIMS);
        return false;
    }
    out->assign(shape, shape + nd);
    for (int64_t d : *out)
        if (d < 0) { set_error(MNI_ERR_INVALID, "negative extent"); return false; }
    return true;
}

// ---- matmul ------------------------------------------------------------------------
// Describe the last two dims of `t` as a GEMM operand; leading dims collapse
// to one batch stride when they can, otherwise the tensor is gathered once on
// the device.  `keep` holds whatever buffer the descriptor points into.
static int make_operand(const Tensor &t, bool transpose, mni_operand *op, BufP *keep) {
    const int nd = (int)t.shape.size();
    Shape strides = t.strides;
    *keep = t.buf;
    int64_t bcount = 1;
    for (int i = 0; i < nd - 2; ++i) bcount *= t.shape[i];
    if (bcount < 1) bcount = 1;
    int64_t bstride = 0;
    bool ok = true;
    if (bcount > 1) {
        // innermost non-unit batch dim gives the stride; outer ones must nest
        int64_t expect = -1;
        for (int i = nd - 3; i >= 0; --i) {
            if (t.shape[i] == 1) continue;
            if (expect < 0) { bstride = strides[i]; expect = bstride * t.shape[i]; }
            else { if (strides[i] != expect) ok = false; expect *= t.shape[i]; }
        }
    }
    if (!ok) {
        BufP c = contiguous_buf(t);
        if (!c) return MNI_ERR_NOMEM;
        *keep = c;
        strides = compute_strides(t.shape);
        bstride = t.shape[nd - 2] * t.shape[nd - 1];
    }
    op->ptr = (*keep)->p;
    op->row_stride = strides[nd - 2];
    op->col_stride = strides[nd - 1];
    if (transpose) std::swap(op->row_stride, op->col_stride);
    op->batch_stride = bstride;
    op->batch_count = bcount;
    return MNI_OK;
}

// C = op(A) * op(B) on tensors, batch rule of ops/matmul.rs:54-60.
// ta / tb: use the operand with its last two dims swapped (transpose_last2,
// ops/matmul.rs:258-284, without the copy).
// aux / colsum_part: the second buffer and the strip sums of the MNI_EPI_BIAS_GELU_DUAL / MNI_EPI_DGELU epilogues.
struct PreparedMatmul {
    mni_gemm_desc d;
    BufP out, keep_a, keep_b;  // the result buffer; contiguous copies the operands needed, alive until the launch is issued
    Shape out_shape;
};

// Everything of a product but the launch: checks, broadcast of the batch dims, operand descriptors, result buffer.
static bool prepare_matmul(uint32_t a, bool ta, uint32_t b, bool tb, const float *bias, int epilogue, float *aux, float *colsum_part,
                           PreparedMatmul *pm) {
    Tensor *A = get(a), *B = get(b);
    if (!A || !B) return false;
    const int and_ = (int)A->shape.size(), bnd = (int)B->shape.size();
    if (and_ < 2 || bnd < 2) {
        set_error(MNI_ERR_INVALID, "matmul requires at least 2D tensors");
        return false;
    }
    int64_t m = A->shape[and_ - 2], k = A->shape[and_ - 1];
    if (ta) std::swap(m, k);
    int64_t k2 = B->shape[bnd - 2], n = B->shape[bnd - 1];
    if (tb) std::swap(k2, n);
    if (k != k2) {
        set_error(MNI_ERR_INVALID, "matmul inner dimensions must match: %lld vs %lld", (long long)k, (long long)k2);
        return false;
    }
    const Shape a_batch(A->shape.begin(), A->shape.end() - 2), b_batch(B->shape.begin(), B->shape.end() - 2);
    Shape &out_shape = pm->out_shape;
    if (!broadcast_shape(a_batch, b_batch, &out_shape)) {
        set_error(MNI_ERR_INVALID, "matmul batch shapes are not broadcastable");
        return false;
    }
    if (out_shape.size() + 2 > MNI_MAX_DIMS) {
        set_error(MNI_ERR_INVALID, "matmul result rank exceeds %d", MNI_MAX_DIMS);
        return false;
    }
    const int64_t batch = shape_size(out_shape);
    out_shape.push_back(m);
    out_shape.push_back(n);

    mni_gemm_desc &d = pm->d;
    memset(&d, 0, sizeof d);
    if (make_operand(*A, ta, &d.A, &pm->keep_a) != MNI_OK || make_operand(*B, tb, &d.B, &pm->keep_b) != MNI_OK) return false;
    pm->out = new_buf((size_t)shape_size(out_shape));
    if (!pm->out) return false;
    d.M = m; d.N = n; d.K = k; d.batch = batch;
    d.C = pm->out->p; d.ldc = n; d.c_batch_stride = m * n;
    d.bias = bias; d.epilogue = epilogue;
    d.aux = aux; d.colsum_part = colsum_part;
    return true;
}

static uint32_t matmul_tensors(uint32_t a, bool ta, uint32_t b, bool tb, const float *bias, int epilogue, float *aux = nullptr,
                               float *colsum_part = nullptr) {
    PreparedMatmul pm;
    if (!prepare_matmul(a, ta, b, tb, bias, epilogue, aux, colsum_part, &pm)) return MNI_BAD_ID;
    if (sgemm(pm.d) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(pm.out), pm.out_shape);
}

// Sum `full` (contiguous, full_shape) down to `orig_shape`
// (utils::unbroadcast, src/native/src/utils.rs:39-66).  Returns a tensor id;
// when nothing is reduced the result shares full's buffer.
static uint32_t unbroadcast_tensor(uint32_t full, const Shape &orig_shape) {
    Tensor *F = get(full);
    if (!F) return MNI_BAD_ID;
    if (F->shape == orig_shape) return insert_contig(F->buf, orig_shape);
    const Shape fshape = F->shape;
    BufP src = contiguous_buf(*F);
    if (!src) return MNI_BAD_ID;
    const int64_t on = shape_size(orig_shape);
    BufP out = new_buf((size_t)on);
    if (!out) return MNI_BAD_ID;
    // Leading-dims reduction ([R.., C..] -> [C..], or [1.., C..]) is a column sum.
    size_t lead = 0;
    while (lead < orig_shape.size() && orig_shape[lead] == 1) ++lead;
    const size_t core = orig_shape.size() - lead;
    bool suffix = fshape.size() >= orig_shape.size();
    for (size_t i = 0; suffix && i < core; ++i) suffix = fshape[fshape.size() - core + i] == orig_shape[lead + i];
    int rc;
    if (suffix) {
        rc = k_colsum(out->p, src->p, shape_size(fshape) / on, on);
    } else {
        rc = k_unbroadcast(out->p, src->p, fshape.data(), (int)fshape.size(), orig_shape.data(), (int)orig_shape.size());
    }
    if (rc != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(out), orig_shape);
}

// ops/matmul.rs:199-222 matmul_backward: dA = unbroadcast(dC * B^T),
// dB = unbroadcast(A^T * dC); both always.
// through_gelu (fused Linear only): A is the output of a GELU Linear with pre-activation z and bias; dA then
// leaves the product already multiplied by gelu'(z + bias), with its strip sums in colsum_part.
struct ThroughGelu {
    const float *bias;
    float *z;
    float *colsum_part;
};
// bias_sums (fused Linear only, may be null): column sums of the upstream gradient wanted along with the two products.
static int matmul_backward(uint32_t grad, const Entry &e, int64_t *out, const ThroughGelu *through_gelu = nullptr, PairColsum *bias_sums = nullptr) {
    const uint32_t a = e.inputs[0], b = e.inputs[1];
    Tensor *A = get(a), *B = get(b), *G = get(grad);
    if (!A || !B || !G) return MNI_ERR_FREED;
    const Shape a_shape = A->shape, b_shape = B->shape;

    // The two products are independent of each other, so both are set up first and issued together
    // (mni_rocm_sgemm_pair's rule decides whether that is one launch or two).
    // dA = dC * B^T
    PreparedMatmul pa;
    if (!(through_gelu ? prepare_matmul(grad, false, b, true, through_gelu->bias, MNI_EPI_DGELU, through_gelu->z, through_gelu->colsum_part, &pa)
                       : prepare_matmul(grad, false, b, true, nullptr, MNI_EPI_NONE, nullptr, nullptr, &pa)))
        return MNI_ERR_INVALID;
    // dB = A^T * dC.  When B has no batch of its own and A / dC stack their batch
    // matrices at a uniform row pitch, sum over the batch inside one product
    // by extending K to batch * M (the split-K path then fills the machine).
    PreparedMatmul pb;
    A = get(a); B = get(b); G = get(grad);
    const int and_ = (int)A->shape.size(), gnd = (int)G->shape.size();
    int64_t b_bcount = 1;
    for (size_t i = 0; i + 2 < b_shape.size(); ++i) b_bcount *= b_shape[i];
    int64_t g_batch = 1;
    for (int i = 0; i < gnd - 2; ++i) g_batch *= G->shape[i];
    bool folded = false;
    if (b_bcount == 1 && g_batch > 1 && is_contiguous(*A) && is_contiguous(*G)) {
        int64_t a_batch = 1;
        for (int i = 0; i < and_ - 2; ++i) a_batch *= A->shape[i];
        if (a_batch == g_batch) {
            const int64_t m = A->shape[and_ - 2], k = A->shape[and_ - 1], n = G->shape[gnd - 1];
            mni_gemm_desc &d = pb.d;
            memset(&d, 0, sizeof d);
            pb.out = new_buf((size_t)(k * n));
            if (!pb.out) return MNI_ERR_NOMEM;
            d.M = k; d.N = n; d.K = g_batch * m; d.batch = 1;
            d.A.ptr = A->buf->p; d.A.row_stride = 1; d.A.col_stride = k; d.A.batch_count = 1;
            d.B.ptr = G->buf->p; d.B.row_stride = n; d.B.col_stride = 1; d.B.batch_count = 1;
            d.C = pb.out->p; d.ldc = n; d.c_batch_stride = k * n;
            pb.out_shape = {k, n};
            folded = true;
        }
    }
    if (!folded && !prepare_matmul(a, true, grad, false, nullptr, MNI_EPI_NONE, nullptr, nullptr, &pb)) return MNI_ERR_INVALID;
    MNI_TRY(sgemm_pair(pa.d, pb.d, bias_sums));

    {
        const uint32_t full = insert_contig(std::move(pa.out), pa.out_shape);
        if (full == MNI_BAD_ID) return MNI_ERR_INVALID;
        const uint32_t ga = unbroadcast_tensor(full, a_shape);
        free_tensor(full);
        if (ga == MNI_BAD_ID) return MNI_ERR_INVALID;
        out[0] = ga;
    }
    {
        const uint32_t full = insert_contig(std::move(pb.out), pb.out_shape);
        if (full == MNI_BAD_ID) return MNI_ERR_INVALID;
        if (folded) {
            // b_shape may carry leading ones ([1, K, N]); same element count.
            Tensor *F = get(full);
            F->shape = b_shape;
            F->strides = compute_strides(b_shape);
            out[1] = full;
        } else {
            const uint32_t gb = unbroadcast_tensor(full, b_shape);
            free_tensor(full);
            if (gb == MNI_BAD_ID) return MNI_ERR_INVALID;
            out[1] = gb;
        }
    }
    return MNI_OK;
}

// ---- elementwise ---------------------------------------------------------------------
// ops/elementwise.rs:20-73,237-248,474-485
// div (:918-928) is recorded like add / sub / mul; the comparisons lt / eq / gt / is_close (:1099-1288)
// produce 1.0 / 0.0 and record nothing.
static uint32_t binary_op(uint32_t a, uint32_t b, int op, float tol = 0.f) {
    Tensor *A = get(a), *B = get(b);
    if (!A || !B) return MNI_BAD_ID;
    Shape out_shape;
    if (!broadcast_shape(A->shape, B->shape, &out_shape)) {
        set_error(MNI_ERR_INVALID, "shapes are not broadcastable");
        return MNI_BAD_ID;
    }
    const int64_t n = shape_size(out_shape);
    BufP out = new_buf((size_t)n);
    if (!out) return MNI_BAD_ID;
    int rc;
    const bool a_c = is_contiguous(*A), b_c = is_contiguous(*B);
    if (A->shape == B->shape && a_c && b_c) {
        rc = k_binary_same(out->p, A->buf->p, B->buf->p, n, op, tol);
    } else if (op == BIN_ADD && a_c && b_c && A->shape == out_shape && B->shape.size() == 1 &&
               B->shape[0] == out_shape.back()) {
        rc = k_add_bias(out->p, A->buf->p, B->buf->p, n / out_shape.back(), out_shape.back());
    } else {
        StridedDesc d;
        d.ndim = (int)out_shape.size();
        const int ao = d.ndim - (int)A->shape.size(), bo = d.ndim - (int)B->shape.size();
        for (int i = 0; i < d.ndim; ++i) {
            d.shape[i] = out_shape[i];
            d.a_strides[i] = (i < ao || A->shape[i - ao] == 1) ? 0 : A->strides[i - ao];
            d.b_strides[i] = (i < bo || B->shape[i - bo] == 1) ? 0 : B->strides[i - bo];
        }
        rc = k_binary_broadcast(out->p, A->buf->p, B->buf->p, d, op, tol);
    }
    if (rc != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), out_shape);
    if (op >= BIN_LT) return id;
    Entry e;
    e.op = op == BIN_ADD ? OP_ADD : op == BIN_SUB ? OP_SUB : op == BIN_MUL ? OP_MUL : OP_DIV;
    e.output_id = id; e.n_inputs = 2; e.inputs[0] = a; e.inputs[1] = b;
    e.saved_shape = out_shape;
    eng().tape.record(std::move(e));
    return id;
}

static uint32_t negated(uint32_t g) {
    Tensor *G = get(g);
    BufP src = contiguous_buf(*G);
    BufP out = src ? new_buf((size_t)G->size) : nullptr;
    if (!out || k_unary(out->p, src->p, G->size, UN_NEG, 0.f) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(out), G->shape);
}

// ops/elementwise.rs:199-211 add_backward, :558-571 sub_backward
static int addsub_backward(uint32_t grad, const Entry &e, int64_t *out, bool is_sub) {
    Tensor *A = get(e.inputs[0]), *B = get(e.inputs[1]);
    if (!A || !B || !get(grad)) return MNI_ERR_FREED;
    const Shape a_shape = A->shape, b_shape = B->shape;
    const uint32_t ga = unbroadcast_tensor(grad, a_shape);
    if (ga == MNI_BAD_ID) return MNI_ERR_INVALID;
    out[0] = ga;
    uint32_t gb;
    if (is_sub) {
        const uint32_t ng = negated(grad);
        if (ng == MNI_BAD_ID) return MNI_ERR_INVALID;
        gb = unbroadcast_tensor(ng, b_shape);
        free_tensor(ng);
    } else {
        gb = unbroadcast_tensor(grad, b_shape);
    }
    if (gb == MNI_BAD_ID) return MNI_ERR_INVALID;
    out[1] = gb;
    return MNI_OK;
}

// ops/elementwise.rs:348-390 mul_backward
static int mul_backward(uint32_t grad, const Entry &e, int64_t *out) {
    const uint32_t a = e.inputs[0], b = e.inputs[1];
    Tensor *A = get(a), *B = get(b), *G = get(grad);
    if (!A || !B || !G) return MNI_ERR_FREED;
    const Shape a_shape = A->shape, b_shape = B->shape, g_shape = G->shape;
    const int64_t n = shape_size(g_shape);
    BufP gsrc = contiguous_buf(*G);
    BufP ga_full = new_buf((size_t)n), gb_full = new_buf((size_t)n);
    if (!gsrc || !ga_full || !gb_full) return MNI_ERR_NOMEM;
    if (a_shape == g_shape && b_shape == g_shape && is_contiguous(*A) && is_contiguous(*B)) {
        MNI_TRY(k_mul_backward_same(ga_full->p, gb_full->p, gsrc->p, A->buf->p, B->buf->p, n));
    } else {
        // ga_full = g * b (b broadcast), gb_full = g * a (a broadcast)
        StridedDesc d;
        d.ndim = (int)g_shape.size();
        const Shape gstr = compute_strides(g_shape);
        const int ao = d.ndim - (int)a_shape.size(), bo = d.ndim - (int)b_shape.size();
        for (int i = 0; i < d.ndim; ++i) {
            d.shape[i] = g_shape[i];
            d.a_strides[i] = gstr[i];
            d.b_strides[i] = (i < bo || b_shape[i - bo] == 1) ? 0 : B->strides[i - bo];
        }
        MNI_TRY(k_binary_broadcast(ga_full->p, gsrc->p, B->buf->p, d, BIN_MUL));
        for (int i = 0; i < d.ndim; ++i)
            d.b_strides[i] = (i < ao || a_shape[i - ao] == 1) ? 0 : A->strides[i - ao];
        MNI_TRY(k_binary_broadcast(gb_full->p, gsrc->p, A->buf->p, d, BIN_MUL));
    }
    const uint32_t fa = insert_contig(std::move(ga_full), g_shape);
    const uint32_t fb = insert_contig(std::move(gb_full), g_shape);
    const uint32_t ga = unbroadcast_tensor(fa, a_shape);
    const uint32_t gb = unbroadcast_tensor(fb, b_shape);
    free_tensor(fa);
    free_tensor(fb);
    if (ga == MNI_BAD_ID || gb == MNI_BAD_ID) return MNI_ERR_INVALID;
    out[0] = ga; out[1] = gb;
    return MNI_OK;
}

// ops/activation.rs:34-44,114-124; elementwise neg / mul_scalar
static uint32_t unary_op(uint32_t a, int un, int tape_op, float s) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)A->size) : nullptr;
    if (!out || k_unary(out->p, src->p, A->size, un, s) != MNI_OK) return MNI_BAD_ID;
    const Shape shape = A->shape;
    const uint32_t id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = tape_op; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a; e.scalar = s;
    eng().tape.record(std::move(e));
    return id;
}

// ops/activation.rs:74-84,154-164 and the neg / mul_scalar backward
static int unary_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad);
    if (!G) return MNI_ERR_FREED;
    const Shape shape = G->shape;
    const int64_t n = G->size;
    BufP g = contiguous_buf(*G);
    BufP o = g ? new_buf((size_t)n) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    if (e.op == OP_RELU || e.op == OP_GELU) {
        Tensor *X = get(e.inputs[0]);
        if (!X) return MNI_ERR_FREED;
        BufP x = contiguous_buf(*X);
        if (!x) return MNI_ERR_NOMEM;
        MNI_TRY(k_unary_backward(o->p, g->p, x->p, n, e.op == OP_RELU ? UN_RELU : UN_GELU));
    } else if (e.op == OP_NEG) {
        MNI_TRY(k_unary(o->p, g->p, n, UN_NEG, 0.f));
    } else {
        MNI_TRY(k_unary(o->p, g->p, n, UN_SCALE, e.scalar));
    }
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// ---- reductions ----------------------------------------------------------------------
static int resolve_dim(int64_t dim, int nd) { return (int)(dim < 0 ? nd + dim : dim); }  // reduce.rs:5-7

// ops/reduce.rs:13-46 sum, :169-184 mean.  The reference's mean also leaves an
// unreachable Sum entry and tensor behind; only the Mean entry is recorded.
static uint32_t reduce_op(uint32_t a, int64_t dim, bool mean) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const int nd = (int)A->shape.size();
    const int d = resolve_dim(dim, nd);
    if (d < 0 || d >= nd) {
        set_error(MNI_ERR_INVALID, "reduce dim %lld out of range for rank %d", (long long)dim, nd);
        return MNI_BAD_ID;
    }
    const Shape a_shape = A->shape;
    Shape out_shape = a_shape;
    out_shape[d] = 1;
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= a_shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= a_shape[i];
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)shape_size(out_shape)) : nullptr;
    if (!out) return MNI_BAD_ID;
    if (k_reduce_dim(out->p, src->p, outer, a_shape[d], inner, mean ? (float)a_shape[d] : 1.0f) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), out_shape);
    Entry e;
    e.op = mean ? OP_MEAN : OP_SUM; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a;
    e.saved_shape = a_shape;
    eng().tape.record(std::move(e));
    return id;
}

// ops/reduce.rs:94-118 sum_backward, :232-263 mean_backward
static int reduce_backward(uint32_t grad, const Entry &e, int64_t *out, bool mean) {
    Tensor *G = get(grad);
    if (!G) return MNI_ERR_FREED;
    const Shape &orig = e.saved_shape;
    const Shape gshape = G->shape;
    if (gshape.size() != orig.size()) return set_error(MNI_ERR_INVALID, "reduce backward: rank mismatch");
    float div = 1.0f;
    if (mean)
        for (size_t d = 0; d < orig.size(); ++d)
            if (gshape[d] == 1 && orig[d] > 1) div = (float)orig[d];
    BufP g = contiguous_buf(*G);
    const int64_t on = shape_size(orig);
    BufP o = g ? new_buf((size_t)on) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    // One expanded dim is the common case; otherwise broadcast generically.
    int nexp = 0, ed = -1;
    for (size_t d = 0; d < orig.size(); ++d)
        if (gshape[d] == 1 && orig[d] != 1) { ++nexp; ed = (int)d; }
    if (nexp <= 1) {
        int64_t outer = 1, inner = 1, dimn = 1;
        if (nexp == 1) {
            for (int i = 0; i < ed; ++i) outer *= orig[i];
            for (size_t i = ed + 1; i < orig.size(); ++i) inner *= orig[i];
            dimn = orig[ed];
        } else {
            inner = on;
        }
        MNI_TRY(k_expand_dim(o->p, g->p, outer, dimn, inner, div));
    } else {
        // g broadcast to orig (as a broadcast multiply by one), then divided.
        BufP one = new_buf(1);
        if (!one) return MNI_ERR_NOMEM;
        MNI_TRY(k_fill(one->p, 1.0f, 1));
        StridedDesc d;
        d.ndim = (int)orig.size();
        const Shape gstr = compute_strides(gshape);
        for (int i = 0; i < d.ndim; ++i) {
            d.shape[i] = orig[i];
            d.a_strides[i] = gshape[i] == 1 ? 0 : gstr[i];
            d.b_strides[i] = 0;
        }
        MNI_TRY(k_binary_broadcast(o->p, g->p, one->p, d, BIN_MUL));
        if (div != 1.0f) MNI_TRY(k_expand_dim(o->p, o->p, 1, 1, on, div));
    }
    out[0] = insert_contig(std::move(o), orig);
    return MNI_OK;
}

// ---- layout ------------------------------------------------------------------------------
// ops/layout.rs:66-89 view: a tensor of the same contents under the new shape.
static uint32_t view_op(uint32_t a, const Shape &new_shape) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const Shape orig = A->shape;
    const int64_t n = A->size;
    if (shape_size(new_shape) != n) {
        set_error(MNI_ERR_INVALID, "view: %lld elements cannot be viewed as %lld", (long long)n, (long long)shape_size(new_shape));
        return MNI_BAD_ID;
    }
    // The reference copies (layout.rs:70-77); with reference-counted buffers a
    // contiguous source is shared instead, and any in-place writer copies first.
    BufP out;
    if (is_contiguous(*A) && (int64_t)A->buf->n == n) {
        out = A->buf;
    } else {
        out = new_buf((size_t)n);
        if (!out) return MNI_BAD_ID;
        const int rc = is_contiguous(*A) ? mni_rocm_d2d(out->p, A->buf->p, (size_t)n * sizeof(float))
                                         : k_strided_copy(out->p, A->buf->p, A->shape.data(), A->strides.data(), (int)A->shape.size());
        if (rc != MNI_OK) return MNI_BAD_ID;
    }
    const uint32_t id = insert_contig(std::move(out), new_shape);
    Entry e;
    e.op = OP_VIEW; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a; e.saved_shape = orig;
    eng().tape.record(std::move(e));
    return id;
}
// ops/layout.rs:92-105 view_backward
static int view_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad);
    if (!G) return MNI_ERR_FREED;
    BufP g = contiguous_buf(*G);
    if (!g) return MNI_ERR_NOMEM;
    out[0] = insert_contig(g, e.saved_shape);  // shares the buffer; writers copy first
    return MNI_OK;
}
// ops/layout.rs:112-134 permute: a view (shared buffer, permuted strides)
static uint32_t permute_op(uint32_t a, const Shape &dims) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const int nd = (int)A->shape.size();
    if ((int)dims.size() != nd) {
        set_error(MNI_ERR_INVALID, "permute: %zu dims given for a rank-%d tensor", dims.size(), nd);
        return MNI_BAD_ID;
    }
    Shape ns(nd), nst(nd);
    std::vector<bool> seen(nd, false);
    for (int i = 0; i < nd; ++i) {
        if (dims[i] < 0 || dims[i] >= nd || seen[dims[i]]) {
            set_error(MNI_ERR_INVALID, "permute: dims are not a permutation");
            return MNI_BAD_ID;
        }
        seen[dims[i]] = true;
        ns[i] = A->shape[dims[i]];
        nst[i] = A->strides[dims[i]];
    }
    const Shape a_shape = A->shape;
    const uint32_t id = insert(A->buf, ns, nst, A->size);
    Entry e;
    e.op = OP_PERMUTE; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a;
    e.saved_shape = a_shape; e.saved_perm = dims;
    eng().tape.record(std::move(e));
    return id;
}
// ops/layout.rs:162-195 permute_backward: grad (contiguous, permuted shape)
// scattered back = a gather of grad through the inverse permutation.
static int permute_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad);
    if (!G) return MNI_ERR_FREED;
    const int nd = (int)e.saved_perm.size();
    BufP g = contiguous_buf(*G);
    if (!g) return MNI_ERR_NOMEM;
    const Shape gstr = compute_strides(G->shape);
    // out[coord_orig] = g[coord_perm], coord_perm[i] = coord_orig[perm[i]]
    Shape src_strides(nd);
    for (int i = 0; i < nd; ++i) src_strides[e.saved_perm[i]] = gstr[i];
    BufP o = new_buf((size_t)shape_size(e.saved_shape));
    if (!o) return MNI_ERR_NOMEM;
    MNI_TRY(k_strided_copy(o->p, g->p, e.saved_shape.data(), src_strides.data(), nd));
    out[0] = insert_contig(std::move(o), e.saved_shape);
    return MNI_OK;
}

// ---- loss ------------------------------------------------------------------------------------
// ops/loss.rs:24-67 cross_entropy
static uint32_t cross_entropy_op(uint32_t logits, const int64_t *targets, size_t nt) {
    Tensor *L = get(logits);
    if (!L) return MNI_BAD_ID;
    const Shape shape = L->shape;
    if (shape.empty()) { set_error(MNI_ERR_INVALID, "cross_entropy: scalar logits"); return MNI_BAD_ID; }
    const int64_t v = shape.back();
    const int64_t n = v ? shape_size(shape) / v : 0;
    if (n <= 0 || v <= 0) { set_error(MNI_ERR_INVALID, "cross_entropy: empty logits"); return MNI_BAD_ID; }
    if ((int64_t)nt < n) { set_error(MNI_ERR_INVALID, "cross_entropy: %zu targets for %lld rows", nt, (long long)n); return MNI_BAD_ID; }
    std::vector<int32_t> t32((size_t)n);
    for (int64_t i = 0; i < n; ++i) {
        if (targets[i] < 0 || targets[i] >= v) {
            set_error(MNI_ERR_INVALID, "cross_entropy: target %lld out of range [0, %lld)", (long long)targets[i], (long long)v);
            return MNI_BAD_ID;
        }
        t32[(size_t)i] = (int32_t)targets[i];
    }
    void *tp = nullptr;
    if (dev_alloc(&tp, (size_t)n * sizeof(int32_t)) != MNI_OK) return MNI_BAD_ID;
    std::shared_ptr<void> tdev(tp, [](void *p) { dev_free(p); });
    BufP x = contiguous_buf(*L);
    BufP sm = x ? new_buf((size_t)(n * v)) : nullptr;
    BufP loss = sm ? new_buf(1) : nullptr;
    if (!loss) return MNI_BAD_ID;
    // (a loss that is differentiated is nearly always the root of backward(): its small-batch kernel writes the
    // gradient for that case while it holds the probabilities)
    BufP dl = eng().tape.enabled && n * v <= 16384 ? new_buf((size_t)(n * v)) : nullptr;
    bool wrote = false;
    if (k_cross_entropy(loss->p, sm->p, x->p, (int32_t *)tp, t32.data(), n, v, dl ? dl->p : nullptr, &wrote) != MNI_OK) return MNI_BAD_ID;
    const uint32_t loss_id = insert_contig(std::move(loss), Shape{1});
    const uint32_t sm_id = insert_contig(std::move(sm), shape);
    Entry e;
    e.op = OP_CROSSENTROPY; e.output_id = loss_id; e.n_inputs = 1; e.inputs[0] = logits;
    e.aux = sm_id; e.targets = tdev; e.ce_n = n; e.ce_v = v;
    if (wrote) e.ce_grad_for_one = std::move(dl);
    eng().tape.record(std::move(e));
    return loss_id;
}
// ops/loss.rs:131-149
static int cross_entropy_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad), *S = get(e.aux);
    if (!G || !S) return MNI_ERR_FREED;
    const Shape shape = S->shape;
    if (e.ce_grad_for_one && eng().one && G->buf == eng().one) {  // the upstream gradient is the constant 1.0
        out[0] = insert_contig(BufP(e.ce_grad_for_one), shape);
        return MNI_OK;
    }
    BufP o = new_buf((size_t)(e.ce_n * e.ce_v));
    if (!o) return MNI_ERR_NOMEM;
    MNI_TRY(k_cross_entropy_backward(o->p, S->buf->p, (const int32_t *)e.targets.get(), G->buf->p, e.ce_n, e.ce_v));
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// Opt-in fused form of mseLoss (src/nn.ts:161-165: sub, mul, mean(-1), mean(-1)): one pass over both operands, one
// tape entry.  The result is what the composition gives, one mean per row of the last dim (the second mean of the
// composition runs over the size-1 dim the first one leaves).
static uint32_t mse_rows_op(uint32_t pred, uint32_t target) {
    Tensor *P = get(pred), *T = get(target);
    if (!P || !T) return MNI_BAD_ID;
    if (P->shape != T->shape || P->shape.empty() || P->size <= 0) {
        set_error(MNI_ERR_INVALID, "mse_loss: prediction and target must have the same non-empty shape (no broadcasting)");
        return MNI_BAD_ID;
    }
    Shape out_shape = P->shape;
    const int64_t dim = out_shape.back();
    out_shape.back() = 1;
    const int64_t rows = P->size / dim;
    BufP p = contiguous_buf(*P);
    BufP t = p ? contiguous_buf(*get(target)) : nullptr;
    BufP o = t ? new_buf((size_t)rows) : nullptr;
    // (a loss that is differentiated is nearly always the root of backward(), whose gradient is ones_like(loss),
    // autograd.rs:143: the forward pass, which holds p - t anyway, writes the gradient for that case: one pass over
    // the operands instead of two)
    BufP seeded = o && eng().tape.enabled ? new_buf((size_t)(rows * dim)) : nullptr;
    if (!o || k_mse_rows(o->p, p->p, t->p, rows, dim, seeded ? seeded->p : nullptr) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(o), out_shape);
    Entry e;
    e.op = OP_MSEROWS; e.output_id = id; e.n_inputs = 2; e.inputs[0] = pred; e.inputs[1] = target;
    e.mse_grad_for_ones = std::move(seeded);
    eng().tape.record(std::move(e));
    return id;
}
static int mse_rows_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad), *P = get(e.inputs[0]), *T = get(e.inputs[1]);
    if (!G || !P || !T) return MNI_ERR_FREED;
    const Shape shape = P->shape;
    const int64_t dim = shape.back(), rows = P->size / dim;
    if (G->size != rows) return set_error(MNI_ERR_INVALID, "mse_loss backward: gradient of %lld values for %lld rows", (long long)G->size, (long long)rows);
    // the target's gradient only where something will take it: a tensor that asks for one, or one the tape produced
    Engine &en = eng();
    const uint32_t tid = e.inputs[1];
    const bool want_t = T->requires_grad || (en.bw_out2entry && tid < en.bw_out2entry->size() && (*en.bw_out2entry)[tid] >= 0);
    if (e.mse_grad_for_ones && !want_t && ((en.ones && G->buf == en.ones) || (en.one && G->buf == en.one))) {
        // the upstream gradient is backward()'s own seed of ones: the forward pass has left the result
        out[0] = insert_contig(BufP(e.mse_grad_for_ones), shape);
        return MNI_OK;
    }
    BufP g = contiguous_buf(*G);
    BufP p = g ? contiguous_buf(*get(e.inputs[0])) : nullptr;
    BufP t = p ? contiguous_buf(*get(e.inputs[1])) : nullptr;
    BufP dp = t ? new_buf((size_t)(rows * dim)) : nullptr;
    BufP dt = dp && want_t ? new_buf((size_t)(rows * dim)) : nullptr;
    if (!dp || (want_t && !dt)) return MNI_ERR_NOMEM;
    MNI_TRY(k_mse_rows_backward(dp->p, dt ? dt->p : nullptr, p->p, t->p, g->p, rows, dim));
    out[0] = insert_contig(std::move(dp), shape);
    if (dt) out[1] = insert_contig(std::move(dt), shape);
    return MNI_OK;
}

// ops/elementwise.rs:991-1029 div_backward: da = g / b, db = -g a / b^2, then unbroadcast
static int div_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *A = get(e.inputs[0]), *B = get(e.inputs[1]), *G = get(grad);
    if (!A || !B || !G) return MNI_ERR_FREED;
    const Shape a_shape = A->shape, b_shape = B->shape, g_shape = G->shape;
    const int64_t n = shape_size(g_shape);
    BufP gsrc = contiguous_buf(*G);
    BufP ga_full = new_buf((size_t)n), gb_full = new_buf((size_t)n);
    if (!gsrc || !ga_full || !gb_full) return MNI_ERR_NOMEM;
    StridedDesc d;
    d.ndim = (int)g_shape.size();
    const int ao = d.ndim - (int)a_shape.size(), bo = d.ndim - (int)b_shape.size();
    for (int i = 0; i < d.ndim; ++i) {
        d.shape[i] = g_shape[i];
        d.a_strides[i] = (i < ao || a_shape[i - ao] == 1) ? 0 : A->strides[i - ao];
        d.b_strides[i] = (i < bo || b_shape[i - bo] == 1) ? 0 : B->strides[i - bo];
    }
    MNI_TRY(k_div_backward(ga_full->p, gb_full->p, gsrc->p, A->buf->p, B->buf->p, d));
    const uint32_t fa = insert_contig(std::move(ga_full), g_shape);
    const uint32_t fb = insert_contig(std::move(gb_full), g_shape);
    const uint32_t ga = unbroadcast_tensor(fa, a_shape);
    const uint32_t gb = unbroadcast_tensor(fb, b_shape);
    free_tensor(fa);
    free_tensor(fb);
    if (ga == MNI_BAD_ID || gb == MNI_BAD_ID) return MNI_ERR_INVALID;
    out[0] = ga; out[1] = gb;
    return MNI_OK;
}

// exp / log / pow (ops/elementwise.rs:760-770, 839-849, 1341-1351) and sigmoid
// (ops/activation.rs:194-204).  exp and sigmoid save their output, log and pow
// their input, as the reference's tape does.
static uint32_t unary2_op(uint32_t a, int un, int tape_op, float s) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)A->size) : nullptr;
    if (!out || k_unary(out->p, src->p, A->size, un, s) != MNI_OK) return MNI_BAD_ID;
    const Shape shape = A->shape;
    const uint32_t id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = tape_op; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a; e.scalar = s;
    e.aux = (un == UN_EXP || un == UN_SIGMOID) ? id : a;
    eng().tape.record(std::move(e));
    return id;
}
static int unary2_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad), *S = get(e.aux);
    if (!G || !S) return MNI_ERR_FREED;
    const Shape shape = G->shape;
    BufP g = contiguous_buf(*G), sv = contiguous_buf(*S);
    BufP o = (g && sv) ? new_buf((size_t)G->size) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    const int un = e.op == OP_EXP ? UN_EXP : e.op == OP_LOG ? UN_LOG : e.op == OP_SIGMOID ? UN_SIGMOID : UN_POW;
    MNI_TRY(k_unary2_backward(o->p, g->p, sv->p, G->size, un, e.scalar));
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// ops/reduce.rs:333-368 max along dim (kept as size 1), :416-447 its backward
static uint32_t max_op(uint32_t a, int64_t dim) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const int nd = (int)A->shape.size();
    const int d = (int)(dim < 0 ? nd + dim : dim);
    if (d < 0 || d >= nd) { set_error(MNI_ERR_INVALID, "max dim %lld out of range for rank %d", (long long)dim, nd); return MNI_BAD_ID; }
    const Shape a_shape = A->shape;
    Shape out_shape = a_shape;
    out_shape[d] = 1;
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= a_shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= a_shape[i];
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)shape_size(out_shape)) : nullptr;
    if (!out || k_max_dim(out->p, src->p, outer, a_shape[d], inner) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), out_shape);
    Entry e;
    e.op = OP_MAX; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a; e.aux = id; e.scalar = (float)d;
    eng().tape.record(std::move(e));
    return id;
}
static int max_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *X = get(e.inputs[0]), *M = get(e.aux), *G = get(grad);
    if (!X || !M || !G) return MNI_ERR_FREED;
    const Shape shape = X->shape;
    const int nd = (int)shape.size(), d = (int)e.scalar;
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= shape[i];
    BufP x = contiguous_buf(*X), m = contiguous_buf(*M), g = contiguous_buf(*G);
    BufP o = (x && m && g) ? new_buf((size_t)X->size) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    MNI_TRY(k_max_backward(o->p, x->p, m->p, g->p, outer, shape[d], inner));
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// ops/norm.rs:167-215 layernorm over the last extent; saves mean and rstd per row
static uint32_t layernorm_op(uint32_t x, uint32_t gamma, uint32_t beta, float eps) {
    Tensor *X = get(x), *Gm = get(gamma), *Bt = get(beta);
    if (!X || !Gm || !Bt) return MNI_BAD_ID;
    if (X->shape.empty()) { set_error(MNI_ERR_INVALID, "layernorm: x must have at least one dim"); return MNI_BAD_ID; }
    const Shape shape = X->shape;
    const int64_t c = shape.back(), rows = c ? X->size / c : 0;
    if (Gm->size < c || Bt->size < c) { set_error(MNI_ERR_INVALID, "layernorm: gamma / beta hold fewer than %lld values", (long long)c); return MNI_BAD_ID; }
    BufP xs = contiguous_buf(*X), gs = contiguous_buf(*Gm), bs = contiguous_buf(*Bt);
    BufP out = (xs && gs && bs) ? new_buf((size_t)X->size) : nullptr;
    BufP mean = out ? new_buf((size_t)rows) : nullptr, rstd = mean ? new_buf((size_t)rows) : nullptr;
    if (!rstd || k_layernorm(out->p, mean->p, rstd->p, xs->p, gs->p, bs->p, rows, c, eps) != MNI_OK) return MNI_BAD_ID;
    const uint32_t out_id = insert_contig(std::move(out), shape);
    const uint32_t mean_id = insert_contig(std::move(mean), Shape{rows});
    const uint32_t rstd_id = insert_contig(std::move(rstd), Shape{rows});
    Entry e;
    e.op = OP_LAYERNORM; e.output_id = out_id; e.n_inputs = 3;
    e.inputs[0] = x; e.inputs[1] = gamma; e.inputs[2] = beta; e.aux = mean_id; e.aux2 = rstd_id;
    eng().tape.record(std::move(e));
    return out_id;
}
// ops/norm.rs:273-322
static int layernorm_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *X = get(e.inputs[0]), *Gm = get(e.inputs[1]), *Mn = get(e.aux), *Rs = get(e.aux2), *G = get(grad);
    if (!X || !Gm || !Mn || !Rs || !G) return MNI_ERR_FREED;
    const Shape shape = X->shape, gshape = Gm->shape;
    const int64_t c = shape.back(), rows = c ? X->size / c : 0;
    BufP xs = contiguous_buf(*X), gs = contiguous_buf(*Gm), g = contiguous_buf(*G);
    BufP dx = (xs && gs && g) ? new_buf((size_t)X->size) : nullptr;
    BufP dgamma = dx ? new_buf((size_t)Gm->size) : nullptr, dbeta = dgamma ? new_buf((size_t)Gm->size) : nullptr;
    if (!dbeta) return MNI_ERR_NOMEM;
    if (Gm->size > c) { MNI_TRY(k_fill(dgamma->p, 0.0f, Gm->size)); MNI_TRY(k_fill(dbeta->p, 0.0f, Gm->size)); }
    MNI_TRY(k_layernorm_backward(dx->p, dgamma->p, dbeta->p, g->p, xs->p, gs->p, Mn->buf->p, Rs->buf->p, rows, c));
    out[0] = insert_contig(std::move(dx), shape);
    out[1] = insert_contig(std::move(dgamma), gshape);
    out[2] = insert_contig(std::move(dbeta), gshape);
    return MNI_OK;
}

// ---- fused bias + GELU ------------------------------------------------------------------------------
// ops/fused.rs:247-273: out = gelu(x + bias[i % c]), c = last extent of x.
static uint32_t bias_gelu_op(uint32_t x, uint32_t bias) {
    Tensor *X = get(x), *Bv = get(bias);
    if (!X || !Bv) return MNI_BAD_ID;
    if (X->shape.empty()) { set_error(MNI_ERR_INVALID, "bias_gelu: x must have at least one dim"); return MNI_BAD_ID; }
    const Shape shape = X->shape;
    const int64_t c = shape.back();
    if (Bv->size < c) { set_error(MNI_ERR_INVALID, "bias_gelu: bias holds %lld values, last extent is %lld", (long long)Bv->size, (long long)c); return MNI_BAD_ID; }
    BufP xs = contiguous_buf(*X), bs = contiguous_buf(*Bv);
    BufP out = (xs && bs) ? new_buf((size_t)X->size) : nullptr;
    if (!out || k_bias_gelu(out->p, xs->p, bs->p, c ? X->size / c : 0, c) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = OP_BIASGELU; e.output_id = id; e.n_inputs = 2; e.inputs[0] = x; e.inputs[1] = bias;
    eng().tape.record(std::move(e));
    return id;
}
// ops/fused.rs:316-351: dx = grad * gelu'(x + bias), dbias = column sums of dx.
static int bias_gelu_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *X = get(e.inputs[0]), *Bv = get(e.inputs[1]), *G = get(grad);
    if (!X || !Bv || !G) return MNI_ERR_FREED;
    const Shape shape = X->shape, bshape = Bv->shape;
    const int64_t c = shape.back(), rows = c ? X->size / c : 0;
    BufP xs = contiguous_buf(*X), bs = contiguous_buf(*Bv), gs = contiguous_buf(*G);
    BufP dx = (xs && bs && gs) ? new_buf((size_t)X->size) : nullptr;
    BufP db = dx ? new_buf((size_t)Bv->size) : nullptr;
    if (!db) return MNI_ERR_NOMEM;
    if (Bv->size > c) MNI_TRY(k_fill(db->p, 0.0f, Bv->size));  // entries past the last extent receive nothing
    MNI_TRY(k_bias_gelu_backward(dx->p, db->p, gs->p, xs->p, bs->p, rows, c));
    out[0] = insert_contig(std::move(dx), shape);
    out[1] = insert_contig(std::move(db), bshape);
    return MNI_OK;
}

// ---- softmax -----------------------------------------------------------------------------------
// ops/norm.rs:10-50.  The tape keeps the dim as it was passed (:47).
static uint32_t softmax_op(uint32_t a, int64_t dim) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const Shape shape = A->shape;
    const int nd = (int)shape.size();
    const int d = (int)(dim < 0 ? nd + dim : dim);
    if (d < 0 || d >= nd) { set_error(MNI_ERR_INVALID, "softmax: dim %lld out of range for %d dims", (long long)dim, nd); return MNI_BAD_ID; }
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= shape[i];
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)A->size) : nullptr;
    if (!out || k_softmax(out->p, src->p, outer, shape[d], inner) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = OP_SOFTMAX; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a; e.scalar = (float)dim; e.aux = id;
    eng().tape.record(std::move(e));
    return id;
}
// ops/norm.rs:96-123.  The saved dim is read back with Rust's saturating
// `as usize`, so a negative dim (the TypeScript default -1, src/nn.ts:77)
// reduces along dim 0 in the reference; kept so that gradients match it.
static int softmax_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *G = get(grad), *S = get(e.aux);
    if (!G || !S) return MNI_ERR_FREED;
    const Shape shape = S->shape;
    const int nd = (int)shape.size();
    const int d = e.scalar > 0.f ? (int)e.scalar : 0;
    if (d >= nd) return set_error(MNI_ERR_INVALID, "softmax backward: dim %d out of range", d);
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < d; ++i) outer *= shape[i];
    for (int i = d + 1; i < nd; ++i) inner *= shape[i];
    BufP g = contiguous_buf(*G), sm = contiguous_buf(*S);
    BufP o = (g && sm) ? new_buf((size_t)S->size) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    MNI_TRY(k_softmax_backward(o->p, sm->p, g->p, outer, shape[d], inner));
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// ---- attention on the batched GEMM ----------------------------------------------------------------
// One batched product through the kernel-level entry: C[b] = op(A)[b] op(B)[b],
// operands given as contiguous [bh, rows, cols] buffers, optionally transposed.
static int attn_gemm(float *c, const float *a, bool ta, const float *b, bool tb, int64_t bh, int64_t m, int64_t n,
                     int64_t k) {
    mni_gemm_desc d;
    memset(&d, 0, sizeof d);
    d.M = m; d.N = n; d.K = k; d.batch = bh;
    // a is stored [bh][m][k] (or [bh][k][m] when ta); b is [bh][k][n] (or [bh][n][k] when tb)
    d.A = ta ? mni_operand{a, 1, m, k * m, bh} : mni_operand{a, k, 1, m * k, bh};
    d.B = tb ? mni_operand{b, 1, k, n * k, bh} : mni_operand{b, n, 1, k * n, bh};
    d.C = c; d.ldc = n; d.c_batch_stride = m * n;
    return sgemm(d);
}

// ops/attention.rs:14-78: q, k, v are taken as [bh, s, d] from their first
// three dims.  Head dims 32, 64, 96 and 128 run the forward in one kernel that
// keeps the scores on the chip; otherwise scores = q k^T and out = P v run on
// the GEMM kernels and the row kernel in between applies scale, the causal
// mask and the normalisation.  Either way lse = max + ln(sum) is left for the
// backward pass, which recomputes P from it.
static uint32_t flash_attention_op(uint32_t q, uint32_t k, uint32_t v, float scale, bool causal) {
    Tensor *Q = get(q), *K = get(k), *V = get(v);
    if (!Q || !K || !V) return MNI_BAD_ID;
    if (Q->shape.size() < 3) { set_error(MNI_ERR_INVALID, "flash_attention: q must be [bh, s, d]"); return MNI_BAD_ID; }
    const int64_t bh = Q->shape[0], s = Q->shape[1], d = Q->shape[2];
    const int64_t total = bh * s * d;
    if (K->size < total || V->size < total) {
        set_error(MNI_ERR_INVALID, "flash_attention: k / v hold fewer than bh*s*d = %lld values", (long long)total);
        return MNI_BAD_ID;
    }
    BufP qc = contiguous_buf(*Q), kc = contiguous_buf(*K), vc = contiguous_buf(*V);
    if (!qc || !kc || !vc) return MNI_BAD_ID;
    BufP lse = new_buf((size_t)(bh * s));
    BufP out = lse ? new_buf((size_t)total) : nullptr;
    if (!out) return MNI_BAD_ID;
    if (total > 0 && attn_fused_supported(d)) {
        // head dims 32 .. 128: one kernel, the scores never reach memory
        if (k_attn_fused_forward(out->p, lse->p, qc->p, kc->p, vc->p, bh, s, d, scale, causal ? 1 : 0) != MNI_OK) return MNI_BAD_ID;
    } else if (total > 0) {
        BufP scores = new_buf((size_t)(bh * s * s));
        if (!scores) return MNI_BAD_ID;
        if (attn_gemm(scores->p, qc->p, false, kc->p, true, bh, s, s, d) != MNI_OK) return MNI_BAD_ID;
        if (k_attn_softmax(scores->p, lse->p, bh * s, s, scale, causal ? 1 : 0) != MNI_OK) return MNI_BAD_ID;
        if (attn_gemm(out->p, scores->p, false, vc->p, false, bh, s, d, s) != MNI_OK) return MNI_BAD_ID;
    }
    const uint32_t out_id = insert_contig(std::move(out), Shape{bh, s, d});
    const uint32_t lse_id = insert_contig(std::move(lse), Shape{bh, s});
    Entry e;
    e.op = OP_FLASHATTENTION; e.output_id = out_id; e.n_inputs = 3;
    e.inputs[0] = q; e.inputs[1] = k; e.inputs[2] = v;
    e.aux = out_id; e.aux2 = lse_id; e.scalar = scale; e.act = causal ? 1 : 0;
    eng().tape.record(std::move(e));
    return out_id;
}
// ops/attention.rs:143-202: di = rowsum(dO * O); P recomputed from lse;
// dV = P^T dO, dP = dO V^T, dS = P (dP - di) scale, dQ = dS K, dK = dS^T Q.
static int flash_attention_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *Q = get(e.inputs[0]), *K = get(e.inputs[1]), *V = get(e.inputs[2]);
    Tensor *O = get(e.aux), *L = get(e.aux2), *G = get(grad);
    if (!Q || !K || !V || !O || !L || !G) return MNI_ERR_FREED;
    const int64_t bh = Q->shape[0], s = Q->shape[1], d = Q->shape[2];
    const int64_t total = bh * s * d;
    BufP qc = contiguous_buf(*Q), kc = contiguous_buf(*K), vc = contiguous_buf(*V);
    BufP oc = contiguous_buf(*O), lc = contiguous_buf(*L), gc = contiguous_buf(*G);
    if (!qc || !kc || !vc || !oc || !lc || !gc) return MNI_ERR_NOMEM;
    BufP di = new_buf((size_t)(bh * s));
    BufP dq = new_buf((size_t)total), dk = new_buf((size_t)total), dv = new_buf((size_t)total);
    if (!di || !dq || !dk || !dv) return MNI_ERR_NOMEM;
    if (total > 0 && attn_fused_supported(d)) {
        // head dims 32 .. 128: two kernels that recompute P from lse, nothing of size s x s is stored
        MNI_TRY(k_rowdot(di->p, gc->p, oc->p, bh * s, d));
        MNI_TRY(k_attn_fused_backward_dq(dq->p, qc->p, kc->p, vc->p, gc->p, lc->p, di->p, bh, s, d, e.scalar, e.act));
        MNI_TRY(k_attn_fused_backward_dkv(dk->p, dv->p, qc->p, kc->p, vc->p, gc->p, lc->p, di->p, bh, s, d, e.scalar, e.act));
    } else if (total > 0) {
        BufP p = new_buf((size_t)(bh * s * s)), ds = new_buf((size_t)(bh * s * s));
        if (!p || !ds) return MNI_ERR_NOMEM;
        MNI_TRY(k_rowdot(di->p, gc->p, oc->p, bh * s, d));
        MNI_TRY(attn_gemm(p->p, qc->p, false, kc->p, true, bh, s, s, d));   // q k^T
        MNI_TRY(attn_gemm(ds->p, gc->p, false, vc->p, true, bh, s, s, d));  // dO v^T
        MNI_TRY(k_attn_backward(p->p, ds->p, lc->p, di->p, bh * s, s, e.scalar, e.act));
        MNI_TRY(attn_gemm(dv->p, p->p, true, gc->p, false, bh, s, d, s));   // P^T dO
        MNI_TRY(attn_gemm(dq->p, ds->p, false, kc->p, false, bh, s, d, s)); // dS k
        MNI_TRY(attn_gemm(dk->p, ds->p, true, qc->p, false, bh, s, d, s));  // dS^T q
    }
    const Shape shape{bh, s, d};
    out[0] = insert_contig(std::move(dq), shape);
    out[1] = insert_contig(std::move(dk), shape);
    out[2] = insert_contig(std::move(dv), shape);
    return MNI_OK;
}

// ---- KV cache ------------------------------------------------------------------------------------
static std::shared_ptr<void> dev_block(size_t bytes) {
    void *p = nullptr;
    if (dev_alloc(&p, bytes ? bytes : 4) != MNI_OK) return nullptr;
    return std::shared_ptr<void>(p, [](void *q) { dev_free(q); });
}
static std::string shape_text(const Shape &s) {  // Rust's {:?} of a slice
    std::string t = "[";
    for (size_t i = 0; i < s.size(); ++i) t += (i ? ", " : "") + std::to_string(s[i]);
    return t + "]";
}
// ops/kv_cache.rs:83-111, 336-349: [B,H,S,D] or [BH,S,D] with S = 1 and the cache's extents
static bool kv_validate(const KvCache &c, const Shape &shape, const char *op, std::string *why) {
    int64_t b, h, sl, d;
    if (shape.size() == 4) { b = shape[0]; h = shape[1]; sl = shape[2]; d = shape[3]; }
    else if (shape.size() == 3) { b = 1; h = shape[0]; sl = shape[1]; d = shape[2]; }
    else { *why = "expected [B,H,S,D] or [BH,S,D], got shape " + shape_text(shape); return false; }
    if (sl != 1) { *why = std::string("kv cache ") + op + " expects seq_len=1, got " + std::to_string(sl); return false; }
    if (b != c.batch || h != c.heads || d != c.d) {
        *why = std::string("kv cache ") + op + " shape mismatch: expected [B=" + std::to_string(c.batch) + ", H=" +
               std::to_string(c.heads) + ", S=1, D=" + std::to_string(c.d) + "], got [B=" + std::to_string(b) + ", H=" +
               std::to_string(h) + ", S=1, D=" + std::to_string(d) + "]";
        return false;
    }
    return true;
}
// ops/kv_cache.rs:113-171 append_inner
static bool kv_append_inner(KvCache &c, const Tensor &K, const Tensor &V, std::string *why) {
    if (c.len >= c.max_seq) {
        *why = "kv cache is full (len=" + std::to_string(c.len) + ", max_seq_len=" + std::to_string(c.max_seq) + ")";
        return false;
    }
    const int64_t bh = c.batch * c.heads;
    BufP kb = contiguous_buf(K), vb = contiguous_buf(V);
    if (!kb || !vb) { *why = mni_rocm_last_error(); return false; }
    if (k_kv_append(c.keys.get(), c.vals.get(), (float *)c.kscale.get(), (float *)c.vscale.get(), kb->p, vb->p, bh, c.d,
                    c.max_seq, c.len, c.quantized ? 1 : 0) != MNI_OK) {
        *why = mni_rocm_last_error();
        return false;
    }
    c.len += 1;
    return true;
}
static uint32_t kv_cache_create(int64_t batch, int64_t heads, int64_t d, int64_t max_seq, bool quantized) {
    if (batch < 0 || heads < 0 || d < 0 || max_seq < 0) { set_error(MNI_ERR_INVALID, "kv cache: negative extent"); return MNI_BAD_ID; }
    KvCache c;
    c.batch = batch; c.heads = heads; c.d = d; c.max_seq = max_seq; c.quantized = quantized;
    const size_t cap = (size_t)(batch * heads * max_seq * d), rows = (size_t)(batch * heads * max_seq);
    c.keys = dev_block(cap * (quantized ? 1 : sizeof(float)));
    c.vals = dev_block(cap * (quantized ? 1 : sizeof(float)));
    if (quantized) { c.kscale = dev_block(rows * sizeof(float)); c.vscale = dev_block(rows * sizeof(float)); }
    if (!c.keys || !c.vals || (quantized && (!c.kscale || !c.vscale))) return MNI_BAD_ID;
    Engine &e = eng();
    const uint32_t id = e.next_kv_cache_id++;
    e.kv_caches[id] = std::move(c);
    return id;
}
static int kv_cache_append(uint32_t id, uint32_t k, uint32_t v) {  // lib.rs:661-676, kv_cache.rs:173-181
    auto it = eng().kv_caches.find(id);
    if (it == eng().kv_caches.end()) return set_error(MNI_ERR_INVALID, "invalid kv cache id: %u", id);
    Tensor *K = get(k), *V = get(v);
    if (!K || !V) return MNI_ERR_FREED;
    std::string why;
    bool ok = true;
    if (K->shape != V->shape) { why = "k/v shapes must match for kv cache append"; ok = false; }
    ok = ok && kv_validate(it->second, K->shape, "append", &why) && kv_append_inner(it->second, *K, *V, &why);
    return ok ? MNI_OK : set_error(MNI_ERR_INVALID, "kv cache append failed: %s", why.c_str());
}
static uint32_t kv_cache_decode_step(uint32_t id, uint32_t q, uint32_t k, uint32_t v, float scale) {  // lib.rs:641-659
    auto it = eng().kv_caches.find(id);
    if (it == eng().kv_caches.end()) { set_error(MNI_ERR_INVALID, "invalid kv cache id: %u", id); return MNI_BAD_ID; }
    KvCache &c = it->second;
    Tensor *Q = get(q), *K = get(k), *V = get(v);
    if (!Q || !K || !V) return MNI_BAD_ID;
    std::string why;
    bool ok = true;
    if (Q->shape != K->shape || Q->shape != V->shape) { why = "q/k/v shapes must match for kv cache decode"; ok = false; }
    ok = ok && kv_validate(c, Q->shape, "decode", &why) && kv_append_inner(c, *K, *V, &why);
    BufP qb, out;
    const int64_t bh = c.batch * c.heads;
    if (ok) {
        qb = contiguous_buf(*Q);
        out = qb ? new_buf((size_t)(bh * c.d)) : nullptr;
        if (!out || k_kv_decode(out->p, c.keys.get(), c.vals.get(), (const float *)c.kscale.get(), (const float *)c.vscale.get(),
                                qb->p, bh, c.d, c.max_seq, c.len, scale, c.quantized ? 1 : 0) != MNI_OK) {
            why = mni_rocm_last_error();
            ok = false;
        }
    }
    if (!ok) { set_error(MNI_ERR_INVALID, "kv cache decode failed: %s", why.c_str()); return MNI_BAD_ID; }
    const Shape out_shape = Q->shape.size() == 4 ? Shape{c.batch, c.heads, 1, c.d} : Shape{bh, 1, c.d};
    return insert_contig(std::move(out), out_shape);
}

// ---- fused Linear ------------------------------------------------------------------------------
static uint32_t linear_op(uint32_t x, uint32_t w, uint32_t bias, int act) {
    Tensor *X = get(x), *W = get(w), *Bv = get(bias);
    if (!X || !W || !Bv) return MNI_BAD_ID;
    if (act < MNI_EPI_BIAS || act > MNI_EPI_BIAS_GELU) { set_error(MNI_ERR_INVALID, "linear: unknown activation %d", act); return MNI_BAD_ID; }
    if (W->shape.size() != 2) { set_error(MNI_ERR_INVALID, "linear: weight must be [in, out]"); return MNI_BAD_ID; }
    if (Bv->shape.size() != 1 || Bv->shape[0] != W->shape[1] || !is_contiguous(*Bv)) {
        set_error(MNI_ERR_INVALID, "linear: bias must be a contiguous [out] vector");
        return MNI_BAD_ID;
    }
    // GELU needs its pre-activation in backward: the product's epilogue writes it (without the bias) and
    // gelu(product + bias) side by side (the reference fuses bias + GELU into one pass after the product,
    // ops/fused.rs:247-273); plain bias and ReLU ride in the epilogue as one output.
    const BufP bias_buf = Bv->buf;
    uint32_t out, aux = MNI_BAD_ID;
    if (act == MNI_EPI_BIAS_GELU) {
        int64_t n_out = W->shape[1];
        for (size_t i = 0; i + 1 < X->shape.size(); ++i) n_out *= X->shape[i];
        BufP o = new_buf((size_t)(n_out > 0 ? n_out : 1));
        if (!o) return MNI_BAD_ID;
        aux = matmul_tensors(x, false, w, false, bias_buf->p, MNI_EPI_BIAS_GELU_DUAL, o->p);
        if (aux == MNI_BAD_ID) return MNI_BAD_ID;
        const Shape zshape = get(aux)->shape;
        out = insert_contig(std::move(o), zshape);
    } else {
        out = matmul_tensors(x, false, w, false, bias_buf->p, act);
        if (out == MNI_BAD_ID) return MNI_BAD_ID;
    }
    Entry e;
    e.op = OP_LINEAR; e.output_id = out; e.n_inputs = 3;
    e.inputs[0] = x; e.inputs[1] = w; e.inputs[2] = bias;
    e.act = act; e.aux = aux;
    eng().tape.record(std::move(e));
    return out;
}
static int linear_backward(uint32_t grad, const Entry &e, int64_t *out) {
    uint32_t g = grad;
    bool own_g = false;
    int64_t db_id = -1;
    Engine &en = eng();
    Engine::PendingStrips pend = {nullptr, 0, 0};
    const auto pre = en.preact_strips.find(e.output_id);
    if (e.act == MNI_EPI_BIAS_GELU && pre != en.preact_strips.end()) {
        // the entry that consumed this layer's output has already taken the gradient through gelu'
        // (in the epilogue of its own product) and left the bias gradient as strip sums
        pend = std::move(pre->second);
        en.preact_strips.erase(pre);
    } else if (e.act == MNI_EPI_BIAS_GELU) {
        // dZ = dOut * gelu'(z + bias) and db = column sums of dZ in one pass (ops/fused.rs:316-351)
        Tensor *G = get(grad), *Z = get(e.aux), *Bv = get(e.inputs[2]);
        if (!G || !Z || !Bv) return MNI_ERR_FREED;
        const int64_t c = Z->shape.back();
        BufP gb = contiguous_buf(*G);
        BufP o = gb ? new_buf((size_t)G->size) : nullptr;
        BufP db = o ? new_buf((size_t)c) : nullptr;
        if (!db) return MNI_ERR_NOMEM;
        MNI_TRY(k_bias_gelu_backward(o->p, db->p, gb->p, Z->buf->p, Bv->buf->p, c ? Z->size / c : 0, c));
        // shapes are copied first: an insert may move the tensor table and leave G / Bv dangling
        const Shape gshape = G->shape, bshape = Bv->shape;
        g = insert_contig(std::move(o), gshape);
        db_id = insert_contig(std::move(db), bshape);
        own_g = true;
    } else if (e.act == MNI_EPI_BIAS_RELU) {
        // dZ = dOut where the output is positive (the output has the sign of z)
        Tensor *G = get(grad), *Z = get(e.output_id);
        if (!G || !Z) return MNI_ERR_FREED;
        BufP gb = contiguous_buf(*G);
        BufP o = gb ? new_buf((size_t)G->size) : nullptr;
        if (!o) return MNI_ERR_NOMEM;
        MNI_TRY(k_unary_backward(o->p, gb->p, Z->buf->p, G->size, UN_RELU));
        g = insert_contig(std::move(o), G->shape);
        own_g = true;
    }
    Entry mm;
    mm.op = OP_MATMUL; mm.n_inputs = 2; mm.inputs[0] = e.inputs[0]; mm.inputs[1] = e.inputs[1];
    // Is the input the output of a GELU Linear that nobody else reads?  Then dX leaves this layer's product
    // as dZ of that one: gelu'(z + bias) applied and the bias gradient's strip sums taken in the epilogue
    // (instead of a pass over dX and z of its own), and that layer's backward starts from dZ.
    ThroughGelu tg = {nullptr, nullptr, nullptr};
    BufP strips;
    uint32_t producer_out = MNI_BAD_ID;
    int64_t strip_rows = 0, strip_cols = 0;
    if (en.bw_tape) {
        const uint32_t x = e.inputs[0];
        Tensor *X = get(x);
        const int64_t pi = x < en.bw_out2entry->size() ? (*en.bw_out2entry)[x] : -1;
        if (X && pi >= 0 && !X->requires_grad && is_contiguous(*X) && X->shape.size() >= 2 && (*en.bw_consumers)[x] == 1 &&
            (*en.bw_grads)[x] < 0) {
            const Entry &P = en.bw_tape->entries[(size_t)pi];
            Tensor *Z = P.op == OP_LINEAR && P.act == MNI_EPI_BIAS_GELU && P.output_id == x ? get(P.aux) : nullptr;
            Tensor *PB = Z ? get(P.inputs[2]) : nullptr;
            if (Z && PB && is_contiguous(*Z) && Z->shape == X->shape && en.preact_strips.find(x) == en.preact_strips.end()) {
                strip_cols = X->shape.back();
                const int64_t m = X->shape[X->shape.size() - 2];
                strip_rows = mni_rocm_sgemm_colsum_rows(m, strip_cols && m ? X->size / (strip_cols * m) : 0);
                if (strip_rows > 0 && strip_cols > 0) strips = new_buf((size_t)(strip_rows * strip_cols));
                if (strips) {
                    tg.bias = PB->buf->p;
                    tg.z = Z->buf->p;
                    tg.colsum_part = strips->p;
                    producer_out = x;
                }
            }
        }
    }
    // The bias gradient (column sums of g over its rows, or of the strip sums left by the consumer) rides in the launch
    // of the two products when they go out as one launch that takes it: a training step of a few thousand parameters
    // is the sum of its launches, and under two big products the sums cost nothing.
    PairColsum sums = {nullptr, nullptr, 0, 0, false};
    BufP db_early;
    if (pend.strips) {
        db_early = new_buf((size_t)pend.cols);
        if (!db_early) return MNI_ERR_NOMEM;
        sums = PairColsum{pend.strips->p, db_early->p, pend.rows, pend.cols, false};
    } else if (db_id < 0) {
        Tensor *G = get(g), *Bv = get(e.inputs[2]);
        if (G && Bv && is_contiguous(*G) && !G->shape.empty() && G->shape.back() == Bv->size && Bv->size > 0) {
            db_early = new_buf((size_t)Bv->size);
            if (db_early) sums = PairColsum{G->buf->p, db_early->p, G->size / Bv->size, Bv->size, false};
        }
    }
    int rc = matmul_backward(g, mm, out, tg.z ? &tg : nullptr, sums.out ? &sums : nullptr);
    if (rc == MNI_OK && tg.z) en.preact_strips[producer_out] = Engine::PendingStrips{strips, strip_rows, strip_cols};
    // (the strips added up in strip order, when the launch above did not take them)
    if (rc == MNI_OK && pend.strips && !sums.done) rc = k_colsum(db_early->p, pend.strips->p, pend.rows, pend.cols);
    if (rc == MNI_OK) {
        if (db_id >= 0) out[2] = db_id;
        else {
            Tensor *Bv = get(e.inputs[2]);
            if (!Bv) rc = MNI_ERR_FREED;
            else {
                const Shape bshape = Bv->shape;
                const uint32_t gb = (sums.done || pend.strips) ? insert_contig(std::move(db_early), bshape) : unbroadcast_tensor(g, bshape);
                if (gb == MNI_BAD_ID) rc = MNI_ERR_INVALID;
                else out[2] = gb;
            }
        }
    } else if (db_id >= 0) free_tensor((uint32_t)db_id);
    if (own_g) free_tensor(g);
    return rc;
}

// ---- random numbers ------------------------------------------------------------------------------
static void rng_init(Engine &e) {
    if (e.rng_ready) return;
    std::random_device rd;
    e.rng_seed = ((uint64_t)rd() << 32) ^ (uint64_t)rd();
    e.rng_offset = 0;
    e.host_rng.seed(e.rng_seed);
    e.rng_ready = true;
}
// Reserve the Philox blocks for n elements and return where they start.
static uint64_t rng_take(int64_t n) {
    Engine &e = eng();
    rng_init(e);
    const uint64_t at = e.rng_offset;
    e.rng_offset += (uint64_t)((n + 3) / 4);
    return at;
}
// tensor.rs:228-250 rand (uniform [0, 1)) / randn (standard normal)
static uint32_t random_tensor(const Shape &shape, int mode) {
    const int64_t n = shape_size(shape);
    BufP b = new_buf((size_t)n);
    if (!b) return MNI_BAD_ID;
    const uint64_t at = rng_take(n);
    if (k_random_fill(b->p, n, eng().rng_seed, at, mode) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(b), shape);
}

// ---- dropout (ops/dropout.rs) --------------------------------------------------------------------
// The mask is not stored: the tape keeps where it starts in the random stream
// and the backward regenerates it.
static uint32_t dropout_op(uint32_t x, float rate, bool training) {
    Tensor *X = get(x);
    if (!X) return MNI_BAD_ID;
    if (!training || rate == 0.0f) return x;  // the same id, dropout.rs:30-32
    const Shape shape = X->shape;
    const int64_t n = X->size;
    BufP src = contiguous_buf(*X);
    BufP out = src ? new_buf((size_t)n) : nullptr;
    if (!out) return MNI_BAD_ID;
    const float scale = 1.0f / (1.0f - rate);
    const uint64_t at = rng_take(n);
    if (k_dropout(out->p, src->p, n, rate, scale, eng().rng_seed, at) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = OP_DROPOUT; e.output_id = id; e.n_inputs = 1; e.inputs[0] = x; e.scalar = rate;
    e.rng_seed = eng().rng_seed; e.rng_offset = at;
    eng().tape.record(std::move(e));
    return id;
}
static int dropout_backward(uint32_t grad, const Entry &e, int64_t *out) {  // dropout.rs:114-126
    Tensor *G = get(grad);
    if (!G) return MNI_ERR_FREED;
    const Shape shape = G->shape;
    BufP g = contiguous_buf(*G);
    BufP o = g ? new_buf((size_t)G->size) : nullptr;
    if (!o) return MNI_ERR_NOMEM;
    const float scale = 1.0f / (1.0f - e.scalar);
    MNI_TRY(k_dropout(o->p, g->p, G->size, e.scalar, scale, e.rng_seed, e.rng_offset));
    out[0] = insert_contig(std::move(o), shape);
    return MNI_OK;
}

// ---- integer buffers and datasets (ops/data.rs) ------------------------------------------------------
static IntBuf *get_int(uint32_t id) {  // data.rs:49-51
    Engine &e = eng();
    if (id >= e.int_bufs.size() || !e.int_bufs[id].live) {
        set_error(MNI_ERR_FREED, "int buffer already freed (id %u)", id);
        return nullptr;
    }
    return &e.int_bufs[id];
}
static uint32_t insert_int(IntBuf &&b) {  // data.rs:37-47: LIFO id recycling
    Engine &e = eng();
    b.live = true;
    if (!e.int_free.empty()) {
        const uint32_t id = e.int_free.back();
        e.int_free.pop_back();
        e.int_bufs[id] = std::move(b);
        return id;
    }
    e.int_bufs.push_back(std::move(b));
    return (uint32_t)e.int_bufs.size() - 1;
}
static std::shared_ptr<void> dev_ints(size_t n) {
    void *p = nullptr;
    if (dev_alloc(&p, (n ? n : 1) * sizeof(int32_t)) != MNI_OK) return nullptr;
    return std::shared_ptr<void>(p, [](void *q) { dev_free(q); });
}
static uint32_t create_dataset(const int32_t *data, size_t len) {  // data.rs:69-77
    IntBuf b;
    b.data = dev_ints(len);
    if (!b.data) return MNI_BAD_ID;
    b.len = (int64_t)len;
    if (len) {
        b.lo = b.hi = data[0];
        for (size_t i = 1; i < len; ++i) {
            if (data[i] < b.lo) b.lo = data[i];
            if (data[i] > b.hi) b.hi = data[i];
        }
        if (mni_rocm_h2d(b.data.get(), data, len * sizeof(int32_t)) != MNI_OK) return MNI_BAD_ID;
    }
    return insert_int(std::move(b));
}
// data.rs:112-155: batch_size windows of block_size tokens, each starting at a
// uniform offset in [0, len - block_size - 1); targets are the inputs shifted
// by one token.  Only the offsets cross the bus.
static int sample_batch(uint32_t dataset, int64_t block, int64_t batch, uint32_t *out_ids) {
    IntBuf *ds = get_int(dataset);
    if (!ds) return MNI_ERR_FREED;
    if (block <= 0 || batch <= 0) return set_error(MNI_ERR_INVALID, "sample_batch: block_size and batch_size must be positive");
    const int64_t range = ds->len - block - 1;
    if (range <= 0)
        return set_error(MNI_ERR_INVALID, "sample_batch: cannot sample empty range (dataset of %lld tokens, block_size %lld)",
                         (long long)ds->len, (long long)block);
    if (ds->len > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sample_batch: dataset too large for 32-bit offsets");
    Engine &e = eng();
    rng_init(e);
    std::vector<int32_t> starts((size_t)batch);
    std::uniform_int_distribution<int64_t> pick(0, range - 1);
    for (auto &s : starts) s = (int32_t)pick(e.host_rng);
    std::shared_ptr<void> dstarts = dev_ints((size_t)batch);
    IntBuf inp, tgt;
    inp.data = dev_ints((size_t)(batch * block));
    tgt.data = dev_ints((size_t)(batch * block));
    if (!dstarts || !inp.data || !tgt.data) return MNI_ERR_NOMEM;
    MNI_TRY(upload_small(dstarts.get(), starts.data(), (size_t)batch * sizeof(int32_t)));
    const std::shared_ptr<void> src = ds->data;
    inp.len = tgt.len = batch * block;
    inp.lo = tgt.lo = ds->lo;
    inp.hi = tgt.hi = ds->hi;
    MNI_TRY(k_sample_windows((int32_t *)inp.data.get(), (int32_t *)tgt.data.get(), (const int32_t *)src.get(),
                             (const int32_t *)dstarts.get(), block, batch));
    // the offsets buffer returns to the allocator here; the stream orders its reuse after the kernel
    out_ids[0] = insert_int(std::move(inp));
    out_ids[1] = insert_int(std::move(tgt));
    return MNI_OK;
}

// ---- embedding (ops/embedding.rs) ------------------------------------------------------------------
static uint32_t embedding_common(uint32_t weight, std::shared_ptr<void> idx, int64_t batch, int64_t seq_len) {
    Tensor *W = get(weight);
    if (!W) return MNI_BAD_ID;
    const int64_t dim = W->shape[1], tokens = batch * seq_len;
    BufP w = contiguous_buf(*W);
    BufP out = w ? new_buf((size_t)(tokens * dim)) : nullptr;
    if (!out) return MNI_BAD_ID;
    if (k_embedding_forward(out->p, w->p, (const int32_t *)idx.get(), tokens, dim) != MNI_OK) return MNI_BAD_ID;
    const uint32_t id = insert_contig(std::move(out), Shape{batch, seq_len, dim});
    Entry e;
    e.op = OP_EMBEDDING; e.output_id = id; e.n_inputs = 1; e.inputs[0] = weight;
    e.targets = std::move(idx); e.ce_n = tokens;
    eng().tape.record(std::move(e));
    return id;
}
static bool embedding_check(uint32_t weight, int64_t batch, int64_t seq_len, int64_t have, int64_t lo, int64_t hi) {
    Tensor *W = get(weight);
    if (!W) return false;
    if (W->shape.size() != 2) { set_error(MNI_ERR_INVALID, "embedding: weight must be [vocab, dim]"); return false; }
    if (batch < 0 || seq_len < 0 || batch * seq_len > have) {
        set_error(MNI_ERR_INVALID, "embedding: %lld indices for batch %lld x seq_len %lld", (long long)have, (long long)batch,
                  (long long)seq_len);
        return false;
    }
    if (batch * seq_len > 0 && (lo < 0 || hi >= W->shape[0])) {
        set_error(MNI_ERR_INVALID, "embedding: index %lld out of range for %lld rows", (long long)(lo < 0 ? lo : hi),
                  (long long)W->shape[0]);
        return false;
    }
    return true;
}
static uint32_t embedding_forward(uint32_t weight, const int64_t *indices, size_t n, int64_t batch, int64_t seq_len) {
    const int64_t tokens = batch * seq_len;
    int64_t lo = 0, hi = 0;
    if (batch >= 0 && seq_len >= 0 && tokens <= (int64_t)n && tokens > 0) {
        lo = hi = indices[0];
        for (int64_t i = 1; i < tokens; ++i) {
            if (indices[i] < lo) lo = indices[i];
            if (indices[i] > hi) hi = indices[i];
        }
    }
    if (!embedding_check(weight, batch, seq_len, (int64_t)n, lo, hi)) return MNI_BAD_ID;
    std::vector<int32_t> i32((size_t)tokens);
    for (int64_t i = 0; i < tokens; ++i) i32[(size_t)i] = (int32_t)indices[i];
    std::shared_ptr<void> dev = dev_ints((size_t)tokens);
    if (!dev) return MNI_BAD_ID;
    if (tokens && upload_small(dev.get(), i32.data(), (size_t)tokens * sizeof(int32_t)) != MNI_OK) return MNI_BAD_ID;
    return embedding_common(weight, std::move(dev), batch, seq_len);
}
static uint32_t embedding_forward_gpu(uint32_t weight, uint32_t int_buf, int64_t batch, int64_t seq_len) {
    IntBuf *b = get_int(int_buf);
    if (!b) return MNI_BAD_ID;
    if (!embedding_check(weight, batch, seq_len, b->len, b->lo, b->hi)) return MNI_BAD_ID;
    return embedding_common(weight, b->data, batch, seq_len);
}
static int embedding_backward(uint32_t grad, const Entry &e, int64_t *out) {  // embedding.rs:104-128
    Tensor *W = get(e.inputs[0]), *G = get(grad);
    if (!W || !G) return MNI_ERR_FREED;
    const Shape wshape = W->shape;
    const int64_t vocab = wshape[0], dim = wshape[1], tokens = e.ce_n;
    if (G->size < tokens * dim) return set_error(MNI_ERR_INVALID, "embedding backward: gradient smaller than the output");
    BufP g = contiguous_buf(*G);
    BufP dw = g ? new_buf((size_t)(vocab * dim)) : nullptr;
    std::shared_ptr<void> work = dw ? dev_ints((size_t)(3 * vocab + 2 + 2 * tokens)) : nullptr;
    if (!work) return MNI_ERR_NOMEM;
    MNI_TRY(k_embedding_backward(dw->p, g->p, (const int32_t *)e.targets.get(), tokens, vocab, dim, (int32_t *)work.get()));
    out[0] = insert_contig(std::move(dw), wshape);
    return MNI_OK;
}

// lib.rs:679-691 + ops/loss.rs:190-229: cross-entropy with the targets in an
// integer buffer; the logits are viewed as [rows, classes] first (a View entry
// on the tape, like the reference).
static uint32_t cross_entropy_gpu_op(uint32_t logits, uint32_t int_buf) {
    Tensor *L = get(logits);
    IntBuf *T = get_int(int_buf);
    if (!L || !T) return MNI_BAD_ID;
    if (L->shape.empty()) { set_error(MNI_ERR_INVALID, "cross_entropy: scalar logits"); return MNI_BAD_ID; }
    const int64_t v = L->shape.back();
    const int64_t n = v ? L->size / v : 0;
    if (n <= 0 || v <= 0) { set_error(MNI_ERR_INVALID, "cross_entropy: empty logits"); return MNI_BAD_ID; }
    if (T->len < n) { set_error(MNI_ERR_INVALID, "cross_entropy: %lld targets for %lld rows", (long long)T->len, (long long)n); return MNI_BAD_ID; }
    if (T->lo < 0 || T->hi >= v) {
        set_error(MNI_ERR_INVALID, "cross_entropy: target %lld out of range [0, %lld)", (long long)(T->lo < 0 ? T->lo : T->hi), (long long)v);
        return MNI_BAD_ID;
    }
    const std::shared_ptr<void> tdev = T->data;
    const uint32_t flat = view_op(logits, Shape{n, v});
    if (flat == MNI_BAD_ID) return MNI_BAD_ID;
    Tensor *F = get(flat);
    BufP x = contiguous_buf(*F);
    BufP sm = x ? new_buf((size_t)(n * v)) : nullptr;
    BufP loss = sm ? new_buf(1) : nullptr;
    if (!loss) return MNI_BAD_ID;
    if (k_cross_entropy(loss->p, sm->p, x->p, (int32_t *)tdev.get(), nullptr, n, v) != MNI_OK) return MNI_BAD_ID;
    const uint32_t loss_id = insert_contig(std::move(loss), Shape{1});
    const uint32_t sm_id = insert_contig(std::move(sm), Shape{n, v});
    Entry e;
    e.op = OP_CROSSENTROPY; e.output_id = loss_id; e.n_inputs = 1; e.inputs[0] = flat;
    e.aux = sm_id; e.targets = tdev; e.ce_n = n; e.ce_v = v;
    eng().tape.record(std::move(e));
    return loss_id;
}

// ---- tile (ops/pooling.rs:276-309; not recorded on the tape there either) ----------------------------
static uint32_t tile_op(uint32_t a, const int64_t *reps, int n) {
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    const int nd = (int)A->shape.size();
    if (n != nd) { set_error(MNI_ERR_INVALID, "tile: reps must match tensor dimensions"); return MNI_BAD_ID; }
    if (nd < 1) { set_error(MNI_ERR_INVALID, "tile: the tensor must have at least one dim"); return MNI_BAD_ID; }
    const Shape shape = A->shape;
    Shape out_shape(nd);
    for (int i = 0; i < nd; ++i) {
        if (reps[i] < 0) { set_error(MNI_ERR_INVALID, "tile: negative repeat count"); return MNI_BAD_ID; }
        out_shape[i] = shape[i] * reps[i];
    }
    BufP src = contiguous_buf(*A);
    BufP out = src ? new_buf((size_t)shape_size(out_shape)) : nullptr;
    if (!out || k_tile(out->p, src->p, shape.data(), reps, nd) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(out), out_shape);
}

// ---- residual + layernorm (ops/fused.rs:23-78, 134-186) ----------------------------------------------
static uint32_t residual_layernorm_op(uint32_t x, uint32_t residual, uint32_t gamma, uint32_t beta, float eps) {
    Tensor *X = get(x), *R = get(residual), *Gm = get(gamma), *Bt = get(beta);
    if (!X || !R || !Gm || !Bt) return MNI_BAD_ID;
    if (X->shape.empty()) { set_error(MNI_ERR_INVALID, "residual_layernorm: x must have at least one dim"); return MNI_BAD_ID; }
    const Shape shape = X->shape;
    const int64_t c = shape.back(), rows = c ? X->size / c : 0;
    if (R->size < X->size) { set_error(MNI_ERR_INVALID, "residual_layernorm: residual holds fewer values than x"); return MNI_BAD_ID; }
    if (Gm->size < c || Bt->size < c) { set_error(MNI_ERR_INVALID, "residual_layernorm: gamma / beta hold fewer than %lld values", (long long)c); return MNI_BAD_ID; }
    BufP xs = contiguous_buf(*X), rs = contiguous_buf(*R), gs = contiguous_buf(*Gm), bs = contiguous_buf(*Bt);
    BufP out = (xs && rs && gs && bs) ? new_buf((size_t)X->size) : nullptr;
    BufP res = out ? new_buf((size_t)X->size) : nullptr;
    BufP mean = res ? new_buf((size_t)rows) : nullptr, rstd = mean ? new_buf((size_t)rows) : nullptr;
    if (!rstd || k_residual_layernorm(out->p, res->p, mean->p, rstd->p, xs->p, rs->p, gs->p, bs->p, rows, c, eps) != MNI_OK)
        return MNI_BAD_ID;
    // ids are handed out in the reference's order: res, mean, rstd, out
    const uint32_t res_id = insert_contig(std::move(res), shape);
    const uint32_t mean_id = insert_contig(std::move(mean), Shape{rows});
    const uint32_t rstd_id = insert_contig(std::move(rstd), Shape{rows});
    const uint32_t out_id = insert_contig(std::move(out), shape);
    Entry e;
    e.op = OP_RESIDUALLAYERNORM; e.output_id = out_id; e.n_inputs = 4;
    e.inputs[0] = x; e.inputs[1] = residual; e.inputs[2] = gamma; e.inputs[3] = beta;
    e.aux = mean_id; e.aux2 = rstd_id; e.aux3 = res_id;
    eng().tape.record(std::move(e));
    return out_id;
}
// The same tensor is returned for x and for the residual, as the reference does.
static int residual_layernorm_backward(uint32_t grad, const Entry &e, int64_t *out) {
    Tensor *S = get(e.aux3), *Gm = get(e.inputs[2]), *Mn = get(e.aux), *Rs = get(e.aux2), *G = get(grad);
    if (!S || !Gm || !Mn || !Rs || !G) return MNI_ERR_FREED;
    const Shape shape = S->shape, gshape = Gm->shape;
    const int64_t c = shape.back(), rows = c ? S->size / c : 0;
    BufP gs = contiguous_buf(*Gm), g = contiguous_buf(*G);
    BufP dx = (gs && g) ? new_buf((size_t)S->size) : nullptr;
    BufP dgamma = dx ? new_buf((size_t)Gm->size) : nullptr, dbeta = dgamma ? new_buf((size_t)Gm->size) : nullptr;
    if (!dbeta) return MNI_ERR_NOMEM;
    if (Gm->size > c) { MNI_TRY(k_fill(dgamma->p, 0.0f, Gm->size)); MNI_TRY(k_fill(dbeta->p, 0.0f, Gm->size)); }
    MNI_TRY(k_layernorm_backward(dx->p, dgamma->p, dbeta->p, g->p, S->buf->p, gs->p, Mn->buf->p, Rs->buf->p, rows, c));
    out[0] = out[1] = insert_contig(std::move(dx), shape);
    out[2] = insert_contig(std::move(dgamma), gshape);
    out[3] = insert_contig(std::move(dbeta), gshape);
    return MNI_OK;
}

// ops/mixed_precision.rs:17-32: grads *= inv_scale, true when any scaled value is inf or NaN
static int scale_grads_checked(const uint32_t *ids, size_t n, float inv_scale, int *found) {
    BufP flag = new_buf(1);
    if (!flag) return MNI_ERR_NOMEM;
    MNI_TRY(k_fill(flag->p, 0.0f, 1));
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (!T) return MNI_ERR_FREED;
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!G) return MNI_ERR_FREED;
        MNI_TRY(make_unique(*G));
        MNI_TRY(k_scale_check(G->buf->p, inv_scale, (int64_t)G->buf->n, flag->p));
    }
    float f = 0.f;
    MNI_TRY(mni_rocm_d2h(&f, flag->p, sizeof(float)));
    *found = f != 0.0f;
    return MNI_OK;
}

// ---- backward --------------------------------------------------------------------------------
static int dispatch_backward(const Entry &e, uint32_t grad, int64_t *out) {  // autograd.rs:180-222
    out[0] = out[1] = out[2] = out[3] = -1;
    switch (e.op) {
    case OP_ADD: return addsub_backward(grad, e, out, false);
    case OP_SUB: return addsub_backward(grad, e, out, true);
    case OP_MUL: return mul_backward(grad, e, out);
    case OP_NEG: case OP_MULSCALAR: case OP_RELU: case OP_GELU: return unary_backward(grad, e, out);
    case OP_MATMUL: return matmul_backward(grad, e, out);
    case OP_SUM: return reduce_backward(grad, e, out, false);
    case OP_MEAN: return reduce_backward(grad, e, out, true);
    case OP_VIEW: return view_backward(grad, e, out);
    case OP_PERMUTE: return permute_backward(grad, e, out);
    case OP_CONTIGUOUS: out[0] = grad; return MNI_OK;  // layout.rs:229-231
    case OP_CROSSENTROPY: return cross_entropy_backward(grad, e, out);
    case OP_LINEAR: return linear_backward(grad, e, out);
    case OP_EXP: case OP_LOG: case OP_SIGMOID: case OP_POW: return unary2_backward(grad, e, out);
    case OP_DIV: return div_backward(grad, e, out);
    case OP_MAX: return max_backward(grad, e, out);
    case OP_LAYERNORM: return layernorm_backward(grad, e, out);
    case OP_BIASGELU: return bias_gelu_backward(grad, e, out);               // autograd.rs BiasGelu
    case OP_SOFTMAX: return softmax_backward(grad, e, out);                  // autograd.rs:204
    case OP_FLASHATTENTION: return flash_attention_backward(grad, e, out);   // autograd.rs:210
    case OP_EMBEDDING: return embedding_backward(grad, e, out);
    case OP_DROPOUT: return dropout_backward(grad, e, out);
    case OP_RESIDUALLAYERNORM: return residual_layernorm_backward(grad, e, out);
    case OP_MSEROWS: return mse_rows_backward(grad, e, out);
    }
    return set_error(MNI_ERR_INVALID, "unknown tape op %d", e.op);
}

// autograd.rs:96-171 Tape::backward
static int tape_backward(Tape &tp, uint32_t loss) {
    if (!get(loss)) return MNI_ERR_FREED;
    const size_t nslots = eng().tensors.size() + 1;
    std::vector<int64_t> out2entry(nslots, -1);
    for (size_t i = 0; i < tp.entries.size(); ++i)
        if (tp.entries[i].output_id < nslots) out2entry[tp.entries[i].output_id] = (int64_t)i;  // later entry wins

    std::vector<char> relevant(nslots, 0), visited(nslots, 0);
    {
        std::vector<uint32_t> stack{loss};
        while (!stack.empty()) {
            const uint32_t tid = stack.back();
            stack.pop_back();
            if (tid >= nslots || relevant[tid]) continue;
            relevant[tid] = 1;
            const int64_t idx = out2entry[tid];
            if (idx >= 0)
                for (int i = 0; i < tp.entries[idx].n_inputs; ++i) stack.push_back(tp.entries[idx].inputs[i]);
        }
    }
    // Post-order DFS, inputs in order (autograd.rs:120-137), without recursion.
    std::vector<uint32_t> order;
    {
        struct Frame { uint32_t tid; int next; };
        std::vector<Frame> st;
        visited[loss] = 1;
        st.push_back({loss, 0});
        while (!st.empty()) {
            Frame &f = st.back();
            const int64_t idx = out2entry[f.tid];
            bool pushed = false;
            if (idx >= 0) {
                const Entry &en = tp.entries[idx];
                while (f.next < en.n_inputs) {
                    const uint32_t inp = en.inputs[f.next++];
                    if (inp < nslots && relevant[inp] && !visited[inp]) {
                        visited[inp] = 1;
                        st.push_back({inp, 0});
                        pushed = true;
                        break;
                    }
                }
            }
            if (!pushed) {
                order.push_back(st.back().tid);
                st.pop_back();
            }
        }
    }
    // how many entries read each tensor (what the fused Linear's backward needs to know, see linear_backward)
    std::vector<int> consumers(nslots, 0);
    for (const Entry &en : tp.entries)
        if (en.output_id < nslots && relevant[en.output_id])
            for (int i = 0; i < en.n_inputs; ++i)
                if (en.inputs[i] < nslots) ++consumers[en.inputs[i]];
    std::vector<int64_t> grads(nslots, -1);
    struct WalkScope {  // publishes the walk to the ops for the duration of this call
        Engine &e;
        WalkScope(Engine &e_, const Tape *t, const std::vector<int64_t> *o, const std::vector<int> *c, const std::vector<int64_t> *g) : e(e_) {
            e.bw_tape = t; e.bw_out2entry = o; e.bw_consumers = c; e.bw_grads = g;
        }
        ~WalkScope() {
            e.bw_tape = nullptr; e.bw_out2entry = nullptr; e.bw_consumers = nullptr; e.bw_grads = nullptr;
            e.preact_strips.clear();  // (none are left when the walk completed)
        }
    } walk_scope(eng(), &tp, &out2entry, &consumers, &grads);
    {
        const Shape shape = get(loss)->shape;
        uint32_t g;  // ones_like for any loss shape, autograd.rs:143
        if (shape_size(shape) == 1) {
            Engine &e = eng();
            if (!e.one) {
                e.one = new_buf(1);
                if (!e.one) return MNI_ERR_NOMEM;
                if (k_fill(e.one->p, 1.0f, 1) != MNI_OK) { e.one = nullptr; return MNI_ERR_HIP; }
            }
            g = insert_contig(BufP(e.one), shape);
        } else if (shape_size(shape) <= (1 << 20)) {
            Engine &e = eng();
            const int64_t n = shape_size(shape);
            if (!e.ones || e.ones_n != n) {
                e.ones = new_buf((size_t)n);
                e.ones_n = n;
                if (!e.ones) { e.ones_n = 0; return MNI_ERR_NOMEM; }
                if (k_fill(e.ones->p, 1.0f, n) != MNI_OK) { e.ones = nullptr; e.ones_n = 0; return MNI_ERR_HIP; }
            }
            g = insert_contig(BufP(e.ones), shape);
        } else {
            g = filled(shape, 1.0f);
        }
        if (g == MNI_BAD_ID) return MNI_ERR_NOMEM;
        grads[loss] = g;
    }
    for (size_t oi = order.size(); oi-- > 0;) {
        const uint32_t tid = order[oi];
        if (grads[tid] < 0) continue;
        const int64_t idx = out2entry[tid];
        if (idx < 0) continue;
        const Entry &en = tp.entries[idx];
        int64_t ig[4];
        MNI_TRY(dispatch_backward(en, (uint32_t)grads[tid], ig));
        for (int i = 0; i < en.n_inputs; ++i) {
            if (ig[i] < 0) continue;
            const uint32_t inp = en.inputs[i];
            Tensor *T = get(inp);
            if (!T) return MNI_ERR_FREED;
            if (T->requires_grad) {
                const int64_t gid = ensure_grad(inp);
                if (gid < 0) return MNI_ERR_NOMEM;
                MNI_TRY(add_into((uint32_t)gid, (uint32_t)ig[i]));
            }
            if (grads[inp] >= 0) MNI_TRY(add_into((uint32_t)grads[inp], (uint32_t)ig[i]));
            else grads[inp] = ig[i];
        }
    }
    return MNI_OK;
}

// ---- optimiser ------------------------------------------------------------------------------------
static float powi_f32(float a, int b) {  // f32::powi (compiler-rt __powisf2)
    const bool recip = b < 0;
    float r = 1.0f;
    while (true) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0f / r : r;
}

// ops/optimizer.rs:126-138 grad_norm
// before_read: issued after the norm's kernels and before the host waits for the value (work that does not
// depend on it then runs while the copy is in flight).
static int grad_norm(const uint32_t *ids, size_t n, float *out, const std::function<int()> &before_read = nullptr) {
    // Workgroups of multi-tensor launches leave one partial sum each in one
    // buffer; a single kernel adds them up.
    std::vector<Tensor *> gs;
    int64_t nparts = 0;
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (!T) return MNI_ERR_FREED;
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!G) return MNI_ERR_FREED;
        if (G->size <= 0) continue;
        gs.push_back(G);
        nparts += multi_tensor_blocks(G->size);
    }
    if (nparts == 0) {  // no gradients
        if (before_read) MNI_TRY(before_read());
        *out = 0.0f;
        return MNI_OK;
    }
    void *acc = nullptr;
    MNI_TRY(dev_alloc(&acc, (size_t)(nparts + 1) * sizeof(double)));
    std::shared_ptr<void> guard(acc, [](void *p) { dev_free(p); });
    double *total = (double *)acc, *part = total + 1;
    // The sum also goes, as a float, to a word of pinned host memory: the host then has it a few microseconds
    // after the kernel that wrote it, with no copy to order and no wait for what was queued behind it.
    const unsigned tag = next_result_tag();
    unsigned long long *word = ctx().result_dev;
    const bool solo = gs.size() <= (size_t)MULTI_MAX && nparts <= SUMSQ_SOLO_BLOCKS;
    int64_t at = 0;
    for (size_t first = 0; first < gs.size(); first += MULTI_MAX) {
        MultiTensor t;
        memset(&t, 0, sizeof t);
        t.count = (int)std::min<size_t>(MULTI_MAX, gs.size() - first);
        int blocks = 0;
        for (int i = 0; i < t.count; ++i) {
            Tensor *G = gs[first + i];
            t.block_start[i] = blocks;
            t.g[i] = G->buf->p;
            t.n[i] = G->size;
            blocks += multi_tensor_blocks(G->size);
        }
        t.block_start[t.count] = blocks;
        if (solo) MNI_TRY(k_sumsq_solo(t, total, word, tag));  // a small model: partial sums and their sum in one launch
        else MNI_TRY(k_sumsq_multi(t, part + at));
        at += blocks;
    }
    if (!solo) MNI_TRY(k_sumsq_finish(total, part, (int)nparts, true, word, tag));
    if (before_read) MNI_TRY(before_read());
    unsigned bits = 0;
    bool delivered = false;
    MNI_TRY(wait_result_word(tag, &bits, &delivered));
    float sq;
    if (delivered) {
        memcpy(&sq, &bits, sizeof sq);
    } else {
        double sq64 = 0.0;
        MNI_TRY(mni_rocm_d2h(&sq64, total, sizeof(double)));
        sq = (float)sq64;
    }
    *out = sqrtf(sq);
    return MNI_OK;
}

// ops/optimizer.rs:21-65 adamw_step
static int adamw_step(const uint32_t *ids, size_t n, float lr, float b1, float b2, float eps, float wd, uint32_t step) {
    const float bc1 = 1.0f - powi_f32(b1, (int)step);
    const float bc2 = 1.0f - powi_f32(b2, (int)step);
    MultiTensor t;
    memset(&t, 0, sizeof t);
    std::vector<BufP> keep;  // gathered copies of non-contiguous gradients, alive until their launch is queued
    int blocks = 0;
    auto flush = [&]() -> int {
        if (t.count == 0) return MNI_OK;
        t.block_start[t.count] = blocks;
        const int rc = k_adamw_multi(t, lr, b1, b2, eps, wd, bc1, bc2);
        memset(&t, 0, sizeof t);
        blocks = 0;
        keep.clear();
        return rc;
    };
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (!T) return MNI_ERR_FREED;
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!G) return MNI_ERR_FREED;
        BufP g = contiguous_buf(*G);
        if (!g) return MNI_ERR_NOMEM;
        const int64_t size = T->size;
        if (size <= 0) continue;
        if ((int64_t)g->n < size) return set_error(MNI_ERR_INVALID, "adamw: gradient smaller than its parameter");
        if (!T->adam_m) {
            T->adam_m = new_buf((size_t)size);
            T->adam_v = new_buf((size_t)size);
            if (!T->adam_m || !T->adam_v) return MNI_ERR_NOMEM;
            MNI_TRY(k_fill(T->adam_m->p, 0.f, size));
            MNI_TRY(k_fill(T->adam_v->p, 0.f, size));
        }
        MNI_TRY(make_unique(*T));
        // the same parameter twice in one list must see its first update: start a new launch
        bool repeated = false;
        for (int i = 0; i < t.count; ++i) repeated = repeated || t.p[i] == T->buf->p;
        if (repeated || t.count == MULTI_MAX) MNI_TRY(flush());
        const int i = t.count++;
        t.block_start[i] = blocks;
        t.p[i] = T->buf->p; t.m[i] = T->adam_m->p; t.v[i] = T->adam_v->p; t.g[i] = g->p; t.n[i] = size;
        blocks += multi_tensor_blocks(size);
        keep.push_back(std::move(g));
    }
    return flush();
}

// A model of a few thousand parameters: gradient norm, clipping and the AdamW update of clip_and_step
// (ops/optimizer.rs:224-245) as one launch of one workgroup.  *handled = false when the parameter list is not of that
// kind (nothing has been launched then).  Same sums and the same update arithmetic as the separate launches.
static int clip_and_step_solo(const uint32_t *ids, size_t n, float lr, float b1, float b2, float eps, float wd, uint32_t step, float max_norm,
                              float *norm_out, bool *handled) {
    *handled = false;
    if (n == 0 || n > (size_t)MULTI_MAX) return MNI_OK;
    MultiTensor t;
    memset(&t, 0, sizeof t);
    int blocks = 0;
    int64_t total = 0;
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (!T) return MNI_ERR_FREED;
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!G) return MNI_ERR_FREED;
        if (T->size <= 0 || G->size != T->size || !is_contiguous(*G) || !G->buf || (int64_t)G->buf->n != G->size) return MNI_OK;
        for (int i = 0; i < t.count; ++i)
            if (t.p[i] == T->buf->p) return MNI_OK;  // (the same parameter twice must see its first update)
        total += T->size;
        blocks += multi_tensor_blocks(T->size);
        if (total > 8192 || blocks > SUMSQ_SOLO_BLOCKS) return MNI_OK;
        ++t.count;
    }
    if (t.count == 0) return MNI_OK;
    // second pass: buffers made private and moments created (launches of their own only on the first step)
    t.count = 0;
    blocks = 0;
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!T->adam_m) {
            T->adam_m = new_buf((size_t)T->size);
            T->adam_v = new_buf((size_t)T->size);
            if (!T->adam_m || !T->adam_v) return MNI_ERR_NOMEM;
            MNI_TRY(k_fill(T->adam_m->p, 0.f, T->size));
            MNI_TRY(k_fill(T->adam_v->p, 0.f, T->size));
        }
        MNI_TRY(make_unique(*T));
        if (max_norm > 0.0f) MNI_TRY(make_unique(*G));  // (clipping scales the gradient in place)
        const int i = t.count++;
        t.block_start[i] = blocks;
        t.p[i] = T->buf->p; t.m[i] = T->adam_m->p; t.v[i] = T->adam_v->p; t.g[i] = G->buf->p; t.n[i] = T->size;
        blocks += multi_tensor_blocks(T->size);
    }
    t.block_start[t.count] = blocks;
    void *acc = nullptr;
    MNI_TRY(dev_alloc(&acc, sizeof(double)));
    std::shared_ptr<void> guard(acc, [](void *q) { dev_free(q); });
    const unsigned tag = next_result_tag();
    const float bc1 = 1.0f - powi_f32(b1, (int)step), bc2 = 1.0f - powi_f32(b2, (int)step);
    MNI_TRY(k_clip_and_step_solo(t, (double *)acc, ctx().result_dev, tag, max_norm, lr, b1, b2, eps, wd, bc1, bc2));
    *handled = true;
    unsigned bits = 0;
    bool delivered = false;
    MNI_TRY(wait_result_word(tag, &bits, &delivered));
    float sq;
    if (delivered) {
        memcpy(&sq, &bits, sizeof sq);
    } else {
        double sq64 = 0.0;
        MNI_TRY(mni_rocm_d2h(&sq64, acc, sizeof(double)));
        sq = (float)sq64;
    }
    *norm_out = sqrtf(sq);
    return MNI_OK;
}

static int scale_grads(const uint32_t *ids, size_t n, float scale) {
    for (size_t p = 0; p < n; ++p) {
        Tensor *T = get(ids[p]);
        if (!T) return MNI_ERR_FREED;
        if (T->grad < 0) continue;
        Tensor *G = get((uint32_t)T->grad);
        if (!G) return MNI_ERR_FREED;
        MNI_TRY(make_unique(*G));
        MNI_TRY(k_scale_inplace(G->buf->p, scale, (int64_t)G->buf->n));
    }
    return MNI_OK;
}

}  // namespace
}  // namespace mni

using namespace mni;

// ============================================================================
// Exported engine surface (one function per #[napi] export of lib.rs)
// ============================================================================
extern "C" {

uint32_t mni_zeros(const int64_t *shape, int ndim) {
    MNI_API_GUARD;
    Shape s;
    if (ensure_init() != MNI_OK || !to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    return zeros(s);
}
uint32_t mni_ones(const int64_t *shape, int ndim) {
    MNI_API_GUARD;
    Shape s;
    if (ensure_init() != MNI_OK || !to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    return filled(s, 1.0f);
}
uint32_t mni_from_float32(const float *data, size_t len, const int64_t *shape, int ndim) {
    MNI_API_GUARD;
    Shape s;
    if (ensure_init() != MNI_OK || !to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    const int64_t n = shape_size(s);
    if ((int64_t)len < n || (n > 0 && !data)) {
        set_error(MNI_ERR_INVALID, "from_float32: %zu values for shape of %lld elements", len, (long long)n);
        return MNI_BAD_ID;
    }
    BufP b = new_buf((size_t)n);
    if (!b || upload_small(b->p, data, (size_t)n * sizeof(float)) != MNI_OK) return MNI_BAD_ID;
    return insert_contig(std::move(b), s);
}
int mni_tensor_shape(uint32_t id, int64_t *out, int cap) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (!t) return -1;
    for (int i = 0; i < (int)t->shape.size() && i < cap; ++i) out[i] = t->shape[i];
    return (int)t->shape.size();
}
int64_t mni_tensor_size(uint32_t id) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    return t ? t->size : -1;
}
int mni_to_float32(uint32_t id, float *out, size_t cap) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (!t) return MNI_ERR_FREED;
    if ((int64_t)cap < t->size) return set_error(MNI_ERR_INVALID, "to_float32: buffer of %zu for %lld elements", cap, (long long)t->size);
    BufP b = contiguous_buf(*t);
    if (!b) return MNI_ERR_NOMEM;
    return mni_rocm_d2h(out, b->p, (size_t)t->size * sizeof(float));
}
int mni_get_scalar(uint32_t id, double *out) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (!t) return MNI_ERR_FREED;
    float v = 0.f;
    MNI_TRY(mni_rocm_d2h(&v, t->buf->p, sizeof(float)));
    *out = (double)v;
    return MNI_OK;
}
void mni_free_tensor(uint32_t id) { MNI_API_GUARD; free_tensor(id); }
int mni_set_requires_grad(uint32_t id, int requires_) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (!t) return MNI_ERR_FREED;
    t->requires_grad = requires_ != 0;
    return MNI_OK;
}
int mni_get_grad(uint32_t id, uint32_t *out) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (!t) return -1;
    if (t->grad < 0) return 0;
    if (out) *out = (uint32_t)t->grad;
    return 1;
}
int mni_backward(uint32_t loss) {
    MNI_API_GUARD;
    // The tape is consumed and replaced by a fresh, enabled one (lib.rs:135).
    Tape old = std::move(eng().tape);
    eng().tape = Tape();
    return tape_backward(old, loss);
}
int mni_zero_grad(const uint32_t *ids, size_t n) {
    MNI_API_GUARD;
    for (size_t p = 0; p < n; ++p) {
        Tensor *t = get(ids[p]);
        if (!t) return MNI_ERR_FREED;
        if (t->grad < 0) continue;
        Tensor *g = peek((uint32_t)t->grad);
        if (!g) return MNI_ERR_FREED;
        if (g->known_zero) continue;
        if (g->buf.use_count() > 1) {  // shared: replace instead of copy + clear
            g->buf = new_buf(g->buf->n);
            if (!g->buf) return MNI_ERR_NOMEM;
        }
        g->known_zero = true;  // the zeros are written when somebody asks for them
        g->zero_filled = false;
    }
    return MNI_OK;
}
void mni_no_grad_start(void) { MNI_API_GUARD; eng().tape.enabled = false; }
void mni_no_grad_end(void) { MNI_API_GUARD; eng().tape.enabled = true; }

uint32_t mni_add(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_ADD); }
uint32_t mni_mul(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_MUL); }
uint32_t mni_sub(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_SUB); }
uint32_t mni_neg(uint32_t a) { MNI_API_GUARD; return unary_op(a, UN_NEG, OP_NEG, 0.f); }
uint32_t mni_mul_scalar(uint32_t a, double s) { MNI_API_GUARD; return unary_op(a, UN_SCALE, OP_MULSCALAR, (float)s); }
uint32_t mni_gelu(uint32_t a) { MNI_API_GUARD; return unary_op(a, UN_GELU, OP_GELU, 0.f); }
uint32_t mni_relu(uint32_t a) { MNI_API_GUARD; return unary_op(a, UN_RELU, OP_RELU, 0.f); }

uint32_t mni_matmul(uint32_t a, uint32_t b) {
    MNI_API_GUARD;
    const uint32_t out = matmul_tensors(a, false, b, false, nullptr, MNI_EPI_NONE);
    if (out == MNI_BAD_ID) return out;
    Entry e;
    e.op = OP_MATMUL; e.output_id = out; e.n_inputs = 2; e.inputs[0] = a; e.inputs[1] = b;
    eng().tape.record(std::move(e));
    return out;
}
uint32_t mni_linear(uint32_t x, uint32_t w, uint32_t bias, int act) { MNI_API_GUARD; return linear_op(x, w, bias, act); }
uint32_t mni_mse_loss(uint32_t pred, uint32_t target) { MNI_API_GUARD; return mse_rows_op(pred, target); }

uint32_t mni_sum_op(uint32_t a, int64_t dim) { MNI_API_GUARD; return reduce_op(a, dim, false); }
uint32_t mni_mean_op(uint32_t a, int64_t dim) { MNI_API_GUARD; return reduce_op(a, dim, true); }
uint32_t mni_sum_all(uint32_t a) {
    MNI_API_GUARD;
    Tensor *t = get(a);
    if (!t) return MNI_BAD_ID;
    uint32_t cur = a;
    for (int d = (int)t->shape.size() - 1; d >= 0 && cur != MNI_BAD_ID; --d) cur = reduce_op(cur, d, false);
    return cur;
}
uint32_t mni_mean_all(uint32_t a) {
    MNI_API_GUARD;
    Tensor *t = get(a);
    if (!t) return MNI_BAD_ID;
    uint32_t cur = a;
    for (int d = (int)t->shape.size() - 1; d >= 0 && cur != MNI_BAD_ID; --d) cur = reduce_op(cur, d, true);
    return cur;
}
uint32_t mni_view(uint32_t a, const int64_t *shape, int ndim) {
    MNI_API_GUARD;
    Shape s;
    if (!to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    return view_op(a, s);
}
uint32_t mni_permute(uint32_t a, const int64_t *dims, int ndim) {
    MNI_API_GUARD;
    Shape s;
    if (!to_shape(dims, ndim, &s)) return MNI_BAD_ID;
    return permute_op(a, s);
}
uint32_t mni_contiguous(uint32_t a) {  // layout.rs:218-227
    MNI_API_GUARD;
    Tensor *A = get(a);
    if (!A) return MNI_BAD_ID;
    if (is_contiguous(*A)) return a;
    BufP b = contiguous_buf(*A);
    if (!b) return MNI_BAD_ID;
    const Shape shape = A->shape;
    const uint32_t id = insert_contig(std::move(b), shape);
    Entry e;
    e.op = OP_CONTIGUOUS; e.output_id = id; e.n_inputs = 1; e.inputs[0] = a;
    eng().tape.record(std::move(e));
    return id;
}
uint32_t mni_exp_op(uint32_t a) { MNI_API_GUARD; return unary2_op(a, UN_EXP, OP_EXP, 0.f); }
uint32_t mni_log_op(uint32_t a) { MNI_API_GUARD; return unary2_op(a, UN_LOG, OP_LOG, 0.f); }
uint32_t mni_sigmoid(uint32_t a) { MNI_API_GUARD; return unary2_op(a, UN_SIGMOID, OP_SIGMOID, 0.f); }
uint32_t mni_pow_op(uint32_t a, double exponent) { MNI_API_GUARD; return unary2_op(a, UN_POW, OP_POW, (float)exponent); }
uint32_t mni_div(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_DIV); }
uint32_t mni_lt(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_LT); }
uint32_t mni_eq_op(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_EQ); }
uint32_t mni_gt(uint32_t a, uint32_t b) { MNI_API_GUARD; return binary_op(a, b, BIN_GT); }
uint32_t mni_is_close(uint32_t a, uint32_t b, double tol) { MNI_API_GUARD; return binary_op(a, b, BIN_CLOSE, (float)tol); }
uint32_t mni_max_op(uint32_t a, int64_t dim) { MNI_API_GUARD; return max_op(a, dim); }
uint32_t mni_layernorm_op(uint32_t x, uint32_t gamma, uint32_t beta, double eps) {
    MNI_API_GUARD;
    return layernorm_op(x, gamma, beta, (float)eps);
}
uint32_t mni_kv_cache_create(int64_t batch_size, int64_t num_heads, int64_t head_dim, int64_t max_seq_len, int quantized) {
    MNI_API_GUARD;
    if (ensure_init() != MNI_OK) return MNI_BAD_ID;
    return kv_cache_create(batch_size, num_heads, head_dim, max_seq_len, quantized != 0);
}
int64_t mni_kv_cache_len(uint32_t cache_id) {
    MNI_API_GUARD;
    auto it = eng().kv_caches.find(cache_id);
    return it == eng().kv_caches.end() ? 0 : it->second.len;
}
int mni_kv_cache_quantized(uint32_t cache_id) {
    MNI_API_GUARD;
    auto it = eng().kv_caches.find(cache_id);
    return it != eng().kv_caches.end() && it->second.quantized ? 1 : 0;
}
void mni_kv_cache_reset(uint32_t cache_id) {
    MNI_API_GUARD;
    auto it = eng().kv_caches.find(cache_id);
    if (it != eng().kv_caches.end()) it->second.len = 0;  // positions past len are never read
}
void mni_kv_cache_free(uint32_t cache_id) { MNI_API_GUARD; eng().kv_caches.erase(cache_id); }
int mni_kv_cache_append(uint32_t cache_id, uint32_t k, uint32_t v) { MNI_API_GUARD; return kv_cache_append(cache_id, k, v); }
uint32_t mni_kv_cache_decode_step(uint32_t cache_id, uint32_t q, uint32_t k, uint32_t v, double scale) {
    MNI_API_GUARD;
    return kv_cache_decode_step(cache_id, q, k, v, (float)scale);
}
uint32_t mni_bias_gelu(uint32_t x, uint32_t bias) { MNI_API_GUARD; return bias_gelu_op(x, bias); }
uint32_t mni_softmax_op(uint32_t a, int64_t dim) { MNI_API_GUARD; return softmax_op(a, dim); }
uint32_t mni_flash_attention(uint32_t q, uint32_t k, uint32_t v, double scale, int causal) {
    MNI_API_GUARD;
    return flash_attention_op(q, k, v, (float)scale, causal != 0);
}
uint32_t mni_cross_entropy_loss(uint32_t logits, const int64_t *targets, size_t n) {
    MNI_API_GUARD;
    if (!targets) { set_error(MNI_ERR_INVALID, "cross_entropy: null targets"); return MNI_BAD_ID; }
    return cross_entropy_op(logits, targets, n);
}
int mni_adamw_step(const uint32_t *ids, size_t n, double lr, double beta1, double beta2, double eps,
                   double weight_decay, int64_t step) {
    MNI_API_GUARD;
    return adamw_step(ids, n, (float)lr, (float)beta1, (float)beta2, (float)eps, (float)weight_decay, (uint32_t)step);
}
double mni_grad_norm(const uint32_t *ids, size_t n) {
    MNI_API_GUARD;
    float norm = 0.f;
    if (grad_norm(ids, n, &norm) != MNI_OK) return -1.0;
    return (double)norm;
}
int mni_clip_grad_norm(const uint32_t *ids, size_t n, double max_norm) {  // optimizer.rs:160-173
    MNI_API_GUARD;
    float norm = 0.f;
    MNI_TRY(grad_norm(ids, n, &norm));
    const float mx = (float)max_norm;
    if (norm > mx) MNI_TRY(scale_grads(ids, n, mx / norm));
    return MNI_OK;
}
double mni_clip_and_step(const uint32_t *ids, size_t n, double lr, double beta1, double beta2, double eps,
                         double weight_decay, int64_t step, double max_grad_norm) {  // optimizer.rs:224-245
    MNI_API_GUARD;
    float norm = 0.f;
    const float mg = (float)max_grad_norm;
    {
        bool handled = false;
        if (clip_and_step_solo(ids, n, (float)lr, (float)beta1, (float)beta2, (float)eps, (float)weight_decay, (uint32_t)step, mg > 0.0f ? mg : 0.0f,
                               &norm, &handled) != MNI_OK)
            return -1.0;
        if (handled) return (double)norm;
    }
    auto update = [&] { return adamw_step(ids, n, (float)lr, (float)beta1, (float)beta2, (float)eps, (float)weight_decay, (uint32_t)step); };
    if (!(mg > 0.0f)) {
        // no clipping asked for: the update does not depend on the norm and is issued before the host waits for it
        if (grad_norm(ids, n, &norm, update) != MNI_OK) return -1.0;
        return (double)norm;
    }
    if (grad_norm(ids, n, &norm) != MNI_OK) return -1.0;
    if (norm > mg)
        if (scale_grads(ids, n, mg / norm) != MNI_OK) return -1.0;
    if (update() != MNI_OK) return -1.0;
    return (double)norm;
}
void mni_reset_engine(void) {
    MNI_API_GUARD;
    Engine &e = eng();
    e.tensors.clear();
    e.free_ids.clear();
    e.tape = Tape();
    e.kv_caches.clear();       // lib.rs:466-467
    e.next_kv_cache_id = 1;
    e.int_bufs.clear();        // lib.rs:465
    e.int_free.clear();
}
int mni_gc_tensors(const uint32_t *keep, size_t n) {
    MNI_API_GUARD;
    Engine &e = eng();
    const size_t len = e.tensors.size();
    std::vector<char> k(len + 1, 0);
    for (size_t i = 0; i < n; ++i)
        if (keep[i] < len) k[keep[i]] = 1;
    for (size_t id = 0; id < len; ++id)
        if (!k[id] && e.tensors[id].live) free_tensor((uint32_t)id);
    e.tape = Tape();
    // The reference drops its allocator cache here (lib.rs:704).  Blocks stay
    // cached for the next step unless the cache has grown large: returning
    // them to the driver every step would cost a device-wide sync per block.
    if (dev_cached_bytes() > ((size_t)64 << 30)) return dev_clear_cache();
    return MNI_OK;
}
// ---- token-side ops ------------------------------------------------------------------------
uint32_t mni_rand_tensor(const int64_t *shape, int ndim) {  // lib.rs:60-64
    MNI_API_GUARD;
    Shape s;
    if (ensure_init() != MNI_OK || !to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    return random_tensor(s, 0);
}
uint32_t mni_randn_tensor(const int64_t *shape, int ndim) {  // lib.rs:67-71
    MNI_API_GUARD;
    Shape s;
    if (ensure_init() != MNI_OK || !to_shape(shape, ndim, &s)) return MNI_BAD_ID;
    return random_tensor(s, 1);
}
int mni_seed(uint64_t seed) {
    MNI_API_GUARD;
    Engine &e = eng();
    e.rng_seed = seed;
    e.rng_offset = 0;
    e.host_rng.seed(seed);
    e.rng_ready = true;
    return MNI_OK;
}
int mni_philox_words(uint64_t seed, uint64_t offset, uint32_t *out, size_t n) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    BufP b = new_buf(n);
    if (!b) return MNI_ERR_NOMEM;
    MNI_TRY(k_random_fill(b->p, (int64_t)n, seed, offset, 2));
    return mni_rocm_d2h(out, b->p, n * sizeof(uint32_t));
}
uint32_t mni_dropout_op(uint32_t x, double rate, int training) {  // lib.rs:388-394
    MNI_API_GUARD;
    return dropout_op(x, (float)rate, training != 0);
}
uint32_t mni_create_dataset(const int32_t *data, size_t len) {  // lib.rs:476-479
    MNI_API_GUARD;
    if (ensure_init() != MNI_OK) return MNI_BAD_ID;
    if (len && !data) { set_error(MNI_ERR_INVALID, "create_dataset: null data"); return MNI_BAD_ID; }
    return create_dataset(data, len);
}
int mni_sample_batch(uint32_t dataset, int64_t block_size, int64_t batch_size, uint32_t *out_ids) {  // lib.rs:483-490
    MNI_API_GUARD;
    return sample_batch(dataset, block_size, batch_size, out_ids);
}
int mni_free_int_buffer(uint32_t id) {  // lib.rs:494-497, data.rs:53-56
    MNI_API_GUARD;
    Engine &e = eng();
    if (id >= e.int_bufs.size()) return set_error(MNI_ERR_INVALID, "int buffer id %u out of range", id);
    e.int_bufs[id] = IntBuf();
    e.int_free.push_back(id);
    return MNI_OK;
}
int64_t mni_int_buffer_len(uint32_t id) {
    MNI_API_GUARD;
    IntBuf *b = get_int(id);
    return b ? b->len : -1;
}
int mni_int_buffer_to_host(uint32_t id, int32_t *out, size_t cap) {
    MNI_API_GUARD;
    IntBuf *b = get_int(id);
    if (!b) return MNI_ERR_FREED;
    if ((int64_t)cap < b->len) return set_error(MNI_ERR_INVALID, "int_buffer_to_host: room for %zu of %lld values", cap, (long long)b->len);
    return b->len ? mni_rocm_d2h(out, b->data.get(), (size_t)b->len * sizeof(int32_t)) : MNI_OK;
}
uint32_t mni_embedding_forward(uint32_t weight, const int64_t *indices, size_t n, int64_t batch, int64_t seq_len) {  // lib.rs:319-326
    MNI_API_GUARD;
    if (n && !indices) { set_error(MNI_ERR_INVALID, "embedding: null indices"); return MNI_BAD_ID; }
    return embedding_forward(weight, indices, n, batch, seq_len);
}
uint32_t mni_embedding_forward_gpu(uint32_t weight, uint32_t int_buf, int64_t batch, int64_t seq_len) {  // lib.rs:501-511
    MNI_API_GUARD;
    return embedding_forward_gpu(weight, int_buf, batch, seq_len);
}
uint32_t mni_cross_entropy_loss_gpu(uint32_t logits, uint32_t int_buf) {  // lib.rs:679-691
    MNI_API_GUARD;
    return cross_entropy_gpu_op(logits, int_buf);
}
uint32_t mni_residual_layernorm(uint32_t x, uint32_t residual, uint32_t gamma, uint32_t beta, double eps) {  // lib.rs:515-523
    MNI_API_GUARD;
    return residual_layernorm_op(x, residual, gamma, beta, (float)eps);
}
int mni_scale_grads(const uint32_t *ids, size_t n, double inv_scale, int *found_inf) {  // lib.rs:450-454
    MNI_API_GUARD;
    int found = 0;
    MNI_TRY(scale_grads_checked(ids, n, (float)inv_scale, &found));
    if (found_inf) *found_inf = found;
    return MNI_OK;
}
uint32_t mni_tile(uint32_t input, const int64_t *reps, int n) {  // lib.rs:568-573
    MNI_API_GUARD;
    if (n > 0 && !reps) { set_error(MNI_ERR_INVALID, "tile: null reps"); return MNI_BAD_ID; }
    return tile_op(input, reps, n);
}

void *mni_dev_ptr(uint32_t id) {
    MNI_API_GUARD;
    Tensor *t = get(id);
    if (t) t->known_zero = false;  // the caller may write through the pointer
    return t ? (void *)t->buf->p : nullptr;
}

}  // extern "C"
