// Node-API addon over the engine-level C ABI of libmni_rocm.so.
//
// Exports the camelCase names that napi-derive generates for the reference's
// #[napi] functions (src/native/src/lib.rs), which is what src/tensor.ts,
// src/nn.ts and src/optimizer.ts call on their `native` object.  Every export
// only converts arguments and forwards ids; where the reference's Rust layer
// would panic, a JavaScript Error carrying mni_rocm_last_error() is thrown.
// Plain C Node-API (node_api.h), no node-addon-api, so it builds with g++ alone.
#include <node_api.h>
#include <stdint.h>
#include <stdlib.h>

#include <vector>

#include "../../include/mni_rocm.h"

namespace {

napi_value throw_last(napi_env env) {
    napi_throw_error(env, nullptr, mni_rocm_last_error());
    return nullptr;
}
napi_value undefined(napi_env env) {
    napi_value v;
    napi_get_undefined(env, &v);
    return v;
}
napi_value make_u32(napi_env env, uint32_t x) {
    napi_value v;
    napi_create_uint32(env, x, &v);
    return v;
}
napi_value make_f64(napi_env env, double x) {
    napi_value v;
    napi_create_double(env, x, &v);
    return v;
}
napi_value ret_id(napi_env env, uint32_t id) { return id == MNI_BAD_ID ? throw_last(env) : make_u32(env, id); }
napi_value ret_rc(napi_env env, int rc) { return rc != MNI_OK ? throw_last(env) : undefined(env); }

struct Args {
    napi_value v[9];
    size_t n = 9;
    Args(napi_env env, napi_callback_info info) { napi_get_cb_info(env, info, &n, v, nullptr, nullptr); }
};
uint32_t get_u32(napi_env env, napi_value v) {
    uint32_t x = 0;
    napi_get_value_uint32(env, v, &x);
    return x;
}
double get_f64(napi_env env, napi_value v) {
    double x = 0;
    napi_get_value_double(env, v, &x);
    return x;
}
int64_t get_i64(napi_env env, napi_value v) { return (int64_t)get_f64(env, v); }
bool get_bool(napi_env env, napi_value v) {
    bool x = false;
    napi_get_value_bool(env, v, &x);
    return x;
}
std::vector<int64_t> get_i64_array(napi_env env, napi_value arr) {
    uint32_t n = 0;
    napi_get_array_length(env, arr, &n);
    std::vector<int64_t> out(n);
    for (uint32_t i = 0; i < n; ++i) {
        napi_value e;
        napi_get_element(env, arr, i, &e);
        out[i] = get_i64(env, e);
    }
    return out;
}
std::vector<uint32_t> get_u32_array(napi_env env, napi_value arr) {
    uint32_t n = 0;
    napi_get_array_length(env, arr, &n);
    std::vector<uint32_t> out(n);
    for (uint32_t i = 0; i < n; ++i) {
        napi_value e;
        napi_get_element(env, arr, i, &e);
        out[i] = get_u32(env, e);
    }
    return out;
}

// ---- signature families ---------------------------------------------------------
#define UNARY(NAME, FN)                                                      \
    napi_value NAME(napi_env env, napi_callback_info info) {                 \
        Args a(env, info);                                                   \
        return ret_id(env, FN(get_u32(env, a.v[0])));                        \
    }
#define BINARY(NAME, FN)                                                     \
    napi_value NAME(napi_env env, napi_callback_info info) {                 \
        Args a(env, info);                                                   \
        return ret_id(env, FN(get_u32(env, a.v[0]), get_u32(env, a.v[1])));  \
    }
#define WITH_DIM(NAME, FN)                                                   \
    napi_value NAME(napi_env env, napi_callback_info info) {                 \
        Args a(env, info);                                                   \
        return ret_id(env, FN(get_u32(env, a.v[0]), get_i64(env, a.v[1])));  \
    }
#define FROM_SHAPE(NAME, FN)                                                 \
    napi_value NAME(napi_env env, napi_callback_info info) {                 \
        Args a(env, info);                                                   \
        std::vector<int64_t> s = get_i64_array(env, a.v[0]);                 \
        return ret_id(env, FN(s.data(), (int)s.size()));                     \
    }
#define WITH_SHAPE(NAME, FN)                                                 \
    napi_value NAME(napi_env env, napi_callback_info info) {                 \
        Args a(env, info);                                                   \
        std::vector<int64_t> s = get_i64_array(env, a.v[1]);                 \
        return ret_id(env, FN(get_u32(env, a.v[0]), s.data(), (int)s.size())); \
    }

FROM_SHAPE(Zeros, mni_zeros)             // lib.rs:45-50
FROM_SHAPE(Ones, mni_ones)               // lib.rs:52-57
BINARY(Add, mni_add)                     // lib.rs:164-169
BINARY(Mul, mni_mul)                     // lib.rs:171-176
BINARY(Sub, mni_sub)                     // lib.rs:178-183
UNARY(Neg, mni_neg)                      // lib.rs:185-190
BINARY(Matmul, mni_matmul)               // lib.rs:199-204
BINARY(BiasGelu, mni_bias_gelu)          // lib.rs:526-531
UNARY(ExpOp, mni_exp_op)                 // lib.rs:220-225
UNARY(LogOp, mni_log_op)                 // lib.rs:227-232
UNARY(Sigmoid, mni_sigmoid)              // lib.rs:374-379
BINARY(Div, mni_div)                     // lib.rs:339-344
BINARY(Lt, mni_lt)                       // lib.rs:346-351
BINARY(EqOp, mni_eq_op)                  // lib.rs:353-358
BINARY(Gt, mni_gt)                       // lib.rs:360-365
WITH_DIM(MaxOp, mni_max_op)              // lib.rs:248-253
UNARY(Gelu, mni_gelu)                    // lib.rs:206-211
UNARY(Relu, mni_relu)                    // lib.rs:213-218
WITH_DIM(SumOp, mni_sum_op)              // lib.rs:234-239
WITH_DIM(MeanOp, mni_mean_op)            // lib.rs:241-246
WITH_DIM(SoftmaxOp, mni_softmax_op)      // lib.rs:302-307
UNARY(SumAll, mni_sum_all)               // lib.rs:255-265
UNARY(MeanAll, mni_mean_all)             // lib.rs:267-277
WITH_SHAPE(View, mni_view)               // lib.rs:279-285
WITH_SHAPE(Permute, mni_permute)         // lib.rs:287-293
UNARY(Contiguous, mni_contiguous)        // lib.rs:295-300

napi_value MulScalar(napi_env env, napi_callback_info info) {  // lib.rs:192-197
    Args a(env, info);
    return ret_id(env, mni_mul_scalar(get_u32(env, a.v[0]), get_f64(env, a.v[1])));
}
napi_value FromFloat32(napi_env env, napi_callback_info info) {  // lib.rs:73-78
    Args a(env, info);
    napi_typedarray_type type;
    size_t len = 0, off = 0;
    void *data = nullptr;
    napi_value ab;
    if (napi_get_typedarray_info(env, a.v[0], &type, &len, &data, &ab, &off) != napi_ok || type != napi_float32_array) {
        napi_throw_type_error(env, nullptr, "fromFloat32 expects a Float32Array");
        return nullptr;
    }
    std::vector<int64_t> s = get_i64_array(env, a.v[1]);
    return ret_id(env, mni_from_float32((const float *)data, len, s.data(), (int)s.size()));
}
napi_value TensorShape(napi_env env, napi_callback_info info) {  // lib.rs:80-84
    Args a(env, info);
    int64_t shape[MNI_MAX_DIMS];
    const int nd = mni_tensor_shape(get_u32(env, a.v[0]), shape, MNI_MAX_DIMS);
    if (nd < 0) return throw_last(env);
    napi_value arr;
    napi_create_array_with_length(env, (size_t)nd, &arr);
    for (int i = 0; i < nd; ++i) napi_set_element(env, arr, (uint32_t)i, make_f64(env, (double)shape[i]));
    return arr;
}
napi_value TensorSize(napi_env env, napi_callback_info info) {  // lib.rs:86-90
    Args a(env, info);
    const int64_t n = mni_tensor_size(get_u32(env, a.v[0]));
    return n < 0 ? throw_last(env) : make_f64(env, (double)n);
}
napi_value ToFloat32(napi_env env, napi_callback_info info) {  // lib.rs:92-97
    Args a(env, info);
    const uint32_t id = get_u32(env, a.v[0]);
    const int64_t n = mni_tensor_size(id);
    if (n < 0) return throw_last(env);
    void *data = nullptr;
    napi_value ab, out;
    napi_create_arraybuffer(env, (size_t)n * sizeof(float), &data, &ab);
    if (mni_to_float32(id, (float *)data, (size_t)n) != MNI_OK) return throw_last(env);
    napi_create_typedarray(env, napi_float32_array, (size_t)n, ab, 0, &out);
    return out;
}
napi_value GetScalar(napi_env env, napi_callback_info info) {  // lib.rs:99-103
    Args a(env, info);
    double v = 0;
    if (mni_get_scalar(get_u32(env, a.v[0]), &v) != MNI_OK) return throw_last(env);
    return make_f64(env, v);
}
napi_value FreeTensor(napi_env env, napi_callback_info info) {  // lib.rs:105-109
    Args a(env, info);
    mni_free_tensor(get_u32(env, a.v[0]));
    return undefined(env);
}
napi_value SetRequiresGrad(napi_env env, napi_callback_info info) {  // lib.rs:115-119
    Args a(env, info);
    return ret_rc(env, mni_set_requires_grad(get_u32(env, a.v[0]), get_bool(env, a.v[1]) ? 1 : 0));
}
napi_value GetGrad(napi_env env, napi_callback_info info) {  // lib.rs:121-125: Option<u32> -> number | null
    Args a(env, info);
    uint32_t g = 0;
    const int r = mni_get_grad(get_u32(env, a.v[0]), &g);
    if (r < 0) return throw_last(env);
    if (r == 0) {
        napi_value v;
        napi_get_null(env, &v);
        return v;
    }
    return make_u32(env, g);
}
napi_value Backward(napi_env env, napi_callback_info info) {  // lib.rs:131-137
    Args a(env, info);
    return ret_rc(env, mni_backward(get_u32(env, a.v[0])));
}
napi_value ZeroGrad(napi_env env, napi_callback_info info) {  // lib.rs:139-146
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    return ret_rc(env, mni_zero_grad(ids.data(), ids.size()));
}
napi_value NoGradStart(napi_env env, napi_callback_info) {  // lib.rs:148-152
    mni_no_grad_start();
    return undefined(env);
}
napi_value NoGradEnd(napi_env env, napi_callback_info) {  // lib.rs:154-158
    mni_no_grad_end();
    return undefined(env);
}
napi_value CrossEntropyLoss(napi_env env, napi_callback_info info) {  // lib.rs:328-336
    Args a(env, info);
    std::vector<int64_t> t = get_i64_array(env, a.v[1]);
    return ret_id(env, mni_cross_entropy_loss(get_u32(env, a.v[0]), t.data(), t.size()));
}
napi_value AdamwStep(napi_env env, napi_callback_info info) {  // lib.rs:400-412
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    return ret_rc(env, mni_adamw_step(ids.data(), ids.size(), get_f64(env, a.v[1]), get_f64(env, a.v[2]), get_f64(env, a.v[3]),
                                      get_f64(env, a.v[4]), get_f64(env, a.v[5]), get_i64(env, a.v[6])));
}
napi_value GradNorm(napi_env env, napi_callback_info info) {  // lib.rs:414-419
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    const double v = mni_grad_norm(ids.data(), ids.size());
    return v < 0 ? throw_last(env) : make_f64(env, v);
}
napi_value ClipGradNorm(napi_env env, napi_callback_info info) {  // lib.rs:421-426
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    return ret_rc(env, mni_clip_grad_norm(ids.data(), ids.size(), get_f64(env, a.v[1])));
}
napi_value ClipAndStep(napi_env env, napi_callback_info info) {  // lib.rs:428-442
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    const double v = mni_clip_and_step(ids.data(), ids.size(), get_f64(env, a.v[1]), get_f64(env, a.v[2]), get_f64(env, a.v[3]),
                                       get_f64(env, a.v[4]), get_f64(env, a.v[5]), get_i64(env, a.v[6]), get_f64(env, a.v[7]));
    return v < 0 ? throw_last(env) : make_f64(env, v);
}
napi_value ResetEngine(napi_env env, napi_callback_info) {  // lib.rs:460-468
    mni_reset_engine();
    return undefined(env);
}
napi_value GcTensors(napi_env env, napi_callback_info info) {  // lib.rs:693-706
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    return ret_rc(env, mni_gc_tensors(ids.data(), ids.size()));
}
// Opt-in fused Linear (no counterpart in lib.rs; feature-detected by callers).
napi_value KvCacheCreate(napi_env env, napi_callback_info info) {  // lib.rs:586-607
    Args a(env, info);
    return ret_id(env, mni_kv_cache_create(get_i64(env, a.v[0]), get_i64(env, a.v[1]), get_i64(env, a.v[2]), get_i64(env, a.v[3]),
                                           get_bool(env, a.v[4]) ? 1 : 0));
}
napi_value KvCacheLen(napi_env env, napi_callback_info info) {  // lib.rs:609-616
    Args a(env, info);
    return make_f64(env, (double)mni_kv_cache_len(get_u32(env, a.v[0])));
}
napi_value KvCacheQuantized(napi_env env, napi_callback_info info) {  // lib.rs:618-625
    Args a(env, info);
    napi_value v;
    napi_get_boolean(env, mni_kv_cache_quantized(get_u32(env, a.v[0])) != 0, &v);
    return v;
}
napi_value KvCacheReset(napi_env env, napi_callback_info info) {  // lib.rs:627-633
    Args a(env, info);
    mni_kv_cache_reset(get_u32(env, a.v[0]));
    return undefined(env);
}
napi_value KvCacheFree(napi_env env, napi_callback_info info) {  // lib.rs:635-639
    Args a(env, info);
    mni_kv_cache_free(get_u32(env, a.v[0]));
    return undefined(env);
}
napi_value KvCacheAppend(napi_env env, napi_callback_info info) {  // lib.rs:661-676
    Args a(env, info);
    return ret_rc(env, mni_kv_cache_append(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2])));
}
napi_value KvCacheDecodeStep(napi_env env, napi_callback_info info) {  // lib.rs:641-659
    Args a(env, info);
    return ret_id(env, mni_kv_cache_decode_step(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2]),
                                                get_u32(env, a.v[3]), get_f64(env, a.v[4])));
}
napi_value PowOp(napi_env env, napi_callback_info info) {  // lib.rs:381-386
    Args a(env, info);
    return ret_id(env, mni_pow_op(get_u32(env, a.v[0]), get_f64(env, a.v[1])));
}
napi_value IsClose(napi_env env, napi_callback_info info) {  // lib.rs:367-372
    Args a(env, info);
    return ret_id(env, mni_is_close(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_f64(env, a.v[2])));
}
napi_value LayernormOp(napi_env env, napi_callback_info info) {  // lib.rs:309-315
    Args a(env, info);
    return ret_id(env, mni_layernorm_op(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2]), get_f64(env, a.v[3])));
}
napi_value FlashAttention(napi_env env, napi_callback_info info) {  // lib.rs:575-584
    Args a(env, info);
    return ret_id(env, mni_flash_attention(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2]),
                                           get_f64(env, a.v[3]), get_bool(env, a.v[4]) ? 1 : 0));
}
napi_value Linear(napi_env env, napi_callback_info info) {
    Args a(env, info);
    const int act = a.n > 3 ? (int)get_i64(env, a.v[3]) : MNI_EPI_BIAS;
    return ret_id(env, mni_linear(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2]), act));
}
napi_value MseLoss(napi_env env, napi_callback_info info) {  // fused form of src/nn.ts:161-165
    Args a(env, info);
    return ret_id(env, mni_mse_loss(get_u32(env, a.v[0]), get_u32(env, a.v[1])));
}

FROM_SHAPE(RandTensor, mni_rand_tensor)    // lib.rs:60-64
FROM_SHAPE(RandnTensor, mni_randn_tensor)  // lib.rs:67-71
WITH_SHAPE(Tile, mni_tile)                 // lib.rs:568-573
BINARY(CrossEntropyLossGpu, mni_cross_entropy_loss_gpu)  // lib.rs:679-691
napi_value Seed(napi_env env, napi_callback_info info) {  // no counterpart in the reference: fixes the random stream
    Args a(env, info);
    return ret_rc(env, mni_seed((uint64_t)get_f64(env, a.v[0])));
}
napi_value PhiloxWords(napi_env env, napi_callback_info info) {  // no counterpart: the raw generator, for known-answer checks
    Args a(env, info);
    const size_t n = (size_t)get_i64(env, a.v[2]);
    napi_value ab, out;
    void *data = nullptr;
    napi_create_arraybuffer(env, n * sizeof(uint32_t), &data, &ab);
    if (mni_philox_words((uint64_t)get_f64(env, a.v[0]), (uint64_t)get_f64(env, a.v[1]), (uint32_t *)data, n) != MNI_OK)
        return throw_last(env);
    napi_create_typedarray(env, napi_uint32_array, n, ab, 0, &out);
    return out;
}
napi_value DropoutOp(napi_env env, napi_callback_info info) {  // lib.rs:388-394
    Args a(env, info);
    return ret_id(env, mni_dropout_op(get_u32(env, a.v[0]), get_f64(env, a.v[1]), get_bool(env, a.v[2]) ? 1 : 0));
}
napi_value CreateDataset(napi_env env, napi_callback_info info) {  // lib.rs:476-479
    Args a(env, info);
    napi_typedarray_type type;
    size_t len = 0, off = 0;
    void *data = nullptr;
    napi_value ab;
    if (napi_get_typedarray_info(env, a.v[0], &type, &len, &data, &ab, &off) != napi_ok || type != napi_int32_array) {
        napi_throw_type_error(env, nullptr, "createDataset expects an Int32Array");
        return nullptr;
    }
    return ret_id(env, mni_create_dataset((const int32_t *)data, len));
}
napi_value SampleBatch(napi_env env, napi_callback_info info) {  // lib.rs:483-490
    Args a(env, info);
    uint32_t ids[2] = {0, 0};
    if (mni_sample_batch(get_u32(env, a.v[0]), get_i64(env, a.v[1]), get_i64(env, a.v[2]), ids) != MNI_OK) return throw_last(env);
    napi_value arr;
    napi_create_array_with_length(env, 2, &arr);
    napi_set_element(env, arr, 0, make_u32(env, ids[0]));
    napi_set_element(env, arr, 1, make_u32(env, ids[1]));
    return arr;
}
napi_value FreeIntBuffer(napi_env env, napi_callback_info info) {  // lib.rs:494-497
    Args a(env, info);
    return ret_rc(env, mni_free_int_buffer(get_u32(env, a.v[0])));
}
napi_value IntBufferToInt32(napi_env env, napi_callback_info info) {  // no counterpart in the reference: reads a buffer back
    Args a(env, info);
    const uint32_t id = get_u32(env, a.v[0]);
    const int64_t n = mni_int_buffer_len(id);
    if (n < 0) return throw_last(env);
    napi_value ab, out;
    void *data = nullptr;
    napi_create_arraybuffer(env, (size_t)n * sizeof(int32_t), &data, &ab);
    if (mni_int_buffer_to_host(id, (int32_t *)data, (size_t)n) != MNI_OK) return throw_last(env);
    napi_create_typedarray(env, napi_int32_array, (size_t)n, ab, 0, &out);
    return out;
}
napi_value EmbeddingForward(napi_env env, napi_callback_info info) {  // lib.rs:319-326
    Args a(env, info);
    std::vector<int64_t> idx = get_i64_array(env, a.v[1]);
    return ret_id(env, mni_embedding_forward(get_u32(env, a.v[0]), idx.data(), idx.size(), get_i64(env, a.v[2]), get_i64(env, a.v[3])));
}
napi_value EmbeddingForwardGpu(napi_env env, napi_callback_info info) {  // lib.rs:501-511
    Args a(env, info);
    return ret_id(env, mni_embedding_forward_gpu(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_i64(env, a.v[2]), get_i64(env, a.v[3])));
}
napi_value ResidualLayernorm(napi_env env, napi_callback_info info) {  // lib.rs:515-523
    Args a(env, info);
    return ret_id(env, mni_residual_layernorm(get_u32(env, a.v[0]), get_u32(env, a.v[1]), get_u32(env, a.v[2]), get_u32(env, a.v[3]),
                                              get_f64(env, a.v[4])));
}
napi_value ScaleGrads(napi_env env, napi_callback_info info) {  // lib.rs:450-454
    Args a(env, info);
    std::vector<uint32_t> ids = get_u32_array(env, a.v[0]);
    int found = 0;
    if (mni_scale_grads(ids.data(), ids.size(), get_f64(env, a.v[1]), &found) != MNI_OK) return throw_last(env);
    napi_value v;
    napi_get_boolean(env, found != 0, &v);
    return v;
}

}  // namespace

NAPI_MODULE_INIT() {
    const napi_property_descriptor props[] = {
#define EXPORT(NAME, FN) {NAME, nullptr, FN, nullptr, nullptr, nullptr, napi_enumerable, nullptr}
        EXPORT("zeros", Zeros), EXPORT("ones", Ones), EXPORT("fromFloat32", FromFloat32),
        EXPORT("tensorShape", TensorShape), EXPORT("tensorSize", TensorSize), EXPORT("toFloat32", ToFloat32),
        EXPORT("getScalar", GetScalar), EXPORT("freeTensor", FreeTensor), EXPORT("setRequiresGrad", SetRequiresGrad),
        EXPORT("getGrad", GetGrad), EXPORT("backward", Backward), EXPORT("zeroGrad", ZeroGrad),
        EXPORT("noGradStart", NoGradStart), EXPORT("noGradEnd", NoGradEnd), EXPORT("add", Add), EXPORT("mul", Mul),
        EXPORT("sub", Sub), EXPORT("neg", Neg), EXPORT("mulScalar", MulScalar), EXPORT("matmul", Matmul),
        EXPORT("gelu", Gelu), EXPORT("relu", Relu), EXPORT("sumOp", SumOp), EXPORT("meanOp", MeanOp),
        EXPORT("sumAll", SumAll), EXPORT("meanAll", MeanAll), EXPORT("view", View), EXPORT("permute", Permute),
        EXPORT("contiguous", Contiguous), EXPORT("crossEntropyLoss", CrossEntropyLoss), EXPORT("adamwStep", AdamwStep),
        EXPORT("gradNorm", GradNorm), EXPORT("clipGradNorm", ClipGradNorm), EXPORT("clipAndStep", ClipAndStep),
        EXPORT("resetEngine", ResetEngine), EXPORT("gcTensors", GcTensors), EXPORT("linear", Linear), EXPORT("mseLoss", MseLoss),
        EXPORT("softmaxOp", SoftmaxOp), EXPORT("biasGelu", BiasGelu),
        EXPORT("expOp", ExpOp), EXPORT("logOp", LogOp), EXPORT("sigmoid", Sigmoid), EXPORT("powOp", PowOp),
        EXPORT("div", Div), EXPORT("lt", Lt), EXPORT("eqOp", EqOp), EXPORT("gt", Gt), EXPORT("isClose", IsClose),
        EXPORT("maxOp", MaxOp), EXPORT("layernormOp", LayernormOp),
        EXPORT("kvCacheCreate", KvCacheCreate), EXPORT("kvCacheLen", KvCacheLen), EXPORT("kvCacheQuantized", KvCacheQuantized),
        EXPORT("kvCacheReset", KvCacheReset), EXPORT("kvCacheFree", KvCacheFree), EXPORT("kvCacheAppend", KvCacheAppend),
        EXPORT("kvCacheDecodeStep", KvCacheDecodeStep), EXPORT("flashAttention", FlashAttention),
        EXPORT("randTensor", RandTensor), EXPORT("randnTensor", RandnTensor), EXPORT("seed", Seed), EXPORT("philoxWords", PhiloxWords), EXPORT("tile", Tile),
        EXPORT("dropoutOp", DropoutOp), EXPORT("createDataset", CreateDataset), EXPORT("sampleBatch", SampleBatch),
        EXPORT("freeIntBuffer", FreeIntBuffer), EXPORT("intBufferToInt32", IntBufferToInt32),
        EXPORT("embeddingForward", EmbeddingForward), EXPORT("embeddingForwardGpu", EmbeddingForwardGpu),
        EXPORT("crossEntropyLossGpu", CrossEntropyLossGpu), EXPORT("residualLayernorm", ResidualLayernorm),
        EXPORT("scaleGrads", ScaleGrads),
#undef EXPORT
    };
    napi_define_properties(env, exports, sizeof(props) / sizeof(props[0]), props);
    return exports;
}
