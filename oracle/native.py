"""ctypes binding of the CPU oracle (oracle/liboracle.so) under the same
camelCase names as the HIP engine's binding, so one test script can drive
both.  TEST INFRASTRUCTURE: only tests/, the smoke check and the cpu_baseline
leg of the benchmark may import this."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
BAD_ID = 0xFFFFFFFF
_i64p = C.POINTER(C.c_int64)
_u32p = C.POINTER(C.c_uint32)


class OracleError(RuntimeError):
    pass


def build():
    subprocess.run(["make", "-s", "-C", _HERE, "liboracle.so"], check=True)
    return LIB_PATH


def _i64(values):
    return (C.c_int64 * max(len(values), 1))(*[int(v) for v in values])


def _u32(values):
    return (C.c_uint32 * max(len(values), 1))(*[int(v) for v in values])


class OracleNative:
    name = "oracle"

    def __init__(self):
        if not os.path.exists(LIB_PATH):
            build()
        lib = C.CDLL(LIB_PATH)
        u32 = C.c_uint32
        sig = {
            "orc_last_error": (C.c_char_p, []),
            "orc_zeros": (u32, [_i64p, C.c_int]), "orc_ones": (u32, [_i64p, C.c_int]),
            "orc_from_float32": (u32, [C.c_void_p, C.c_size_t, _i64p, C.c_int]),
            "orc_tensor_shape": (C.c_int, [u32, _i64p, C.c_int]), "orc_tensor_size": (C.c_int64, [u32]),
            "orc_to_float32": (C.c_int, [u32, C.c_void_p, C.c_size_t]),
            "orc_get_scalar": (C.c_int, [u32, C.POINTER(C.c_double)]),
            "orc_free_tensor": (None, [u32]), "orc_set_requires_grad": (C.c_int, [u32, C.c_int]),
            "orc_get_grad": (C.c_int, [u32, _u32p]), "orc_backward": (C.c_int, [u32]),
            "orc_zero_grad": (C.c_int, [_u32p, C.c_size_t]),
            "orc_no_grad_start": (None, []), "orc_no_grad_end": (None, []),
            "orc_add": (u32, [u32, u32]), "orc_sub": (u32, [u32, u32]), "orc_mul": (u32, [u32, u32]),
            "orc_neg": (u32, [u32]), "orc_mul_scalar": (u32, [u32, C.c_double]),
            "orc_matmul": (u32, [u32, u32]), "orc_gelu": (u32, [u32]), "orc_relu": (u32, [u32]),
            "orc_sum_op": (u32, [u32, C.c_int64]), "orc_mean_op": (u32, [u32, C.c_int64]),
            "orc_sum_all": (u32, [u32]), "orc_mean_all": (u32, [u32]),
            "orc_view": (u32, [u32, _i64p, C.c_int]), "orc_permute": (u32, [u32, _i64p, C.c_int]),
            "orc_contiguous": (u32, [u32]),
            "orc_cross_entropy_loss": (u32, [u32, _i64p, C.c_size_t]),
            "orc_softmax_op": (u32, [u32, C.c_int64]),
            "orc_bias_gelu": (u32, [u32, u32]),
            "orc_kv_cache_create": (u32, [C.c_int64] * 4 + [C.c_int]), "orc_kv_cache_len": (C.c_int64, [u32]),
            "orc_kv_cache_quantized": (C.c_int, [u32]), "orc_kv_cache_reset": (None, [u32]), "orc_kv_cache_free": (None, [u32]),
            "orc_kv_cache_append": (C.c_int, [u32, u32, u32]),
            "orc_kv_cache_decode_step": (u32, [u32, u32, u32, u32, C.c_double]),
            "orc_exp_op": (u32, [u32]), "orc_log_op": (u32, [u32]), "orc_sigmoid": (u32, [u32]),
            "orc_pow_op": (u32, [u32, C.c_double]), "orc_div": (u32, [u32, u32]),
            "orc_lt": (u32, [u32, u32]), "orc_eq_op": (u32, [u32, u32]), "orc_gt": (u32, [u32, u32]),
            "orc_is_close": (u32, [u32, u32, C.c_double]), "orc_max_op": (u32, [u32, C.c_int64]),
            "orc_layernorm_op": (u32, [u32, u32, u32, C.c_double]),
            "orc_flash_attention": (u32, [u32, u32, u32, C.c_double, C.c_int]),
            "orc_adamw_step": (None, [_u32p, C.c_size_t] + [C.c_double] * 5 + [C.c_int64]),
            "orc_grad_norm": (C.c_double, [_u32p, C.c_size_t]),
            "orc_clip_and_step": (C.c_double, [_u32p, C.c_size_t] + [C.c_double] * 5 + [C.c_int64, C.c_double]),
            "orc_reset_engine": (None, []), "orc_gc_tensors": (None, [_u32p, C.c_size_t]),
            "orc_sgemm_ikj": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]),
            "orc_philox4x32_10": (None, [_u32p, _u32p, _u32p]),
            "orc_philox_words": (None, [C.c_uint64, C.c_uint64, C.c_void_p, C.c_size_t]),
            "orc_seed": (None, [C.c_uint64]),
            "orc_rand_tensor": (u32, [_i64p, C.c_int]), "orc_randn_tensor": (u32, [_i64p, C.c_int]),
            "orc_dropout_op": (u32, [u32, C.c_double, C.c_int]),
            "orc_create_dataset": (u32, [C.c_void_p, C.c_size_t]), "orc_free_int_buffer": (None, [u32]),
            "orc_int_buffer_len": (C.c_int64, [u32]), "orc_int_buffer_to_host": (C.c_int, [u32, C.c_void_p, C.c_size_t]),
            "orc_sample_batch_at": (C.c_int, [u32, C.c_int64, C.c_int64, _i64p, _u32p]),
            "orc_embedding_forward": (u32, [u32, _i64p, C.c_size_t, C.c_int64, C.c_int64]),
            "orc_embedding_forward_gpu": (u32, [u32, u32, C.c_int64, C.c_int64]),
            "orc_cross_entropy_loss_gpu": (u32, [u32, u32]),
            "orc_residual_layernorm": (u32, [u32, u32, u32, u32, C.c_double]),
            "orc_scale_grads": (C.c_int, [_u32p, C.c_size_t, C.c_double]),
            "orc_tile": (u32, [u32, _i64p, C.c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        self.lib = lib

    def _err(self):
        return OracleError(self.lib.orc_last_error().decode())

    def _id(self, v):
        if v == BAD_ID:
            raise self._err()
        return v

    def _rc(self, rc):
        if rc != 0:
            raise self._err()

    def zeros(self, shape):
        return self._id(self.lib.orc_zeros(_i64(shape), len(shape)))

    def ones(self, shape):
        return self._id(self.lib.orc_ones(_i64(shape), len(shape)))

    def fromFloat32(self, data, shape):
        a = np.ascontiguousarray(data, dtype=np.float32)
        return self._id(self.lib.orc_from_float32(a.ctypes.data, a.size, _i64(shape), len(shape)))

    def tensorShape(self, id):
        out = (C.c_int64 * 8)()
        nd = self.lib.orc_tensor_shape(id, out, 8)
        if nd < 0:
            raise self._err()
        return [int(out[i]) for i in range(nd)]

    def tensorSize(self, id):
        n = self.lib.orc_tensor_size(id)
        if n < 0:
            raise self._err()
        return int(n)

    def toFloat32(self, id):
        out = np.empty(self.tensorSize(id), dtype=np.float32)
        self._rc(self.lib.orc_to_float32(id, out.ctypes.data, out.size))
        return out

    def getScalar(self, id):
        v = C.c_double(0)
        self._rc(self.lib.orc_get_scalar(id, C.byref(v)))
        return v.value

    def freeTensor(self, id):
        self.lib.orc_free_tensor(id)

    def setRequiresGrad(self, id, requires):
        self._rc(self.lib.orc_set_requires_grad(id, 1 if requires else 0))

    def getGrad(self, id):
        out = C.c_uint32(0)
        r = self.lib.orc_get_grad(id, C.byref(out))
        if r < 0:
            raise self._err()
        return out.value if r == 1 else None

    def backward(self, loss):
        self._rc(self.lib.orc_backward(loss))

    def zeroGrad(self, ids):
        self._rc(self.lib.orc_zero_grad(_u32(ids), len(ids)))

    def noGradStart(self):
        self.lib.orc_no_grad_start()

    def noGradEnd(self):
        self.lib.orc_no_grad_end()

    def add(self, a, b):
        return self._id(self.lib.orc_add(a, b))

    def sub(self, a, b):
        return self._id(self.lib.orc_sub(a, b))

    def mul(self, a, b):
        return self._id(self.lib.orc_mul(a, b))

    def neg(self, a):
        return self._id(self.lib.orc_neg(a))

    def mulScalar(self, a, s):
        return self._id(self.lib.orc_mul_scalar(a, float(s)))

    def matmul(self, a, b):
        return self._id(self.lib.orc_matmul(a, b))

    def gelu(self, a):
        return self._id(self.lib.orc_gelu(a))

    def relu(self, a):
        return self._id(self.lib.orc_relu(a))

    def sumOp(self, a, dim):
        return self._id(self.lib.orc_sum_op(a, dim))

    def meanOp(self, a, dim):
        return self._id(self.lib.orc_mean_op(a, dim))

    def sumAll(self, a):
        return self._id(self.lib.orc_sum_all(a))

    def meanAll(self, a):
        return self._id(self.lib.orc_mean_all(a))

    def view(self, a, shape):
        return self._id(self.lib.orc_view(a, _i64(shape), len(shape)))

    def permute(self, a, dims):
        return self._id(self.lib.orc_permute(a, _i64(dims), len(dims)))

    def contiguous(self, a):
        return self._id(self.lib.orc_contiguous(a))

    def crossEntropyLoss(self, logits, targets):
        return self._id(self.lib.orc_cross_entropy_loss(logits, _i64(targets), len(targets)))

    def softmaxOp(self, a, dim):
        return self._id(self.lib.orc_softmax_op(a, dim))

    def biasGelu(self, x, bias):
        return self._id(self.lib.orc_bias_gelu(x, bias))

    def kvCacheCreate(self, batchSize, numHeads, headDim, maxSeqLen, quantized):
        return self.lib.orc_kv_cache_create(batchSize, numHeads, headDim, maxSeqLen, 1 if quantized else 0)

    def kvCacheLen(self, cacheId):
        return self.lib.orc_kv_cache_len(cacheId)

    def kvCacheQuantized(self, cacheId):
        return bool(self.lib.orc_kv_cache_quantized(cacheId))

    def kvCacheReset(self, cacheId):
        self.lib.orc_kv_cache_reset(cacheId)

    def kvCacheFree(self, cacheId):
        self.lib.orc_kv_cache_free(cacheId)

    def kvCacheAppend(self, cacheId, k, v):
        if self.lib.orc_kv_cache_append(cacheId, k, v) != 0:
            raise self._err()

    def kvCacheDecodeStep(self, cacheId, q, k, v, scale):
        return self._id(self.lib.orc_kv_cache_decode_step(cacheId, q, k, v, scale))

    def expOp(self, a):
        return self._id(self.lib.orc_exp_op(a))

    def logOp(self, a):
        return self._id(self.lib.orc_log_op(a))

    def sigmoid(self, a):
        return self._id(self.lib.orc_sigmoid(a))

    def powOp(self, a, exponent):
        return self._id(self.lib.orc_pow_op(a, exponent))

    def div(self, a, b):
        return self._id(self.lib.orc_div(a, b))

    def lt(self, a, b):
        return self._id(self.lib.orc_lt(a, b))

    def eqOp(self, a, b):
        return self._id(self.lib.orc_eq_op(a, b))

    def gt(self, a, b):
        return self._id(self.lib.orc_gt(a, b))

    def isClose(self, a, b, tol):
        return self._id(self.lib.orc_is_close(a, b, tol))

    def maxOp(self, a, dim):
        return self._id(self.lib.orc_max_op(a, dim))

    def layernormOp(self, x, gamma, beta, eps):
        return self._id(self.lib.orc_layernorm_op(x, gamma, beta, eps))

    def flashAttention(self, q, k, v, scale, causal):
        return self._id(self.lib.orc_flash_attention(q, k, v, scale, 1 if causal else 0))

    def adamwStep(self, ids, lr, beta1, beta2, eps, weight_decay, step):
        self.lib.orc_adamw_step(_u32(ids), len(ids), lr, beta1, beta2, eps, weight_decay, step)

    def gradNorm(self, ids):
        return self.lib.orc_grad_norm(_u32(ids), len(ids))

    def clipAndStep(self, ids, lr, beta1, beta2, eps, weight_decay, step, max_grad_norm):
        return self.lib.orc_clip_and_step(_u32(ids), len(ids), lr, beta1, beta2, eps, weight_decay, step, max_grad_norm)

    def resetEngine(self):
        self.lib.orc_reset_engine()

    def gcTensors(self, keep):
        self.lib.orc_gc_tensors(_u32(keep), len(keep))

    # token-side ops
    def philox(self, ctr, key):
        out = (C.c_uint32 * 4)()
        self.lib.orc_philox4x32_10(_u32(ctr), _u32(key), out)
        return [int(v) for v in out]

    def philoxWords(self, seed, offset, n):
        out = np.empty(n, dtype=np.uint32)
        self.lib.orc_philox_words(seed, offset, out.ctypes.data, n)
        return out

    def seed(self, seed):
        self.lib.orc_seed(seed)

    def randTensor(self, shape):
        return self._id(self.lib.orc_rand_tensor(_i64(shape), len(shape)))

    def randnTensor(self, shape):
        return self._id(self.lib.orc_randn_tensor(_i64(shape), len(shape)))

    def dropoutOp(self, x, rate, training):
        return self._id(self.lib.orc_dropout_op(x, rate, 1 if training else 0))

    def createDataset(self, data):
        a = np.ascontiguousarray(data, dtype=np.int32)
        return self._id(self.lib.orc_create_dataset(a.ctypes.data, a.size))

    def freeIntBuffer(self, id):
        self.lib.orc_free_int_buffer(id)

    def intBufferToHost(self, id):
        n = self.lib.orc_int_buffer_len(id)
        if n < 0:
            raise self._err()
        out = np.empty(n, dtype=np.int32)
        self._rc(self.lib.orc_int_buffer_to_host(id, out.ctypes.data, n))
        return out

    # the reference draws the window starts from its thread RNG; the oracle takes them as an argument
    def sampleBatchAt(self, datasetId, blockSize, batchSize, starts):
        out = (C.c_uint32 * 2)()
        self._rc(self.lib.orc_sample_batch_at(datasetId, blockSize, batchSize, _i64(starts), out))
        return [int(out[0]), int(out[1])]

    def embeddingForward(self, weight, indices, batch, seqLen):
        return self._id(self.lib.orc_embedding_forward(weight, _i64(indices), len(indices), batch, seqLen))

    def embeddingForwardGpu(self, weight, intBufId, batch, seqLen):
        return self._id(self.lib.orc_embedding_forward_gpu(weight, intBufId, batch, seqLen))

    def crossEntropyLossGpu(self, logits, intBufId):
        return self._id(self.lib.orc_cross_entropy_loss_gpu(logits, intBufId))

    def residualLayernorm(self, x, residual, gamma, beta, eps):
        return self._id(self.lib.orc_residual_layernorm(x, residual, gamma, beta, eps))

    def scaleGrads(self, ids, invScale):
        return bool(self.lib.orc_scale_grads(_u32(ids), len(ids), invScale))

    def tile(self, a, reps):
        return self._id(self.lib.orc_tile(a, _i64(reps), len(reps)))

    # raw loop of ops/matmul.rs:62-69 on host arrays
    def sgemm_ikj(self, a, b):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        m, k = a.shape
        k2, n = b.shape
        assert k == k2
        c = np.empty((m, n), dtype=np.float32)
        self.lib.orc_sgemm_ikj(a.ctypes.data, b.ctypes.data, c.ctypes.data, m, n, k)
        return c
