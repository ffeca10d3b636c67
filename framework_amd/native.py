"""ctypes binding of libmni_rocm.so.

Two objects are exposed:

* ``rocm`` -- the kernel-level C ABI (``mni_rocm_*``): device buffers, copies,
  timing marks and ``sgemm`` on raw pointers.
* ``native`` -- the engine-level C ABI (``mni_*``) under the camelCase names the
  reference's N-API addon exports to JavaScript (``matmul``, ``fromFloat32``,
  ``clipAndStep`` ...; src/native/src/lib.rs, consumer src/tensor.ts), so the
  ``Tensor`` / ``Linear`` / ``Adam`` wrappers read like the reference's.

There is no CPU fallback: if the shared library is missing or fails to load,
importing a symbol from it raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmni_rocm.so")

BAD_ID = 0xFFFFFFFF
MAX_DIMS = 8
EPI_NONE, EPI_BIAS, EPI_BIAS_RELU, EPI_BIAS_GELU, EPI_BIAS_GELU_DUAL, EPI_DGELU = 0, 1, 2, 3, 4, 5
ALGO_AUTO, ALGO_MFMA, ALGO_SKINNY, ALGO_MFMA_SMALL, ALGO_SKINNY_TWO_PASS, ALGO_MFMA_STREAMK, ALGO_DIRECT, ALGO_PANEL, ALGO_TINY, ALGO_FEWROWS, ALGO_OUTER, ALGO_GEMV, ALGO_FEWROWS_NT = 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12

_f32p = C.POINTER(C.c_float)
_i64p = C.POINTER(C.c_int64)
_u32p = C.POINTER(C.c_uint32)


class MniError(RuntimeError):
    """Raised where the reference's Rust layer would panic."""


class Operand(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("row_stride", C.c_int64), ("col_stride", C.c_int64),
                ("batch_stride", C.c_int64), ("batch_count", C.c_int64)]


class GemmDesc(C.Structure):
    _fields_ = [("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64), ("batch", C.c_int64),
                ("A", Operand), ("B", Operand),
                ("C", C.c_void_p), ("ldc", C.c_int64), ("c_batch_stride", C.c_int64),
                ("bias", C.c_void_p), ("epilogue", C.c_int32), ("accumulate", C.c_int32),
                ("split_k", C.c_int32), ("algo", C.c_int32), ("aux", C.c_void_p), ("colsum_part", C.c_void_p)]


# name -> (restype, argtypes): every symbol include/mni_rocm.h declares.
SIGNATURES = {
    "mni_rocm_init": (C.c_int, [C.c_int]),
    "mni_rocm_device_info": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mni_rocm_device_xcds": (C.c_int, []),
    "mni_rocm_last_error": (C.c_char_p, []),
    "mni_rocm_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "mni_rocm_free": (C.c_int, [C.c_void_p]),
    "mni_rocm_clear_cache": (C.c_int, []),
    "mni_rocm_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mni_rocm_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mni_rocm_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mni_rocm_sync": (C.c_int, []),
    "mni_rocm_test_raise_device_status": (C.c_int, [C.c_uint]),
    "mni_rocm_launch_count": (C.c_uint64, []),
    "mni_rocm_alloc_stats": (C.c_int, [C.POINTER(C.c_uint64)] * 4),
    "mni_rocm_event_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "mni_rocm_event_record": (C.c_int, [C.c_void_p]),
    "mni_rocm_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "mni_rocm_event_destroy": (C.c_int, [C.c_void_p]),
    "mni_rocm_sgemm": (C.c_int, [C.POINTER(GemmDesc)]),
    "mni_rocm_sgemm_colsum_rows": (C.c_int64, [C.c_int64, C.c_int64]),
    "mni_rocm_sgemm_noalloc": (C.c_int, [C.POINTER(GemmDesc)]),
    "mni_rocm_sgemm_noalloc_workspace_bytes": (C.c_size_t, []),
    "mni_rocm_sgemm_timed": (C.c_int, [C.POINTER(GemmDesc), C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "mni_rocm_sgemm_pair_timed": (C.c_int, [C.POINTER(GemmDesc), C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "mni_rocm_sgemm_pair": (C.c_int, [C.POINTER(GemmDesc), C.POINTER(GemmDesc)]),
    "mni_rocm_yardstick_timed": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_size_t, C.c_int, C.c_int,
                                           C.c_int, C.POINTER(C.c_float)]),
    "mni_rocm_mfma_yardstick_timed": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "mni_rocm_strided_copy": (C.c_int, [C.c_void_p, C.c_void_p, _i64p, _i64p, C.c_int]),
    "mni_rocm_add_bias": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]),
    "mni_rocm_colsum": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]),
    "mni_rocm_unbroadcast": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int, C.POINTER(C.c_int64), C.c_int]),
    "mni_rocm_axpy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_float, C.c_int64]),
    "mni_rocm_fill": (C.c_int, [C.c_void_p, C.c_float, C.c_int64]),
    "mni_zeros": (C.c_uint32, [_i64p, C.c_int]),
    "mni_ones": (C.c_uint32, [_i64p, C.c_int]),
    "mni_from_float32": (C.c_uint32, [C.c_void_p, C.c_size_t, _i64p, C.c_int]),
    "mni_tensor_shape": (C.c_int, [C.c_uint32, _i64p, C.c_int]),
    "mni_tensor_size": (C.c_int64, [C.c_uint32]),
    "mni_to_float32": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t]),
    "mni_get_scalar": (C.c_int, [C.c_uint32, C.POINTER(C.c_double)]),
    "mni_free_tensor": (None, [C.c_uint32]),
    "mni_set_requires_grad": (C.c_int, [C.c_uint32, C.c_int]),
    "mni_get_grad": (C.c_int, [C.c_uint32, _u32p]),
    "mni_backward": (C.c_int, [C.c_uint32]),
    "mni_zero_grad": (C.c_int, [_u32p, C.c_size_t]),
    "mni_no_grad_start": (None, []),
    "mni_no_grad_end": (None, []),
    "mni_add": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_mul": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_sub": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_neg": (C.c_uint32, [C.c_uint32]),
    "mni_mul_scalar": (C.c_uint32, [C.c_uint32, C.c_double]),
    "mni_matmul": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_gelu": (C.c_uint32, [C.c_uint32]),
    "mni_relu": (C.c_uint32, [C.c_uint32]),
    "mni_sum_op": (C.c_uint32, [C.c_uint32, C.c_int64]),
    "mni_mean_op": (C.c_uint32, [C.c_uint32, C.c_int64]),
    "mni_sum_all": (C.c_uint32, [C.c_uint32]),
    "mni_mean_all": (C.c_uint32, [C.c_uint32]),
    "mni_view": (C.c_uint32, [C.c_uint32, _i64p, C.c_int]),
    "mni_permute": (C.c_uint32, [C.c_uint32, _i64p, C.c_int]),
    "mni_contiguous": (C.c_uint32, [C.c_uint32]),
    "mni_softmax_op": (C.c_uint32, [C.c_uint32, C.c_int64]),
    "mni_bias_gelu": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_kv_cache_create": (C.c_uint32, [C.c_int64] * 4 + [C.c_int]), "mni_kv_cache_len": (C.c_int64, [C.c_uint32]),
    "mni_kv_cache_quantized": (C.c_int, [C.c_uint32]), "mni_kv_cache_reset": (None, [C.c_uint32]),
    "mni_kv_cache_free": (None, [C.c_uint32]), "mni_kv_cache_append": (C.c_int, [C.c_uint32] * 3),
    "mni_kv_cache_decode_step": (C.c_uint32, [C.c_uint32] * 4 + [C.c_double]),
    "mni_exp_op": (C.c_uint32, [C.c_uint32]), "mni_log_op": (C.c_uint32, [C.c_uint32]),
    "mni_sigmoid": (C.c_uint32, [C.c_uint32]), "mni_pow_op": (C.c_uint32, [C.c_uint32, C.c_double]),
    "mni_div": (C.c_uint32, [C.c_uint32, C.c_uint32]), "mni_lt": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_eq_op": (C.c_uint32, [C.c_uint32, C.c_uint32]), "mni_gt": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_is_close": (C.c_uint32, [C.c_uint32, C.c_uint32, C.c_double]),
    "mni_max_op": (C.c_uint32, [C.c_uint32, C.c_int64]),
    "mni_layernorm_op": (C.c_uint32, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_double]),
    "mni_flash_attention": (C.c_uint32, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_double, C.c_int]),
    "mni_rand_tensor": (C.c_uint32, [_i64p, C.c_int]), "mni_randn_tensor": (C.c_uint32, [_i64p, C.c_int]),
    "mni_seed": (C.c_int, [C.c_uint64]),
    "mni_philox_words": (C.c_int, [C.c_uint64, C.c_uint64, C.c_void_p, C.c_size_t]),
    "mni_dropout_op": (C.c_uint32, [C.c_uint32, C.c_double, C.c_int]),
    "mni_create_dataset": (C.c_uint32, [C.c_void_p, C.c_size_t]),
    "mni_sample_batch": (C.c_int, [C.c_uint32, C.c_int64, C.c_int64, _u32p]),
    "mni_free_int_buffer": (C.c_int, [C.c_uint32]),
    "mni_int_buffer_len": (C.c_int64, [C.c_uint32]),
    "mni_int_buffer_to_host": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t]),
    "mni_embedding_forward": (C.c_uint32, [C.c_uint32, _i64p, C.c_size_t, C.c_int64, C.c_int64]),
    "mni_embedding_forward_gpu": (C.c_uint32, [C.c_uint32, C.c_uint32, C.c_int64, C.c_int64]),
    "mni_cross_entropy_loss_gpu": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_residual_layernorm": (C.c_uint32, [C.c_uint32] * 4 + [C.c_double]),
    "mni_scale_grads": (C.c_int, [_u32p, C.c_size_t, C.c_double, C.POINTER(C.c_int)]),
    "mni_tile": (C.c_uint32, [C.c_uint32, _i64p, C.c_int]),
    "mni_cross_entropy_loss": (C.c_uint32, [C.c_uint32, _i64p, C.c_size_t]),
    "mni_adamw_step": (C.c_int, [_u32p, C.c_size_t, C.c_double, C.c_double, C.c_double, C.c_double, C.c_double, C.c_int64]),
    "mni_grad_norm": (C.c_double, [_u32p, C.c_size_t]),
    "mni_clip_grad_norm": (C.c_int, [_u32p, C.c_size_t, C.c_double]),
    "mni_clip_and_step": (C.c_double, [_u32p, C.c_size_t, C.c_double, C.c_double, C.c_double, C.c_double, C.c_double, C.c_int64, C.c_double]),
    "mni_reset_engine": (None, []),
    "mni_gc_tensors": (C.c_int, [_u32p, C.c_size_t]),
    "mni_linear": (C.c_uint32, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_int]),
    "mni_mse_loss": (C.c_uint32, [C.c_uint32, C.c_uint32]),
    "mni_dev_ptr": (C.c_void_p, [C.c_uint32]),
}

_lib = None


def load_library(path=LIB_PATH):
    """Loads libmni_rocm.so and types every exported symbol.  Raises if the
    library is absent: there is no other implementation to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise MniError("%s not found: build it with `python -m framework_amd.build`" % path)
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _i64_array(values):
    return (C.c_int64 * max(len(values), 1))(*[int(v) for v in values])


def _u32_array(values):
    return (C.c_uint32 * max(len(values), 1))(*[int(v) for v in values])


class Rocm:
    """Kernel-level ABI on raw device pointers."""

    def __init__(self):
        self.lib = load_library()

    def _check(self, rc):
        if rc != 0:
            raise MniError(self.lib.mni_rocm_last_error().decode())

    def init(self, device=0):
        self._check(self.lib.mni_rocm_init(device))

    def device_info(self):
        name = C.create_string_buffer(256)
        cus, khz = C.c_int(0), C.c_int(0)
        self._check(self.lib.mni_rocm_device_info(name, 256, C.byref(cus), C.byref(khz)))
        return {"name": name.value.decode(), "compute_units": cus.value, "clock_khz": khz.value}

    def device_xcds(self):
        n = self.lib.mni_rocm_device_xcds()
        if n < 0:
            raise MniError(self.lib.mni_rocm_last_error().decode())
        return n

    def malloc(self, nbytes):
        p = C.c_void_p()
        self._check(self.lib.mni_rocm_malloc(C.byref(p), nbytes))
        return p.value

    def free(self, ptr):
        self._check(self.lib.mni_rocm_free(ptr))

    def clear_cache(self):
        self._check(self.lib.mni_rocm_clear_cache())

    def to_device(self, array):
        a = np.ascontiguousarray(array)
        p = self.malloc(max(a.nbytes, 4))
        self._check(self.lib.mni_rocm_h2d(p, a.ctypes.data, a.nbytes))
        return p

    def to_host(self, ptr, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self._check(self.lib.mni_rocm_d2h(out.ctypes.data, ptr, out.nbytes))
        return out

    def sync(self):
        self._check(self.lib.mni_rocm_sync())

    def test_raise_device_status(self, code):
        self._check(self.lib.mni_rocm_test_raise_device_status(code))

    def launch_count(self):
        return int(self.lib.mni_rocm_launch_count())

    def alloc_stats(self):
        """(requests, driver allocations, releases, cached bytes) of the library's device allocator."""
        v = [C.c_uint64(0) for _ in range(4)]
        self._check(self.lib.mni_rocm_alloc_stats(*[C.byref(x) for x in v]))
        return tuple(int(x.value) for x in v)

    def event(self):
        e = C.c_void_p()
        self._check(self.lib.mni_rocm_event_create(C.byref(e)))
        return e.value

    def record(self, event):
        self._check(self.lib.mni_rocm_event_record(event))

    def elapsed_ms(self, start, stop):
        ms = C.c_float(0)
        self._check(self.lib.mni_rocm_event_elapsed_ms(start, stop, C.byref(ms)))
        return ms.value

    def event_destroy(self, event):
        self._check(self.lib.mni_rocm_event_destroy(event))

    def sgemm(self, M, N, K, A, B, Cptr, **kw):
        """C = epilogue(op(A) * op(B)).  a_strides / b_strides are (row, col)
        element strides of op(A) (M x K) and op(B) (K x N); default row-major."""
        d = self.gemm_desc(M, N, K, A, B, Cptr, **kw)
        self._check(self.lib.mni_rocm_sgemm(C.byref(d)))

    def sgemm_noalloc(self, M, N, K, A, B, Cptr, **kw):
        """sgemm with the plan's workspace taken from the library's fixed block: no allocation during the call."""
        d = self.gemm_desc(M, N, K, A, B, Cptr, **kw)
        self._check(self.lib.mni_rocm_sgemm_noalloc(C.byref(d)))

    def sgemm_noalloc_workspace_bytes(self):
        return int(self.lib.mni_rocm_sgemm_noalloc_workspace_bytes())

    def sgemm_colsum_rows(self, M, batch=1):
        return int(self.lib.mni_rocm_sgemm_colsum_rows(M, batch))

    def sgemm_timed(self, descs, warmup, iters):
        """Average ms per launch of the products in `descs` (made by gemm_desc),
        cycled back to back and issued from C."""
        arr = (GemmDesc * len(descs))(*descs)
        ms = C.c_float(0)
        self._check(self.lib.mni_rocm_sgemm_timed(arr, len(descs), warmup, iters, C.byref(ms)))
        return ms.value

    def sgemm_pair(self, first, second):
        """Two independent products (descriptors made by gemm_desc), in one launch where the library pairs them."""
        self._check(self.lib.mni_rocm_sgemm_pair(C.byref(first), C.byref(second)))

    def sgemm_pair_timed(self, descs, warmup, iters):
        """Average ms per pair: descs holds pairs (0 with 1, 2 with 3, ...), cycled back to back and issued from C."""
        arr = (GemmDesc * len(descs))(*descs)
        ms = C.c_float(0)
        self._check(self.lib.mni_rocm_sgemm_pair_timed(arr, len(descs), warmup, iters, C.byref(ms)))
        return ms.value

    @staticmethod
    def gemm_desc(M, N, K, A, B, Cptr, *, batch=1, a_strides=None, b_strides=None, a_batch=(0, 1), b_batch=(0, 1),
                  ldc=None, c_batch_stride=None, bias=None, epilogue=EPI_NONE, accumulate=False, split_k=0, algo=ALGO_AUTO,
                  aux=None, colsum_part=None):
        d = GemmDesc()
        d.M, d.N, d.K, d.batch = M, N, K, batch
        ars, acs = a_strides if a_strides is not None else (K, 1)
        brs, bcs = b_strides if b_strides is not None else (N, 1)
        d.A = Operand(A, ars, acs, a_batch[0], a_batch[1])
        d.B = Operand(B, brs, bcs, b_batch[0], b_batch[1])
        d.C = Cptr
        d.ldc = N if ldc is None else ldc
        d.c_batch_stride = M * N if c_batch_stride is None else c_batch_stride
        d.bias = bias
        d.epilogue = epilogue
        d.accumulate = 1 if accumulate else 0
        d.split_k = split_k
        d.algo = algo
        d.aux = aux
        d.colsum_part = colsum_part
        return d

    def yardstick_timed(self, kind, nbytes, dst=None, srcs=(), nontemporal=True, blocks_per_cu=8, warmup=5, iters=50):
        """Average ms per launch of a streaming kernel: kind "empty", "read", "write" or "copy"."""
        code = {"empty": 0, "read": 1, "write": 2, "copy": 3}[kind]
        arr = (C.c_void_p * max(len(srcs), 1))(*srcs)
        ms = C.c_float(0)
        self._check(self.lib.mni_rocm_yardstick_timed(code, 1 if nontemporal else 0, dst, arr, len(srcs), nbytes, blocks_per_cu,
                                                      warmup, iters, C.byref(ms)))
        return ms.value

    def mfma_yardstick(self, valu_per_mfma=0, waves_per_simd=2, mfmas_per_wave=32768, warmup=2, iters=5):
        """TFLOP/s of a loop of nothing but fp32 MFMAs with `valu_per_mfma` independent v_mov_b32 behind each."""
        ms = C.c_float(0)
        self._check(self.lib.mni_rocm_mfma_yardstick_timed(valu_per_mfma, waves_per_simd, mfmas_per_wave, warmup, iters, C.byref(ms)))
        cus = self.device_info()["compute_units"]
        return cus * 4 * waves_per_simd * mfmas_per_wave * 4096.0 / (ms.value * 1e-3) / 1e12

    def strided_copy(self, dst, src, shape, strides):
        self._check(self.lib.mni_rocm_strided_copy(dst, src, _i64_array(shape), _i64_array(strides), len(shape)))

    def add_bias(self, out, a, bias, rows, cols):
        self._check(self.lib.mni_rocm_add_bias(out, a, bias, rows, cols))

    def colsum(self, out, a, rows, cols):
        self._check(self.lib.mni_rocm_colsum(out, a, rows, cols))

    def unbroadcast(self, out, g, g_shape, to_shape):
        gs = (C.c_int64 * max(len(g_shape), 1))(*g_shape)
        ts = (C.c_int64 * max(len(to_shape), 1))(*to_shape)
        self._check(self.lib.mni_rocm_unbroadcast(out, g, gs, len(g_shape), ts, len(to_shape)))

    def axpy(self, dst, src, alpha, n):
        self._check(self.lib.mni_rocm_axpy(dst, src, alpha, n))

    def fill(self, dst, value, n):
        self._check(self.lib.mni_rocm_fill(dst, value, n))


class Native:
    """Engine-level ABI under the reference's N-API export names."""

    name = "rocm"

    def __init__(self):
        self.lib = load_library()

    def _err(self):
        return MniError(self.lib.mni_rocm_last_error().decode())

    def _id(self, v):
        if v == BAD_ID:
            raise self._err()
        return v

    def _rc(self, rc):
        if rc != 0:
            raise self._err()

    # creation / transfer
    def zeros(self, shape):
        return self._id(self.lib.mni_zeros(_i64_array(shape), len(shape)))

    def ones(self, shape):
        return self._id(self.lib.mni_ones(_i64_array(shape), len(shape)))

    def fromFloat32(self, data, shape):
        a = np.ascontiguousarray(data, dtype=np.float32)
        return self._id(self.lib.mni_from_float32(a.ctypes.data, a.size, _i64_array(shape), len(shape)))

    def tensorShape(self, id):
        out = (C.c_int64 * MAX_DIMS)()
        nd = self.lib.mni_tensor_shape(id, out, MAX_DIMS)
        if nd < 0:
            raise self._err()
        return [int(out[i]) for i in range(nd)]

    def tensorSize(self, id):
        n = self.lib.mni_tensor_size(id)
        if n < 0:
            raise self._err()
        return int(n)

    def toFloat32(self, id):
        out = np.empty(self.tensorSize(id), dtype=np.float32)
        self._rc(self.lib.mni_to_float32(id, out.ctypes.data, out.size))
        return out

    def getScalar(self, id):
        v = C.c_double(0)
        self._rc(self.lib.mni_get_scalar(id, C.byref(v)))
        return v.value

    def freeTensor(self, id):
        self.lib.mni_free_tensor(id)

    def setRequiresGrad(self, id, requires):
        self._rc(self.lib.mni_set_requires_grad(id, 1 if requires else 0))

    def getGrad(self, id):
        out = C.c_uint32(0)
        r = self.lib.mni_get_grad(id, C.byref(out))
        if r < 0:
            raise self._err()
        return out.value if r == 1 else None

    # autograd
    def backward(self, loss):
        self._rc(self.lib.mni_backward(loss))

    def zeroGrad(self, ids):
        self._rc(self.lib.mni_zero_grad(_u32_array(ids), len(ids)))

    def noGradStart(self):
        self.lib.mni_no_grad_start()

    def noGradEnd(self):
        self.lib.mni_no_grad_end()

    # ops
    def add(self, a, b):
        return self._id(self.lib.mni_add(a, b))

    def mul(self, a, b):
        return self._id(self.lib.mni_mul(a, b))

    def sub(self, a, b):
        return self._id(self.lib.mni_sub(a, b))

    def neg(self, a):
        return self._id(self.lib.mni_neg(a))

    def mulScalar(self, a, s):
        return self._id(self.lib.mni_mul_scalar(a, float(s)))

    def matmul(self, a, b):
        return self._id(self.lib.mni_matmul(a, b))

    def linear(self, x, w, bias, act=EPI_BIAS):
        return self._id(self.lib.mni_linear(x, w, bias, act))

    def mseLoss(self, pred, target):
        return self._id(self.lib.mni_mse_loss(pred, target))

    def gelu(self, a):
        return self._id(self.lib.mni_gelu(a))

    def relu(self, a):
        return self._id(self.lib.mni_relu(a))

    def sumOp(self, a, dim):
        return self._id(self.lib.mni_sum_op(a, dim))

    def meanOp(self, a, dim):
        return self._id(self.lib.mni_mean_op(a, dim))

    def sumAll(self, a):
        return self._id(self.lib.mni_sum_all(a))

    def meanAll(self, a):
        return self._id(self.lib.mni_mean_all(a))

    def view(self, a, shape):
        return self._id(self.lib.mni_view(a, _i64_array(shape), len(shape)))

    def permute(self, a, dims):
        return self._id(self.lib.mni_permute(a, _i64_array(dims), len(dims)))

    def contiguous(self, a):
        return self._id(self.lib.mni_contiguous(a))

    def softmaxOp(self, a, dim):
        return self._id(self.lib.mni_softmax_op(a, dim))

    def biasGelu(self, x, bias):
        return self._id(self.lib.mni_bias_gelu(x, bias))

    def kvCacheCreate(self, batchSize, numHeads, headDim, maxSeqLen, quantized):
        return self._id(self.lib.mni_kv_cache_create(batchSize, numHeads, headDim, maxSeqLen, 1 if quantized else 0))

    def kvCacheLen(self, cacheId):
        return self.lib.mni_kv_cache_len(cacheId)

    def kvCacheQuantized(self, cacheId):
        return bool(self.lib.mni_kv_cache_quantized(cacheId))

    def kvCacheReset(self, cacheId):
        self.lib.mni_kv_cache_reset(cacheId)

    def kvCacheFree(self, cacheId):
        self.lib.mni_kv_cache_free(cacheId)

    def kvCacheAppend(self, cacheId, k, v):
        self._rc(self.lib.mni_kv_cache_append(cacheId, k, v))

    def kvCacheDecodeStep(self, cacheId, q, k, v, scale):
        return self._id(self.lib.mni_kv_cache_decode_step(cacheId, q, k, v, scale))

    def expOp(self, a):
        return self._id(self.lib.mni_exp_op(a))

    def logOp(self, a):
        return self._id(self.lib.mni_log_op(a))

    def sigmoid(self, a):
        return self._id(self.lib.mni_sigmoid(a))

    def powOp(self, a, exponent):
        return self._id(self.lib.mni_pow_op(a, exponent))

    def div(self, a, b):
        return self._id(self.lib.mni_div(a, b))

    def lt(self, a, b):
        return self._id(self.lib.mni_lt(a, b))

    def eqOp(self, a, b):
        return self._id(self.lib.mni_eq_op(a, b))

    def gt(self, a, b):
        return self._id(self.lib.mni_gt(a, b))

    def isClose(self, a, b, tol):
        return self._id(self.lib.mni_is_close(a, b, tol))

    def maxOp(self, a, dim):
        return self._id(self.lib.mni_max_op(a, dim))

    def layernormOp(self, x, gamma, beta, eps):
        return self._id(self.lib.mni_layernorm_op(x, gamma, beta, eps))

    def flashAttention(self, q, k, v, scale, causal):
        return self._id(self.lib.mni_flash_attention(q, k, v, scale, 1 if causal else 0))

    def crossEntropyLoss(self, logits, targets):
        return self._id(self.lib.mni_cross_entropy_loss(logits, _i64_array(targets), len(targets)))

    # token-side ops
    def randTensor(self, shape):
        return self._id(self.lib.mni_rand_tensor(_i64_array(shape), len(shape)))

    def randnTensor(self, shape):
        return self._id(self.lib.mni_randn_tensor(_i64_array(shape), len(shape)))

    def seed(self, seed):
        self._rc(self.lib.mni_seed(seed))

    def philoxWords(self, seed, offset, n):
        out = np.empty(n, dtype=np.uint32)
        self._rc(self.lib.mni_philox_words(seed, offset, out.ctypes.data, n))
        return out

    def dropoutOp(self, x, rate, training):
        return self._id(self.lib.mni_dropout_op(x, rate, 1 if training else 0))

    def createDataset(self, data):
        a = np.ascontiguousarray(data, dtype=np.int32)
        return self._id(self.lib.mni_create_dataset(a.ctypes.data, a.size))

    def sampleBatch(self, datasetId, blockSize, batchSize):
        out = (C.c_uint32 * 2)()
        self._rc(self.lib.mni_sample_batch(datasetId, blockSize, batchSize, out))
        return [int(out[0]), int(out[1])]

    def freeIntBuffer(self, id):
        self._rc(self.lib.mni_free_int_buffer(id))

    def intBufferToHost(self, id):
        n = self.lib.mni_int_buffer_len(id)
        if n < 0:
            raise self._err()
        out = np.empty(n, dtype=np.int32)
        self._rc(self.lib.mni_int_buffer_to_host(id, out.ctypes.data, n))
        return out

    def embeddingForward(self, weight, indices, batch, seqLen):
        idx = np.ascontiguousarray(indices, dtype=np.int64)  # a numpy array passes through without a per-element copy
        return self._id(self.lib.mni_embedding_forward(weight, idx.ctypes.data_as(_i64p), idx.size, batch, seqLen))

    def embeddingForwardGpu(self, weight, intBufId, batch, seqLen):
        return self._id(self.lib.mni_embedding_forward_gpu(weight, intBufId, batch, seqLen))

    def crossEntropyLossGpu(self, logits, intBufId):
        return self._id(self.lib.mni_cross_entropy_loss_gpu(logits, intBufId))

    def residualLayernorm(self, x, residual, gamma, beta, eps):
        return self._id(self.lib.mni_residual_layernorm(x, residual, gamma, beta, eps))

    def scaleGrads(self, ids, invScale):
        found = C.c_int(0)
        self._rc(self.lib.mni_scale_grads(_u32_array(ids), len(ids), invScale, C.byref(found)))
        return bool(found.value)

    def tile(self, a, reps):
        return self._id(self.lib.mni_tile(a, _i64_array(reps), len(reps)))

    # optimiser
    def adamwStep(self, ids, lr, beta1, beta2, eps, weight_decay, step):
        self._rc(self.lib.mni_adamw_step(_u32_array(ids), len(ids), lr, beta1, beta2, eps, weight_decay, step))

    def gradNorm(self, ids):
        v = self.lib.mni_grad_norm(_u32_array(ids), len(ids))
        if v < 0:
            raise self._err()
        return v

    def clipGradNorm(self, ids, max_norm):
        self._rc(self.lib.mni_clip_grad_norm(_u32_array(ids), len(ids), max_norm))

    def clipAndStep(self, ids, lr, beta1, beta2, eps, weight_decay, step, max_grad_norm):
        v = self.lib.mni_clip_and_step(_u32_array(ids), len(ids), lr, beta1, beta2, eps, weight_decay, step, max_grad_norm)
        if v < 0:
            raise self._err()
        return v

    # lifecycle
    def resetEngine(self):
        self.lib.mni_reset_engine()

    def gcTensors(self, keep):
        self._rc(self.lib.mni_gc_tensors(_u32_array(keep), len(keep)))

    def devPtr(self, id):
        p = self.lib.mni_dev_ptr(id)
        if not p:
            raise self._err()
        return p
