"""ctypes binding of libfoundry_attn.so (the C ABI declared in include/foundry_attn.h).

Host-side plumbing for tests, the smoke check and the benchmark: it loads the library, declares the
prototypes and keeps device buffers alive. It does no arithmetic of its own and has no fallback: if the
library is missing or a call fails, it raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FOUNDRY_ATTN_LIB") or os.path.join(HERE, "libfoundry_attn.so")  # the override is for development builds

FA_OK = 0
STATUS_NAMES = {
    0: "Ok", 1: "DeviceNotFound", 2: "NullPointer", 3: "InvalidShape", 4: "OutOfMemory",
    5: "OperationNotSupported", 6: "InvalidOperation", 7: "UnsupportedDtype", 8: "OperationFailed",
    9: "InputNotFound",
}
DTYPE_F32, DTYPE_F16, DTYPE_BF16, DTYPE_I8, DTYPE_I32, DTYPE_U32 = 0, 1, 2, 15, 17, 20
DTYPE_Q4_0, DTYPE_Q8_0, DTYPE_U8 = 3, 7, 18  # block-quantised weight policies (metallic-sdk's Dtype order), raw bytes
ROPE_NEOX, ROPE_NORMAL = 0, 1


class FoundryError(RuntimeError):
    """The library's error convention: a MetalError-like variant name plus message."""

    def __init__(self, status, message):
        self.status = status
        self.variant = STATUS_NAMES.get(status, "Unknown")
        self.dtype = load().fa_last_error_dtype() if status == 7 else None  # UnsupportedDtype names the refused dtype
        super().__init__("%s: %s" % (self.variant, message))


class TensorArg(C.Structure):
    _fields_ = [("buffer", C.c_void_p), ("offset", C.c_size_t), ("dtype", C.c_uint32), ("rank", C.c_uint32),
                ("dims", C.c_size_t * 4), ("strides", C.c_size_t * 4)]


class KvPrepFusedParams(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "d_model", "kv_dim", "head_dim", "n_heads", "n_kv_heads", "group_size", "seq_len", "position_offset",
        "max_seq_len", "total_elements", "rope_mode", "layer_idx", "no_rope_layer_step")]

    @classmethod
    def make(cls, n_heads, n_kv_heads, head_dim, seq_len, position_offset, max_seq_len, rope_mode=ROPE_NORMAL,
             layer_idx=0, no_rope_layer_step=0):
        return cls(n_heads * head_dim, n_kv_heads * head_dim, head_dim, n_heads, n_kv_heads, n_heads // n_kv_heads,
                   seq_len, position_offset, max_seq_len, n_heads * seq_len * head_dim, rope_mode, layer_idx,
                   no_rope_layer_step)


class FusedQkvParams(C.Structure):
    """fa_fused_qkv_params (FusedQkvArgs scalars, src/metals/gemv/qkv_step.rs:57-99)."""
    _fields_ = [("k_dim", C.c_uint32), ("n_dim", C.c_uint32), ("n_kv", C.c_uint32), ("m", C.c_uint32),
                ("weights_per_block", C.c_uint32), ("layout", C.c_uint32), ("epsilon", C.c_float)]


WEIGHT_LAYOUT_ROW_MAJOR, WEIGHT_LAYOUT_CANONICAL = 0, 1


class MatMulParams(C.Structure):
    """fa_matmul_params (MatMulStep scalars, src/metals/matmul.rs:11-31)."""
    _fields_ = [("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("transpose_a", C.c_uint32),
                ("transpose_b", C.c_uint32), ("alpha", C.c_float), ("beta", C.c_float), ("weights_per_block", C.c_uint32),
                ("activation", C.c_uint32)]


class SageCache(C.Structure):
    _fields_ = [("k_q", C.c_void_p), ("k_scale", C.c_void_p), ("k_tail", C.c_void_p), ("v", C.c_void_p), ("q_q", C.c_void_p),
                ("k_mean", C.c_void_p), ("q_scale", C.c_void_p), ("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32),
                ("capacity", C.c_uint32), ("head_dim", C.c_uint32)]


class DecodeVariant(C.Structure):
    _fields_ = [("keys_per_split", C.c_uint32), ("merge", C.c_uint32)]


class PagedKv(C.Structure):
    _fields_ = [("k_pool", C.c_void_p), ("v_pool", C.c_void_p), ("block_table", C.c_void_p),
                ("seq_lens", C.c_void_p), ("n_blocks", C.c_uint32), ("n_kv_heads", C.c_uint32),
                ("block_size", C.c_uint32), ("head_dim", C.c_uint32), ("n_seqs", C.c_uint32),
                ("max_blocks_per_seq", C.c_uint32)]


_PT = C.POINTER(TensorArg)
_vp, _u32, _sz, _i = C.c_void_p, C.c_uint32, C.c_size_t, C.c_int

# name -> argtypes (restype is int status unless listed in _RESTYPES)
PROTOTYPES = {
    "fa_status_name": [_i],
    "fa_last_error_string": [],
    "fa_last_error_dtype": [],
    "fa_version": [],
    "fa_ctx_create": [_i, C.POINTER(_vp)],
    "fa_ctx_destroy": [_vp],
    "fa_synchronize": [_vp],
    "fa_ctx_stream": [_vp],
    "fa_ctx_reserve_workspace": [_vp, _sz],
    "fa_start_capture": [_vp],
    "fa_end_capture": [_vp, C.POINTER(_vp)],
    "fa_graph_launch": [_vp, _vp],
    "fa_graph_destroy": [_vp],
    "fa_is_capturing": [_vp],
    "fa_profile_enable": [_vp, _i],
    "fa_profile_reset": [_vp],
    "fa_profile_query": [_vp, C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_double)],
    "fa_profile_clock_buffer": [_vp, _vp, _u32],
    "fa_compute_units": [_vp, C.POINTER(_u32)],
    "fa_stream_timer_start": [_vp],
    "fa_stream_timer_stop": [_vp, C.POINTER(C.c_float)],
    "fa_device_alloc": [_vp, _sz, C.POINTER(_vp)],
    "fa_device_free": [_vp, _vp],
    "fa_upload": [_vp, _vp, _sz, _vp, _sz],
    "fa_download": [_vp, _vp, _vp, _sz, _sz],
    "fa_device_memset": [_vp, _vp, _i, _sz],
    "fa_device_copy": [_vp, _vp, _sz, _vp, _sz, _sz],
    "fa_u32_add": [_vp, _vp, _u32, _u32],
    "fa_rope_tables_f16": [C.c_float, _u32, _u32, _u32, _vp, _vp, _vp],
    "fa_kv_prep_fused": [_vp, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, C.POINTER(KvPrepFusedParams)],
    "fa_kv_prep_fused_dyn": [_vp, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, C.POINTER(KvPrepFusedParams), _vp],
    "fa_flash_attention": [_vp, _PT, _PT, _PT, _PT, _i, _u32, _u32, _u32, _u32, _u32, _i],
    "fa_flash_decode_dyn": [_vp, _PT, _PT, _PT, _PT, _u32, _u32, _vp, _u32, _u32],
    "fa_decode_step_fused": [_vp, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, C.POINTER(KvPrepFusedParams), _vp, _u32],
    "fa_decode_step_fused_noalloc": [_vp, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, _PT, C.POINTER(KvPrepFusedParams), _vp, _u32],
    "fa_noalloc_scratch_bytes": [],
    "fa_decode_step_fused_paged": [_vp, _PT, _PT, _PT, _PT, C.POINTER(PagedKv), _PT, _PT, _PT,
                                   C.POINTER(KvPrepFusedParams), _u32],
    "fa_set_decode_variant": [_vp, C.POINTER(DecodeVariant)],
    "fa_set_decode_poll_spin_us": [_vp, C.c_uint32],
    "fa_set_prefill_split_k": [_vp, C.c_uint32],
    "fa_set_prefill_variant": [_vp, C.c_uint32],
    "fa_set_sage_step_variant": [_vp, C.c_uint32],
    "fa_set_gemm_min_m": [_vp, C.c_uint32],
    "fa_set_gemm_variant": [_vp, C.c_uint32],
    "fa_kv_prep_fused_paged": [_vp, _PT, _PT, _PT, _PT, C.POINTER(PagedKv), _u32, _PT, _PT,
                               C.POINTER(KvPrepFusedParams)],
    "fa_kv_prep_decode_paged": [_vp, _PT, _PT, _PT, _PT, C.POINTER(PagedKv), _PT, _PT, C.POINTER(KvPrepFusedParams)],
    "fa_flash_decode_paged": [_vp, _PT, C.POINTER(PagedKv), _PT, _u32, _u32, _u32],
    "fa_flash_prefill_paged": [_vp, _PT, C.POINTER(PagedKv), _u32, _PT, _i, _u32, _u32, _u32, _u32],
    "fa_paged_gather": [_vp, C.POINTER(PagedKv), _u32, _u32, _vp, _vp, _u32],
    "fa_paged_copy_blocks": [_vp, C.POINTER(PagedKv), _vp, _vp, _u32],
    "fa_fused_qkv": [_vp] + [_PT] * 14 + [C.POINTER(FusedQkvParams)],
    "fa_fused_qkv_kv_prep": [_vp] + [_PT] * 11 + [C.POINTER(FusedQkvParams)] + [_PT] * 5 + [C.POINTER(KvPrepFusedParams)],
    "fa_fused_qkv_kv_prep_paged": [_vp] + [_PT] * 11 + [C.POINTER(FusedQkvParams), _PT, C.POINTER(PagedKv), _u32, _PT, _PT,
                                   C.POINTER(KvPrepFusedParams)],
    "fa_matmul": [_vp] + [_PT] * 6 + [C.POINTER(MatMulParams)],
    "fa_kv_prefix_copy": [_vp, _PT, _PT, _sz],
    "fa_kv_prefix_copy_batch": [_vp, _PT, _PT, _u32, _sz],
    "fa_align_capacity": [_sz],
    "fa_grown_capacity": [_sz, _sz, _sz, C.c_float],
    "fa_sage_k_mean": [_vp, _vp, _u32, _u32, _u32, _u32, _vp],
    "fa_sage_quantize_k": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _vp, _vp],
    "fa_sage_quantize_q": [_vp, _vp, _u32, _u32, _vp, _vp],
    "fa_sage_decode": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32],
    "fa_sage_cache_build": [_vp, _vp, _u32, C.POINTER(SageCache)],
    "fa_sage_decode_step": [_vp, _PT, _PT, _PT, C.POINTER(SageCache), _PT, _PT, _PT, C.POINTER(KvPrepFusedParams), _vp, _u32],
    "fa_rope": [_vp, _PT, _PT, _PT, _PT, _vp],
    "fa_kv_cache_write": [_vp, _PT, _PT, _vp],
    "fa_kv_cache_write_repeat_kv_heads": [_vp, _PT, _PT, _vp],
    "fa_kv_cache_read": [_vp, _PT, _PT, _vp],
    "fa_kv_rearrange": [_vp, _PT, _PT, _vp],
    "fa_repeat_kv_heads": [_vp, _PT, _PT, _vp],
    "fa_sdpa_reference": [_vp, _PT, _PT, _PT, _PT, _i, _u32, _u32, _u32, _u32, _u32, _i],
    "fa_measure_clock": [_vp, _i, _u32, C.POINTER(C.c_float), C.POINTER(C.c_float)],
    "fa_device_info": [_vp, C.c_char_p, _sz, C.POINTER(_u32), C.POINTER(C.c_uint64)],
    "fa_device_mem_info": [_vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
}
_RESTYPES = {"fa_status_name": C.c_char_p, "fa_last_error_string": C.c_char_p, "fa_version": C.c_char_p,
             "fa_ctx_stream": _vp, "fa_is_capturing": _i, "fa_align_capacity": _sz, "fa_grown_capacity": _sz,
             "fa_noalloc_scratch_bytes": _sz, "fa_last_error_dtype": _u32}

_lib = None


def canonical_layout(w, weights_per_block=32):
    """[n_rows, k_dim] row-major weights -> the flat canonical blocked order FusedQkv and MatMul read
    (element (row, k) at (k % wpb) + wpb * (row + (k // wpb) * n_rows); metallic-loader lays tensors out this way)."""
    n, k = w.shape
    kk = np.arange(k)
    idx = (kk % weights_per_block)[None, :] + weights_per_block * (np.arange(n)[:, None] + (kk // weights_per_block)[None, :] * n)
    out = np.empty(n * k, w.dtype)
    out[idx.reshape(-1)] = w.reshape(-1)
    return out


def align_capacity(capacity):
    return load().fa_align_capacity(capacity)


def grown_capacity(allocated, required_len, max_context_len, growth_factor=2.0):
    """0 = required_len exceeds max_context_len (the reference raises InvalidOperation there)."""
    return load().fa_grown_capacity(allocated, required_len, max_context_len, growth_factor)


def load():
    """Loads the shared library and declares every prototype; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `python test-burn_amd/build.py` (there is no CPU fallback)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, argtypes in PROTOTYPES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, _i)
        _lib = lib
    return _lib


def check(status):
    if status != FA_OK:
        raise FoundryError(status, load().fa_last_error_string().decode())


_NP_DTYPE = {np.dtype(np.float16): DTYPE_F16, np.dtype(np.float32): DTYPE_F32, np.dtype(np.int8): DTYPE_I8,
             np.dtype(np.int32): DTYPE_I32, np.dtype(np.uint32): DTYPE_U32, np.dtype(np.uint8): DTYPE_U8}


class DevBuf:
    """A device allocation with numpy-style shape/dtype metadata."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = _vp()
        check(ctx.lib.fa_device_alloc(ctx.h, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.nbytes == self.nbytes, (arr.shape, self.shape)
        check(self.ctx.lib.fa_upload(self.ctx.h, self.ptr, 0, arr.ctypes.data, arr.nbytes))
        return self

    def download(self):
        out = np.empty(self.shape, self.dtype)
        check(self.ctx.lib.fa_download(self.ctx.h, out.ctypes.data, self.ptr, 0, self.nbytes))
        return out

    def zero(self):
        check(self.ctx.lib.fa_device_memset(self.ctx.h, self.ptr, 0, self.nbytes))
        return self

    def arg(self, dims=None, strides=None, offset=0, dtype=None):
        """TensorArg view: dims default to the buffer shape, strides to row-major."""
        dims = self.shape if dims is None else tuple(dims)
        if strides is None:
            strides, acc = [], 1
            for d in reversed(dims):
                strides.append(acc)
                acc *= d
            strides = tuple(reversed(strides))
        t = TensorArg()
        t.buffer, t.offset = self.ptr, offset
        t.dtype = _NP_DTYPE[self.dtype] if dtype is None else dtype
        t.rank = len(dims)
        for i, (d, s) in enumerate(zip(dims, strides)):
            t.dims[i], t.strides[i] = d, s
        return t

    def free(self):
        if self.ptr:
            check(self.ctx.lib.fa_device_free(self.ctx.h, self.ptr))
            self.ptr = None


class Graph:
    def __init__(self, ctx, handle):
        self.ctx, self.h = ctx, handle

    def launch(self):
        check(self.ctx.lib.fa_graph_launch(self.ctx.h, self.h))

    def destroy(self):
        if self.h:
            self.ctx.lib.fa_graph_destroy(self.h)
            self.h = None


class Foundry:
    """Context handle: the counterpart of the reference's `Foundry` for this path."""

    def __init__(self, device=0):
        self.lib = load()
        h = _vp()
        check(self.lib.fa_ctx_create(device, C.byref(h)))
        self.h = h.value

    # -- lifecycle
    def close(self):
        if self.h:
            self.lib.fa_ctx_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def synchronize(self):
        check(self.lib.fa_synchronize(self.h))

    def start_capture(self):
        check(self.lib.fa_start_capture(self.h))

    def end_capture(self):
        g = _vp()
        check(self.lib.fa_end_capture(self.h, C.byref(g)))
        return Graph(self, g.value)

    def reserve_workspace(self, nbytes):
        check(self.lib.fa_ctx_reserve_workspace(self.h, nbytes))

    def set_decode_variant(self, keys_per_split=0, merge=2):
        """No arguments: the library's defaults (partition size by the launch rule, separate merge kernel)."""
        v = DecodeVariant(keys_per_split, merge)
        check(self.lib.fa_set_decode_variant(self.h, C.byref(v)))

    def set_decode_poll_spin_us(self, spin_us):
        """How long a merging workgroup of the polled decode merge waits for the other partitions' records."""
        check(self.lib.fa_set_decode_poll_spin_us(self.h, spin_us))

    def set_gemm_variant(self, variant=0):
        """0 = auto; 1 = GEMM operand tiles through registers; 2 / 3 = straight into LDS in steps of 64 / 32 features."""
        check(self.lib.fa_set_gemm_variant(self.h, variant))

    def set_gemm_min_m(self, min_m=0):
        """Input rows from which FusedQkv / MatMul run as a GEMM; 0 = the library's default."""
        check(self.lib.fa_set_gemm_min_m(self.h, min_m))

    def set_prefill_split_k(self, split_k=0):
        check(self.lib.fa_set_prefill_split_k(self.h, split_k))

    def set_prefill_variant(self, variant):
        check(self.lib.fa_set_prefill_variant(self.h, variant))

    def profile_enable(self, on=True):
        check(self.lib.fa_profile_enable(self.h, int(on)))

    def profile_reset(self):
        check(self.lib.fa_profile_reset(self.h))

    def profile_query(self, prefix):
        n, ms = C.c_uint64(), C.c_double()
        check(self.lib.fa_profile_query(self.h, prefix.encode(), C.byref(n), C.byref(ms)))
        return n.value, ms.value

    def device_info(self):
        name = C.create_string_buffer(256)
        cus, mem = _u32(), C.c_uint64()
        check(self.lib.fa_device_info(self.h, name, 256, C.byref(cus), C.byref(mem)))
        return name.value.decode(), cus.value, mem.value

    def device_mem_info(self):
        """(free, total) bytes of device memory right now."""
        free, total = C.c_uint64(), C.c_uint64()
        check(self.lib.fa_device_mem_info(self.h, C.byref(free), C.byref(total)))
        return free.value, total.value

    # -- memory
    def empty(self, shape, dtype=np.float16):
        return DevBuf(self, shape, dtype)

    def zeros(self, shape, dtype=np.float16):
        return DevBuf(self, shape, dtype).zero()

    def array(self, arr):
        arr = np.ascontiguousarray(arr)
        return DevBuf(self, arr.shape, arr.dtype).upload(arr)

    def u32_add(self, buf, n, delta):
        check(self.lib.fa_u32_add(self.h, buf.ptr, n, delta))

    # -- ops (thin: build the structs, call, check)
    def kv_prep_fused(self, q, k, v, q_rot, k_cache, v_cache, cos, sin, params, d_position=None):
        a = [C.byref(x) for x in (q, k, v, q_rot, k_cache, v_cache, cos, sin)]
        if d_position is None:
            check(self.lib.fa_kv_prep_fused(self.h, *a, C.byref(params)))
        else:
            check(self.lib.fa_kv_prep_fused_dyn(self.h, *a, C.byref(params), d_position.ptr))

    def flash_attention(self, q, k, v, out, causal, query_offset, n_heads, head_dim, kv_seq_len, m,
                        kv_head_major=True):
        check(self.lib.fa_flash_attention(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(out), int(causal),
                                          query_offset, n_heads, head_dim, kv_seq_len, m, int(kv_head_major)))

    def flash_decode_dyn(self, q, k, v, out, n_heads, head_dim, d_position, kv_len_add, kv_len_bound):
        check(self.lib.fa_flash_decode_dyn(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(out), n_heads, head_dim,
                                           d_position.ptr, kv_len_add, kv_len_bound))

    def decode_step_fused(self, q, k, v, q_rot, k_cache, v_cache, cos, sin, out, params, d_position=None,
                          kv_len_bound=0, noalloc=False):
        if q_rot is None:
            q_rot = TensorArg()
        a = [C.byref(x) for x in (q, k, v, q_rot, k_cache, v_cache, cos, sin, out)]
        fn = self.lib.fa_decode_step_fused_noalloc if noalloc else self.lib.fa_decode_step_fused
        check(fn(self.h, *a, C.byref(params), None if d_position is None else d_position.ptr, kv_len_bound))

    def decode_step_fused_paged(self, q, k, v, q_rot, cache, cos, sin, out, params, kv_len_bound):
        if q_rot is None:
            q_rot = TensorArg()
        check(self.lib.fa_decode_step_fused_paged(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(q_rot),
                                                  C.byref(cache), C.byref(cos), C.byref(sin), C.byref(out),
                                                  C.byref(params), kv_len_bound))

    def kv_prep_fused_paged(self, q, k, v, q_rot, cache, seq_index, cos, sin, params):
        check(self.lib.fa_kv_prep_fused_paged(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(q_rot),
                                              C.byref(cache), seq_index, C.byref(cos), C.byref(sin), C.byref(params)))

    def kv_prep_decode_paged(self, q, k, v, q_rot, cache, cos, sin, params):
        check(self.lib.fa_kv_prep_decode_paged(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(q_rot),
                                               C.byref(cache), C.byref(cos), C.byref(sin), C.byref(params)))

    def flash_decode_paged(self, q, cache, out, n_heads, kv_len_add, kv_len_bound):
        check(self.lib.fa_flash_decode_paged(self.h, C.byref(q), C.byref(cache), C.byref(out), n_heads, kv_len_add,
                                             kv_len_bound))

    def flash_prefill_paged(self, q, cache, seq_index, out, causal, query_offset, n_heads, kv_seq_len, m):
        check(self.lib.fa_flash_prefill_paged(self.h, C.byref(q), C.byref(cache), seq_index, C.byref(out), int(causal),
                                              query_offset, n_heads, kv_seq_len, m))

    def paged_gather(self, cache, seq_index, seq_len, k_out, v_out, out_capacity):
        check(self.lib.fa_paged_gather(self.h, C.byref(cache), seq_index, seq_len, k_out.ptr, v_out.ptr, out_capacity))

    def fused_qkv(self, x, w_q, w_k, w_v, out_q, out_k, out_v, k_dim, n_dim, n_kv, m=1, gamma=None, biases=None,
                  layout=WEIGHT_LAYOUT_CANONICAL, weights_per_block=32, epsilon=1e-6, scales=None):
        """All tensors as TensorArg; gamma None = no RMSNorm; biases None or (bias_q, bias_k, bias_v); scales None (F16
        weights) or (s_q, s_k, s_v) for Q8_0 weights."""
        p = FusedQkvParams(k_dim, n_dim, n_kv, m, weights_per_block, layout, epsilon)
        none = TensorArg()
        g = gamma if gamma is not None else none
        bq, bk, bv = biases if biases is not None else (none, none, none)
        sq, sk, sv = scales if scales is not None else (none, none, none)
        check(self.lib.fa_fused_qkv(self.h, C.byref(w_q), C.byref(sq), C.byref(w_k), C.byref(sk), C.byref(w_v), C.byref(sv),
                                    C.byref(x), C.byref(out_q), C.byref(out_k), C.byref(out_v), C.byref(bq), C.byref(bk),
                                    C.byref(bv), C.byref(g), C.byref(p)))

    def fused_qkv_kv_prep(self, x, w_q, w_k, w_v, k_dim, q_rot, cos, sin, params, k_cache=None, v_cache=None, paged=None,
                          seq_index=0, gamma=None, biases=None, layout=WEIGHT_LAYOUT_CANONICAL, weights_per_block=32,
                          epsilon=1e-6, scales=None):
        """FusedQkv + KvPrepFused in one op (params: KvPrepFusedParams; m = params.seq_len). Either k_cache and v_cache
        (contiguous) or paged (a PagedKv) and seq_index."""
        p = FusedQkvParams(k_dim, params.d_model, params.kv_dim, params.seq_len, weights_per_block, layout, epsilon)
        none = TensorArg()
        g = gamma if gamma is not None else none
        bq, bk, bv = biases if biases is not None else (none, none, none)
        sq, sk, sv = scales if scales is not None else (none, none, none)
        head = [C.byref(t) for t in (w_q, sq, w_k, sk, w_v, sv, x, bq, bk, bv, g)] + [C.byref(p), C.byref(q_rot)]
        if paged is None:
            check(self.lib.fa_fused_qkv_kv_prep(self.h, *head, C.byref(k_cache), C.byref(v_cache), C.byref(cos), C.byref(sin),
                                                C.byref(params)))
        else:
            check(self.lib.fa_fused_qkv_kv_prep_paged(self.h, *head, C.byref(paged), seq_index, C.byref(cos), C.byref(sin),
                                                      C.byref(params)))

    def matmul(self, a, b, output, m, n, k, bias=None, c=None, transpose_b=True, alpha=1.0, beta=0.0, transpose_a=False,
               weights_per_block=32, activation=0, b_scales=None):
        """output[m, n] = alpha * a[m, k] . b^T + bias + beta * c; b row-major [n, k] (transpose_b) or canonical; b_scales
        for Q8_0 weights."""
        p = MatMulParams(m, n, k, int(transpose_a), int(transpose_b), alpha, beta, weights_per_block, activation)
        none = TensorArg()
        check(self.lib.fa_matmul(self.h, C.byref(a), C.byref(b), C.byref(b_scales if b_scales is not None else none),
                                 C.byref(output), C.byref(bias if bias is not None else none),
                                 C.byref(c if c is not None else none), C.byref(p)))

    def paged_copy_blocks(self, cache, src_ids, dst_ids, n_pairs):
        """src_ids / dst_ids: device i32 buffers."""
        check(self.lib.fa_paged_copy_blocks(self.h, C.byref(cache), src_ids.ptr, dst_ids.ptr, n_pairs))

    def kv_prefix_copy(self, src, dst, prefix_len):
        """src, dst: TensorArg [heads, capacity, head_dim] (snapshot, restore and growth are this one copy)."""
        check(self.lib.fa_kv_prefix_copy(self.h, C.byref(src), C.byref(dst), prefix_len))

    def kv_prefix_copy_batch(self, srcs, dsts, prefix_len):
        n = len(srcs)
        assert n == len(dsts)
        sa, da = (TensorArg * max(n, 1))(*srcs), (TensorArg * max(n, 1))(*dsts)
        check(self.lib.fa_kv_prefix_copy_batch(self.h, sa, da, n, prefix_len))

    def sage_k_mean(self, k, n_kv_heads, capacity, head_dim, kv_len, mean_out):
        check(self.lib.fa_sage_k_mean(self.h, k.ptr, n_kv_heads, capacity, head_dim, kv_len, mean_out.ptr))

    def sage_quantize_k(self, k, mean, n_kv_heads, capacity, head_dim, row_begin, row_end, k_q, k_scale):
        check(self.lib.fa_sage_quantize_k(self.h, k.ptr, mean.ptr, n_kv_heads, capacity, head_dim, row_begin, row_end,
                                          k_q.ptr, k_scale.ptr))

    def sage_quantize_q(self, q, n_heads, head_dim, q_q, q_scale):
        check(self.lib.fa_sage_quantize_q(self.h, q.ptr, n_heads, head_dim, q_q.ptr, q_scale.ptr))

    def profile_clock_buffer(self, buf, n_workgroups):
        check(self.lib.fa_profile_clock_buffer(self.h, None if buf is None else buf.ptr, n_workgroups))

    def timer_start(self):
        check(self.lib.fa_stream_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        check(self.lib.fa_stream_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def n_cus(self):
        n = C.c_uint32()
        check(self.lib.fa_compute_units(self.h, C.byref(n)))
        return n.value

    def measure_clock(self, matrix_load, iterations):
        """(shader MHz, milliseconds the waves ran) under back-to-back MFMAs (matrix_load) or dependent FMAs."""
        mhz, ms = C.c_float(), C.c_float()
        check(self.lib.fa_measure_clock(self.h, int(matrix_load), iterations, C.byref(mhz), C.byref(ms)))
        return mhz.value, ms.value

    def legacy_op(self, name, tensors, params):
        """One of the un-fused ops (fa_rope, fa_kv_cache_write, ...): `params` is the tuple of u32 fields of its struct."""
        arr = (C.c_uint32 * len(params))(*params)
        check(getattr(self.lib, name)(self.h, *[C.byref(t) for t in tensors], C.cast(arr, C.c_void_p)))

    def sdpa_reference(self, q, k, v, out, causal, query_offset, n_heads, head_dim, kv_seq_len, m, kv_head_major=True):
        check(self.lib.fa_sdpa_reference(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(out), int(causal), query_offset,
                                         n_heads, head_dim, kv_seq_len, m, int(kv_head_major)))

    def sage_cache_build(self, k_f16, kv_len, cache):
        check(self.lib.fa_sage_cache_build(self.h, k_f16.ptr, kv_len, C.byref(cache)))

    def set_sage_step_variant(self, variant=0):
        """1 (default) = the int8 decode step as one launch, 2 = append kernel + decode kernel."""
        check(self.lib.fa_set_sage_step_variant(self.h, variant))

    def sage_decode_step(self, q, k, v, cache, cos, sin, out, params, d_position=None, kv_len_bound=0):
        check(self.lib.fa_sage_decode_step(self.h, C.byref(q), C.byref(k), C.byref(v), C.byref(cache), C.byref(cos),
                                           C.byref(sin), C.byref(out), C.byref(params),
                                           None if d_position is None else d_position.ptr, kv_len_bound))

    def sage_decode(self, q_q, q_scale, k_q, k_scale, v, out, n_heads, n_kv_heads, head_dim, capacity, kv_len):
        check(self.lib.fa_sage_decode(self.h, q_q.ptr, q_scale.ptr, k_q.ptr, k_scale.ptr, v.ptr, out.ptr, n_heads,
                                      n_kv_heads, head_dim, capacity, kv_len))


def sage_cache(ctx, n_heads, n_kv_heads, capacity, head_dim, v_buf):
    """Allocates the int8 state of one layer around an existing f16 V cache buffer; returns (descriptor, buffers)."""
    bufs = dict(k_q=ctx.zeros((n_kv_heads, capacity, head_dim), np.int8),
                k_scale=ctx.zeros((n_kv_heads, (capacity + 31) // 32), np.float16),
                k_tail=ctx.zeros((n_kv_heads, 32, head_dim), np.float16),
                q_q=ctx.zeros((n_heads, head_dim), np.int8), k_mean=ctx.zeros((n_kv_heads, head_dim), np.float32),
                q_scale=ctx.zeros((n_heads,), np.float32), v=v_buf)
    d = SageCache(bufs["k_q"].ptr, bufs["k_scale"].ptr, bufs["k_tail"].ptr, v_buf.ptr, bufs["q_q"].ptr, bufs["k_mean"].ptr,
                  bufs["q_scale"].ptr, n_heads, n_kv_heads, capacity, head_dim)
    return d, bufs


def rope_tables(rope_base, head_dim, n_pos, freq_factors=None, pos_begin=0):
    """Host RoPE tables through the library (fa_rope_tables_f16)."""
    half = head_dim // 2
    cos = np.empty((n_pos - pos_begin, half), np.float16)
    sin = np.empty((n_pos - pos_begin, half), np.float16)
    ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, dtype=np.float32)
    check(load().fa_rope_tables_f16(rope_base, head_dim, pos_begin, n_pos, None if ff is None else ff.ctypes.data,
                                    cos.ctypes.data, sin.ctypes.data))
    return cos, sin


def paged_kv(k_pool, v_pool, block_table, seq_lens, n_blocks, n_kv_heads, block_size, head_dim, n_seqs,
             max_blocks_per_seq):
    return PagedKv(k_pool.ptr, v_pool.ptr, block_table.ptr, None if seq_lens is None else seq_lens.ptr, n_blocks,
                   n_kv_heads, block_size, head_dim, n_seqs, max_blocks_per_seq)
