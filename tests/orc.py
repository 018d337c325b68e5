"""ctypes loader for the CPU oracle (oracle/liboracle_attn.so). Test infrastructure only.

The oracle takes IEEE binary16 tensors as uint16 buffers; the wrappers here accept and return
numpy float16 arrays.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_ORACLE_DIR = os.path.join(_ROOT, "oracle")
_SO = os.path.join(_ORACLE_DIR, "liboracle_attn.so")

u16p = C.POINTER(C.c_uint16)
f32p = C.POINTER(C.c_float)
i8p = C.POINTER(C.c_int8)
i32p = C.POINTER(C.c_int32)


class KvPrepParams(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "d_model", "kv_dim", "head_dim", "n_heads", "n_kv_heads", "group_size", "seq_len", "position_offset",
        "max_seq_len", "total_elements", "rope_mode", "layer_idx", "no_rope_layer_step")]


def build():
    subprocess.check_call(["make", "-s", "-C", _ORACLE_DIR, "liboracle_attn.so"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_max_threads.restype = C.c_int
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_set_elem_type.argtypes = [C.c_int]
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(t)


def _h(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


def f16_to_f32_n(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_f16_to_f32_n(_p(h, u16p), _p(out, f32p), C.c_size_t(h.size))
    return out


def f32_to_f16_n(f):
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().orc_f32_to_f16_n(_p(f, f32p), _p(out, u16p), C.c_size_t(f.size))
    return out


def rope_tables(base, head_dim, n_pos, freq_factors=None, pos_begin=0):
    half = head_dim // 2
    cos = np.empty((n_pos - pos_begin, half), np.float16)
    sin = np.empty((n_pos - pos_begin, half), np.float16)
    ff = None
    if freq_factors is not None:
        ff = np.ascontiguousarray(freq_factors, dtype=np.float32)
    lib().orc_rope_tables(C.c_float(base), C.c_uint32(head_dim), C.c_uint32(pos_begin), C.c_uint32(n_pos),
                          _p(ff, f32p) if ff is not None else None, _p(cos, u16p), _p(sin, u16p))
    return cos, sin


def rope_neox(x, cos, sin, dim, seq_len, position_offset):
    x = _h(x)
    out = np.empty_like(x)
    lib().orc_rope_neox(_p(x, u16p), _p(out, u16p), _p(_h(cos), u16p), _p(_h(sin), u16p), C.c_uint32(dim),
                        C.c_uint32(seq_len), C.c_uint32(position_offset), C.c_size_t(x.size))
    return out


def kv_rearrange(x, n_heads, n_kv_heads, head_dim, seq, batch=1):
    """[batch*seq, n_kv_heads*head_dim] -> [batch*n_heads, seq, head_dim] (GQA map h -> h/group)."""
    x = _h(x)
    kv_dim = n_kv_heads * head_dim
    out = np.zeros((batch * n_heads, seq, head_dim), np.float16)
    lib().orc_kv_rearrange(_p(x, u16p), _p(out, u16p), C.c_uint32(kv_dim), C.c_uint32(kv_dim), C.c_uint32(head_dim),
                           C.c_uint32(n_heads), C.c_uint32(n_kv_heads), C.c_uint32(head_dim), C.c_uint32(seq),
                           C.c_size_t(out.size))
    return out


def kv_cache_write(cache, x, n_kv_heads, head_dim, input_seq_len, position_offset, max_seq_len):
    assert cache.dtype == np.float16 and cache.flags.c_contiguous
    lib().orc_kv_cache_write(_p(cache, u16p), _p(_h(x), u16p), C.c_uint32(n_kv_heads), C.c_uint32(head_dim),
                             C.c_uint32(input_seq_len), C.c_uint32(position_offset), C.c_uint32(max_seq_len))


def kv_cache_write_repeat(cache, x, n_kv_heads, n_heads, head_dim, input_seq_len, position_offset, max_seq_len):
    assert cache.dtype == np.float16 and cache.flags.c_contiguous
    lib().orc_kv_cache_write_repeat(_p(cache, u16p), _p(_h(x), u16p), C.c_uint32(n_kv_heads), C.c_uint32(n_heads),
                                    C.c_uint32(n_heads // n_kv_heads), C.c_uint32(head_dim),
                                    C.c_uint32(input_seq_len), C.c_uint32(position_offset), C.c_uint32(max_seq_len))


def kv_cache_read(cache, n_kv_heads, head_dim, seq_len, max_seq_len):
    out = np.empty((n_kv_heads, seq_len, head_dim), np.float16)
    lib().orc_kv_cache_read(_p(_h(cache), u16p), _p(out, u16p), C.c_uint32(n_kv_heads), C.c_uint32(head_dim),
                            C.c_uint32(seq_len), C.c_uint32(max_seq_len))
    return out


def repeat_kv_heads(x, n_kv_heads, n_heads, seq, head_dim, cache_stride, batch=1):
    out = np.empty((batch * n_heads, seq, head_dim), np.float16)
    lib().orc_repeat_kv_heads(_p(_h(x), u16p), _p(out, u16p), C.c_uint32(n_heads // n_kv_heads), C.c_uint32(batch),
                              C.c_uint32(n_kv_heads), C.c_uint32(n_heads), C.c_uint32(seq), C.c_uint32(head_dim),
                              C.c_uint32(cache_stride))
    return out


def make_params(n_heads, n_kv_heads, head_dim, seq_len, position_offset, max_seq_len, rope_mode=0, layer_idx=0,
                no_rope_layer_step=0):
    return KvPrepParams(n_heads * head_dim, n_kv_heads * head_dim, head_dim, n_heads, n_kv_heads,
                        n_heads // n_kv_heads, seq_len, position_offset, max_seq_len,
                        n_heads * seq_len * head_dim, rope_mode, layer_idx, no_rope_layer_step)


def kv_prep_fused(q, k, v, k_cache, v_cache, cos, sin, params):
    """Appends into k_cache / v_cache in place and returns q_rot [n_heads, seq_len, head_dim]."""
    q_rot = np.empty((params.n_heads, params.seq_len, params.head_dim), np.float16)
    assert k_cache.dtype == np.float16 and k_cache.flags.c_contiguous
    assert v_cache.dtype == np.float16 and v_cache.flags.c_contiguous
    lib().orc_kv_prep_fused(_p(_h(q), u16p), _p(_h(k), u16p), _p(_h(v), u16p), _p(q_rot, u16p), _p(k_cache, u16p),
                            _p(v_cache, u16p), _p(_h(cos), u16p), _p(_h(sin), u16p), C.byref(params))
    return q_rot


def sdpa_decode(q, k, v, n_heads, n_kv_heads, head_dim, capacity, kv_len, scale=None, block_keys=256, warps=16,
                tg_out_half=False, n_threads=1):
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    out = np.empty((n_heads * head_dim,), np.float16)
    lib().orc_sdpa_decode(_p(_h(q), u16p), _p(_h(k), u16p), _p(_h(v), u16p), _p(out, u16p), C.c_uint32(n_heads),
                          C.c_uint32(n_kv_heads), C.c_uint32(head_dim), C.c_uint32(capacity), C.c_uint32(kv_len),
                          C.c_float(scale), C.c_uint32(block_keys), C.c_uint32(warps), C.c_int(int(tg_out_half)),
                          C.c_int(n_threads))
    return out


def sdpa_prefill(q, k, v, n_heads, n_kv_heads, head_dim, q_len, kv_len, query_offset, capacity, causal=True,
                 q_layout="head_major", out_layout="token_major", scale=None, tile_keys=32, n_threads=1):
    """q: head-major [H, q_len, D] or token-major [q_len, H*D]; K/V [Hkv, capacity, D]; out token-major
    [q_len, H*D] (the reference's attn_out layout) or head-major [H, q_len, D]."""
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    D = head_dim
    if q_layout == "head_major":
        qsh, qsm = q_len * D, D
    else:
        qsh, qsm = D, n_heads * D
    if out_layout == "token_major":
        out = np.zeros((q_len, n_heads * D), np.float16)
        osh, osm = D, n_heads * D
    else:
        out = np.zeros((n_heads, q_len, D), np.float16)
        osh, osm = q_len * D, D
    u64 = C.c_uint64
    lib().orc_sdpa_prefill(_p(_h(q), u16p), _p(_h(k), u16p), _p(_h(v), u16p), _p(out, u16p), C.c_uint32(n_heads),
                           C.c_uint32(n_heads // n_kv_heads), C.c_uint32(D), C.c_uint32(q_len), C.c_uint32(kv_len),
                           C.c_uint32(query_offset), C.c_int(int(causal)), C.c_float(scale), u64(qsh), u64(qsm),
                           u64(capacity * D), u64(D), u64(capacity * D), u64(D), u64(osh), u64(osm),
                           C.c_uint32(tile_keys), C.c_int(n_threads))
    return out


def sdpa_row_splitk(q_row, k_head, v_head, head_dim, kv_len, causal_limit, split_k, tile_keys=32, scale=None):
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    acc = np.zeros((split_k, head_dim), np.float32)
    m = np.zeros((split_k,), np.float32)
    l = np.zeros((split_k,), np.float32)
    lib().orc_sdpa_row_partials(_p(_h(q_row), u16p), _p(_h(k_head), u16p), _p(_h(v_head), u16p), C.c_uint32(head_dim),
                                C.c_uint64(head_dim), C.c_uint64(head_dim), C.c_uint32(kv_len),
                                C.c_uint32(causal_limit), C.c_float(scale), C.c_uint32(split_k), C.c_uint32(tile_keys),
                                _p(acc, f32p), _p(m, f32p), _p(l, f32p))
    out = np.empty((head_dim,), np.float16)
    lib().orc_splitk_merge(_p(acc, f32p), _p(m, f32p), _p(l, f32p), C.c_uint32(split_k), C.c_uint32(head_dim),
                           _p(out, u16p))
    return out, acc, m, l


def paged_gather(pool, block_table, n_kv_heads, block_size, head_dim, seq_len, out_capacity=None):
    if out_capacity is None:
        out_capacity = seq_len
    out = np.zeros((n_kv_heads, out_capacity, head_dim), np.float16)
    bt = np.ascontiguousarray(block_table, dtype=np.int32)
    lib().orc_paged_gather(_p(_h(pool), u16p), _p(bt, i32p), C.c_uint32(n_kv_heads), C.c_uint32(block_size),
                           C.c_uint32(head_dim), C.c_uint32(seq_len), C.c_uint32(out_capacity), _p(out, u16p))
    return out


def weight_index(layout, row, k, k_dim, n_rows, wpb=32):
    L = lib()
    L.orc_weight_index.restype = C.c_size_t
    return L.orc_weight_index(C.c_int(layout), C.c_size_t(row), C.c_size_t(k), C.c_size_t(k_dim), C.c_size_t(n_rows),
                              C.c_size_t(wpb))


def to_canonical(w, wpb=32):
    """[n_rows, k_dim] row-major -> the canonical blocked order (flat), by the layout's own index formula."""
    n, k = w.shape
    kk = np.arange(k)
    idx = (kk % wpb)[None, :] + wpb * (np.arange(n)[:, None] + (kk // wpb)[None, :] * n)
    out = np.empty(n * k, w.dtype)
    out[idx.reshape(-1)] = w.reshape(-1)
    return out


def fused_qkv(x, w_q, w_k, w_v, gamma=None, biases=None, layout=0, wpb=32, eps=1e-6, n_threads=8):
    """x [m, K]; w_* flat or 2-D in `layout`; returns (q [m, n_dim], k [m, n_kv], v [m, n_kv])."""
    x = _h(x)
    m, K = x.shape
    wq, wk, wv = (_h(np.asarray(w).reshape(-1)) for w in (w_q, w_k, w_v))
    n_dim, n_kv = wq.size // K, wk.size // K
    oq, ok, ov = np.zeros((m, n_dim), np.float16), np.zeros((m, n_kv), np.float16), np.zeros((m, n_kv), np.float16)
    g = _h(gamma) if gamma is not None else None
    bs = [_h(b) for b in biases] if biases is not None else [None] * 3
    nul = C.cast(None, u16p)
    lib().orc_fused_qkv(_p(x, u16p), _p(wq, u16p), _p(wk, u16p), _p(wv, u16p), _p(g, u16p) if g is not None else nul,
                        *[(_p(b, u16p) if b is not None else nul) for b in bs], _p(oq, u16p), _p(ok, u16p), _p(ov, u16p),
                        C.c_uint32(K), C.c_uint32(n_dim), C.c_uint32(n_kv), C.c_uint32(m), C.c_int(layout), C.c_uint32(wpb),
                        C.c_float(eps), C.c_int(n_threads))
    return oq, ok, ov


def matmul_gemv(x, w, bias=None, residual=None, layout=0, wpb=32, alpha=1.0, beta=0.0, n_threads=8):
    """x [m, K]; w flat or 2-D in `layout`; returns out [m, n]."""
    x = _h(x)
    m, K = x.shape
    wf = _h(np.asarray(w).reshape(-1))
    n = wf.size // K
    out = np.zeros((m, n), np.float16)
    nul = C.cast(None, u16p)
    b = _h(bias) if bias is not None else None
    r = _h(residual) if residual is not None else None
    lib().orc_matmul_gemv(_p(x, u16p), _p(wf, u16p), _p(b, u16p) if b is not None else nul, _p(r, u16p) if r is not None else nul,
                          _p(out, u16p), C.c_uint32(m), C.c_uint32(n), C.c_uint32(K), C.c_int(layout), C.c_uint32(wpb),
                          C.c_float(alpha), C.c_float(beta), C.c_int(n_threads))
    return out


def quantize_q8_0(w, wpb=32):
    """GGUF Q8_0 of a row-major [n, k] matrix: per 32 weights of a row, scale = max|w| / 127 stored as f16 and
    q = round(w / scale) in [-127, 127] (the generator of tests/gemv_v2_parity.rs' Q8 cases). Returns (int8 [n, k],
    f16 scales [n, k / wpb])."""
    w = np.asarray(w, np.float32)
    n, k = w.shape
    blocks = w.reshape(n, k // wpb, wpb)
    scale = (np.abs(blocks).max(axis=2) / 127.0).astype(np.float16)
    sf = np.where(scale == 0, np.float16(1.0), scale).astype(np.float32)
    q = np.clip(np.rint(blocks / sf[:, :, None]), -127, 127).astype(np.int8)
    return q.reshape(n, k), scale


def quantize_q4_0(w, wpb=32):
    """Q4_0 of a row-major [n, k] matrix as the reference's test helper makes it (tests/gemm_v2_parity.rs:112-199): per 32
    weights of a row, scale = max|w| / 7 stored as f16, q = round-half-away(w / scale) clamped to [-8, 7] (with the
    unrounded scale). Returns (int8 [n, k] with values -8..7, f16 scales [n, k / wpb])."""
    w = np.asarray(w, np.float16).astype(np.float32)
    n, k = w.shape
    blocks = w.reshape(n, k // wpb, wpb)
    scale = (np.abs(blocks).max(axis=2) / np.float32(7.0)).astype(np.float32)
    t = np.where(scale[:, :, None] > 0, blocks / np.where(scale == 0, np.float32(1), scale)[:, :, None], 0.0)
    q = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), -8, 7).astype(np.int8)
    return q.reshape(n, k), scale.astype(np.float16)


def pack_q4_0(q_flat):
    """Integers -8..7 in the buffer's element order -> the policy's bytes: element 2i in the low nibble of byte i."""
    u = (np.asarray(q_flat, np.int16).reshape(-1) + 8).astype(np.uint8)
    return (u[0::2] | (u[1::2] << 4)).astype(np.uint8)


def unpack_q4_0(packed):
    """The oracle's reading of Q4_0 bytes (policy_q4_0.metal:70-98): int8 values in element order."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    out = np.zeros(packed.size * 2, np.int8)
    lib().orc_unpack_q4_0(packed.ctypes.data_as(C.c_void_p), C.c_size_t(out.size), out.ctypes.data_as(C.c_void_p))
    return out


def dequantize_blocks(q, scales, wpb=32):
    """Block-quantised integers [n, k] (row-major) and their f16 scales [n, k / wpb] -> the f16 weights the reference's
    GEMM works on: f16(q * scale), one rounding (src/metals/mma/tile_loader.metal:100-120; the CPU reference of
    tests/gemm_v2_parity.rs:295-350 dequantises the same way). q * scale is exact in f32 (8-bit integer times an 11-bit
    significand), so this is a single f32 -> f16 rounding."""
    q = np.asarray(q)
    n, k = q.shape
    sf = np.asarray(scales, np.float16).astype(np.float32).reshape(n, k // wpb)
    return (q.astype(np.float32).reshape(n, k // wpb, wpb) * sf[:, :, None]).reshape(n, k).astype(np.float16)


def _i8(a):
    return np.ascontiguousarray(a, dtype=np.int8)


def matmul_gemv_q8(x, w8, scales, bias=None, residual=None, layout=0, wpb=32, alpha=1.0, beta=0.0, n_threads=8):
    x = _h(x)
    m, K = x.shape
    wf = _i8(np.asarray(w8).reshape(-1))
    n = wf.size // K
    sc = _h(scales)
    out = np.zeros((m, n), np.float16)
    nul = C.cast(None, u16p)
    b = _h(bias) if bias is not None else None
    r = _h(residual) if residual is not None else None
    lib().orc_matmul_gemv_q8(_p(x, u16p), _p(wf, i8p), _p(sc, u16p), _p(b, u16p) if b is not None else nul,
                             _p(r, u16p) if r is not None else nul, _p(out, u16p), C.c_uint32(m), C.c_uint32(n), C.c_uint32(K),
                             C.c_int(layout), C.c_uint32(wpb), C.c_float(alpha), C.c_float(beta), C.c_int(n_threads))
    return out


def fused_qkv_q8(x, ws8, scales, gamma=None, biases=None, layout=0, wpb=32, eps=1e-6, n_threads=8):
    """ws8: three int8 matrices (flat or 2-D in `layout`), scales: three f16 [rows, K / wpb]."""
    x = _h(x)
    m, K = x.shape
    w = [_i8(np.asarray(a).reshape(-1)) for a in ws8]
    sc = [_h(a) for a in scales]
    n_dim, n_kv = w[0].size // K, w[1].size // K
    oq, ok, ov = np.zeros((m, n_dim), np.float16), np.zeros((m, n_kv), np.float16), np.zeros((m, n_kv), np.float16)
    g = _h(gamma) if gamma is not None else None
    bs = [_h(b) for b in biases] if biases is not None else [None] * 3
    nul = C.cast(None, u16p)
    lib().orc_fused_qkv_q8(_p(x, u16p), _p(w[0], i8p), _p(sc[0], u16p), _p(w[1], i8p), _p(sc[1], u16p), _p(w[2], i8p),
                           _p(sc[2], u16p), _p(g, u16p) if g is not None else nul,
                           *[(_p(b, u16p) if b is not None else nul) for b in bs], _p(oq, u16p), _p(ok, u16p), _p(ov, u16p),
                           C.c_uint32(K), C.c_uint32(n_dim), C.c_uint32(n_kv), C.c_uint32(m), C.c_int(layout), C.c_uint32(wpb),
                           C.c_float(eps), C.c_int(n_threads))
    return oq, ok, ov


def paged_copy_blocks(pool, n_kv_heads, block_size, head_dim, src_ids, dst_ids):
    """In place on `pool` [n_blocks, n_kv_heads, block_size, head_dim] f16."""
    assert pool.dtype == np.float16 and pool.flags.c_contiguous
    s = np.ascontiguousarray(src_ids, dtype=np.int32)
    d = np.ascontiguousarray(dst_ids, dtype=np.int32)
    lib().orc_paged_copy_blocks(_p(pool, u16p), C.c_uint32(pool.shape[0]), C.c_uint32(n_kv_heads), C.c_uint32(block_size),
                                C.c_uint32(head_dim), _p(s, i32p), _p(d, i32p), C.c_uint32(len(s)))


def kv_prefix_copy(src, dst, prefix_len):
    """Rows [0, prefix_len) of every head of src [heads, cap_s, D] into dst [heads, cap_d, D] (in place); any dtype."""
    assert src.flags.c_contiguous and dst.flags.c_contiguous and src.dtype == dst.dtype
    assert src.shape[0] == dst.shape[0] and src.shape[2] == dst.shape[2]
    L = lib()
    L.orc_kv_prefix_copy.restype = C.c_int
    return L.orc_kv_prefix_copy(C.c_void_p(src.ctypes.data), C.c_void_p(dst.ctypes.data), C.c_size_t(src.shape[0]),
                                C.c_size_t(src.shape[1]), C.c_size_t(dst.shape[1]), C.c_size_t(src.shape[2]),
                                C.c_size_t(src.dtype.itemsize), C.c_size_t(prefix_len))


def align_capacity(capacity):
    L = lib()
    L.orc_align_capacity.restype = C.c_size_t
    return L.orc_align_capacity(C.c_size_t(capacity))


def grown_capacity(allocated, required_len, max_context_len, growth_factor=2.0):
    L = lib()
    L.orc_grown_capacity.restype = C.c_size_t
    return L.orc_grown_capacity(C.c_size_t(allocated), C.c_size_t(required_len), C.c_size_t(max_context_len),
                                C.c_float(growth_factor))


def paged_scatter(pool, block_table, n_kv_heads, block_size, head_dim, pos_begin, pos_end, src):
    assert pool.dtype == np.float16 and pool.flags.c_contiguous
    bt = np.ascontiguousarray(block_table, dtype=np.int32)
    src = _h(src)
    lib().orc_paged_scatter(_p(pool, u16p), _p(bt, i32p), C.c_uint32(n_kv_heads), C.c_uint32(block_size),
                            C.c_uint32(head_dim), C.c_uint32(pos_begin), C.c_uint32(pos_end),
                            C.c_uint32(src.shape[1]), _p(src, u16p))


def sage_k_mean(k, n_kv_heads, capacity, head_dim, kv_len):
    mean = np.zeros((n_kv_heads, head_dim), np.float32)
    lib().orc_sage_k_mean(_p(_h(k), u16p), C.c_uint32(n_kv_heads), C.c_uint32(capacity), C.c_uint32(head_dim),
                          C.c_uint32(kv_len), _p(mean, f32p))
    return mean


def sage_quantize_k(k, mean, n_kv_heads, capacity, head_dim, kv_len, block=32):
    kq = np.zeros((n_kv_heads, capacity, head_dim), np.int8)
    ks = np.zeros((n_kv_heads, (capacity + block - 1) // block), np.float16)
    mean = np.ascontiguousarray(mean, dtype=np.float32)
    lib().orc_sage_quantize_k(_p(_h(k), u16p), _p(mean, f32p), C.c_uint32(n_kv_heads), C.c_uint32(capacity),
                              C.c_uint32(head_dim), C.c_uint32(kv_len), C.c_uint32(block), _p(kq, i8p), _p(ks, u16p))
    return kq, ks


def sage_quantize_q(q, n_heads, head_dim):
    qq = np.zeros((n_heads, head_dim), np.int8)
    qs = np.zeros((n_heads,), np.float32)
    lib().orc_sage_quantize_q(_p(_h(q), u16p), C.c_uint32(n_heads), C.c_uint32(head_dim), _p(qq, i8p), _p(qs, f32p))
    return qq, qs


def sage_decode(qq, qs, kq, ks, v, n_heads, n_kv_heads, head_dim, capacity, kv_len, block=32, scale=None,
                n_threads=1):
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    out = np.empty((n_heads * head_dim,), np.float16)
    lib().orc_sage_decode(_p(np.ascontiguousarray(qq), i8p), _p(np.ascontiguousarray(qs), f32p),
                          _p(np.ascontiguousarray(kq), i8p), _p(_h(ks), u16p), _p(_h(v), u16p), _p(out, u16p),
                          C.c_uint32(n_heads), C.c_uint32(n_kv_heads), C.c_uint32(head_dim), C.c_uint32(capacity),
                          C.c_uint32(kv_len), C.c_uint32(block), C.c_float(scale), C.c_int(n_threads))
    return out


def lcg_fill_f16(state, n, scale):
    """Returns (array, new_state): the reference tests' LCG stream."""
    st = C.c_uint32(state)
    out = np.empty((n,), np.float16)
    lib().orc_lcg_fill_f16(C.byref(st), _p(out, u16p), C.c_size_t(n), C.c_float(scale))
    return out, st.value


class bf16_mode:
    """Context manager: the oracle's data tensors are bf16 inside (arrays are still passed as 16-bit patterns in
    numpy float16 containers: use bf16_pack / bf16_unpack)."""

    def __enter__(self):
        lib().orc_set_elem_type(1)

    def __exit__(self, *a):
        lib().orc_set_elem_type(0)


def bf16_pack(x):
    """float32 array -> bf16 bit patterns (round to nearest even) in a float16-typed container."""
    import torch  # an implementation independent of the oracle's

    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.float16).copy()


def bf16_unpack(h):
    """bf16 bit patterns (float16-typed or uint16 container) -> float32."""
    u = np.ascontiguousarray(h).view(np.uint16).astype(np.uint32) << 16
    return u.view(np.float32)
