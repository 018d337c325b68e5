"""Independent float64 restatements used to pin the oracle (library routines only: numpy / scipy)."""
import numpy as np
from scipy.special import softmax


def attn_f64(q, k, v, scale, mask=None):
    """q [M, D], k/v [N, D] (any float dtype) -> [M, D] float64 softmax(scale q k^T + mask) v."""
    s = (q.astype(np.float64) @ k.astype(np.float64).T) * float(scale)
    if mask is not None:
        s = np.where(mask, s, -np.inf)
    return softmax(s, axis=-1) @ v.astype(np.float64)


def causal_mask(m, n, query_offset):
    r = np.arange(m)[:, None] + query_offset
    return np.arange(n)[None, :] <= r


def gqa_decode_f64(q, k, v, n_heads, n_kv_heads, head_dim, kv_len, scale=None):
    """q [H*D] or [H, D]; k, v [Hkv, cap, D] -> [H, D] float64."""
    if scale is None:
        scale = 1.0 / np.sqrt(head_dim)
    q = q.reshape(n_heads, head_dim)
    g = n_heads // n_kv_heads
    out = np.empty((n_heads, head_dim))
    for h in range(n_heads):
        out[h] = attn_f64(q[h:h + 1], k[h // g, :kv_len], v[h // g, :kv_len], scale)[0]
    return out


def gqa_prefill_f64(q_hm, k, v, n_heads, n_kv_heads, head_dim, kv_len, query_offset, causal=True, scale=None):
    """q_hm [H, M, D]; k, v [Hkv, cap, D] -> [H, M, D] float64."""
    if scale is None:
        scale = 1.0 / np.sqrt(head_dim)
    g = n_heads // n_kv_heads
    m = q_hm.shape[1]
    mask = causal_mask(m, kv_len, query_offset) if causal else None
    out = np.empty((n_heads, m, head_dim))
    for h in range(n_heads):
        out[h] = attn_f64(q_hm[h], k[h // g, :kv_len], v[h // g, :kv_len], scale, mask)
    return out


def rope_rotate_f64(x, cos, sin, pos, mode):
    """x [..., D] float16 rows at positions `pos` (broadcastable to x.shape[:-1]); cos/sin [P, D/2] f16 tables.
    Complex-multiplication form of the rotation; returns float64."""
    D = x.shape[-1]
    half = D // 2
    x64 = x.astype(np.float64)
    c = cos.astype(np.float64)[pos]
    s = sin.astype(np.float64)[pos]
    if mode == "neox":
        z = x64[..., :half] + 1j * x64[..., half:]
    else:
        z = x64[..., 0::2] + 1j * x64[..., 1::2]
    z = z * (c + 1j * s)
    out = np.empty_like(x64)
    if mode == "neox":
        out[..., :half], out[..., half:] = z.real, z.imag
    else:
        out[..., 0::2], out[..., 1::2] = z.real, z.imag
    return out


def f16_ulp(x):
    """Spacing of binary16 at |x| (float64 array)."""
    ax = np.maximum(np.abs(x), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(ax)) - 10)
