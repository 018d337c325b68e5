"""Regenerates tests/golden/known_answer_sdpa.npz.

The inputs are the closed-form patterns the reference's own known-answer tests use
(/root/reference/crates/metallic-foundry/tests/sdpa_oob_repro.rs:16-38 and
tests/sdpa_head_stride_misaligned.rs:15-36): q = (h+1)(t+1)(d+1)*1e-3, k = (h+1)(t+1)(d+1)*1e-5,
v = (h+1)(t+1)((d%7)+1)*1e-4, rounded to f16. Expected outputs are the textbook
softmax(q k^T / sqrt(D)) v evaluated in float64 with scipy (library routine, not the oracle),
on the f16-rounded inputs. Nothing from the reference is imported or executed.

Run: python tests/golden/make_known_answer.py
"""
import os

import numpy as np
from scipy.special import softmax


def pattern(n_heads, m, seq_k, head_dim):
    h = np.arange(n_heads, dtype=np.float32)[:, None, None] + 1
    d = np.arange(head_dim, dtype=np.float32)[None, None, :]
    tq = np.arange(m, dtype=np.float32)[None, :, None] + 1
    tk = np.arange(seq_k, dtype=np.float32)[None, :, None] + 1
    q = (h * tq * (d + 1) * np.float32(0.001)).astype(np.float16)
    k = (h * tk * (d + 1) * np.float32(0.00001)).astype(np.float16)
    v = (h * tk * ((d % 7) + 1) * np.float32(0.0001)).astype(np.float16)
    return q, k, v


def expected(q, k, v):
    q64, k64, v64 = (a.astype(np.float64) for a in (q, k, v))
    s = np.einsum("hmd,hnd->hmn", q64, k64) / np.sqrt(q.shape[-1])
    return np.einsum("hmn,hnd->hmd", softmax(s, axis=-1), v64)


def main():
    out = {}
    for name, (H, M, N, D) in {"oob_m1": (2, 1, 15, 64), "misaligned_m17": (2, 17, 15, 64)}.items():
        q, k, v = pattern(H, M, N, D)
        out[name + "_q"], out[name + "_k"], out[name + "_v"] = q, k, v
        out[name + "_expected_f64"] = expected(q, k, v)  # [H, M, D] head-major
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answer_sdpa.npz"), **out)


if __name__ == "__main__":
    main()
