"""GPU parity: Sage-style int8 Q/K decode. The reference holds only a prose design (docs/SAGE.md), so parity is
unpinned by reference tests: the quantisers are checked bit-exactly against the oracle's int8 model, the decode
against that model, and the end-to-end error against f16 SDPA on the unquantised tensors is measured."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
import refmath as rm
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu


def outlier_normal(rng, shape, frac=0.01, sigma=8.0):
    x = rng.normal(size=shape)
    mask = rng.random(size=shape) < frac
    return h16(np.where(mask, sigma * np.sign(x), x))


@pytest.mark.parametrize("H,Hkv,D,N,cap", [(16, 4, 128, 4096, 4096), (16, 4, 128, 1000, 1024), (14, 2, 64, 333, 352),
                                           (8, 8, 128, 31, 64),
                                           (16, 4, 128, 32768, 32768)])  # SmolLM3 shape at the full 32K context
def test_sage_quantize_and_decode(H, Hkv, D, N, cap):
    announce("sage", H, Hkv, D, N)
    f = ctx()
    rng = np.random.default_rng(N + D)
    k = outlier_normal(rng, (Hkv, cap, D))
    v = outlier_normal(rng, (Hkv, cap, D))
    q = outlier_normal(rng, (H, D))
    dk, dv, dq = f.array(k), f.array(v), f.array(q)
    dmean = f.zeros((Hkv, D), np.float32)
    dkq, dks = f.zeros((Hkv, cap, D), np.int8), f.zeros((Hkv, (cap + 31) // 32), np.float16)
    dqq, dqs = f.zeros((H, D), np.int8), f.zeros((H,), np.float32)
    dout = f.zeros((H * D,))
    f.sage_k_mean(dk, Hkv, cap, D, N, dmean)
    f.sage_quantize_k(dk, dmean, Hkv, cap, D, 0, N, dkq, dks)
    f.sage_quantize_q(dq, H, D, dqq, dqs)
    f.sage_decode(dqq, dqs, dkq, dks, dv, dout, H, Hkv, D, cap, N)
    f.synchronize()
    mean = dmean.download()
    assert max_abs(mean, orc.sage_k_mean(k, Hkv, cap, D, N)) <= 2e-5
    want_kq, want_ks = orc.sage_quantize_k(k, mean, Hkv, cap, D, N)  # same mean -> bit-exact quantisation
    got_kq, got_ks = dkq.download(), dks.download()
    nb = (N + 31) // 32
    assert np.array_equal(bits(got_ks[:, :nb]), bits(want_ks[:, :nb]))
    assert np.array_equal(got_kq[:, :N], want_kq[:, :N])
    want_qq, want_qs = orc.sage_quantize_q(q, H, D)
    assert np.array_equal(dqq.download(), want_qq) and np.array_equal(dqs.download(), want_qs)
    got = dout.download().reshape(H, D)
    model = orc.sage_decode(want_qq, want_qs, want_kq, want_ks, v, H, Hkv, D, cap, N, n_threads=8).reshape(H, D)
    assert max_abs(got, model) <= 2e-3
    # int8 quantisation error against f16 SDPA on the unquantised tensors: a measured quantity (with 1 % of
    # entries at 8 sigma every 32-token block's scale is 8/127, so the logits carry ~0.02 of noise)
    full = rm.gqa_decode_f64(q, k, v, H, Hkv, D, N)
    err = max_abs(got, full)
    mean_err = float(np.mean(np.abs(got.astype(np.float64) - full)))
    cos_sim = float(np.sum(got.astype(np.float64) * full) / np.sqrt(np.sum(got.astype(np.float64) ** 2) * np.sum(full ** 2)))
    print("sage vs f16-sdpa: max abs err %.4f mean abs err %.5f cosine %.5f" % (err, mean_err, cos_sim), flush=True)
    assert err <= 0.15 and mean_err <= 0.03 and cos_sim >= 0.98
    for b in (dk, dv, dq, dmean, dkq, dks, dqq, dqs, dout):
        b.free()


def test_sage_incremental_block_quantisation_and_errors():
    announce("sage incremental")
    f = ctx()
    rng = np.random.default_rng(1)
    Hkv, D, cap, N = 2, 128, 128, 100
    k = h16(rng.normal(size=(Hkv, cap, D)))
    dk = f.array(k)
    dmean = f.zeros((Hkv, D), np.float32)
    f.sage_k_mean(dk, Hkv, cap, D, N, dmean)
    a_q, a_s = f.zeros((Hkv, cap, D), np.int8), f.zeros((Hkv, 4), np.float16)
    b_q, b_s = f.zeros((Hkv, cap, D), np.int8), f.zeros((Hkv, 4), np.float16)
    f.sage_quantize_k(dk, dmean, Hkv, cap, D, 0, N, a_q, a_s)
    f.sage_quantize_k(dk, dmean, Hkv, cap, D, 0, 64, b_q, b_s)
    f.sage_quantize_k(dk, dmean, Hkv, cap, D, 64, N, b_q, b_s)
    f.synchronize()
    assert np.array_equal(a_q.download(), b_q.download()) and np.array_equal(bits(a_s.download()), bits(b_s.download()))
    with pytest.raises(fa.FoundryError) as e:
        f.sage_quantize_k(dk, dmean, Hkv, cap, D, 10, N, b_q, b_s)
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:
        f.sage_k_mean(dk, Hkv, cap, 96, N, dmean)
    assert e.value.variant == "OperationNotSupported"
    f.synchronize()
