"""GPU parity in bf16 (an extension: the reference is f16 only, so this dtype is PARITY UNPINNED by any reference
test). The oracle runs the same recurrences with bf16 element conversions (pinned against torch's bfloat16 in
tests/test_oracle_cpu.py). Bars: RoPE'd rows and cache slots bit-exact; attention outputs within 1.6e-2 max-abs
(bf16 keeps 8 significand bits: one output rounding alone is up to 2^-9 relative, and the PV operand P is rounded to
bf16 as well), tables stay f16."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
import refmath as rm
from gpu_util import announce, bits, ctx, max_abs

pytestmark = pytest.mark.gpu
TOL_BF16 = 1.6e-2
BF = fa.DTYPE_BF16


def up(f, a):
    """Uploads bf16 bit patterns (float16-typed container) and returns the buffer."""
    return f.array(np.ascontiguousarray(a))


@pytest.mark.parametrize("mode", [fa.ROPE_NEOX, fa.ROPE_NORMAL])
@pytest.mark.parametrize("H,Hkv,D,T,pos,cap", [(14, 2, 64, 1, 5, 16), (24, 8, 128, 7, 3, 32), (4, 2, 20, 3, 0, 8)])
def test_kv_prep_bf16_bit_exact(mode, H, Hkv, D, T, pos, cap):
    announce("kv_prep bf16", H, D, T, mode)
    f = ctx()
    rng = np.random.default_rng(H * D + T)
    q, k, v = (orc.bf16_pack(rng.normal(size=(T, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(1e4, D, cap)
    kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    with orc.bf16_mode():
        want_qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, T, pos, cap, rope_mode=mode))
    dq, dk, dv, dqr = up(f, q), up(f, k), up(f, v), f.zeros((H, T, D))
    dkc, dvc, dcos, dsin = f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.array(cos), f.array(sin)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, T, pos, cap, mode)
    f.kv_prep_fused(dq.arg(dtype=BF), dk.arg(dtype=BF), dv.arg(dtype=BF), dqr.arg(dtype=BF), dkc.arg(dtype=BF),
                    dvc.arg(dtype=BF), dcos.arg(), dsin.arg(), p)
    f.synchronize()
    assert np.array_equal(bits(dqr.download()), bits(want_qr))
    assert np.array_equal(bits(dkc.download()), bits(kc))
    assert np.array_equal(bits(dvc.download()), bits(vc))
    with pytest.raises(fa.FoundryError) as e:  # mixed element types are refused
        f.kv_prep_fused(dq.arg(dtype=BF), dk.arg(), dv.arg(dtype=BF), dqr.arg(dtype=BF), dkc.arg(dtype=BF),
                        dvc.arg(dtype=BF), dcos.arg(), dsin.arg(), p)
    assert e.value.variant == "UnsupportedDtype"
    for b in (dq, dk, dv, dqr, dkc, dvc, dcos, dsin):
        b.free()


@pytest.mark.parametrize("H,Hkv,D,N,cap", [(14, 2, 64, 1025, 1152), (24, 8, 128, 8200, 8448), (16, 2, 128, 1, 16),
                                            (6, 6, 128, 333, 400)])
def test_decode_bf16_vs_oracle(H, Hkv, D, N, cap):
    announce("decode bf16", H, Hkv, D, N)
    f = ctx()
    rng = np.random.default_rng(N + D)
    q = orc.bf16_pack(rng.normal(size=(H, D)))
    k = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    v = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    with orc.bf16_mode():
        want = orc.bf16_unpack(orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N, n_threads=8)).reshape(H, D)
    dq, dk, dv, do = up(f, q), up(f, k), up(f, v), f.zeros((1, H * D))
    f.flash_attention(dq.arg((1, H * D), dtype=BF), dk.arg(dtype=BF), dv.arg(dtype=BF), do.arg(dtype=BF), True, N - 1, H,
                      D, N, 1)
    f.synchronize()
    got = orc.bf16_unpack(do.download()).reshape(H, D)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL_BF16
    full = rm.gqa_decode_f64(orc.bf16_unpack(q), orc.bf16_unpack(k), orc.bf16_unpack(v), H, Hkv, D, N)
    assert max_abs(got, full) <= TOL_BF16
    for b in (dq, dk, dv, do):
        b.free()


def test_fused_decode_step_bf16_contiguous_and_paged():
    """RoPE + append + decode in one launch on bf16 tensors: appended rows and q_rot bit-exact, output within bound."""
    announce("fused step bf16")
    f = ctx()
    rng = np.random.default_rng(21)
    H, Hkv, D, pos, cap = 24, 8, 128, 700, 768
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    kc[:, :pos] = orc.bf16_pack(rng.normal(size=(Hkv, pos, D)))
    vc[:, :pos] = orc.bf16_pack(rng.normal(size=(Hkv, pos, D)))
    q, k, v = (orc.bf16_pack(rng.normal(size=(1, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(5e5, D, cap)
    dkc, dvc = up(f, kc), up(f, vc)
    dq, dk, dv, dqr, do = up(f, q), up(f, k), up(f, v), f.zeros((H, 1, D)), f.zeros((1, H * D))
    dcos, dsin = f.array(cos), f.array(sin)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NORMAL)
    f.decode_step_fused(dq.arg(dtype=BF), dk.arg(dtype=BF), dv.arg(dtype=BF), dqr.arg(dtype=BF), dkc.arg(dtype=BF),
                        dvc.arg(dtype=BF), dcos.arg(), dsin.arg(), do.arg(dtype=BF), p)
    f.synchronize()
    with orc.bf16_mode():
        want_qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=1))
        want = orc.bf16_unpack(orc.sdpa_decode(want_qr[:, 0].copy(), kc, vc, H, Hkv, D, cap, pos + 1, n_threads=8))
    assert np.array_equal(bits(dqr.download()), bits(want_qr))
    assert np.array_equal(bits(dkc.download()), bits(kc)) and np.array_equal(bits(dvc.download()), bits(vc))
    assert max_abs(orc.bf16_unpack(do.download()).reshape(-1), want.reshape(-1)) <= TOL_BF16
    for b in (dq, dk, dv, dqr, do, dkc, dvc, dcos, dsin):
        b.free()


@pytest.mark.usefixtures("prefill_variant")
@pytest.mark.parametrize("D,H,Hkv,M,prefix", [(128, 6, 2, 200, 333), (64, 14, 2, 70, 0), (128, 24, 8, 33, 2000)])
def test_prefill_bf16_vs_oracle(D, H, Hkv, M, prefix):
    announce("prefill bf16", D, M, prefix)
    f = ctx()
    rng = np.random.default_rng(M + prefix)
    N, cap = M + prefix, M + prefix + 3
    q = orc.bf16_pack(rng.normal(size=(H, M, D)))
    k = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    v = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    with orc.bf16_mode():
        want = orc.bf16_unpack(orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True,
                                                out_layout="head_major", n_threads=8))
    dq, dk, dv, do = up(f, q), up(f, k), up(f, v), f.zeros((M, H * D))
    f.flash_attention(dq.arg((H, M, D), dtype=BF), dk.arg(dtype=BF), dv.arg(dtype=BF), do.arg(dtype=BF), True, prefix, H,
                      D, N, M)
    f.synchronize()
    got = orc.bf16_unpack(do.download()).reshape(M, H, D).transpose(1, 0, 2)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL_BF16
    for b in (dq, dk, dv, do):
        b.free()
