"""GPU: fa_decode_step_fused_noalloc (partition partials in the library's static device array, nothing allocated)
gives the bits of fa_decode_step_fused and stays within the attention tolerance of the oracle, on two calls in a row
of which the second is smaller, so that it runs over what the first left in the array."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu

TOL = 2e-3  # max-abs bound of attention outputs against the oracle


def _one_step(f, rng, H, Hkv, D, cap, pos, use_dpos):
    """Runs the step through both entry points on identical copies of the caches; returns what each produced plus the
    oracle's result."""
    cos, sin = fa.rope_tables(5e5, D, cap)
    kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    kc[:, :pos] = h16(rng.normal(size=(Hkv, pos, D)))
    vc[:, :pos] = h16(rng.normal(size=(Hkv, pos, D)))
    q, k, v = (h16(rng.normal(size=(1, n * D))) for n in (H, Hkv, Hkv))
    dcos, dsin, dq, dk, dv = f.array(cos), f.array(sin), f.array(q), f.array(k), f.array(v)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0 if use_dpos else pos, cap, fa.ROPE_NORMAL)
    dpos = f.array(np.array([pos], np.uint32)) if use_dpos else None
    got = {}
    # the entry point that allocates nothing always merges with the second launch: the existing entry point is given the
    # same merge form, so both run the same kernels over the same partitions
    f.set_decode_variant(0, 1)
    for noalloc in (False, True):
        dkc, dvc, dqr, dout = f.array(kc), f.array(vc), f.zeros((H, 1, D)), f.zeros((1, H * D))
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(),
                            dout.arg(), p, d_position=dpos, kv_len_bound=cap if use_dpos else 0, noalloc=noalloc)
        f.synchronize()
        got[noalloc] = (dout.download(), dkc.download(), dvc.download(), dqr.download())
        for b in (dkc, dvc, dqr, dout):
            b.free()
    f.set_decode_variant()
    ok, ov = kc.copy(), vc.copy()
    want_qr = orc.kv_prep_fused(q, k, v, ok, ov, cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=1))
    want = orc.sdpa_decode(want_qr[:, 0].copy(), ok, ov, H, Hkv, D, cap, pos + 1)
    for b in (dcos, dsin, dq, dk, dv) + ((dpos,) if dpos is not None else ()):
        b.free()
    return got, (want, ok, ov, want_qr)


def _check(got, want):
    out_a, kc_a, vc_a, qr_a = got[False]
    out_n, kc_n, vc_n, qr_n = got[True]
    w_out, w_k, w_v, w_qr = want
    # against the existing entry point: the same kernels over the same partitions, so the same bits
    assert np.array_equal(bits(out_n), bits(out_a))
    assert np.array_equal(bits(kc_n), bits(kc_a)) and np.array_equal(bits(vc_n), bits(vc_a))
    assert np.array_equal(bits(qr_n), bits(qr_a))
    # against the oracle: cache rows and rotated q bit-exact, attention within tolerance
    assert np.array_equal(bits(kc_n), bits(w_k)) and np.array_equal(bits(vc_n), bits(w_v))
    assert np.array_equal(bits(qr_n.reshape(w_qr.shape)), bits(w_qr))
    assert max_abs(out_n.reshape(-1), w_out.reshape(-1)) <= TOL


def test_noalloc_two_calls_second_smaller():
    f = ctx()
    assert f.lib.fa_noalloc_scratch_bytes() == 4 << 20
    rng = np.random.default_rng(0x5C4A)
    announce("noalloc decode step: H24/Hkv8/D128, position 8200 of capacity 8448 (32 partitions), device position")
    got, want = _one_step(f, rng, 24, 8, 128, 8448, 8200, True)
    _check(got, want)
    announce("noalloc decode step: H24/Hkv8/D128, position 1100 of capacity 1280 (fewer, shorter partitions)")
    got, want = _one_step(f, rng, 24, 8, 128, 1280, 1100, False)
    _check(got, want)
    announce("noalloc decode step: H14/Hkv2/D64, position 40 (one partition: the scratch is not used)")
    got, want = _one_step(f, rng, 14, 2, 64, 128, 40, False)
    _check(got, want)


def test_noalloc_rejects_what_does_not_fit():
    f = ctx()
    announce("noalloc decode step: a partition size that needs more partials than the static array holds")
    rng = np.random.default_rng(3)
    H, Hkv, D, cap, pos = 32, 32, 128, 8192, 8100
    cos, sin = fa.rope_tables(1e4, D, cap)
    dkc, dvc = f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D))
    dq, dk, dv = (f.array(h16(rng.normal(size=(1, n * D)))) for n in (H, Hkv, Hkv))
    dcos, dsin, dout = f.array(cos), f.array(sin), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NEOX)
    f.set_decode_variant(64, 1)  # 127 partitions x 32 heads x 130 floats x 4 B = 2.1 MB fits
    try:
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), dout.arg(),
                            p, noalloc=True)
        f.synchronize()
    finally:
        f.set_decode_variant(0, 1)
    # 64 heads x 127 partitions x 130 floats x 4 B = 4.23 MB does not
    H2 = 64
    dq2, dout2 = f.array(h16(rng.normal(size=(1, H2 * D)))), f.zeros((1, H2 * D))
    p2 = fa.KvPrepFusedParams.make(H2, Hkv, D, 1, pos, cap, fa.ROPE_NEOX)
    f.set_decode_variant(64, 1)
    try:
        with pytest.raises(fa.FoundryError) as e:
            f.decode_step_fused(dq2.arg(), dk.arg(), dv.arg(), None, dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(),
                                dout2.arg(), p2, noalloc=True)
        assert e.value.variant == "InvalidShape" and "static scratch" in str(e.value)
        # the existing entry point takes the same launch
        f.decode_step_fused(dq2.arg(), dk.arg(), dv.arg(), None, dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), dout2.arg(), p2)
        f.synchronize()
    finally:
        f.set_decode_variant(0, 1)
    for b in (dkc, dvc, dq, dk, dv, dcos, dsin, dout, dq2, dout2):
        b.free()


def test_noalloc_leaves_device_memory_untouched():
    """The property the entry point is named for: between two readings of the device's free memory, a call of it (and the
    wait for its kernels) allocates and frees nothing. The allocating entry point runs the same shape first, so that the
    kernels' code is resident before the first reading."""
    f = ctx()
    announce("noalloc decode step: free device memory before and after")
    rng = np.random.default_rng(11)
    H, Hkv, D, cap, pos = 24, 8, 128, 4096, 4000
    cos, sin = fa.rope_tables(5e5, D, cap)
    dkc, dvc = f.array(h16(rng.normal(size=(Hkv, cap, D)))), f.array(h16(rng.normal(size=(Hkv, cap, D))))
    dq, dk, dv = (f.array(h16(rng.normal(size=(1, n * D)))) for n in (H, Hkv, Hkv))
    dcos, dsin, dout = f.array(cos), f.array(sin), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NORMAL)
    args = (dq.arg(), dk.arg(), dv.arg(), None, dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p)
    f.set_decode_variant(0, 1)
    try:
        f.decode_step_fused(*args)
        f.synchronize()
        before = f.device_mem_info()[0]
        for _ in range(3):
            f.decode_step_fused(*args, noalloc=True)
        f.synchronize()
        assert f.device_mem_info()[0] == before
    finally:
        f.set_decode_variant()
    for b in (dkc, dvc, dq, dk, dv, dcos, dsin, dout):
        b.free()
