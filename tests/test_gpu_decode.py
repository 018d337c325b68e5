"""GPU parity: flash decode (fa_flash_attention with m = 1, fa_flash_decode_dyn) against the CPU oracle.
Tolerance: max-abs <= 2e-3 on f16 outputs with f32 accumulation (N(0,1) inputs)."""
import os

import numpy as np
import pytest

import foundry_attn as fa
import orc
import refmath as rm
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-3
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gpu_decode(q, k, v, H, D, N, causal=True, query_offset=None, q_arg_dims=None):
    f = ctx()
    Hkv, cap = k.shape[0], k.shape[1]
    dq, dk, dv, do = f.array(q), f.array(k), f.array(v), f.zeros((1, H * D))
    qa = dq.arg(q_arg_dims) if q_arg_dims else dq.arg((1, H * D))
    f.flash_attention(qa, dk.arg(), dv.arg(), do.arg(), causal, N - 1 if query_offset is None else query_offset, H, D,
                      N, 1)
    f.synchronize()
    out = do.download().reshape(H, D)
    for b in (dq, dk, dv, do):
        b.free()
    return out


@pytest.mark.parametrize("H,Hkv,D,N,cap", [
    (14, 2, 64, 1025, 1152),    # benchmark configuration 1 (Qwen2.5-0.5B shape)
    (24, 8, 128, 8193, 8448),   # benchmark configuration 2 (Llama-3.2-3B shape, one layer)
    (16, 2, 128, 3000, 3008),   # Qwen2.5-3B shape
    (16, 4, 128, 5000, 5120),   # SmolLM3 shape
    (32, 8, 128, 777, 1024),
    (24, 8, 128, 70000, 70016),  # a long context at batch 1: whole partitions, one per compute unit, merged inside the launch
    (8, 8, 64, 130, 130), (2, 1, 128, 64, 64), (12, 2, 64, 333, 400), (10, 2, 128, 100, 128), (16, 1, 64, 70, 96),
])
def test_decode_vs_oracle(H, Hkv, D, N, cap):
    announce("decode", H, Hkv, D, N, cap)
    rng = np.random.default_rng(H * 1000 + N)
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    got = gpu_decode(q, k, v, H, D, N)
    want = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N, n_threads=8).reshape(H, D)
    assert max_abs(got, want) <= TOL
    assert max_abs(got, rm.gqa_decode_f64(q, k, v, H, Hkv, D, N)) <= TOL


@pytest.mark.parametrize("N", [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 257, 1000])
@pytest.mark.parametrize("D,H,Hkv", [(64, 14, 2), (128, 6, 2)])
def test_decode_ragged_lengths_and_splits(N, D, H, Hkv):
    announce("decode ragged", N, D)
    f = ctx()
    rng = np.random.default_rng(N)
    cap = 1024
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    k[:, N:], v[:, N:] = np.float16(np.nan), np.float16(np.nan)  # rows past kv_len must never contribute
    want = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N).reshape(H, D)
    try:
        for kps, merge in [(0, 0), (64, 0), (64, 1), (128, 0), (1024, 1), (0, 2), (64, 2), (128, 2), (1024, 2)]:
            f.set_decode_variant(kps, merge)
            got = gpu_decode(q, k, v, H, D, N)
            assert np.all(np.isfinite(got)), (kps, merge)
            assert max_abs(got, want) <= TOL, (kps, merge)
    finally:
        f.set_decode_variant()


def test_decode_known_answer_fixture():
    announce("decode known-answer fixture")
    g = np.load(os.path.join(GOLD, "known_answer_sdpa.npz"))
    q, k, v, want = g["oob_m1_q"], g["oob_m1_k"], g["oob_m1_v"], g["oob_m1_expected_f64"]
    H, _, D = q.shape
    N = k.shape[1]
    got = gpu_decode(q.reshape(H, D), k, v, H, D, N, causal=False, query_offset=0)
    assert np.all(np.abs(got.astype(np.float64) - want[:, 0]) <= rm.f16_ulp(want[:, 0]) + 1e-6)


@pytest.mark.parametrize("seed,H,D,N", [(1, 14, 64, 128), (7, 14, 64, 257), (42, 8, 128, 300)])
def test_decode_reference_lcg_inputs(seed, H, D, N):
    """Inputs of tests/flashattention_decode_parity.rs (LCG, MHA cache); the reference accepts 6e-2 there."""
    announce("decode lcg", seed)
    st = seed
    q, st = orc.lcg_fill_f16(st, H * D, 0.25)
    k, st = orc.lcg_fill_f16(st, H * N * D, 0.25)
    v, st = orc.lcg_fill_f16(st, H * N * D, 0.25)
    k, v = k.reshape(H, N, D), v.reshape(H, N, D)
    got = gpu_decode(q.reshape(H, D), k, v, H, D, N, q_arg_dims=(1, H * D))
    assert max_abs(got, rm.gqa_decode_f64(q, k, v, H, H, D, N)) <= 5e-4


def test_decode_group_sizes_and_invariants():
    announce("decode group sizes")
    rng = np.random.default_rng(5)
    D, N, cap = 128, 200, 256
    for G in (1, 2, 3, 4, 5, 6, 7, 8, 12, 16):
        Hkv = 2
        H = G * Hkv
        q = h16(rng.normal(size=(H, D)))
        k = h16(rng.normal(size=(Hkv, cap, D)))
        v = h16(rng.normal(size=(Hkv, cap, D)))
        got = gpu_decode(q, k, v, H, D, N)
        assert max_abs(got, orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N).reshape(H, D)) <= TOL, G
        # GQA(compact) == MHA(expanded)
        ke = orc.repeat_kv_heads(k, Hkv, H, cap, D, cap)
        ve = orc.repeat_kv_heads(v, Hkv, H, cap, D, cap)
        assert max_abs(got, gpu_decode(q, ke, ve, H, D, N)) <= 1e-3, G
    # equal keys -> mean of V ; single key -> V[0]
    H, Hkv = 6, 2
    q = h16(rng.normal(size=(H, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    ks = np.broadcast_to(h16(rng.normal(size=(Hkv, 1, D))), (Hkv, cap, D)).copy()
    got = gpu_decode(q, ks, v, H, D, N)
    for h in range(H):
        assert max_abs(got[h], v[h // 3, :N].astype(np.float64).mean(0)) <= 1e-3
    got1 = gpu_decode(q, ks, v, H, D, 1)
    for h in range(H):
        assert np.array_equal(bits(got1[h]), bits(v[h // 3, 0]))


def test_decode_causal_offset_and_rank4_cache():
    """m = 1 with query_offset + 1 < kv_seq_len (the reference routes this to its materialized path,
    src/metals/sdpa/step.rs:268-290): only keys j <= query_offset are visible."""
    announce("decode causal offset")
    f = ctx()
    rng = np.random.default_rng(9)
    H, Hkv, D, N, cap = 8, 2, 64, 90, 96
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    got = gpu_decode(q, k, v, H, D, N, causal=True, query_offset=40)
    assert max_abs(got, orc.sdpa_decode(q, k, v, H, Hkv, D, cap, 41).reshape(H, D)) <= TOL
    got = gpu_decode(q, k, v, H, D, N, causal=False, query_offset=40)
    assert max_abs(got, orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N).reshape(H, D)) <= TOL
    dq, dk, dv, do = f.array(q), f.array(k), f.array(v), f.zeros((H * D,))
    f.flash_attention(dq.arg((H * D,)), dk.arg((1, Hkv, cap, D)), dv.arg((1, Hkv, cap, D)), do.arg(), True, N - 1, H, D,
                      N, 1)
    f.synchronize()
    assert max_abs(do.download().reshape(H, D), orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N).reshape(H, D)) <= TOL


def test_decode_device_position_matches_static():
    announce("decode dyn")
    f = ctx()
    rng = np.random.default_rng(11)
    H, Hkv, D, cap = 24, 8, 128, 1024
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    dq, dk, dv, do = f.array(q), f.array(k), f.array(v), f.zeros((1, H * D))
    dpos = f.array(np.array([0], np.uint32))
    for pos in (0, 63, 64, 500, 1023):
        dpos.upload(np.array([pos], np.uint32))
        f.flash_decode_dyn(dq.arg(), dk.arg(), dv.arg(), do.arg(), H, D, dpos, 1, cap)
        f.synchronize()
        got = do.download().reshape(H, D)
        assert max_abs(got, orc.sdpa_decode(q, k, v, H, Hkv, D, cap, pos + 1).reshape(H, D)) <= TOL, pos
    # a bound smaller than the device length clamps instead of reading past it
    dpos.upload(np.array([900], np.uint32))
    f.flash_decode_dyn(dq.arg(), dk.arg(), dv.arg(), do.arg(), H, D, dpos, 1, 256)
    f.synchronize()
    assert max_abs(do.download().reshape(H, D), orc.sdpa_decode(q, k, v, H, Hkv, D, cap, 256).reshape(H, D)) <= TOL


def test_decode_errors():
    announce("decode errors")
    f = ctx()
    H, Hkv, cap = 4, 2, 32
    for D, variant in [(96, "OperationNotSupported"), (32, "OperationNotSupported")]:
        dq, dk, dv, do = f.zeros((1, H * D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.zeros((1, H * D))
        with pytest.raises(fa.FoundryError) as e:
            f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, 1, 1)
        assert e.value.variant == variant and "head_dim" in str(e.value)
    D = 64
    dq, dk, dv, do = f.zeros((1, H * D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.zeros((1, H * D))
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, 1, 1, kv_head_major=False)
    assert e.value.variant == "OperationNotSupported" and "kv_head_major" in str(e.value)
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, cap + 1, 1)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, 0, 1)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg((Hkv, cap, D), (cap * D * 2, 2 * D, 1)), dv.arg(), do.arg(), True, 0, H, D, 4, 1)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:
        f.set_decode_variant(100, 0)
    assert e.value.variant == "OperationNotSupported"
    f.synchronize()


@pytest.mark.parametrize("H,Hkv,D,mode,base,layer,step", [
    (14, 2, 64, fa.ROPE_NEOX, 1e6, 0, 0),      # Qwen2.5-0.5B
    (24, 8, 128, fa.ROPE_NORMAL, 5e5, 0, 0),   # Llama-3.2-3B
    (16, 4, 128, fa.ROPE_NORMAL, 5e6, 3, 4),   # SmolLM3 NoPE layer
    (16, 4, 128, fa.ROPE_NORMAL, 5e6, 4, 4),   # SmolLM3 RoPE layer
    (16, 2, 128, fa.ROPE_NEOX, 1e6, 0, 0),     # Qwen2.5-3B
    (24, 2, 64, fa.ROPE_NEOX, 1e4, 0, 0),      # group 12: three workgroups share a KV head
])
def test_fused_decode_step_equals_separate_ops(H, Hkv, D, mode, base, layer, step):
    """fa_decode_step_fused == fa_kv_prep_fused + fa_flash_attention: caches and q_rot bit-exact against the
    oracle; outputs read the same f16 values and agree with the two-op path up to f32 summation order."""
    announce("fused step", H, Hkv, D, mode, layer, step)
    f = ctx()
    rng = np.random.default_rng(H + D + layer)
    cap = 704
    cos, sin = fa.rope_tables(base, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    f.set_decode_variant(64, 0)
    try:
        for pos in (0, 1, 62, 63, 64, 127, 128, 300, 703):
            kc0 = h16(rng.normal(size=(Hkv, cap, D)))
            vc0 = h16(rng.normal(size=(Hkv, cap, D)))
            q, k, v = (h16(rng.normal(size=(1, n * D))) for n in (H, Hkv, Hkv))
            ok, ov = kc0.copy(), vc0.copy()
            want_qr = orc.kv_prep_fused(q, k, v, ok, ov, cos, sin,
                                        orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=mode, layer_idx=layer,
                                                        no_rope_layer_step=step))
            want = orc.sdpa_decode(want_qr[:, 0].copy(), ok, ov, H, Hkv, D, cap, pos + 1).reshape(H, D)
            dq, dk, dv = f.array(q), f.array(k), f.array(v)
            # two-op path
            kc_a, vc_a, qr_a, out_a = f.array(kc0), f.array(vc0), f.zeros((H, 1, D)), f.zeros((1, H * D))
            p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, mode, layer, step)
            f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), qr_a.arg(), kc_a.arg(), vc_a.arg(), dcos.arg(), dsin.arg(), p)
            f.flash_attention(qr_a.arg((1, H * D)), kc_a.arg(), vc_a.arg(), out_a.arg(), True, pos, H, D, pos + 1, 1)
            # fused, static position
            kc_b, vc_b, qr_b, out_b = f.array(kc0), f.array(vc0), f.zeros((H, 1, D)), f.zeros((1, H * D))
            f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), qr_b.arg(), kc_b.arg(), vc_b.arg(), dcos.arg(), dsin.arg(),
                                out_b.arg(), p)
            # fused, device position, no q_rot output
            kc_c, vc_c, out_c = f.array(kc0), f.array(vc0), f.zeros((1, H * D))
            dpos = f.array(np.array([pos], np.uint32))
            p0 = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, mode, layer, step)
            f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, kc_c.arg(), vc_c.arg(), dcos.arg(), dsin.arg(),
                                out_c.arg(), p0, d_position=dpos, kv_len_bound=cap)
            f.synchronize()
            for kc_x, vc_x in ((kc_a, vc_a), (kc_b, vc_b), (kc_c, vc_c)):
                assert np.array_equal(bits(kc_x.download()), bits(ok)), pos
                assert np.array_equal(bits(vc_x.download()), bits(ov)), pos
            assert np.array_equal(bits(qr_a.download()), bits(want_qr)), pos
            assert np.array_equal(bits(qr_b.download()), bits(want_qr)), pos
            oa, ob, oc = out_a.download(), out_b.download(), out_c.download()
            assert max_abs(oa.reshape(H, D), want) <= TOL, pos
            assert max_abs(ob, oa) <= 2e-3 and max_abs(ob.reshape(H, D), want) <= TOL, pos
            assert np.array_equal(bits(oc), bits(ob)), pos  # static and device position: same kernel, same bits
            for b in (dq, dk, dv, kc_a, vc_a, qr_a, out_a, kc_b, vc_b, qr_b, out_b, kc_c, vc_c, out_c, dpos):
                b.free()
    finally:
        f.set_decode_variant()


def test_fused_step_errors_and_overflow_guard():
    announce("fused step errors")
    f = ctx()
    H, Hkv, D, cap = 8, 2, 64, 64
    q, k, v = f.zeros((1, H * D)), f.zeros((1, Hkv * D)), f.zeros((1, Hkv * D))
    kc, vc, out = f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.zeros((1, H * D))
    cos, sin = f.zeros((cap, D // 2)), f.zeros((cap, D // 2))
    with pytest.raises(fa.FoundryError) as e:
        f.decode_step_fused(q.arg(), k.arg(), v.arg(), None, kc.arg(), vc.arg(), cos.arg(), sin.arg(), out.arg(),
                            fa.KvPrepFusedParams.make(H, Hkv, D, 1, cap, cap))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:
        f.decode_step_fused(q.arg(), k.arg(), v.arg(), None, kc.arg(), vc.arg(), cos.arg(), sin.arg(), out.arg(),
                            fa.KvPrepFusedParams.make(H, Hkv, D, 2, 0, cap))
    assert e.value.variant == "InvalidShape"
    # a device position beyond the capacity appends nothing, and the next synchronize reports the dropped token
    dpos = f.array(np.array([cap + 5], np.uint32))
    f.decode_step_fused(q.arg(), k.arg(), v.arg(), None, kc.arg(), vc.arg(), cos.arg(), sin.arg(), out.arg(),
                        fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap), d_position=dpos, kv_len_bound=cap)
    with pytest.raises(fa.FoundryError) as e:
        f.synchronize()
    assert e.value.variant == "InvalidOperation"
    f.synchronize()
    assert not kc.download().any()


def test_in_kernel_merge_equals_merge_kernel_over_many_launches():
    """The merge by the last-arriving workgroup reads partials written by other workgroups of the same launch. It
    folds the same partials as the two-launch merge in another f32 order (one workgroup per head group there, one
    per head here), so the outputs agree to one f16 unit in the last place; and it is deterministic: repeated
    launches give the same bits (a stale partial would show in either check)."""
    announce("merge stress")
    f = ctx()
    rng = np.random.default_rng(123)
    H, Hkv, D, cap = 24, 8, 128, 4096
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    oa, ob = f.zeros((1, H * D)), f.zeros((1, H * D))
    lens = [int(x) for x in rng.integers(65, cap, size=40)] + [cap, 64 * 17 + 1]
    try:
        for kps in (64, 128, 0):
            for n in lens:
                f.set_decode_variant(kps, 1)
                f.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), oa.arg(), True, n - 1, H, D, n, 1)
                f.set_decode_variant(kps, 0)
                a = oa.download().astype(np.float32)
                first = None
                for _ in range(3):
                    f.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), ob.arg(), True, n - 1, H, D, n, 1)
                    f.synchronize()
                    got = ob.download()
                    if first is None:
                        first = bits(got)
                    assert np.array_equal(bits(got), first), (kps, n)
                    g = got.astype(np.float32)
                    assert np.all(np.abs(g - a) <= np.maximum(np.abs(a), 2.0 ** -14) * 2.0 ** -10), (kps, n)
    finally:
        f.set_decode_variant()


def test_polled_merge_equals_merge_kernel_over_many_launches():
    """The polled merge (every partition's workgroup merges a share of the columns as soon as the other partitions'
    records have arrived in the pattern-filled buffer) against the two-launch merge: one f16 unit in the last place
    (another f32 order), the same bits on every repetition, and the buffer is left ready for the next launch - a
    record that was not reset, or one taken before it had arrived, would show in one of the checks. Launch shapes on
    both sides of what the polled form takes (it needs all workgroups resident at once)."""
    announce("polled merge stress")
    f = ctx()
    rng = np.random.default_rng(321)
    for H, Hkv, D, cap in [(24, 8, 128, 4096), (14, 2, 64, 2048), (16, 4, 128, 8192), (32, 32, 128, 1024), (16, 1, 64, 4096)]:
        q = h16(rng.normal(size=(H, D)))
        k = h16(rng.normal(size=(Hkv, cap, D)))
        v = h16(rng.normal(size=(Hkv, cap, D)))
        dq, dk, dv = f.array(q), f.array(k), f.array(v)
        oa, ob = f.zeros((1, H * D)), f.zeros((1, H * D))
        lens = [int(x) for x in rng.integers(17, cap, size=12)] + [cap, min(cap, 64 * 17 + 1)]
        try:
            for kps in (0, 64, 256):
                for n in lens:
                    f.set_decode_variant(kps, 1)
                    f.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), oa.arg(), True, n - 1, H, D, n, 1)
                    f.set_decode_variant(kps, 2)
                    a = oa.download().astype(np.float32)
                    first = None
                    for _ in range(3):
                        f.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), ob.arg(), True, n - 1, H, D, n, 1)
                        f.synchronize()
                        got = ob.download()
                        if first is None:
                            first = bits(got)
                        assert np.array_equal(bits(got), first), (H, Hkv, D, kps, n)
                        g = got.astype(np.float32)
                        assert np.all(np.abs(g - a) <= np.maximum(np.abs(a), 2.0 ** -14) * 2.0 ** -10), (H, Hkv, D, kps, n)
        finally:
            f.set_decode_variant()
        for b in (dq, dk, dv, oa, ob):
            b.free()


def test_polled_merge_gives_up_cleanly():
    """Failure handling of the polled merge, forced from the host: with a wait bound of zero a merging workgroup gives
    up at its first look unless every record is already there. Every kernel still ends normally. The give-up is
    reported by whichever call waits for the stream next (here a download, with no synchronize in between), the record
    buffer is restored, and the context falls back to the two-launch merge until the polled form is selected again -
    which, with the normal bound, is then right on the SAME context."""
    announce("polled merge, zero wait bound")
    H, Hkv, D, cap, n = 24, 8, 128, 4096, 4000
    rng = np.random.default_rng(77)
    q, k, v = h16(rng.normal(size=(H, D))), h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, n).reshape(H, D)
    g = fa.Foundry(0)
    try:
        dq, dk, dv, do = g.array(q), g.array(k), g.array(v), g.zeros((1, H * D))
        dropped = g.array(np.array([cap + 5], np.uint32))
        kc, vc = g.zeros((Hkv, cap, D)), g.zeros((Hkv, cap, D))
        cos, sin, raw = g.zeros((cap, D // 2)), g.zeros((cap, D // 2)), g.zeros((1, H * D))
        failures = 0
        for it in range(4):
            g.set_decode_variant(0, 2)
            g.set_decode_poll_spin_us(0)
            g.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), do.arg(), True, n - 1, H, D, n, 1)
            if it == 0:
                # a second condition raised behind the first (a fused step at a position past its cache) must not erase it
                g.decode_step_fused(raw.arg(), raw.arg((1, Hkv * D)), raw.arg((1, Hkv * D)), None, kc.arg(), vc.arg(), cos.arg(),
                                    sin.arg(), raw.arg(), fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap), d_position=dropped,
                                    kv_len_bound=cap)
            try:
                got = do.download().reshape(H, D)  # waits for the stream: the report comes from here
                assert it > 0, "the dropped step of the first iteration was not reported"
                assert max_abs(got, want) <= TOL   # nobody had to wait: the result must be right
            except fa.FoundryError as e:
                if it == 0 and "waited longer" not in str(e):
                    assert e.variant == "InvalidOperation"  # only the dropped step was flagged (nobody had to wait)
                    continue
                failures += 1
                assert e.variant == "OperationFailed" and "waited longer" in str(e)
                assert it > 0 or "also dropped" in str(e)  # both conditions of the first iteration survive
                # the context has fallen back to the two-launch merge
                g.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), do.arg(), True, n - 1, H, D, n, 1)
                assert max_abs(do.download().reshape(H, D), want) <= TOL
            g.synchronize()  # nothing is left over
        # the polled form again on the same context, normal bound: right, repeatedly (the record buffer was restored)
        g.set_decode_poll_spin_us(5000)
        g.set_decode_variant(0, 2)
        for _ in range(3):
            g.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), do.arg(), True, n - 1, H, D, n, 1)
            assert max_abs(do.download().reshape(H, D), want) <= TOL
        g.synchronize()
    finally:
        g.close()
