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


def test_sage_quantiser_special_blocks_match_the_oracle_bit_for_bit():
    """The quantiser divides a block by its one scale through a shared reciprocal, which holds for a finite positive
    scale; other blocks take the plain division. Blocks of every kind against the oracle: all rows equal to the mean
    (scale 0), one infinity (scale infinite: finite values quantise to 0, the infinity - a NaN quotient - to -127, which is
    what a clamp with maxNum / minNum makes of a NaN), one NaN (ignored by the block's maximum, -127 itself), tiny values (a scale that is a subnormal f16), the largest f16 values, and
    values exactly half way between two steps of the grid."""
    announce("sage quantiser special blocks")
    f = ctx()
    rng = np.random.default_rng(7)
    Hkv, D, cap = 2, 128, 32 * 8
    k = h16(rng.normal(size=(Hkv, cap, D)))
    k[:, 0:32] = 0                                       # block 0: zeros (the mean below is zero, too)
    k[:, 40, 5] = np.float16(np.inf)                     # block 1: an infinity
    k[:, 70, 9] = np.float16(np.nan)                     # block 2: a NaN
    k[:, 96:128] = h16(rng.normal(size=(Hkv, 32, D)) * 1e-7)   # block 3: subnormal-scale values
    k[:, 128:160] = h16(rng.uniform(-65504, 65504, size=(Hkv, 32, D)))  # block 4: the f16 range
    half = (np.arange(D) % 255 - 127).astype(np.float32) + 0.5          # block 5: k / scale = n + 1/2 with scale 1: max |k| = 127
    k[:, 160:192] = h16(np.clip(half, -126.5, 126.5))[None, None, :]
    k[:, 160, 0] = np.float16(127.0)
    mean = np.zeros((Hkv, D), np.float32)
    dk, dmean = f.array(k), f.array(mean)
    dkq, dks = f.zeros((Hkv, cap, D), np.int8), f.zeros((Hkv, cap // 32), np.float16)
    f.sage_quantize_k(dk, dmean, Hkv, cap, D, 0, cap, dkq, dks)
    f.synchronize()
    with np.errstate(all="ignore"):
        want_kq, want_ks = orc.sage_quantize_k(k, mean, Hkv, cap, D, cap)
    got_q, got_s = dkq.download(), dks.download()
    assert np.array_equal(bits(got_s), bits(want_ks))
    assert np.array_equal(got_q, want_kq)
    assert not got_q[:, 0:32].any() and got_q[0, 40, 5] == -127 and got_q[0, 41, 5] == 0 and got_q[0, 70, 9] == -127
    for b in (dk, dmean, dkq, dks):
        b.free()


@pytest.mark.parametrize("launches", [1, 2], ids=["one_launch", "two_launches"])
@pytest.mark.parametrize("H,Hkv,D,start,cap,steps,mode,layer,nope_step,dyn", [
    (16, 4, 128, 90, 256, 40, fa.ROPE_NEOX, 0, 0, False),    # crosses the block boundaries at 96 and 128
    (14, 2, 64, 64, 160, 34, fa.ROPE_NORMAL, 0, 0, True),    # starts on an empty open block, device-side position
    (16, 4, 128, 37, 128, 6, fa.ROPE_NEOX, 3, 4, False),     # layer 3 of a model with every 4th layer un-rotated
    (16, 4, 128, 32760, 32800, 12, fa.ROPE_NEOX, 0, 0, True),   # SmolLM3 shape around the full 32K context
    (32, 8, 128, 49980, 50016, 5, fa.ROPE_NORMAL, 0, 0, True)])  # more partitions than compute units: 4-wave workgroups, merge kernel
def test_sage_decode_step_over_consecutive_tokens(H, Hkv, D, start, cap, steps, mode, layer, nope_step, dyn, launches):
    """fa_sage_decode_step: RoPE + append into the int8 cache (open block quantised anew from its exact rows, fixed
    mean) + int8 decode, over consecutive positions. After every step the int8 rows and scales must be bit for bit what
    the oracle's quantiser gives for the oracle's rotated f16 cache with the same mean, the V rows and the quantised
    query bit-exact, and the output within tolerance of the oracle's int8 model; the error against f16 SDPA on the
    unquantised cache is measured."""
    announce("sage decode step", H, Hkv, D, start, cap, steps, mode, layer, nope_step, dyn, launches)
    f = ctx()
    f.set_sage_step_variant(launches)
    rng = np.random.default_rng(start + cap + D)
    cos, sin = fa.rope_tables(1e6, D, cap)
    kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    kc[:, :start] = outlier_normal(rng, (Hkv, start, D))
    vc[:, :start] = outlier_normal(rng, (Hkv, start, D))
    dk, dv = f.array(kc), f.array(vc)
    desc, bufs = fa.sage_cache(f, H, Hkv, cap, D, dv)
    f.sage_cache_build(dk, start, desc)
    f.synchronize()
    mean = bufs["k_mean"].download()
    assert max_abs(mean, orc.sage_k_mean(kc, Hkv, cap, D, start)) <= 2e-5
    dcos, dsin, dout = f.array(cos), f.array(sin), f.zeros((H * D,))
    dpos = f.array(np.array([start], np.uint32)) if dyn else None
    rope_mode = 0 if mode == fa.ROPE_NEOX else 1
    worst_model, worst_full = 0.0, 0.0
    for t in range(steps):
        P = start + t
        q, k, v = (outlier_normal(rng, (1, n * D)) for n in (H, Hkv, Hkv))
        dq, dkn, dvn = f.array(q), f.array(k), f.array(v)
        p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0 if dyn else P, cap, mode, layer_idx=layer, no_rope_layer_step=nope_step)
        f.sage_decode_step(dq.arg(), dkn.arg(), dvn.arg(), desc, dcos.arg(), dsin.arg(), dout.arg(), p, d_position=dpos,
                           kv_len_bound=cap if dyn else 0)
        if dyn:
            f.u32_add(dpos, 1, 1)
        f.synchronize()
        # the oracle's f16 path appends the rotated row to its f16 cache; the int8 state is its quantisation
        qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin,
                               orc.make_params(H, Hkv, D, 1, P, cap, rope_mode=rope_mode, layer_idx=layer, no_rope_layer_step=nope_step))
        N = P + 1
        check_state = t < 3 or t == steps - 1 or N % 32 in (0, 1)
        if check_state:
            want_kq, want_ks = orc.sage_quantize_k(kc, mean, Hkv, cap, D, N)
            nb = (N + 31) // 32
            assert np.array_equal(bits(bufs["k_scale"].download()[:, :nb]), bits(want_ks[:, :nb])), (t, "scales")
            assert np.array_equal(bufs["k_q"].download()[:, :N], want_kq[:, :N]), (t, "int8 rows")
            assert np.array_equal(bits(dv.download()[:, :N]), bits(vc[:, :N])), (t, "v rows")
            want_qq, want_qs = orc.sage_quantize_q(np.ascontiguousarray(qr[:, 0]), H, D)
            assert np.array_equal(bufs["q_q"].download(), want_qq) and np.array_equal(bufs["q_scale"].download(), want_qs)
            got = dout.download().reshape(H, D)
            model = orc.sage_decode(want_qq, want_qs, want_kq, want_ks, vc, H, Hkv, D, cap, N, n_threads=8).reshape(H, D)
            # the bound scales with the outputs: at a few dozen keys with 8-sigma values they reach 2 .. 4, where one f16
            # unit in the last place is already 2e-3 .. 4e-3
            worst_model = max(worst_model, max_abs(got, model) / max(1.0, float(np.max(np.abs(model)))))
            full = rm.gqa_decode_f64(np.ascontiguousarray(qr[:, 0]), kc, vc, H, Hkv, D, N)
            worst_full = max(worst_full, max_abs(got, full))
        for b in (dq, dkn, dvn):
            b.free()
    f.set_sage_step_variant()
    print("sage decode step: max abs err vs int8 model (relative to max(1, |out|)) %.2e, vs f16 sdpa %.4f" % (worst_model, worst_full), flush=True)
    assert worst_model <= 2e-3
    assert worst_full <= 0.2
    # untouched rows past the last position stay zero
    assert not bufs["k_q"].download()[:, start + steps:].any()
    for b in list(bufs.values()) + [dk, dcos, dsin, dout] + ([dpos] if dyn else []):
        b.free()


def test_sage_decode_step_errors():
    announce("sage decode step errors")
    f = ctx()
    H, Hkv, D, cap = 8, 2, 128, 64
    dv = f.zeros((Hkv, cap, D))
    desc, bufs = fa.sage_cache(f, H, Hkv, cap, D, dv)
    q, k, v, out = f.zeros((1, H * D)), f.zeros((1, Hkv * D)), f.zeros((1, Hkv * D)), f.zeros((H * D,))
    cos, sin = f.zeros((cap, D // 2)), f.zeros((cap, D // 2))
    with pytest.raises(fa.FoundryError) as e:  # position at the capacity
        f.sage_decode_step(q.arg(), k.arg(), v.arg(), desc, cos.arg(), sin.arg(), out.arg(), fa.KvPrepFusedParams.make(H, Hkv, D, 1, cap, cap))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:  # params of another shape
        f.sage_decode_step(q.arg(), k.arg(), v.arg(), desc, cos.arg(), sin.arg(), out.arg(), fa.KvPrepFusedParams.make(H, Hkv, 64, 1, 0, cap))
    assert e.value.variant == "InvalidShape"
    dpos = f.array(np.array([cap + 3], np.uint32))  # a device position past the cache: dropped and reported
    f.sage_decode_step(q.arg(), k.arg(), v.arg(), desc, cos.arg(), sin.arg(), out.arg(), fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap),
                       d_position=dpos, kv_len_bound=cap)
    with pytest.raises(fa.FoundryError) as e:
        f.synchronize()
    assert e.value.variant == "InvalidOperation"
    f.synchronize()
    for b in list(bufs.values()) + [q, k, v, out, cos, sin, dpos]:
        b.free()
