"""GPU parity: fused RoPE + KV-cache append (fa_kv_prep_fused*) against the CPU oracle.
Bar: cache slots and values bit-exact; q_rot bit-exact too (same f32 op order, one RNE convert)."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16

pytestmark = pytest.mark.gpu

SHAPES = [  # (seq, pos, cap, H, Hkv, D): first three are tests/kv_prep_fused.rs:249-267
    (1, 5, 16, 14, 2, 64), (4, 0, 16, 14, 2, 64), (2, 0, 64, 32, 8, 128),
    (1, 1024, 1152, 14, 2, 64),      # Qwen2.5-0.5B decode step of benchmark configuration 1
    (1, 8192, 8448, 24, 8, 128),     # Llama-3.2-3B decode step
    (33, 100, 256, 24, 8, 128), (7, 3, 32, 16, 4, 128), (5, 0, 8, 16, 2, 128),
]


def _run(S, off, cap, H, Hkv, D, mode, layer=0, step=0, base=10000.0, dyn=False, seed=0):
    f = ctx()
    rng = np.random.default_rng(seed + S * 7 + off)
    q, k, v = (h16(rng.normal(size=(S, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(base, D, cap)
    pre_k = h16(rng.normal(size=(Hkv, cap, D)))  # existing cache contents must survive
    pre_v = h16(rng.normal(size=(Hkv, cap, D)))
    ok, ov = pre_k.copy(), pre_v.copy()
    want_q = orc.kv_prep_fused(q, k, v, ok, ov, cos, sin,
                               orc.make_params(H, Hkv, D, S, off, cap, rope_mode=mode, layer_idx=layer,
                                               no_rope_layer_step=step))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    dqr = f.zeros((H, S, D))
    dkc, dvc = f.array(pre_k), f.array(pre_v)
    dcos, dsin = f.array(cos), f.array(sin)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, S, 0 if dyn else off, cap, mode, layer, step)
    dpos = f.array(np.array([off], np.uint32)) if dyn else None
    f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), p, dpos)
    f.synchronize()
    got_q, got_k, got_v = dqr.download(), dkc.download(), dvc.download()
    for b in (dq, dk, dv, dqr, dkc, dvc, dcos, dsin):
        b.free()
    assert np.array_equal(bits(got_q), bits(want_q)), "q_rot differs"
    assert np.array_equal(bits(got_k), bits(ok)), "k_cache differs"
    assert np.array_equal(bits(got_v), bits(ov)), "v_cache differs"


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mode", [fa.ROPE_NEOX, fa.ROPE_NORMAL])
def test_kv_prep_fused_bit_exact(shape, mode):
    announce("kv_prep_fused", shape, "mode", mode)
    _run(*shape, mode)


@pytest.mark.parametrize("layer", [0, 3, 7, 8])
def test_kv_prep_nope_layers(layer):
    announce("kv_prep nope layer", layer)
    _run(3, 9, 32, 16, 4, 128, fa.ROPE_NORMAL, layer=layer, step=4, base=5e6)


def test_kv_prep_device_position_and_odd_head_dim():
    announce("kv_prep dyn position")
    _run(1, 77, 128, 24, 8, 128, fa.ROPE_NORMAL, base=5e5, dyn=True)
    _run(4, 60, 128, 14, 2, 64, fa.ROPE_NEOX, base=1e6, dyn=True)
    announce("kv_prep element path (head_dim 24, 6)")
    _run(3, 2, 16, 6, 2, 24, fa.ROPE_NEOX)
    _run(2, 1, 8, 4, 4, 6, fa.ROPE_NORMAL)


def test_kv_prep_consecutive_appends_build_the_same_cache():
    """Appending 1 row at a time and appending the block at once give identical caches."""
    announce("kv_prep consecutive appends")
    f = ctx()
    H, Hkv, D, cap, T = 14, 2, 64, 64, 9
    rng = np.random.default_rng(3)
    q, k, v = (h16(rng.normal(size=(T, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(1e6, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    kc1, vc1, kc2, vc2 = (f.zeros((Hkv, cap, D)) for _ in range(4))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    qr = f.zeros((H, T, D))
    f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), qr.arg(), kc1.arg(), vc1.arg(), dcos.arg(), dsin.arg(),
                    fa.KvPrepFusedParams.make(H, Hkv, D, T, 5, cap, fa.ROPE_NEOX))
    qr1 = f.zeros((H, 1, D))
    for t in range(T):
        f.kv_prep_fused(dq.arg((1, H * D), offset=t * H * D * 2), dk.arg((1, Hkv * D), offset=t * Hkv * D * 2),
                        dv.arg((1, Hkv * D), offset=t * Hkv * D * 2), qr1.arg(), kc2.arg(), vc2.arg(), dcos.arg(),
                        dsin.arg(), fa.KvPrepFusedParams.make(H, Hkv, D, 1, 5 + t, cap, fa.ROPE_NEOX))
    f.synchronize()
    assert np.array_equal(bits(kc1.download()), bits(kc2.download()))
    assert np.array_equal(bits(vc1.download()), bits(vc2.download()))
    assert np.array_equal(bits(qr.download()[:, T - 1]), bits(qr1.download()[:, 0]))


def test_kv_prep_errors():
    announce("kv_prep error paths")
    f = ctx()
    H, Hkv, D, cap = 4, 2, 64, 16
    bufs = dict(q=f.zeros((1, H * D)), k=f.zeros((1, Hkv * D)), v=f.zeros((1, Hkv * D)), qr=f.zeros((H, 1, D)),
                kc=f.zeros((Hkv, cap, D)), vc=f.zeros((Hkv, cap, D)), cos=f.zeros((cap, D // 2)),
                sin=f.zeros((cap, D // 2)))

    def call(p, **over):
        a = {n: b.arg() for n, b in bufs.items()}
        a.update(over)
        f.kv_prep_fused(a["q"], a["k"], a["v"], a["qr"], a["kc"], a["vc"], a["cos"], a["sin"], p)

    good = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap)
    call(good)
    with pytest.raises(fa.FoundryError) as e:  # context overflow
        call(fa.KvPrepFusedParams.make(H, Hkv, D, 1, cap, cap))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:
        bad = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap)
        bad.group_size = 3
        call(bad)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:
        none = fa.TensorArg()
        call(good, k=none)
    assert e.value.variant == "InputNotFound" and "k" in str(e.value)
    with pytest.raises(fa.FoundryError) as e:
        call(good, q=bufs["q"].arg(dtype=fa.DTYPE_F32))
    assert e.value.variant == "UnsupportedDtype" and e.value.dtype == fa.DTYPE_F32  # the refused dtype travels with the error
    with pytest.raises(fa.FoundryError) as e:
        call(good, kc=bufs["kc"].arg((Hkv, cap // 2, D)))
    assert e.value.variant == "InvalidShape"
    f.synchronize()
    for b in bufs.values():
        b.free()
