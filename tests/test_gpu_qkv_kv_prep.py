"""GPU parity: FusedQkv + KvPrepFused as one op (fa_fused_qkv_kv_prep, fa_fused_qkv_kv_prep_paged).

The contract is bit equality with the two ops run one after the other on the same context (src/metals/gemv/qkv_step.rs:14-120
then src/metals/kv_prep/kv_prep_fused.metal:26-123, whose own parity test tests/kv_prep_fused.rs:239-244 is bit exact too):
q_rot, and every cache row, must hold the same 16 bits. The chain is in turn checked against the oracle - the projections
within the FusedQkv tolerance, KvPrepFused applied to the library's own projections bit for bit."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx
from test_gpu_paged import Paged
from test_gpu_qkv import _close, _data

pytestmark = pytest.mark.gpu


def _paths(m):
    """(GEMM threshold, GEMM variant): the defaults, every GEMM kernel, and - for short chunks - the weight-stream form."""
    if m < 12:
        return [(0, 0), (1, 0), (1, 1)]
    if m <= 64:
        paths = [(0, 0), (0, 1), (0, 2), (0, 3), (1 << 30, 0)]
        if 12 <= m <= 32:  # an explicit threshold: the GEMM also where the one-launch kernel for up to 32 rows takes the chunk
            paths += [(12, 0), (12, 1), (12, 2), (12, 3)]
        return paths
    return [(0, 0), (0, 1), (0, 2), (0, 3)]


@pytest.mark.parametrize("H,Hkv,D,K,m,pos,cap,mode,norm,bias,layout,layer,step", [
    (24, 8, 128, 3072, 256, 0, 512, fa.ROPE_NORMAL, True, False, 1, 0, 0),     # Llama-3.2-3B, a 256-token chunk
    (24, 8, 128, 3072, 32, 8160, 8448, fa.ROPE_NORMAL, True, False, 1, 0, 0),  # the reference's default chunk after a prefix (split-K)
    (14, 2, 64, 896, 200, 37, 384, fa.ROPE_NEOX, True, True, 0, 0, 0),         # Qwen2.5-0.5B: NeoX pairs, biases, 2 heads per tile, ragged tiles
    (14, 2, 64, 896, 32, 5, 128, fa.ROPE_NEOX, True, True, 1, 0, 0),           # same through split-K: the mate piece summed a second time
    (16, 4, 128, 1024, 130, 3, 256, fa.ROPE_NEOX, False, False, 1, 3, 4),      # SmolLM3 rule: layer 3 of every 4 is not rotated
    (16, 4, 128, 1024, 130, 3, 256, fa.ROPE_NEOX, False, True, 1, 2, 4),       # ... layer 2 is
    (8, 8, 64, 512, 5, 100, 128, fa.ROPE_NORMAL, True, True, 1, 0, 0),         # a few rows: weight stream, then KvPrepFused, inside the op
    (3, 1, 64, 256, 17, 0, 32, fa.ROPE_NEOX, True, False, 0, 0, 0),            # 192 weight rows: a tile and a half
    # chunks of 12 to 32 rows against 2048 or 3072 features: KvPrepFused as the write stage of the one-launch weight stream
    (16, 2, 128, 2048, 17, 40, 128, fa.ROPE_NEOX, True, True, 1, 0, 0),        # NeoX pairs (a workgroup takes both halves), biases, ragged rows
    (14, 2, 128, 2048, 32, 5, 64, fa.ROPE_NEOX, False, False, 0, 0, 0),        # row-major weights, a last workgroup with two pairs
    (32, 8, 64, 2048, 24, 3, 64, fa.ROPE_NEOX, True, True, 1, 0, 0),           # 64-wide heads: pairs of one workgroup across two heads
    (32, 8, 64, 3072, 12, 50, 64, fa.ROPE_NORMAL, True, True, 1, 0, 0),        # adjacent pairs, 64-wide heads, biases
    (16, 4, 128, 2048, 20, 3, 64, fa.ROPE_NEOX, True, False, 1, 3, 4),         # a layer that is not rotated
    (16, 4, 128, 2048, 20, 3, 64, fa.ROPE_NEOX, True, False, 1, 2, 4),         # ... and one that is
])
def test_fused_op_equals_the_two_ops(H, Hkv, D, K, m, pos, cap, mode, norm, bias, layout, layer, step):
    announce("fused qkv + kv prep", H, Hkv, D, K, m, pos, cap, mode, norm, bias, layout, layer, step)
    f = ctx()
    rng = np.random.default_rng(H * 1000 + K + m)
    N, NK = H * D, Hkv * D
    x, g, ws, bs = _data(rng, K, N, NK, m)
    kc0, vc0 = (rng.normal(size=(Hkv, cap, D)).astype(np.float16) for _ in range(2))
    cos, sin = fa.rope_tables(5e5, D, cap)
    dev_w = [f.array(orc.to_canonical(w) if layout == 1 else w.reshape(-1)) for w in ws]
    dx, dg, db = f.array(x), f.array(g), [f.array(b) for b in bs]
    dcos, dsin = f.array(cos), f.array(sin)
    dq, dk, dv = (f.zeros((m, n)) for n in (N, NK, NK))
    dqr = [f.zeros((H, m, D)) for _ in range(2)]
    dkc = [f.array(kc0) for _ in range(2)]
    dvc = [f.array(vc0) for _ in range(2)]
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, pos, cap, mode, layer_idx=layer, no_rope_layer_step=step)
    kw = dict(gamma=dg.arg() if norm else None, biases=[b.arg() for b in db] if bias else None, layout=layout)
    try:
        for min_m, variant in _paths(m):
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            for d, src in ((dkc[0], kc0), (dkc[1], kc0), (dvc[0], vc0), (dvc[1], vc0)):
                d.upload(src)
            for d in dqr:
                d.upload(np.zeros((H, m, D), np.float16))
            # the two ops
            f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), dq.arg(), dk.arg(), dv.arg(), K, N, NK, m, **kw)
            f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), dqr[0].arg(), dkc[0].arg(), dvc[0].arg(), dcos.arg(), dsin.arg(), p)
            # the one op
            f.fused_qkv_kv_prep(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), K, dqr[1].arg(), dcos.arg(), dsin.arg(), p,
                                k_cache=dkc[1].arg(), v_cache=dvc[1].arg(), **kw)
            f.synchronize()
            tag = (min_m, variant)
            assert np.array_equal(bits(dqr[0].download()), bits(dqr[1].download())), tag
            assert np.array_equal(bits(dkc[0].download()), bits(dkc[1].download())), tag
            assert np.array_equal(bits(dvc[0].download()), bits(dvc[1].download())), tag
            # the chain itself against the oracle: projections within the FusedQkv bar, KvPrepFused on them exact
            q, k, v = dq.download(), dk.download(), dv.download()
            want = orc.fused_qkv(x, *ws, gamma=g if norm else None, biases=bs if bias else None, layout=0)
            for got, w in zip((q, k, v), want):
                assert _close(got, w, K), tag
            kc_w, vc_w = kc0.copy(), vc0.copy()
            qr_w = orc.kv_prep_fused(q, k, v, kc_w, vc_w, cos, sin,
                                     orc.make_params(H, Hkv, D, m, pos, cap, rope_mode=mode, layer_idx=layer, no_rope_layer_step=step))
            assert np.array_equal(bits(dqr[1].download()), bits(qr_w)), tag
            assert np.array_equal(bits(dkc[1].download()), bits(kc_w)), tag
            assert np.array_equal(bits(dvc[1].download()), bits(vc_w)), tag
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    for b in dev_w + [dx, dg, dcos, dsin, dq, dk, dv] + db + dqr + dkc + dvc:
        b.free()


@pytest.mark.parametrize("H,Hkv,D,K,m,pos,bs,mode", [
    (24, 8, 128, 3072, 150, 0, 16, fa.ROPE_NORMAL),   # an empty sequence of a batch of three
    (16, 2, 128, 2048, 64, 40, 16, fa.ROPE_NEOX),     # after a prefix that ends inside a block
    (14, 2, 64, 896, 7, 9, 32, fa.ROPE_NEOX),         # a few rows (the weight-stream form)
    (16, 2, 128, 2048, 30, 40, 16, fa.ROPE_NEOX),     # a chunk of the one-launch weight stream: rows across three blocks
    (24, 8, 128, 3072, 32, 37, 16, fa.ROPE_NORMAL),
])
def test_fused_op_into_a_paged_cache(H, Hkv, D, K, m, pos, bs, mode):
    announce("fused qkv + kv prep, paged", H, Hkv, D, K, m, pos, bs, mode)
    f = ctx()
    rng = np.random.default_rng(K + m + pos)
    N, NK = H * D, Hkv * D
    x, g, ws, _ = _data(rng, K, N, NK, m)
    cos, sin = fa.rope_tables(1e6, D, pos + m + 8)
    pgs = [Paged(f, np.random.default_rng(5), [0, pos, 0], Hkv, D, bs, extra_tokens=m + 1).upload() for _ in range(2)]
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dx, dg, dcos, dsin = f.array(x), f.array(g), f.array(cos), f.array(sin)
    dq, dk, dv = (f.zeros((m, n)) for n in (N, NK, NK))
    dqr = [f.zeros((H, m, D)) for _ in range(2)]
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, pos, 0, mode)
    f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), dq.arg(), dk.arg(), dv.arg(), K, N, NK, m, gamma=dg.arg())
    f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr[0].arg(), pgs[0].desc, 1, dcos.arg(), dsin.arg(), p)
    f.fused_qkv_kv_prep(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), K, dqr[1].arg(), dcos.arg(), dsin.arg(), p,
                        paged=pgs[1].desc, seq_index=1, gamma=dg.arg())
    f.synchronize()
    assert np.array_equal(pgs[0].bt, pgs[1].bt)  # same seed: same block tables
    assert np.array_equal(bits(dqr[0].download()), bits(dqr[1].download()))
    kp, vp = pgs[1].dk.download(), pgs[1].dv.download()
    assert np.array_equal(bits(pgs[0].dk.download()), bits(kp))
    assert np.array_equal(bits(pgs[0].dv.download()), bits(vp))
    # and against the oracle on the library's projections; rows outside [pos, pos + m) and other sequences stay empty
    kc_w, vc_w = np.zeros((Hkv, pos + m, D), np.float16), np.zeros((Hkv, pos + m, D), np.float16)
    qr_w = orc.kv_prep_fused(dq.download(), dk.download(), dv.download(), kc_w, vc_w, cos, sin,
                             orc.make_params(H, Hkv, D, m, pos, pos + m, rope_mode=mode))
    assert np.array_equal(bits(dqr[1].download()), bits(qr_w))
    assert np.array_equal(bits(orc.paged_gather(kp, pgs[1].bt[1], Hkv, bs, D, pos + m)), bits(kc_w))
    assert np.array_equal(bits(orc.paged_gather(vp, pgs[1].bt[1], Hkv, bs, D, pos + m)), bits(vc_w))
    for s in (0, 2):
        assert not orc.paged_gather(kp, pgs[1].bt[s], Hkv, bs, D, m).any()
    for pg in pgs:
        pg.free()
    for b in dev_w + [dx, dg, dcos, dsin, dq, dk, dv] + dqr:
        b.free()


def test_fused_op_of_a_short_chunk_is_one_launch():
    """A chunk of 12 to 32 rows (the reference's default prefill chunk, src/model/executor.rs:232-250) against 2048 or 3072
    features: RMSNorm, projections, RoPE and the cache append leave ONE kernel (the profiler's launch counts)."""
    announce("fused qkv + kv prep, launches of a short chunk")
    f = ctx()
    H, Hkv, D, K, m, pos, cap = 24, 8, 128, 3072, 32, 100, 256
    rng = np.random.default_rng(11)
    x, g, ws, _ = _data(rng, K, H * D, Hkv * D, m)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dx, dg, dcos, dsin = f.array(x), f.array(g), f.array(cos), f.array(sin)
    dqr, dkc, dvc = f.zeros((H, m, D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, pos, cap, fa.ROPE_NORMAL)
    f.profile_reset()
    f.profile_enable(True)
    try:
        f.fused_qkv_kv_prep(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), K, dqr.arg(), dcos.arg(), dsin.arg(), p,
                            k_cache=dkc.arg(), v_cache=dvc.arg(), gamma=dg.arg())
        f.synchronize()
        assert f.profile_query("fused_qkv_rows32_rope_kernel")[0] == 1
        for other in ("fused_qkv_rows32_kernel", "kv_prep_fused_elem_kernel", "kv_prep_fused_vec_kernel", "fused_qkv_gemm_kernel"):
            assert f.profile_query(other)[0] == 0, other
    finally:
        f.profile_enable(False)
    kc, vc = dkc.download(), dvc.download()
    assert not kc[:, :pos].any() and not kc[:, pos + m:].any() and kc[:, pos:pos + m].any()  # only the chunk's rows are written
    assert not vc[:, :pos].any() and not vc[:, pos + m:].any() and vc[:, pos:pos + m].any()
    for b in dev_w + [dx, dg, dcos, dsin, dqr, dkc, dvc]:
        b.free()


def test_fused_op_errors():
    announce("fused qkv + kv prep errors")
    f = ctx()
    H, Hkv, D, K, m, cap = 4, 2, 64, 128, 16, 64
    rng = np.random.default_rng(3)
    x, g, ws, _ = _data(rng, K, H * D, Hkv * D, m)
    cos, sin = fa.rope_tables(1e4, D, cap)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dx, dcos, dsin = f.array(x), f.array(cos), f.array(sin)
    dqr, dkc, dvc = f.zeros((H, m, D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D))

    def run(p, **kw):
        f.fused_qkv_kv_prep(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), K, dqr.arg(), dcos.arg(), dsin.arg(), p,
                            k_cache=dkc.arg(), v_cache=dvc.arg(), **kw)

    run(fa.KvPrepFusedParams.make(H, Hkv, D, m, 0, cap, fa.ROPE_NEOX))  # the well-formed call
    with pytest.raises(fa.FoundryError) as e:  # rows past the cache
        run(fa.KvPrepFusedParams.make(H, Hkv, D, m, cap - 3, cap, fa.ROPE_NEOX))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:  # a head size the write stage is not built for
        p = fa.KvPrepFusedParams.make(H * 2, Hkv * 2, 32, m, 0, cap, fa.ROPE_NEOX)
        run(p)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:  # inconsistent geometry
        p = fa.KvPrepFusedParams.make(H, Hkv, D, m, 0, cap, fa.ROPE_NEOX)
        p.group_size = 3
        run(p)
    assert e.value.variant == "InvalidShape"
    f.synchronize()
    for b in dev_w + [dx, dcos, dsin, dqr, dkc, dvc]:
        b.free()
