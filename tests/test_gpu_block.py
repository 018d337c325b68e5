"""GPU parity of the whole attention block as the reference's model graph runs it (models/llama.json:509-585):
FusedQkv -> KvPrepFused -> FlashAttention -> MatMul (o_proj + residual), decode step and prefill chunk, each stage
checked against the oracle on the stage's actual inputs and the block's output end to end."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu


def _ulp_close(got, want, ulps=2, slack=1e-3):
    g, w = got.astype(np.float64), want.astype(np.float64)
    return bool(np.all(np.abs(g - w) <= ulps * np.maximum(np.abs(w), 2.0 ** -10) * 2.0 ** -10 + slack))


@pytest.mark.parametrize("m,prefix,q8", [(1, 300, False), (1, 300, True), (24, 100, False), (32, 0, True)])
def test_attention_block_stage_by_stage_and_end_to_end(m, prefix, q8):
    announce("attention block", m, prefix, q8)
    f = ctx()
    rng = np.random.default_rng(m * 1000 + prefix + int(q8))
    H, Hkv, D, cap = 8, 2, 64, 512
    dm, kvd = H * D, Hkv * D
    hidden = rng.uniform(-1, 1, (m, dm)).astype(np.float16)
    gamma = rng.uniform(0.5, 1.5, dm).astype(np.float16)
    ws = [rng.uniform(-0.1, 0.1, (n, dm)).astype(np.float16) for n in (dm, kvd, kvd)]
    wo = rng.uniform(-0.1, 0.1, (dm, dm)).astype(np.float16)
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    kc[:, :prefix], vc[:, :prefix] = h16(rng.normal(size=(Hkv, prefix, D))), h16(rng.normal(size=(Hkv, prefix, D)))
    cos, sin = fa.rope_tables(1e4, D, cap)
    if q8:
        qw = [orc.quantize_q8_0(w) for w in ws]
        qo = orc.quantize_q8_0(wo)
        dev_w = [f.array(orc.to_canonical(w)) for w, _ in qw]
        dev_s = [f.array(s) for _, s in qw]
        dwo, dso = f.array(orc.to_canonical(qo[0])), f.array(qo[1])
    else:
        dev_w, dev_s = [f.array(orc.to_canonical(w)) for w in ws], None
        dwo, dso = f.array(orc.to_canonical(wo)), None
    dh, dg = f.array(hidden), f.array(gamma)
    dq, dk, dv = f.zeros((m, dm)), f.zeros((m, kvd)), f.zeros((m, kvd))
    dqr, dkc, dvc, dcos, dsin = f.zeros((H, m, D)), f.array(kc), f.array(vc), f.array(cos), f.array(sin)
    dattn, dres = f.zeros((m, dm)), f.zeros((m, dm))
    # the four steps of the layer
    f.fused_qkv(dh.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), dq.arg(), dk.arg(), dv.arg(), dm, dm, kvd, m,
                gamma=dg.arg(), scales=[s.arg() for s in dev_s] if q8 else None)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, prefix, cap, fa.ROPE_NEOX)
    f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), p)
    f.flash_attention(dqr.arg(), dkc.arg(), dvc.arg(), dattn.arg(), True, prefix, H, D, prefix + m, m)
    f.matmul(dattn.arg(), dwo.arg(), dres.arg(), m, dm, dm, c=dh.arg(), transpose_b=False, alpha=1.0, beta=1.0,
             b_scales=dso.arg() if q8 else None)
    f.synchronize()
    gq, gk, gv, gattn, gres = dq.download(), dk.download(), dv.download(), dattn.download(), dres.download()

    # stage 1 against the oracle
    if q8 and m >= 12:  # a chunk: the GEMM's arithmetic, f16(q * scale) weights (src/metals/mma/tile_loader.metal:100-120)
        wq, wk, wv = orc.fused_qkv(hidden, *[orc.dequantize_blocks(w, s) for w, s in qw], gamma=gamma)
    elif q8:
        wq, wk, wv = orc.fused_qkv_q8(hidden, [w for w, _ in qw], [s for _, s in qw], gamma=gamma)
    else:
        wq, wk, wv = orc.fused_qkv(hidden, *ws, gamma=gamma)
    assert _ulp_close(gq, wq) and _ulp_close(gk, wk) and _ulp_close(gv, wv)
    # stage 2 on the GPU's q, k, v: bit-exact
    kw, vw = kc.copy(), vc.copy()
    qr = orc.kv_prep_fused(gq, gk, gv, kw, vw, cos, sin, orc.make_params(H, Hkv, D, m, prefix, cap, rope_mode=0))
    assert np.array_equal(bits(dqr.download()), bits(qr))
    assert np.array_equal(bits(dkc.download()), bits(kw)) and np.array_equal(bits(dvc.download()), bits(vw))
    # stage 3 on those caches
    want_attn = np.stack([orc.sdpa_decode(qr[:, r].copy(), kw, vw, H, Hkv, D, cap, prefix + r + 1).reshape(dm) for r in range(m)])
    assert max_abs(gattn, want_attn) <= 2e-3
    # stage 4 on the GPU's attention output
    def o_proj(attn):
        if q8 and m >= 12:
            return orc.matmul_gemv(attn, orc.dequantize_blocks(qo[0], qo[1]), None, hidden, 0, 32, 1.0, 1.0)
        if q8:
            return orc.matmul_gemv_q8(attn, qo[0], qo[1], None, hidden, 0, 32, 1.0, 1.0)
        return orc.matmul_gemv(attn, wo, None, hidden, 0, 32, 1.0, 1.0)

    want_res = o_proj(gattn)
    assert _ulp_close(gres, want_res)
    # end to end: the oracle's own chain from `hidden`
    kw2, vw2 = kc.copy(), vc.copy()
    qr2 = orc.kv_prep_fused(wq, wk, wv, kw2, vw2, cos, sin, orc.make_params(H, Hkv, D, m, prefix, cap, rope_mode=0))
    attn2 = np.stack([orc.sdpa_decode(qr2[:, r].copy(), kw2, vw2, H, Hkv, D, cap, prefix + r + 1).reshape(dm) for r in range(m)])
    res2 = o_proj(attn2)
    assert max_abs(gres, res2) <= 2e-2  # f16 roundings of q, k, v and attn_out carried through two projections
    for b in dev_w + (dev_s or []) + [dwo, dh, dg, dq, dk, dv, dqr, dkc, dvc, dcos, dsin, dattn, dres] + ([dso] if q8 else []):
        b.free()


@pytest.mark.parametrize("mode,paired_prefix", [(fa.ROPE_NORMAL, 2100), (fa.ROPE_NEOX, 2049)])
def test_prefill_chunk_block_as_graph_replays(mode, paired_prefix):
    """The attention block of the reference's default prefill mode (a chunk of 32 rows after a prefix,
    src/model/executor.rs:232-250) on the kernels that shape takes - FusedQkv + KvPrepFused as ONE launch, the short-chunk
    attention kernel, the one-launch o_proj - captured as a HIP graph and replayed: every replay against the oracle's chain on
    the same inputs (the chunk's cache rows are rewritten with the same values by every replay)."""
    announce("prefill chunk block, graph replays", mode, paired_prefix)
    f = ctx()
    m, prefix = 32, paired_prefix
    H, Hkv, D, cap = 16, 4, 128, prefix + 64
    dm, kvd = H * D, Hkv * D
    rng = np.random.default_rng(prefix + mode)
    hidden = rng.uniform(-1, 1, (m, dm)).astype(np.float16)
    gamma = rng.uniform(0.5, 1.5, dm).astype(np.float16)
    ws = [rng.uniform(-0.05, 0.05, (n, dm)).astype(np.float16) for n in (dm, kvd, kvd)]
    wo = rng.uniform(-0.05, 0.05, (dm, dm)).astype(np.float16)
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    kc[:, :prefix], vc[:, :prefix] = h16(rng.normal(size=(Hkv, prefix, D))), h16(rng.normal(size=(Hkv, prefix, D)))
    cos, sin = fa.rope_tables(5e5, D, cap)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dwo, dh, dg = f.array(orc.to_canonical(wo)), f.array(hidden), f.array(gamma)
    dqr, dkc, dvc, dcos, dsin = f.zeros((H, m, D)), f.array(kc), f.array(vc), f.array(cos), f.array(sin)
    dattn, dres = f.zeros((m, dm)), f.zeros((m, dm))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, prefix, cap, mode)

    def enqueue():
        f.fused_qkv_kv_prep(dh.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), dm, dqr.arg(), dcos.arg(), dsin.arg(), p,
                            k_cache=dkc.arg(), v_cache=dvc.arg(), gamma=dg.arg())
        f.flash_attention(dqr.arg(), dkc.arg(), dvc.arg(), dattn.arg(), True, prefix, H, D, prefix + m, m)
        f.matmul(dattn.arg(), dwo.arg(), dres.arg(), m, dm, dm, c=dh.arg(), transpose_b=False, alpha=1.0, beta=1.0)

    # the launches this shape takes, from the profiler's counts of one eager pass (which also sizes the workspaces)
    f.profile_reset()
    f.profile_enable(True)
    try:
        enqueue()
        f.synchronize()
        counts = {k: f.profile_query(k)[0] for k in ("fused_qkv_rows32_rope_kernel", "flash_chunk_kernel", "matmul_rows32_kernel")}
    finally:
        f.profile_enable(False)
    assert counts == {"fused_qkv_rows32_rope_kernel": 1, "flash_chunk_kernel": 1, "matmul_rows32_kernel": 1}, counts
    # the oracle's chain: projections, rotation + append, causal attention of every row, o_proj with residual
    wq, wk, wv = orc.fused_qkv(hidden, *ws, gamma=gamma)
    kw, vw = kc.copy(), vc.copy()
    qr = orc.kv_prep_fused(wq, wk, wv, kw, vw, cos, sin, orc.make_params(H, Hkv, D, m, prefix, cap, rope_mode=mode))
    attn = np.stack([orc.sdpa_decode(qr[:, r].copy(), kw, vw, H, Hkv, D, cap, prefix + r + 1).reshape(dm) for r in range(m)])
    want = orc.matmul_gemv(attn, wo, None, hidden, 0, 32, 1.0, 1.0)
    f.start_capture()
    enqueue()
    graph = f.end_capture()
    try:
        for replay in range(3):
            for d in (dqr, dattn, dres):  # eager work between the replays: the outputs are cleared
                d.upload(np.zeros(d.shape, np.float16))
            graph.launch()
            f.synchronize()
            assert _ulp_close(dqr.download(), qr, ulps=4, slack=4e-3), replay
            assert max_abs(dkc.download()[:, :prefix + m], kw[:, :prefix + m]) <= 4e-3, replay  # (rotated projections: within the FusedQkv bar)
            assert np.array_equal(bits(dkc.download()[:, :prefix]), bits(kc[:, :prefix])), replay   # the prefix is untouched
            assert max_abs(dattn.download(), attn) <= 2e-3, replay
            assert max_abs(dres.download(), want) <= 2e-2, replay
    finally:
        graph.destroy()
    for b in dev_w + [dwo, dh, dg, dqr, dkc, dvc, dcos, dsin, dattn, dres]:
        b.free()
