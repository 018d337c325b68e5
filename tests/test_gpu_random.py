"""GPU parity on seeded random configurations: head counts, group sizes, lengths, capacities, partition sizes, merge
forms, RoPE modes and chunk positions drawn at random, each checked against the oracle. The fixed-shape tests pin the
cases the reference tests; these sweep the combinations in between."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-3
HEADS = [(8, 8), (8, 2), (14, 2), (24, 8), (32, 4), (16, 1), (12, 4), (6, 3), (16, 16), (28, 4), (40, 8), (9, 3)]


@pytest.mark.parametrize("seed", range(24))
def test_random_fused_decode_step(seed):
    """RoPE + append + decode in one launch at a random shape, position, partition size and merge form."""
    rng = np.random.default_rng(1000 + seed)
    H, Hkv = HEADS[rng.integers(len(HEADS))]
    D = int(rng.choice([64, 128]))
    pos = int(rng.integers(0, 3000))
    cap = (pos + 1 + int(rng.integers(0, 300)) + 15) // 16 * 16
    kps = int(rng.choice([0, 0, 64, 128, 256, 1024]))
    merge = int(rng.integers(0, 3))
    mode = int(rng.choice([fa.ROPE_NEOX, fa.ROPE_NORMAL]))
    step = int(rng.choice([0, 0, 4]))
    layer = int(rng.integers(0, 8))
    announce("random fused step", seed, H, Hkv, D, pos, cap, kps, merge, mode, step, layer)
    f = ctx()
    cos, sin = fa.rope_tables(float(rng.choice([1e4, 5e5, 1e6])), D, cap)
    kc = h16(rng.normal(size=(Hkv, cap, D)))
    vc = h16(rng.normal(size=(Hkv, cap, D)))
    kc[:, pos:], vc[:, pos:] = np.float16(np.nan), np.float16(np.nan)  # nothing past the position may contribute
    q, k, v = (h16(rng.normal(size=(1, n * D))) for n in (H, Hkv, Hkv))
    kw, vw = kc.copy(), vc.copy()
    qr = orc.kv_prep_fused(q, k, v, kw, vw, cos, sin,
                           orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=0 if mode == fa.ROPE_NEOX else 1, layer_idx=layer,
                                           no_rope_layer_step=step))
    want = orc.sdpa_decode(qr[:, 0].copy(), kw, vw, H, Hkv, D, cap, pos + 1).reshape(H, D)
    dq, dk, dv, dkc, dvc = f.array(q), f.array(k), f.array(v), f.array(kc), f.array(vc)
    dcos, dsin, dqr, dout = f.array(cos), f.array(sin), f.zeros((H, 1, D)), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, mode, layer_idx=layer, no_rope_layer_step=step)
    try:
        f.set_decode_variant(kps, merge)
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p)
        f.synchronize()
    finally:
        f.set_decode_variant()
    got = dout.download().reshape(H, D)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    gk, gv = dkc.download(), dvc.download()
    assert np.array_equal(bits(gk[:, :pos + 1]), bits(kw[:, :pos + 1])) and np.array_equal(bits(gv[:, :pos + 1]), bits(vw[:, :pos + 1]))
    assert np.array_equal(bits(dqr.download()), bits(qr))
    for b in (dq, dk, dv, dkc, dvc, dcos, dsin, dqr, dout):
        b.free()


@pytest.mark.parametrize("seed", range(16))
def test_random_prefill_chunk_with_prefix(seed, prefill_variant):
    """KvPrepFused + FlashAttention for a chunk of m tokens after a random prefix (the chunked prefill's call shape)."""
    rng = np.random.default_rng(2000 + seed)
    H, Hkv = HEADS[rng.integers(len(HEADS))]
    D = int(rng.choice([64, 128]))
    m = int(rng.choice([2, 7, 24, 32, 33, 64, 130, 257]))
    prefix = int(rng.choice([0, 0, 1, 31, 100, 513, 1500]))
    cap = (prefix + m + int(rng.integers(0, 100)) + 127) // 128 * 128
    mode = int(rng.choice([fa.ROPE_NEOX, fa.ROPE_NORMAL]))
    announce("random prefill chunk", seed, H, Hkv, D, m, prefix, cap, mode)
    f = ctx()
    cos, sin = fa.rope_tables(1e4, D, cap)
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    kc[:, :prefix] = h16(rng.normal(size=(Hkv, prefix, D)))
    vc[:, :prefix] = h16(rng.normal(size=(Hkv, prefix, D)))
    q, k, v = (h16(rng.normal(size=(m, n * D))) for n in (H, Hkv, Hkv))
    kw, vw = kc.copy(), vc.copy()
    qr = orc.kv_prep_fused(q, k, v, kw, vw, cos, sin, orc.make_params(H, Hkv, D, m, prefix, cap, rope_mode=0 if mode == fa.ROPE_NEOX else 1))
    want = np.stack([orc.sdpa_decode(qr[:, r].copy(), kw, vw, H, Hkv, D, cap, prefix + r + 1).reshape(H * D) for r in range(m)])
    dq, dk, dv, dkc, dvc = f.array(q), f.array(k), f.array(v), f.array(kc), f.array(vc)
    dcos, dsin, dqr, dout = f.array(cos), f.array(sin), f.zeros((H, m, D)), f.zeros((m, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, prefix, cap, mode)
    f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), p)
    f.flash_attention(dqr.arg(), dkc.arg(), dvc.arg(), dout.arg(), True, prefix, H, D, prefix + m, m)
    f.synchronize()
    got = dout.download()
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    assert np.array_equal(bits(dkc.download()), bits(kw)) and np.array_equal(bits(dvc.download()), bits(vw))
    for b in (dq, dk, dv, dkc, dvc, dcos, dsin, dqr, dout):
        b.free()


@pytest.mark.parametrize("seed", range(12))
def test_random_paged_batch_step(seed):
    """A ragged batch on a paged cache with a random block size and a permuted block table: one fused step."""
    rng = np.random.default_rng(3000 + seed)
    H, Hkv = HEADS[rng.integers(len(HEADS))]
    D = int(rng.choice([64, 128]))
    bs = int(rng.choice([16, 32, 48, 64, 128]))
    B = int(rng.integers(1, 9))
    lens = [int(x) for x in rng.integers(0, 1200, size=B)]
    announce("random paged step", seed, H, Hkv, D, bs, lens)
    f = ctx()
    need = [(n + 1 + bs - 1) // bs for n in lens]
    mb, nblk = max(need), sum(need) + 2
    perm = rng.permutation(nblk).astype(np.int32)
    bt = np.zeros((B, mb), np.int32)
    o = 0
    for s, n in enumerate(need):
        bt[s, :n] = perm[o:o + n]
        o += n
    k_pool = h16(rng.normal(size=(nblk, Hkv, bs, D)))
    v_pool = h16(rng.normal(size=(nblk, Hkv, bs, D)))
    cos, sin = fa.rope_tables(1e6, D, max(lens) + 2)
    q, kn, vn = (h16(rng.normal(size=(B, n * D))) for n in (H, Hkv, Hkv))
    wk, wv = k_pool.copy(), v_pool.copy()
    want = np.zeros((B, H * D), np.float16)
    for s, n in enumerate(lens):
        kc = orc.paged_gather(wk, bt[s], Hkv, bs, D, n, n + 1)
        vc = orc.paged_gather(wv, bt[s], Hkv, bs, D, n, n + 1)
        qr = orc.kv_prep_fused(q[s:s + 1], kn[s:s + 1], vn[s:s + 1], kc, vc, cos, sin, orc.make_params(H, Hkv, D, 1, n, n + 1, rope_mode=0))
        want[s] = orc.sdpa_decode(qr[:, 0].copy(), kc, vc, H, Hkv, D, n + 1, n + 1).reshape(-1)
        orc.paged_scatter(wk, bt[s], Hkv, bs, D, n, n + 1, kc)
        orc.paged_scatter(wv, bt[s], Hkv, bs, D, n, n + 1, vc)
    dk, dv, dbt, dl = f.array(k_pool), f.array(v_pool), f.array(bt), f.array(np.array(lens, np.uint32))
    desc = fa.paged_kv(dk, dv, dbt, dl, nblk, Hkv, bs, D, B, mb)
    dq, dkn, dvn, dcos, dsin, dout = f.array(q), f.array(kn), f.array(vn), f.array(cos), f.array(sin), f.zeros((B, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, B, 0, 0, fa.ROPE_NEOX)
    f.decode_step_fused_paged(dq.arg(), dkn.arg(), dvn.arg(), None, desc, dcos.arg(), dsin.arg(), dout.arg(), p, mb * bs)
    f.synchronize()
    got = dout.download()
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    assert np.array_equal(bits(dk.download()), bits(wk)) and np.array_equal(bits(dv.download()), bits(wv))
    for b in (dk, dv, dbt, dl, dq, dkn, dvn, dcos, dsin, dout):
        b.free()
