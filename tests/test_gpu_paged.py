"""GPU parity: paged KV cache (block table, per-sequence lengths). The reference has no paged cache; the
contract is gather(paged) == the contiguous cache the reference would hold, bit for bit, and attention over
the paged cache == attention over that contiguous cache."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-3


class Paged:
    """Host mirror of a paged pool with a seeded random permutation of physical blocks."""

    def __init__(self, f, rng, lens, Hkv, D, bs, extra_tokens=1, slack_blocks=3):
        self.f, self.Hkv, self.D, self.bs = f, Hkv, D, bs
        self.lens = np.asarray(lens, np.uint32)
        self.n_seqs = len(lens)
        need = [(int(n) + extra_tokens + bs - 1) // bs for n in lens]
        self.mb = max(need)
        self.n_blocks = sum(need) + slack_blocks
        perm = rng.permutation(self.n_blocks).astype(np.int32)
        self.bt = np.full((self.n_seqs, self.mb), -1, np.int32)
        o = 0
        for s, n in enumerate(need):
            self.bt[s, :n] = perm[o:o + n]
            o += n
        self.bt_dev_host = np.where(self.bt < 0, 0, self.bt).astype(np.int32)
        self.k_pool = np.zeros((self.n_blocks, Hkv, bs, D), np.float16)
        self.v_pool = np.zeros((self.n_blocks, Hkv, bs, D), np.float16)

    def fill_from(self, ks, vs):
        for s in range(self.n_seqs):
            orc.paged_scatter(self.k_pool, self.bt[s], self.Hkv, self.bs, self.D, 0, int(self.lens[s]), ks[s])
            orc.paged_scatter(self.v_pool, self.bt[s], self.Hkv, self.bs, self.D, 0, int(self.lens[s]), vs[s])

    def upload(self):
        f = self.f
        self.dk, self.dv = f.array(self.k_pool), f.array(self.v_pool)
        self.dbt, self.dlens = f.array(self.bt_dev_host), f.array(self.lens)
        self.desc = fa.paged_kv(self.dk, self.dv, self.dbt, self.dlens, self.n_blocks, self.Hkv, self.bs, self.D,
                                self.n_seqs, self.mb)
        return self

    def free(self):
        for b in (self.dk, self.dv, self.dbt, self.dlens):
            b.free()


@pytest.mark.parametrize("H,Hkv,D,bs,lens", [
    (16, 2, 128, 16, [512, 777, 16, 1, 4095, 1000, 33, 2049]),   # Qwen2.5-3B shape (benchmark configuration 3), ragged
    (14, 2, 64, 16, [100, 5, 64]),
    (24, 8, 128, 32, [300, 31]),
    (8, 8, 64, 64, [129]),
    (24, 8, 128, 16, [40000]),  # one long sequence: whole partitions, one per compute unit, merged inside the launch
])
def test_paged_batched_decode_step(H, Hkv, D, bs, lens):
    """One batched decode step: append one token per sequence at seq_lens[b], then ragged flash decode."""
    announce("paged decode step", H, Hkv, D, bs, lens)
    f = ctx()
    rng = np.random.default_rng(len(lens) * 100 + D)
    B = len(lens)
    ks = [h16(rng.normal(size=(Hkv, n + 1, D))) for n in lens]
    vs = [h16(rng.normal(size=(Hkv, n + 1, D))) for n in lens]
    pg = Paged(f, rng, lens, Hkv, D, bs)
    pg.fill_from(ks, vs)
    pg.upload()
    q = h16(rng.normal(size=(B, H * D)))
    kn = h16(rng.normal(size=(B, Hkv * D)))
    vn = h16(rng.normal(size=(B, Hkv * D)))
    maxpos = int(max(lens)) + 1
    cos, sin = fa.rope_tables(1e6, D, maxpos)
    dq, dkn, dvn, dqr, dout = f.array(q), f.array(kn), f.array(vn), f.zeros((B, H, D)), f.zeros((B, H * D))
    dcos, dsin = f.array(cos), f.array(sin)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, B, 0, 0, fa.ROPE_NEOX)
    f.kv_prep_decode_paged(dq.arg(), dkn.arg(), dvn.arg(), dqr.arg(), pg.desc, dcos.arg(), dsin.arg(), p)
    f.flash_decode_paged(dqr.arg(), pg.desc, dout.arg(), H, 1, maxpos)
    f.synchronize()
    got_qr, got_out = dqr.download(), dout.download().reshape(B, H, D)
    got_kp, got_vp = pg.dk.download(), pg.dv.download()
    gk, gv = f.zeros((Hkv, maxpos, D)), f.zeros((Hkv, maxpos, D))
    for b, n in enumerate(lens):
        # oracle: the reference's contiguous cache after the same append
        kc = np.zeros((Hkv, n + 1, D), np.float16)
        vc = np.zeros((Hkv, n + 1, D), np.float16)
        kc[:, :n], vc[:, :n] = ks[b][:, :n], vs[b][:, :n]
        want_qr = orc.kv_prep_fused(q[b:b + 1], kn[b:b + 1], vn[b:b + 1], kc, vc, cos, sin,
                                    orc.make_params(H, Hkv, D, 1, n, n + 1, rope_mode=0))
        assert np.array_equal(bits(got_qr[b]), bits(want_qr[:, 0])), b
        # host-side gather of the downloaded pools and the device gather kernel agree with it bit for bit
        assert np.array_equal(bits(orc.paged_gather(got_kp, pg.bt[b], Hkv, bs, D, n + 1)), bits(kc)), b
        assert np.array_equal(bits(orc.paged_gather(got_vp, pg.bt[b], Hkv, bs, D, n + 1)), bits(vc)), b
        f.paged_gather(pg.desc, b, n + 1, gk, gv, maxpos)
        f.synchronize()
        assert np.array_equal(bits(gk.download()[:, :n + 1]), bits(kc)), b
        assert np.array_equal(bits(gv.download()[:, :n + 1]), bits(vc)), b
        want = orc.sdpa_decode(want_qr[:, 0].copy(), kc, vc, H, Hkv, D, n + 1, n + 1).reshape(H, D)
        assert max_abs(got_out[b], want) <= TOL, b
    # blocks outside every block table were not touched
    used = set(pg.bt[pg.bt >= 0].tolist())
    for blk in range(pg.n_blocks):
        if blk not in used:
            assert not got_kp[blk].any() and not got_vp[blk].any()
    pg.free()
    for b in (dq, dkn, dvn, dqr, dout, dcos, dsin, gk, gv):
        b.free()


@pytest.mark.usefixtures("prefill_variant")
def test_paged_prefill_append_then_decode_equals_contiguous():
    """Multi-token append into an empty paged cache (one sequence of a batch), compared with the contiguous op."""
    announce("paged prefill append")
    f = ctx()
    rng = np.random.default_rng(77)
    H, Hkv, D, bs, T = 24, 8, 128, 16, 150
    pg = Paged(f, rng, [0, 0, 0], Hkv, D, bs, extra_tokens=T + 1).upload()
    q, k, v = (h16(rng.normal(size=(T, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(5e5, D, 256)
    dq, dk, dv, dqr = f.array(q), f.array(k), f.array(v), f.zeros((H, T, D))
    dcos, dsin = f.array(cos), f.array(sin)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, T, 0, 0, fa.ROPE_NORMAL)
    f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), pg.desc, 1, dcos.arg(), dsin.arg(), p)
    f.synchronize()
    kc, vc = np.zeros((Hkv, T, D), np.float16), np.zeros((Hkv, T, D), np.float16)
    want_qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, T, 0, T, rope_mode=1))
    assert np.array_equal(bits(dqr.download()), bits(want_qr))
    assert np.array_equal(bits(orc.paged_gather(pg.dk.download(), pg.bt[1], Hkv, bs, D, T)), bits(kc))
    assert np.array_equal(bits(orc.paged_gather(pg.dv.download(), pg.bt[1], Hkv, bs, D, T)), bits(vc))
    # sequences 0 and 2 own other blocks: still empty
    for s in (0, 2):
        assert not orc.paged_gather(pg.dk.download(), pg.bt[s], Hkv, bs, D, T).any()
    with pytest.raises(fa.FoundryError) as e:  # beyond the block table
        f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), pg.desc, 1, dcos.arg(), dsin.arg(),
                              fa.KvPrepFusedParams.make(H, Hkv, D, T, pg.mb * bs - 3, 0, fa.ROPE_NORMAL))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:
        f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), pg.desc, 3, dcos.arg(), dsin.arg(), p)
    assert e.value.variant == "InvalidShape"
    f.synchronize()
    pg.free()


def test_paged_decode_multi_step_advances_lengths():
    """Three decode steps with device-side length advance between them (fa_u32_add)."""
    announce("paged multi-step")
    f = ctx()
    rng = np.random.default_rng(5)
    H, Hkv, D, bs, steps = 16, 2, 128, 16, 3
    lens = [30, 47, 16]
    B = len(lens)
    ks = [h16(rng.normal(size=(Hkv, n + steps, D))) for n in lens]
    vs = [h16(rng.normal(size=(Hkv, n + steps, D))) for n in lens]
    pg = Paged(f, rng, lens, Hkv, D, bs, extra_tokens=steps)
    pg.fill_from(ks, vs)
    pg.upload()
    cos, sin = fa.rope_tables(1e6, D, 128)
    dcos, dsin = f.array(cos), f.array(sin)
    kc = [np.zeros((Hkv, n + steps, D), np.float16) for n in lens]
    vc = [np.zeros((Hkv, n + steps, D), np.float16) for n in lens]
    for b, n in enumerate(lens):
        kc[b][:, :n], vc[b][:, :n] = ks[b][:, :n], vs[b][:, :n]
    dqr, dout = f.zeros((B, H, D)), f.zeros((B, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, B, 0, 0, fa.ROPE_NEOX)
    for t in range(steps):
        q, kn, vn = (h16(rng.normal(size=(B, n * D))) for n in (H, Hkv, Hkv))
        dq, dkn, dvn = f.array(q), f.array(kn), f.array(vn)
        f.kv_prep_decode_paged(dq.arg(), dkn.arg(), dvn.arg(), dqr.arg(), pg.desc, dcos.arg(), dsin.arg(), p)
        f.flash_decode_paged(dqr.arg(), pg.desc, dout.arg(), H, 1, 64)
        f.u32_add(pg.dlens, B, 1)
        f.synchronize()
        got = dout.download().reshape(B, H, D)
        for b, n in enumerate(lens):
            qr = orc.kv_prep_fused(q[b:b + 1], kn[b:b + 1], vn[b:b + 1], kc[b], vc[b], cos, sin,
                                   orc.make_params(H, Hkv, D, 1, n + t, n + steps, rope_mode=0))
            want = orc.sdpa_decode(qr[:, 0].copy(), kc[b], vc[b], H, Hkv, D, n + steps, n + t + 1).reshape(H, D)
            assert max_abs(got[b], want) <= TOL, (t, b)
    assert np.array_equal(pg.dlens.download(), np.asarray(lens, np.uint32) + steps)
    pg.free()


def test_paged_fused_step_equals_separate_ops():
    """fa_decode_step_fused_paged == fa_kv_prep_decode_paged + fa_flash_decode_paged: q_rot and pools bit-identical,
    outputs equal up to f32 summation order."""
    announce("paged fused step")
    f = ctx()
    rng = np.random.default_rng(17)
    H, Hkv, D, bs = 16, 2, 128, 16
    lens = [512, 15, 16, 1, 1000, 63, 64, 0]
    B = len(lens)
    ks = [h16(rng.normal(size=(Hkv, n + 1, D))) for n in lens]
    vs = [h16(rng.normal(size=(Hkv, n + 1, D))) for n in lens]
    q, kn, vn = (h16(rng.normal(size=(B, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(1e6, D, 1024)
    dcos, dsin = f.array(cos), f.array(sin)
    dq, dkn, dvn = f.array(q), f.array(kn), f.array(vn)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, B, 0, 0, fa.ROPE_NEOX)
    outs = []
    for fused in (False, True):
        pg = Paged(f, np.random.default_rng(3), lens, Hkv, D, bs)
        pg.fill_from(ks, vs)
        pg.upload()
        dqr, dout = f.zeros((B, H, D)), f.zeros((B, H * D))
        if fused:
            f.decode_step_fused_paged(dq.arg(), dkn.arg(), dvn.arg(), dqr.arg(), pg.desc, dcos.arg(), dsin.arg(),
                                      dout.arg(), p, 1024)
        else:
            f.kv_prep_decode_paged(dq.arg(), dkn.arg(), dvn.arg(), dqr.arg(), pg.desc, dcos.arg(), dsin.arg(), p)
            f.flash_decode_paged(dqr.arg(), pg.desc, dout.arg(), H, 1, 1024)
        f.synchronize()
        outs.append((dqr.download(), dout.download(), pg.dk.download(), pg.dv.download()))
        pg.free()
    for i, (a, b) in enumerate(zip(outs[0], outs[1])):
        if i == 1:
            assert max_abs(a, b) <= 2e-3
        else:
            assert np.array_equal(bits(a), bits(b))
    # and against the oracle for two of the sequences
    for b in (0, 7):
        n = lens[b]
        kc, vc = np.zeros((Hkv, n + 1, D), np.float16), np.zeros((Hkv, n + 1, D), np.float16)
        kc[:, :n], vc[:, :n] = ks[b][:, :n], vs[b][:, :n]
        qr = orc.kv_prep_fused(q[b:b + 1], kn[b:b + 1], vn[b:b + 1], kc, vc, cos, sin,
                               orc.make_params(H, Hkv, D, 1, n, n + 1, rope_mode=0))
        want = orc.sdpa_decode(qr[:, 0].copy(), kc, vc, H, Hkv, D, n + 1, n + 1).reshape(H, D)
        assert max_abs(outs[1][1].reshape(B, H, D)[b], want) <= TOL


def test_paged_decode_full_batch_of_32_ragged_sequences():
    """The Qwen2.5-3B-shaped batched paged decode at full size: 32 sequences with lengths drawn from 512..16384,
    16-token blocks behind a random block permutation. Every sequence against the oracle over its gathered cache."""
    announce("paged decode, 32 ragged sequences")
    f = ctx()
    rng = np.random.default_rng(2024)
    H, Hkv, D, bs, B = 16, 2, 128, 16, 32
    lens = [int(x) for x in rng.integers(512, 16385, size=B)]
    ks = [h16(rng.normal(size=(Hkv, n, D))) for n in lens]
    vs = [h16(rng.normal(size=(Hkv, n, D))) for n in lens]
    pg = Paged(f, rng, lens, Hkv, D, bs, extra_tokens=0)
    pg.fill_from(ks, vs)
    pg.upload()
    q = h16(rng.normal(size=(B, H, D)))
    dq, dout = f.array(q), f.zeros((B, H * D))
    f.flash_decode_paged(dq.arg(), pg.desc, dout.arg(), H, 0, max(lens))
    f.synchronize()
    got = dout.download().reshape(B, H, D)
    assert np.all(np.isfinite(got))
    worst = 0.0
    for b, n in enumerate(lens):
        want = orc.sdpa_decode(q[b], ks[b], vs[b], H, Hkv, D, n, n, n_threads=8).reshape(H, D)
        worst = max(worst, max_abs(got[b], want))
    print("32 ragged sequences, %d keys in total: max abs err %.2e" % (sum(lens), worst), flush=True)
    assert worst <= TOL
    pg.free()
    for b in (dq, dout):
        b.free()


@pytest.mark.usefixtures("prefill_variant")
@pytest.mark.parametrize("H,Hkv,D,bs,prefix,M", [
    (6, 2, 128, 16, 333, 100),    # context ends inside a block and inside a key tile
    (14, 2, 64, 48, 70, 37),      # block size not a power of two, head_dim 64
    (8, 8, 128, 32, 0, 129),      # no prefix, one row into a second query tile
    (4, 2, 128, 16, 2000, 32),    # a 32-row chunk after a long prefix: few query tiles, split over the keys
    (24, 8, 128, 16, 1111, 32),   # the same at the Llama-3.2-3B shape: the three heads of a KV group share an item
    (14, 2, 64, 32, 500, 9),      # nine rows, groups of seven heads
])
def test_paged_prefill_chunk_after_prefix(H, Hkv, D, bs, prefix, M):
    """A prefill chunk attending a paged cache that already holds a prefix (sequence 1 of 3, random block
    permutation), against the oracle over the gathered contiguous cache."""
    announce("paged prefill chunk", H, Hkv, D, bs, prefix, M)
    f = ctx()
    rng = np.random.default_rng(prefix * 7 + M)
    N = prefix + M
    lens = [5, N, 40]
    ks = [h16(rng.normal(size=(Hkv, n, D))) for n in lens]
    vs = [h16(rng.normal(size=(Hkv, n, D))) for n in lens]
    pg = Paged(f, rng, lens, Hkv, D, bs, extra_tokens=0)
    pg.fill_from(ks, vs)
    pg.upload()
    q = h16(rng.normal(size=(H, M, D)))
    dq, dout = f.array(q), f.zeros((M, H * D))
    f.flash_prefill_paged(dq.arg(), pg.desc, 1, dout.arg(), True, prefix, H, N, M)
    f.synchronize()
    got = dout.download()
    want = orc.sdpa_prefill(q, ks[1], vs[1], H, Hkv, D, M, N, prefix, N, causal=True, n_threads=8)  # token-major
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    pg.free()
    for b in (dq, dout):
        b.free()
