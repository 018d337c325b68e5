"""GPU parity: KV-cache prefix copies (snapshot, restore, growth) and paged block copies against the oracle's
byte copies. Bit-exact: these are index maps."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16

pytestmark = pytest.mark.gpu


def _rand(rng, shape, dtype):
    dtype = np.dtype(dtype)
    if dtype.kind == "f":
        return rng.normal(size=shape).astype(dtype)
    return rng.integers(-100, 100, size=shape).astype(dtype)


@pytest.mark.parametrize("heads,cap_s,cap_d,D,dtype,n", [
    (8, 2048, 4096, 128, np.float16, 2048),   # growth of a Llama-3.2-3B layer cache, full prefix
    (8, 2048, 4096, 128, np.float16, 1337),
    (2, 1152, 1152, 64, np.float16, 1025),    # same capacity (restore into a live cache)
    (2, 777, 1152, 64, np.float16, 777),      # snapshot buffer -> live cache
    (2, 1152, 777, 64, np.float16, 777),      # live cache -> snapshot buffer
    (4, 256, 512, 128, np.int8, 200),         # int8 K of the quantised variant
    (4, 16, 32, 128, np.float32, 5),
    (3, 40, 48, 20, np.float16, 7),           # 40-byte rows: head pitches not multiples of 16 -> byte kernel
    (1, 128, 128, 64, np.float16, 1),
    (8, 128, 256, 128, np.float16, 0),        # empty prefix: nothing moves
])
def test_kv_prefix_copy_equals_oracle(heads, cap_s, cap_d, D, dtype, n):
    announce("kv prefix copy", heads, cap_s, cap_d, D, np.dtype(dtype).name, n)
    f = ctx()
    rng = np.random.default_rng(heads * 1000 + n)
    src = _rand(rng, (heads, cap_s, D), dtype)
    dst = _rand(rng, (heads, cap_d, D), dtype)
    want = dst.copy()
    assert orc.kv_prefix_copy(src, want, n) == 0
    ds, dd = f.array(src), f.array(dst)
    f.kv_prefix_copy(ds.arg(), dd.arg(), n)
    got = dd.download()
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    assert np.array_equal(ds.download().view(np.uint8), src.view(np.uint8))  # source untouched
    ds.free(), dd.free()


def test_kv_prefix_copy_with_byte_offsets_takes_the_unaligned_path():
    """TensorArg.offset shifts the views by 2 bytes: no 16-byte alignment, same bytes."""
    announce("kv prefix copy, offsets")
    f = ctx()
    rng = np.random.default_rng(5)
    heads, cap_s, cap_d, D, n = 2, 64, 96, 64, 50
    src_flat = h16(rng.normal(size=heads * cap_s * D + 8))
    dst_flat = h16(rng.normal(size=heads * cap_d * D + 8))
    src = src_flat[1:1 + heads * cap_s * D].reshape(heads, cap_s, D).copy()
    want_view = dst_flat[3:3 + heads * cap_d * D].reshape(heads, cap_d, D).copy()
    orc.kv_prefix_copy(src, want_view, n)
    want = dst_flat.copy()
    want[3:3 + heads * cap_d * D] = want_view.reshape(-1)
    ds, dd = f.array(src_flat), f.array(dst_flat)
    f.kv_prefix_copy(ds.arg((heads, cap_s, D), offset=2), dd.arg((heads, cap_d, D), offset=6), n)
    assert np.array_equal(bits(dd.download()), bits(want))  # including the words before and after the view
    ds.free(), dd.free()


def test_snapshot_clobber_restore_round_trip_and_growth_of_all_layers():
    """capture -> overwrite the live caches -> restore gives the captured prefix back and leaves rows past it as they
    were; growth moves the prefix of every layer's K and V into larger caches in one batched call."""
    announce("kv snapshot / restore / growth")
    f = ctx()
    rng = np.random.default_rng(11)
    L, Hkv, D, cap, pos = 3, 8, 128, 256, 201
    live = [h16(rng.normal(size=(Hkv, cap, D))) for _ in range(2 * L)]
    d_live = [f.array(a) for a in live]
    d_snap = [f.zeros((Hkv, pos, D)) for _ in range(2 * L)]
    f.kv_prefix_copy_batch([b.arg() for b in d_live], [b.arg() for b in d_snap], pos)
    for a, b in zip(live, d_snap):
        assert np.array_equal(bits(b.download()), bits(a[:, :pos]))
    clobber = [h16(rng.normal(size=(Hkv, cap, D))) for _ in range(2 * L)]
    for b, c in zip(d_live, clobber):
        b.upload(c)
    f.kv_prefix_copy_batch([b.arg() for b in d_snap], [b.arg() for b in d_live], pos)
    for a, c, b in zip(live, clobber, d_live):
        got = b.download()
        assert np.array_equal(bits(got[:, :pos]), bits(a[:, :pos]))
        assert np.array_equal(bits(got[:, pos:]), bits(c[:, pos:]))
    # growth: new capacity from the reference's policy, prefix = current_pos
    new_cap = fa.grown_capacity(cap, pos + 100, 4096)
    assert new_cap == orc.grown_capacity(cap, pos + 100, 4096) == 512
    d_new = [f.zeros((Hkv, new_cap, D)) for _ in range(2 * L)]
    f.kv_prefix_copy_batch([b.arg() for b in d_live], [b.arg() for b in d_new], pos)
    for a, b in zip(live, d_new):
        got = b.download()
        want = np.zeros((Hkv, new_cap, D), np.float16)
        orc.kv_prefix_copy(a, want, pos)
        assert np.array_equal(bits(got), bits(want))
    for b in d_live + d_snap + d_new:
        b.free()


def test_kv_prefix_copy_batch_of_mixed_geometries_and_more_tensors_than_one_launch_holds():
    announce("kv prefix copy, batch")
    f = ctx()
    rng = np.random.default_rng(3)
    shapes = [(2, 32, 64)] * 70 + [(4, 48, 128)] * 3 + [(2, 32, 64)] * 2
    n = 17
    srcs = [h16(rng.normal(size=s)) for s in shapes]
    dsts = [h16(rng.normal(size=(s[0], s[1] + 16, s[2]))) for s in shapes]
    ds, dd = [f.array(a) for a in srcs], [f.array(a) for a in dsts]
    f.kv_prefix_copy_batch([b.arg() for b in ds], [b.arg() for b in dd], n)
    for a, d0, b in zip(srcs, dsts, dd):
        want = d0.copy()
        orc.kv_prefix_copy(a, want, n)
        assert np.array_equal(bits(b.download()), bits(want))
    for b in ds + dd:
        b.free()


def test_kv_prefix_copy_errors_follow_the_reference():
    announce("kv prefix copy errors")
    f = ctx()
    a, b = f.zeros((2, 64, 64)), f.zeros((2, 128, 64))
    with pytest.raises(fa.FoundryError) as e:  # prefix_len exceeds capacity (executor.rs:1115-1120)
        f.kv_prefix_copy(a.arg(), b.arg(), 65)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:  # rank (executor.rs:1106-1111)
        f.kv_prefix_copy(a.arg((2 * 64, 64)), b.arg(), 1)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:  # strides (executor.rs:1123-1131)
        f.kv_prefix_copy(a.arg((2, 32, 64), (64 * 64, 128, 1)), b.arg(), 1)
    assert e.value.variant == "InvalidShape"
    c = f.zeros((2, 64, 64), np.float32)
    with pytest.raises(fa.FoundryError) as e:  # dtype mismatch (executor.rs:1281-1286)
        f.kv_prefix_copy(a.arg(), c.arg(), 1)
    assert e.value.variant == "InvalidShape"
    d = f.zeros((4, 64, 64))
    with pytest.raises(fa.FoundryError) as e:  # heads mismatch (executor.rs:1287-1292)
        f.kv_prefix_copy(a.arg(), d.arg(), 1)
    assert e.value.variant == "InvalidShape"
    t = a.arg()
    t.buffer = None
    with pytest.raises(fa.FoundryError) as e:
        f.kv_prefix_copy(t, b.arg(), 1)
    assert e.value.variant == "InputNotFound"
    f.synchronize()
    for x in (a, b, c, d):
        x.free()


@pytest.mark.parametrize("Hkv,D,bs", [(2, 128, 16), (8, 128, 32), (2, 64, 48)])
def test_paged_copy_blocks_equals_oracle_and_forks_a_sequence(Hkv, D, bs):
    """A fork shares its parent's full blocks by block-table entry and owns a copy of the partly filled tail block;
    gathering the fork gives the parent's rows. Out-of-range ids and src == dst are skipped."""
    announce("paged copy blocks", Hkv, D, bs)
    f = ctx()
    rng = np.random.default_rng(Hkv + bs)
    n_blocks, n_tok = 12, 2 * bs + 5
    k_pool = h16(rng.normal(size=(n_blocks, Hkv, bs, D)))
    v_pool = h16(rng.normal(size=(n_blocks, Hkv, bs, D)))
    parent = np.array([7, 2, 9], np.int32)       # 3 blocks hold n_tok rows
    fork = np.array([7, 2, 4], np.int32)         # shares 7 and 2, owns 4
    src = np.array([9, 3, -1, 5, 12, 1], np.int32)
    dst = np.array([4, 3, 6, 99, 0, 11], np.int32)  # 9->4 and 1->11 are the only valid pairs
    wk, wv = k_pool.copy(), v_pool.copy()
    orc.paged_copy_blocks(wk, Hkv, bs, D, src, dst)
    orc.paged_copy_blocks(wv, Hkv, bs, D, src, dst)
    bt = np.stack([parent, fork])
    dk, dv, dbt, dl = f.array(k_pool), f.array(v_pool), f.array(bt), f.array(np.array([n_tok, n_tok], np.uint32))
    desc = fa.paged_kv(dk, dv, dbt, dl, n_blocks, Hkv, bs, D, 2, 3)
    dsrc, ddst = f.array(src), f.array(dst)
    f.paged_copy_blocks(desc, dsrc, ddst, len(src))
    assert np.array_equal(bits(dk.download()), bits(wk))
    assert np.array_equal(bits(dv.download()), bits(wv))
    assert np.array_equal(bits(wk[4]), bits(k_pool[9])) and np.array_equal(bits(wk[0]), bits(k_pool[0]))
    ko = [f.zeros((Hkv, n_tok, D)) for _ in range(2)]
    vo = [f.zeros((Hkv, n_tok, D)) for _ in range(2)]
    for s in range(2):
        f.paged_gather(desc, s, n_tok, ko[s], vo[s], n_tok)
    assert np.array_equal(bits(ko[0].download()), bits(ko[1].download()))
    assert np.array_equal(bits(vo[0].download()), bits(vo[1].download()))
    assert np.array_equal(bits(ko[1].download()), bits(orc.paged_gather(k_pool, parent, Hkv, bs, D, n_tok)))
    for b in [dk, dv, dbt, dl, dsrc, ddst] + ko + vo:
        b.free()


def test_forked_sequence_shares_prefix_blocks_and_decodes_independently():
    """Prefix sharing on the paged cache: a fork points at its parent's full blocks, owns a copy of the partly filled
    tail block (fa_paged_copy_blocks), and then both sequences append and attend different tokens in one batched step.
    Each must equal the oracle over its own contiguous history; the parent's tail block must not see the fork's token."""
    announce("paged fork + decode")
    f = ctx()
    rng = np.random.default_rng(404)
    H, Hkv, D, bs, n = 8, 2, 128, 16, 16 * 5 + 9   # 5 full blocks + 9 rows in the tail block
    nblk, mb = 16, 7
    k_hist = h16(rng.normal(size=(Hkv, n, D)))
    v_hist = h16(rng.normal(size=(Hkv, n, D)))
    parent = np.array([3, 11, 0, 7, 14, 5, 9], np.int32)          # block 5 is the tail, 9 is room to grow
    fork = np.array([3, 11, 0, 7, 14, 2, 13], np.int32)           # shares five blocks, owns 2 (copy of 5) and 13
    k_pool = h16(rng.normal(size=(nblk, Hkv, bs, D)))
    v_pool = h16(rng.normal(size=(nblk, Hkv, bs, D)))
    orc.paged_scatter(k_pool, parent, Hkv, bs, D, 0, n, k_hist)
    orc.paged_scatter(v_pool, parent, Hkv, bs, D, 0, n, v_hist)
    bt = np.stack([parent, fork])
    dk, dv, dbt, dl = f.array(k_pool), f.array(v_pool), f.array(bt), f.array(np.array([n, n], np.uint32))
    desc = fa.paged_kv(dk, dv, dbt, dl, nblk, Hkv, bs, D, 2, mb)
    dsrc, ddst = f.array(np.array([5], np.int32)), f.array(np.array([2], np.int32))
    f.paged_copy_blocks(desc, dsrc, ddst, 1)
    cos, sin = fa.rope_tables(1e6, D, 256)
    q, kn, vn = (h16(rng.normal(size=(2, m * D))) for m in (H, Hkv, Hkv))   # different new tokens for the two sequences
    dq, dkn, dvn, dcos, dsin, dout = f.array(q), f.array(kn), f.array(vn), f.array(cos), f.array(sin), f.zeros((2, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 2, 0, 0, fa.ROPE_NEOX)
    f.decode_step_fused_paged(dq.arg(), dkn.arg(), dvn.arg(), None, desc, dcos.arg(), dsin.arg(), dout.arg(), p, mb * bs)
    f.synchronize()
    got = dout.download().reshape(2, H, D)
    gk, gv = dk.download(), dv.download()
    for s, table in enumerate((parent, fork)):
        kc, vc = np.zeros((Hkv, n + 1, D), np.float16), np.zeros((Hkv, n + 1, D), np.float16)
        kc[:, :n], vc[:, :n] = k_hist, v_hist
        qr = orc.kv_prep_fused(q[s:s + 1], kn[s:s + 1], vn[s:s + 1], kc, vc, cos, sin, orc.make_params(H, Hkv, D, 1, n, n + 1, rope_mode=0))
        want = orc.sdpa_decode(qr[:, 0].copy(), kc, vc, H, Hkv, D, n + 1, n + 1).reshape(H, D)
        assert float(np.max(np.abs(got[s].astype(np.float64) - want.astype(np.float64)))) <= 2e-3, s
        assert np.array_equal(bits(orc.paged_gather(gk, table, Hkv, bs, D, n + 1)), bits(kc)), s
        assert np.array_equal(bits(orc.paged_gather(gv, table, Hkv, bs, D, n + 1)), bits(vc)), s
    assert not np.array_equal(bits(gk[5][:, 9]), bits(gk[2][:, 9]))   # the two tails diverged at the new row
    for b in (dk, dv, dbt, dl, dsrc, ddst, dq, dkn, dvn, dcos, dsin, dout):
        b.free()
