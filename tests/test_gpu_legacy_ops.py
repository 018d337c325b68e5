"""GPU parity of the un-fused chain's ops (Rope, KvCacheWrite, KvCacheWriteRepeatKvHeads, KvCacheRead, KvRearrange,
RepeatKvHeads) and of SdpaReference: index maps and the NeoX rotation bit-exact against the oracle's restatements,
which the CPU tests pin by the reference tests' own CPU helpers (tests/rope.rs:31-63, tests/kv_cache.rs:14-46,
tests/kv_rearrange.rs:33-68, tests/repeat_kv_heads.rs:32-61, tests/kv_cache_write_repeat_kv_heads.rs:57-70); shapes are
those of the reference tests plus ragged ones."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
import refmath as rm
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,dim,seq_len,offset", [(8, 64, 8, 0), (6, 128, 3, 5), (14 * 7, 64, 7, 100), (1, 2, 1, 0)])
def test_rope_op(rows, dim, seq_len, offset):
    announce("rope op", rows, dim, seq_len, offset)
    f = ctx()
    rng = np.random.default_rng(rows + dim)
    x = h16(rng.normal(size=(rows, dim)))
    cos, sin = fa.rope_tables(1e4, dim, offset + seq_len)
    dx, dy, dc, ds = f.array(x), f.zeros((rows, dim)), f.array(cos), f.array(sin)
    f.legacy_op("fa_rope", (dx.arg(), dy.arg(), dc.arg(), ds.arg()), (dim, seq_len, offset, rows * dim))
    f.synchronize()
    assert np.array_equal(bits(dy.download()), bits(orc.rope_neox(x, cos, sin, dim, seq_len, offset)))
    with pytest.raises(fa.FoundryError) as e:  # tables too short for the positions
        f.legacy_op("fa_rope", (dx.arg(), dy.arg(), dc.arg(), ds.arg()), (dim, seq_len, offset + 1, rows * dim))
    assert e.value.variant == "InvalidShape"
    for b in (dx, dy, dc, ds):
        b.free()


@pytest.mark.parametrize("Hkv,H,D,S,pos,cap", [(2, 14, 64, 1, 1024, 1152), (8, 24, 128, 5, 3, 16), (4, 4, 32, 7, 0, 7)])
def test_cache_write_read_and_repeat(Hkv, H, D, S, pos, cap):
    announce("cache write/read/repeat ops", Hkv, H, D, S, pos, cap)
    f = ctx()
    rng = np.random.default_rng(Hkv * H + S)
    x = h16(rng.normal(size=(Hkv, S, D)))
    base = h16(rng.normal(size=(Hkv, cap, D)))
    dx, dc = f.array(x), f.array(base)
    f.legacy_op("fa_kv_cache_write", (dx.arg(), dc.arg()), (Hkv, D, S, pos, cap, Hkv * S * D, 0))
    want = base.copy()
    orc.kv_cache_write(want, x, Hkv, D, S, pos, cap)
    f.synchronize()
    assert np.array_equal(bits(dc.download()), bits(want))
    n = pos + S
    dout = f.zeros((Hkv, n, D))
    f.legacy_op("fa_kv_cache_read", (dc.arg(), dout.arg()), (Hkv, D, n, cap, Hkv * n * D))
    f.synchronize()
    assert np.array_equal(bits(dout.download()), bits(orc.kv_cache_read(want, Hkv, D, n, cap)))
    # expanded cache
    big = h16(rng.normal(size=(H, cap, D)))
    db = f.array(big)
    f.legacy_op("fa_kv_cache_write_repeat_kv_heads", (dx.arg(), db.arg()), (Hkv, H, H // Hkv, D, S, pos, cap, Hkv * S * D, 0))
    want_big = big.copy()
    orc.kv_cache_write_repeat(want_big, x, Hkv, H, D, S, pos, cap)
    f.synchronize()
    assert np.array_equal(bits(db.download()), bits(want_big))
    # RepeatKvHeads over the contiguous cache
    drep = f.zeros((H, n, D))
    f.legacy_op("fa_repeat_kv_heads", (dc.arg(), drep.arg()), (H // Hkv, 1, Hkv, H, n, D, cap, H * n * D))
    f.synchronize()
    assert np.array_equal(bits(drep.download()), bits(orc.repeat_kv_heads(want, Hkv, H, n, D, cap)))
    with pytest.raises(fa.FoundryError) as e:  # a write past the capacity
        f.legacy_op("fa_kv_cache_write", (dx.arg(), dc.arg()), (Hkv, D, S, cap - S + 1, cap, Hkv * S * D, 0))
    assert e.value.variant == "InvalidOperation"
    with pytest.raises(fa.FoundryError) as e:  # total_elements that is not the product
        f.legacy_op("fa_kv_cache_read", (dc.arg(), dout.arg()), (Hkv, D, n, cap, Hkv * n * D - 1))
    assert e.value.variant == "InvalidShape"
    for b in (dx, dc, dout, db, drep):
        b.free()


@pytest.mark.parametrize("H,Hkv,D,seq,batch", [(14, 2, 64, 5, 1), (24, 8, 128, 3, 2), (4, 4, 32, 1, 1)])
def test_kv_rearrange_op(H, Hkv, D, seq, batch):
    announce("kv_rearrange op", H, Hkv, D, seq, batch)
    f = ctx()
    rng = np.random.default_rng(H + seq)
    x = h16(rng.normal(size=(batch * seq, Hkv * D)))
    dx, dy = f.array(x), f.zeros((batch * H, seq, D))
    f.legacy_op("fa_kv_rearrange", (dx.arg(), dy.arg()), (Hkv * D, Hkv * D, D, H, Hkv, D, seq, batch * H * seq * D))
    f.synchronize()
    assert np.array_equal(bits(dy.download()), bits(orc.kv_rearrange(x, H, Hkv, D, seq, batch)))
    for b in (dx, dy):
        b.free()


def test_sdpa_reference_op_runs_on_the_flash_kernels():
    """SdpaReference binds and gives the flash result: decode and a non-causal prefill (a case the reference routes to its
    materialized path), both against float64."""
    announce("SdpaReference op")
    f = ctx()
    rng = np.random.default_rng(9)
    H, Hkv, D, cap, N, M = 8, 2, 64, 256, 200, 17
    k, v = h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    q1, qm = h16(rng.normal(size=(H, D))), h16(rng.normal(size=(H, M, D)))
    dk, dv, dq1, dqm = f.array(k), f.array(v), f.array(q1), f.array(qm)
    o1, om = f.zeros((1, H * D)), f.zeros((M, H * D))
    f.sdpa_reference(dq1.arg((1, H * D)), dk.arg(), dv.arg(), o1.arg(), True, N - 1, H, D, N, 1)
    f.sdpa_reference(dqm.arg(), dk.arg(), dv.arg(), om.arg(), False, 0, H, D, N, M)
    f.synchronize()
    assert max_abs(o1.download().reshape(H, D), rm.gqa_decode_f64(q1, k, v, H, Hkv, D, N)) <= 2e-3
    want = rm.gqa_prefill_f64(qm, k, v, H, Hkv, D, N, 0, causal=False)
    assert max_abs(om.download().reshape(M, H, D).transpose(1, 0, 2), want) <= 2e-3
    with pytest.raises(fa.FoundryError) as e:
        f.sdpa_reference(dq1.arg((1, H * D)), dk.arg(), dv.arg(), o1.arg(), True, N - 1, H, D, N, 1, kv_head_major=False)
    assert e.value.variant == "OperationNotSupported"
    for b in (dk, dv, dq1, dqm, o1, om):
        b.free()
