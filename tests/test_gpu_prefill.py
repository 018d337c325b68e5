"""GPU parity: causal flash prefill on MFMA (fa_flash_attention with m > 1, fa_flash_prefill_paged) against the
CPU oracle. Tolerance: max-abs <= 2e-3 (f32 accumulation; probabilities are rounded to f16 for the PV MFMA)."""
import os

import numpy as np
import pytest

import foundry_attn as fa
import orc
import refmath as rm
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("prefill_variant")]  # every case under both kernels
TOL = 2e-3
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gpu_prefill(q_hm, k, v, H, D, M, N, offset, causal=True, q_layout="head_major", out_layout="token_major"):
    f = ctx()
    if q_layout == "head_major":
        dq = f.array(q_hm)
        qa = dq.arg((H, M, D))
    elif q_layout == "token_meta_head_contents":  # [1, M_cap, d_model] metadata over head-major packed contents
        cap_m = M + 5
        buf = np.zeros((cap_m * H * D,), np.float16)
        buf[:H * M * D] = q_hm.reshape(-1)
        dq = f.array(buf)
        qa = dq.arg((1, cap_m, H * D))
    else:  # token-major [M, H, D] with explicit head dim
        dq = f.array(np.ascontiguousarray(q_hm.transpose(1, 0, 2)))
        qa = dq.arg((M, H, D))
    dk, dv = f.array(k), f.array(v)
    if out_layout == "token_major":
        do = f.zeros((M, H * D))
        oa = do.arg()
    else:
        do = f.zeros((H, M, D))
        oa = do.arg()
    f.flash_attention(qa, dk.arg(), dv.arg(), oa, causal, offset, H, D, N, M)
    f.synchronize()
    out = do.download()
    for b in (dq, dk, dv, do):
        b.free()
    if out_layout == "token_major":
        out = out.reshape(M, H, D).transpose(1, 0, 2)
    return out


@pytest.mark.parametrize("M,prefix", [(2, 0), (7, 0), (16, 0), (17, 5), (26, 0), (31, 100), (32, 0), (33, 64),
                                      (128, 0), (129, 31), (200, 1000), (257, 0)])
@pytest.mark.parametrize("D,H,Hkv", [(64, 14, 2), (128, 6, 2)])
def test_prefill_causal_vs_oracle(M, prefix, D, H, Hkv):
    announce("prefill", M, prefix, D)
    rng = np.random.default_rng(M * 31 + prefix)
    N = prefix + M
    cap = N + 7
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    k[:, N:], v[:, N:] = np.float16(np.nan), np.float16(np.nan)
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    got = gpu_prefill(q, k, v, H, D, M, N, prefix)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    assert max_abs(got, rm.gqa_prefill_f64(q, k, v, H, Hkv, D, N, prefix)) <= TOL


def test_prefill_layouts_and_noncausal():
    announce("prefill layouts")
    rng = np.random.default_rng(2)
    H, Hkv, D, M, prefix = 8, 2, 128, 45, 19
    N, cap = M + prefix, 80
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major")
    base = gpu_prefill(q, k, v, H, D, M, N, prefix)
    assert max_abs(base, want) <= TOL
    for ql in ("token_meta_head_contents", "token_major_hd"):
        for ol in ("token_major", "head_major"):
            got = gpu_prefill(q, k, v, H, D, M, N, prefix, q_layout=ql, out_layout=ol)
            assert np.array_equal(bits(got), bits(base)), (ql, ol)  # layouts only move data
    # non-causal and causal-offset-mismatch cases run on the same kernel (no materialized fallback)
    nc = gpu_prefill(q, k, v, H, D, M, N, 0, causal=False)
    assert max_abs(nc, orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, 0, cap, causal=False, out_layout="head_major")) <= TOL
    off = gpu_prefill(q, k, v, H, D, M, N, 3, causal=True)  # query_offset + m != kv_seq_len
    assert max_abs(off, orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, 3, cap, causal=True, out_layout="head_major")) <= TOL


@pytest.mark.parametrize("D", [64, 128])
def test_prefill_output_view_that_is_only_8_byte_aligned(D):
    """The output tensor starts 8 bytes into its buffer: whole-row 16-byte stores are not possible and each group writes its
    half of every row in 8-byte pieces. Same bits as the aligned output; the bytes around the view stay untouched."""
    announce("prefill, 8-byte aligned output view", D)
    f = ctx()
    rng = np.random.default_rng(17 + D)
    H, Hkv, M = 6, 2, 333
    q, k, v = h16(rng.normal(size=(H, M, D))), h16(rng.normal(size=(Hkv, M, D))), h16(rng.normal(size=(Hkv, M, D)))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    aligned = f.zeros((M, H * D))
    f.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), aligned.arg(), True, 0, H, D, M, M)
    pad = 4  # elements = 8 bytes
    sentinel = np.float16(3.25)
    shifted = f.array(np.full((M * H * D + 2 * pad,), sentinel, np.float16))
    f.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), shifted.arg((M, H * D), offset=pad * 2), True, 0, H, D, M, M)
    f.synchronize()
    got = shifted.download()
    assert np.all(got[:pad] == sentinel) and np.all(got[-pad:] == sentinel)
    assert np.array_equal(bits(got[pad:-pad].reshape(M, H * D)), bits(aligned.download()))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, M, 0, M, causal=True)
    assert max_abs(got[pad:-pad].reshape(M, H * D), want) <= TOL
    for b in (dq, dk, dv, aligned, shifted):
        b.free()


def test_prefill_known_answer_fixture_noncausal():
    announce("prefill fixture")
    g = np.load(os.path.join(GOLD, "known_answer_sdpa.npz"))
    q, k, v, want = (g["misaligned_m17_" + n] for n in ("q", "k", "v", "expected_f64"))
    H, M, D = q.shape
    N = k.shape[1]
    got = gpu_prefill(q, k, v, H, D, M, N, 0, causal=False)
    assert np.all(np.abs(got.astype(np.float64) - want) <= rm.f16_ulp(want) + 2e-4 * np.abs(want) + 1e-6)


def test_prefill_rows_equal_decode_and_first_row():
    announce("prefill rows == decode")
    f = ctx()
    rng = np.random.default_rng(4)
    H, Hkv, D, M = 6, 2, 64, 70
    cap = M
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    got = gpu_prefill(q, k, v, H, D, M, M, 0)
    for h in range(H):
        assert np.array_equal(bits(got[h, 0]), bits(v[h // 3, 0]))
    for r in (1, 33, 69):
        dq, dk, dv, do = f.array(q[:, r].copy()), f.array(k), f.array(v), f.zeros((1, H * D))
        f.flash_attention(dq.arg((1, H * D)), dk.arg(), dv.arg(), do.arg(), True, r, H, D, r + 1, 1)
        f.synchronize()
        assert max_abs(do.download().reshape(H, D), got[:, r]) <= 1.5e-3


@pytest.mark.parametrize("H,Hkv,D,M", [(24, 8, 128, 4133), (14, 2, 64, 5000)])
def test_prefill_many_items_per_workgroup_rows_equal_decode(H, Hkv, D, M):
    """More (query tile, head) items than three times the CUs, the last tile ragged: every resident workgroup works
    through several items in turn. Sampled rows (tile edges, the ragged end) against the decode kernel's answer for the
    same row, which the oracle tests pin; rows of the output nobody should have touched stay as they were."""
    announce("prefill, several items per workgroup", H, Hkv, D, M)
    f = ctx()
    rng = np.random.default_rng(M)
    q, k, v = h16(rng.normal(size=(H, M, D))), h16(rng.normal(size=(Hkv, M, D))), h16(rng.normal(size=(Hkv, M, D)))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    guard = 3
    sentinel = np.float16(-7.5)
    dout = f.array(np.full((M + guard, H * D), sentinel, np.float16))
    f.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), dout.arg((M, H * D)), True, 0, H, D, M, M)
    f.synchronize()
    got = dout.download()
    assert np.all(got[M:] == sentinel), "rows past the last query were written"
    got = got[:M].reshape(M, H, D)
    assert np.isfinite(got.astype(np.float32)).all()
    rows = sorted({0, 1, 127, 128, 129, 2047, 2048, 3000, M - 130, M - 2, M - 1} | set(rng.integers(0, M, 6).tolist()))
    d1 = f.zeros((1, H * D))
    for r in rows:
        dqr = f.array(np.ascontiguousarray(q[:, r]))
        f.flash_attention(dqr.arg((1, H * D)), dk.arg(), dv.arg(), d1.arg(), True, r, H, D, r + 1, 1)
        f.synchronize()
        assert max_abs(d1.download().reshape(H, D), got[r]) <= 1.5e-3, r
        dqr.free()
    for b in (dq, dk, dv, dout, d1):
        b.free()


def test_prefill_llama_shape_full_size_from_paged_cache():
    """benchmark configuration 4: 2048-token prompt, H24/Hkv8/D128, RoPE theta 5e5 on positions 0..2047, all rows
    appended into an empty paged cache, causal flash attention reading through the block table."""
    announce("prefill C4 full size")
    f = ctx()
    rng = np.random.default_rng(0xF0DD + 4)
    H, Hkv, D, M, bs = 24, 8, 128, 2048, 16
    n_blocks = M // bs + 4
    bt = rng.permutation(n_blocks)[:M // bs].astype(np.int32)[None, :]
    q, k, v = (h16(rng.normal(size=(M, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(5e5, D, M)
    dkp, dvp = f.zeros((n_blocks, Hkv, bs, D)), f.zeros((n_blocks, Hkv, bs, D))
    dbt = f.array(bt)
    desc = fa.paged_kv(dkp, dvp, dbt, None, n_blocks, Hkv, bs, D, 1, M // bs)
    dq, dk, dv, dqr, dout = f.array(q), f.array(k), f.array(v), f.zeros((H, M, D)), f.zeros((M, H * D))
    dcos, dsin = f.array(cos), f.array(sin)
    f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), desc, 0, dcos.arg(), dsin.arg(),
                          fa.KvPrepFusedParams.make(H, Hkv, D, M, 0, 0, fa.ROPE_NORMAL))
    f.flash_prefill_paged(dqr.arg(), desc, 0, dout.arg(), True, 0, H, M, M)
    f.synchronize()
    kc, vc = np.zeros((Hkv, M, D), np.float16), np.zeros((Hkv, M, D), np.float16)
    qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, M, 0, M, rope_mode=1))
    assert np.array_equal(bits(dqr.download()), bits(qr))
    assert np.array_equal(bits(orc.paged_gather(dkp.download(), bt[0], Hkv, bs, D, M)), bits(kc))
    assert np.array_equal(bits(orc.paged_gather(dvp.download(), bt[0], Hkv, bs, D, M)), bits(vc))
    want = orc.sdpa_prefill(qr, kc, vc, H, Hkv, D, M, M, 0, M, causal=True, n_threads=16)  # token-major
    got = dout.download()
    assert max_abs(got, want) <= TOL
    # the contiguous entry point on the gathered cache gives the same bits
    dkc, dvc, dout2 = f.array(kc), f.array(vc), f.zeros((M, H * D))
    f.flash_attention(dqr.arg((1, M, H * D)), dkc.arg(), dvc.arg(), dout2.arg(), True, 0, H, D, M, M)
    f.synchronize()
    assert np.array_equal(bits(dout2.download()), bits(got))


def test_prefill_errors():
    announce("prefill errors")
    f = ctx()
    H, Hkv, D, M, cap = 4, 2, 64, 8, 16
    dq, dk, dv, do = f.zeros((H, M, D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.zeros((M, H * D))
    f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, M, M)
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg((H, M, 96)), dk.arg(), dv.arg(), do.arg(), True, 0, H, 96, M, M)
    assert e.value.variant == "OperationNotSupported" and "64 or 128" in str(e.value)
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg((M * H * D,)), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, M, M)
    assert e.value.variant == "OperationNotSupported" and "layout" in str(e.value)
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg((H * M * D,)), True, 0, H, D, M, M)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:
        f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, 0, H, D, cap + 1, M)
    assert e.value.variant == "InvalidShape"
    f.synchronize()


@pytest.mark.parametrize("split_k", [0, 1, 5])
@pytest.mark.parametrize("H,Hkv,D,M,prefix,layout", [
    (24, 8, 128, 32, 4000, "head_major"),   # the reference's default chunk at the Llama-3.2-3B shape: 3 heads per item
    (16, 2, 128, 20, 3000, "token_major"),  # a group of 8: two items of 4 heads per KV head, rows past the chunk's end
    (14, 2, 64, 32, 2500, "head_major"),    # a group of 7: items of 4 and of 3 heads
    (8, 4, 64, 5, 1500, "token_major"),     # a group of 2: two of the four waves of a group have no head
    (12, 3, 128, 2, 900, "head_major"),     # two rows
    (6, 2, 128, 31, 0, "head_major"),       # no prefix: one key tile, nothing to split
    (24, 8, 128, 64, 4000, "head_major"),   # 64 rows: six (head, 32 rows) pairs per KV group in items of four and two
    (14, 2, 64, 40, 700, "token_major"),    # 40 rows, groups of seven heads: fourteen pairs, the second blocks ragged
    (4, 2, 128, 33, 300, "head_major"),     # one row into the second block, groups of two: exactly one item per KV head
])
def test_prefill_short_chunk_packs_the_heads_of_a_kv_group(H, Hkv, D, M, prefix, layout, split_k, prefill_variant):
    """A chunk of at most 64 query rows (the reference's default prefill chunk size is 32, src/model/executor.rs:232-250)
    runs with four (head, 32 rows) pairs of a KV group in one item. Same contract as every other prefill launch: the
    oracle and float64 within the tolerance, for the automatic split count, no split and a forced one."""
    announce("prefill, short chunk", H, Hkv, D, M, prefix, layout, split_k, prefill_variant)
    f = ctx()
    rng = np.random.default_rng(H * 100 + M + prefix)
    N = prefix + M
    cap = N + 3
    q, k, v = h16(rng.normal(size=(H, M, D))), h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    k[:, N:], v[:, N:] = np.float16(np.nan), np.float16(np.nan)
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    f.set_prefill_split_k(split_k)
    try:
        got = gpu_prefill(q, k, v, H, D, M, N, prefix, q_layout=layout)
    finally:
        f.set_prefill_split_k(0)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL
    assert max_abs(got, rm.gqa_prefill_f64(q, k, v, H, Hkv, D, N, prefix)) <= TOL


@pytest.mark.parametrize("split_k", [0, 1, 2, 3, 4, 8])
def test_prefill_split_k_independent_of_split_count(split_k):
    """A prefill chunk after a long prefix, key tiles divided over split_k workgroups + merge kernel
    (flash_prefill.metal:452-457, 843-888): same result for every split count, including splits that get no tile."""
    announce("prefill split-k", split_k)
    f = ctx()
    rng = np.random.default_rng(11)
    H, Hkv, D, M, prefix = 6, 2, 128, 37, 700
    N, cap = M + prefix, 800
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    k[:, N:], v[:, N:] = np.float16(np.nan), np.float16(np.nan)
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    f.set_prefill_split_k(split_k)
    try:
        got = gpu_prefill(q, k, v, H, D, M, N, prefix)
    finally:
        f.set_prefill_split_k(0)
    assert np.all(np.isfinite(got))
    assert max_abs(got, want) <= TOL


def test_prefill_split_k_more_splits_than_tiles_and_d64():
    announce("prefill split-k edge")
    f = ctx()
    rng = np.random.default_rng(12)
    H, Hkv, D, M, prefix = 14, 2, 64, 130, 61   # 2 query tiles; the first sees only 3 key tiles
    N, cap = M + prefix, 256
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    for split_k in (3, 64):
        f.set_prefill_split_k(split_k)
        try:
            got = gpu_prefill(q, k, v, H, D, M, N, prefix)
        finally:
            f.set_prefill_split_k(0)
        assert max_abs(got, want) <= TOL, split_k
    with pytest.raises(fa.FoundryError) as e:
        f.set_prefill_split_k(65)
    assert e.value.variant == "OperationNotSupported"


def test_prefill_chunk_after_long_prefix_auto_split():
    """The reference's default prefill chunk (32 rows) against an 8K prefix: the automatic split-K path."""
    announce("prefill chunk 32 @ 8k")
    rng = np.random.default_rng(13)
    H, Hkv, D, M, prefix = 24, 8, 128, 32, 8160
    N, cap = M + prefix, 8192
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    got = gpu_prefill(q, k, v, H, D, M, N, prefix)
    assert max_abs(got, want) <= TOL


def test_prefill_chunk_after_32k_prefix_ring_wraps():
    """32 rows against a 32K prefix: every workgroup of the chunk kernel takes its partition through the LDS ring
    several times over (1024 keys = 16 rounds of 64 in 4 slots), with the last partition shorter than the others."""
    announce("prefill chunk 32 @ 32k")
    rng = np.random.default_rng(14)
    H, Hkv, D, M, prefix = 24, 8, 128, 32, 32768 - 32 - 40
    N, cap = M + prefix, 32768
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major", n_threads=8)
    got = gpu_prefill(q, k, v, H, D, M, N, prefix)
    assert max_abs(got, want) <= TOL


def test_prefill_chunk_kernel_gives_up_cleanly():
    """Failure handling of the chunk kernel's waits (LDS ring and merge), forced from the host: with a wait bound of
    zero a wave gives up at its first look at anything that is not there yet. Every kernel still ends normally, the
    next stream wait reports it, and with the normal bound the same context is right again (the arrival pattern of
    the partial buffer was restored)."""
    announce("prefill chunk kernel, zero wait bound")
    rng = np.random.default_rng(15)
    H, Hkv, D, M, prefix = 24, 8, 128, 32, 4000
    N, cap = M + prefix, 4096
    q, k, v = h16(rng.normal(size=(H, M, D))), h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="token_major", n_threads=8)
    g = fa.Foundry(0)
    try:
        dq, dk, dv, do = g.array(q), g.array(k), g.array(v), g.zeros((M, H * D))
        g.set_prefill_variant(3)
        g.set_decode_poll_spin_us(0)
        reported = 0
        for _ in range(3):
            g.set_prefill_variant(3)  # (a give-up takes the kernel out until it is selected again)
            g.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), do.arg(), True, prefix, H, D, N, M)
            try:
                g.synchronize()
            except fa.FoundryError as e:
                reported += 1
                assert e.variant == "OperationFailed" and "waited longer" in str(e)
        assert reported >= 1  # (a wave cannot find a whole round in LDS at its first look)
        # after a give-up the context leaves the kernel out: right again at once, zero bound or not (tiled kernel + merge launch)
        g.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), do.arg(), True, prefix, H, D, N, M)
        assert max_abs(do.download().reshape(M, H * D), want.reshape(M, H * D)) <= TOL
        # ... and selecting the variant again brings the kernel back, which with the normal bound is right
        g.set_prefill_variant(3)
        g.set_decode_poll_spin_us(5000)
        for _ in range(3):
            g.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), do.arg(), True, prefix, H, D, N, M)
            assert max_abs(do.download().reshape(M, H * D), want.reshape(M, H * D)) <= TOL
        g.synchronize()
    finally:
        g.close()


def test_prefill_chunk_kernel_repeated_launches_give_the_same_bits():
    """The chunk kernel's producer and consumer waves run rounds apart, held together only by the ring's counters, and
    its result does not depend on the order in which anything arrives: 40 launches over a 32K prefix (16 rounds through
    4 slots per workgroup) must give the same bits every time, and those of a launch that is known to be right."""
    announce("prefill chunk 32 @ 32k, repeated")
    rng = np.random.default_rng(16)
    H, Hkv, D, M, prefix = 24, 8, 128, 32, 32768 - 32
    N, cap = M + prefix, 32768
    q, k, v = h16(rng.normal(size=(H, M, D))), h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    want = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="token_major", n_threads=8)
    f = ctx()
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    outs = [f.zeros((M, H * D)) for _ in range(40)]
    for do in outs:
        f.flash_attention(dq.arg((H, M, D)), dk.arg(), dv.arg(), do.arg(), True, prefix, H, D, N, M)
    f.synchronize()
    first = outs[0].download()
    assert max_abs(first.reshape(M, H * D), want.reshape(M, H * D)) <= TOL
    for i, do in enumerate(outs[1:]):
        assert np.array_equal(bits(do.download()), bits(first)), i + 1
    for b in [dq, dk, dv] + outs:
        b.free()
