"""Pins the CPU oracle (oracle/oracle_attn.c) without a GPU.

Each check is independent of the oracle's own formulae: exhaustive comparison with numpy's binary16,
closed forms, float64 library softmax / complex rotation, index brute force, the reference tests' own
closed-form known-answer inputs (tests/golden/known_answer_sdpa.npz) and algebraic invariants.
Reference citations are paths under /root/reference/crates/metallic-foundry/.
"""
import os

import numpy as np
import pytest

import orc
import refmath as rm

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
rng_global = np.random.default_rng(0xF0DD)


def h16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


# ----------------------------------------------------------------------------- f16 conversions

def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.f16_to_f32_n(bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_rne_against_numpy():
    rng = np.random.default_rng(1)
    # random bit patterns, midpoints between adjacent halves, subnormal and overflow boundaries
    rand = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    halves = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)  # exact ties
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e30, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, 5.96e-8, 6.1e-5], np.float32)
    x = np.concatenate([rand, mids, -mids, near, edge, -edge])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = orc.f32_to_f16_n(x)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (x[bad[:5]], got[bad[:5]], want[bad[:5]])
    assert np.isnan(np.array([orc.lib().orc_f32_to_f16(float("nan"))], np.uint16).view(np.float16))[0]


# ----------------------------------------------------------------------------- RoPE tables (src/model/executor.rs:1981-2006)

@pytest.mark.parametrize("base,D,P", [(1e6, 64, 1100), (5e5, 128, 8500), (1e4, 128, 64)])
def test_rope_tables_closed_forms(base, D, P):
    cos, sin = orc.rope_tables(base, D, P)
    assert cos.shape == (P, D // 2)
    assert np.all(cos[0] == np.float16(1)) and np.all(sin[0] == np.float16(0))
    # column 0: exponent 0 -> inv_freq 1 -> angle = p exactly (p < 2^24)
    p = np.arange(P, dtype=np.float64)
    assert np.all(np.abs(cos[:, 0].astype(np.float64) - np.cos(p)) <= 0.5 * rm.f16_ulp(np.cos(p)) + 1e-7)
    assert np.all(np.abs(sin[:, 0].astype(np.float64) - np.sin(p)) <= 0.5 * rm.f16_ulp(np.sin(p)) + 1e-7)
    # all columns against float64 cos/sin of the f32 angle
    i = np.arange(D // 2)
    inv = (np.float32(1) / np.power(np.float32(base), (2 * i).astype(np.float32) / np.float32(D))).astype(np.float32)
    ang = (p.astype(np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
    # a few f32 ulp of slack on inv_freq (libm powf vs numpy power) scale with the angle
    slack = 4e-7 * np.abs(ang) + 0.5 * 2.0 ** -11 + 1e-6
    assert np.all(np.abs(cos.astype(np.float64) - np.cos(ang)) <= slack)
    assert np.all(np.abs(sin.astype(np.float64) - np.sin(ang)) <= slack)
    # cos^2 + sin^2 = 1 within f16 rounding
    assert np.all(np.abs(cos.astype(np.float64) ** 2 + sin.astype(np.float64) ** 2 - 1) < 2e-3)


def test_rope_tables_freq_factors_and_window():
    ff = np.linspace(1.0, 8.0, 32).astype(np.float32)
    c_all, s_all = orc.rope_tables(5e5, 64, 300, ff)
    c_win, s_win = orc.rope_tables(5e5, 64, 300, ff, pos_begin=200)
    assert np.array_equal(c_all[200:], c_win) and np.array_equal(s_all[200:], s_win)
    c_one, _ = orc.rope_tables(5e5, 64, 300, np.ones(32, np.float32))
    c_none, _ = orc.rope_tables(5e5, 64, 300)
    assert np.array_equal(c_one, c_none)
    # dividing inv_freq by f == evaluating the unscaled column at angle/f
    i = np.arange(32)
    inv = 1.0 / np.power(5e5, 2 * i / 64.0) / ff
    ang = np.arange(300)[:, None] * inv[None, :]
    assert np.max(np.abs(c_all.astype(np.float64) - np.cos(ang))) < 1e-3


# ----------------------------------------------------------------------------- NeoX RoPE (tests/rope.rs:31-63)

@pytest.mark.parametrize("dim,seq,rows,off", [(64, 1, 1, 0), (64, 16, 16, 0), (128, 8, 32, 0), (256, 4, 8, 0),
                                              (64, 1, 14, 1024), (128, 7, 21, 5), (64, 128, 128, 0), (2, 4, 4, 1)])
def test_rope_neox_is_complex_rotation(dim, seq, rows, off):
    rng = np.random.default_rng(dim * 131 + seq)
    x = h16(rng.uniform(-1, 1, size=(rows, dim)))
    cos, sin = orc.rope_tables(10000.0, dim, seq + off)
    got = orc.rope_neox(x, cos, sin, dim, seq, off)
    pos = (np.arange(rows) % seq) + off
    want = rm.rope_rotate_f64(x, cos, sin, pos, "neox")
    err = np.abs(got.astype(np.float64) - want)
    assert np.all(err <= 0.5 * rm.f16_ulp(want) + 2e-7)  # f32 products/sum then one RNE to f16


def test_rope_neox_invariants():
    rng = np.random.default_rng(7)
    dim, seq = 64, 9
    x = h16(rng.normal(size=(seq, dim)))
    cos, sin = orc.rope_tables(1e6, dim, seq)
    y = orc.rope_neox(x, cos, sin, dim, seq, 0)
    assert np.array_equal(y[0], x[0])  # position 0: cos 1, sin 0
    nx = x.astype(np.float64)[:, :32] ** 2 + x.astype(np.float64)[:, 32:] ** 2
    ny = y.astype(np.float64)[:, :32] ** 2 + y.astype(np.float64)[:, 32:] ** 2
    assert np.all(np.abs(nx - ny) <= 4e-3 * (1 + nx))  # table cos^2+sin^2 != 1 exactly in f16
    back = orc.rope_neox(y, cos, (-sin.astype(np.float32)).astype(np.float16), dim, seq, 0)
    assert np.max(np.abs(back.astype(np.float32) - x.astype(np.float32))) < 6e-3
    ident = orc.rope_neox(x, np.ones_like(cos), np.zeros_like(sin), dim, seq, 0)
    assert np.array_equal(ident, x)  # tests/sdpa_v2_parity.rs:153-155 identity tables


# ----------------------------------------------------------------------------- index maps of the legacy chain

def test_kv_rearrange_brute_force():
    # tests/kv_rearrange.rs:33-68: out[b*H + h, s, d] = in[b*seq + s, (h / G)*D + d]
    H, Hkv, D, S, B = 6, 2, 8, 5, 2
    x = h16(np.arange(B * S * Hkv * D).reshape(B * S, Hkv * D) % 2048)
    got = orc.kv_rearrange(x, H, Hkv, D, S, batch=B)
    for b in range(B):
        for h in range(H):
            for s in range(S):
                assert np.array_equal(got[b * H + h, s], x[b * S + s, (h // 3) * D:(h // 3 + 1) * D])


def test_kv_cache_write_read_brute_force():
    Hkv, D, S, off, cap = 3, 4, 5, 7, 16
    x = h16(np.arange(Hkv * S * D).reshape(Hkv, S, D))
    cache = np.zeros((Hkv, cap, D), np.float16)
    orc.kv_cache_write(cache, x, Hkv, D, S, off, cap)
    want = np.zeros_like(cache)
    want[:, off:off + S] = x
    assert np.array_equal(cache, want)
    assert np.array_equal(orc.kv_cache_read(cache, Hkv, D, off + S, cap), want[:, :off + S])


def test_kv_cache_write_repeat_and_repeat_kv_heads():
    # tests/kv_cache_write_repeat_kv_heads.rs:57-70 and tests/repeat_kv_heads.rs:32-61
    Hkv, H, D, S, off, cap = 2, 6, 4, 3, 2, 8
    x = h16(np.arange(Hkv * S * D).reshape(Hkv, S, D) + 1)
    cache = np.zeros((H, cap, D), np.float16)
    orc.kv_cache_write_repeat(cache, x, Hkv, H, D, S, off, cap)
    for h in range(H):
        assert np.array_equal(cache[h, off:off + S], x[h // 3])
        assert not cache[h, :off].any() and not cache[h, off + S:].any()
    compact = np.zeros((Hkv, cap, D), np.float16)
    orc.kv_cache_write(compact, x, Hkv, D, S, off, cap)
    rep = orc.repeat_kv_heads(compact, Hkv, H, off + S, D, cap)
    assert np.array_equal(rep, cache[:, :off + S])


# ----------------------------------------------------------------------------- fused kv_prep

def _chain_reference(q, k, v, H, Hkv, D, S, off, cap, cos, sin):
    """The un-fused chain the reference's parity test compares against (tests/kv_prep_fused.rs:60-200):
    rearrange -> NeoX rope -> compact cache write."""
    q_r = orc.kv_rearrange(q, H, H, D, S)
    q_rot = orc.rope_neox(q_r, cos, sin, D, S, off)
    k_r = orc.kv_rearrange(k, Hkv, Hkv, D, S)
    k_rot = orc.rope_neox(k_r, cos, sin, D, S, off)
    v_r = orc.kv_rearrange(v, Hkv, Hkv, D, S)
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    orc.kv_cache_write(kc, k_rot, Hkv, D, S, off, cap)
    orc.kv_cache_write(vc, v_r, Hkv, D, S, off, cap)
    return q_rot, kc, vc


@pytest.mark.parametrize("S,off,cap,H,Hkv,D", [(1, 5, 16, 14, 2, 64), (4, 0, 16, 14, 2, 64), (2, 0, 64, 32, 8, 128),
                                               (3, 9, 12, 24, 8, 128), (1, 1024, 1152, 14, 2, 64)])
def test_kv_prep_fused_neox_equals_chain_bitwise(S, off, cap, H, Hkv, D):
    rng = np.random.default_rng(S * 1000 + off)
    q = h16(rng.uniform(-1, 1, (S, H * D)))
    k = h16(rng.uniform(-1, 1, (S, Hkv * D)))
    v = h16(rng.uniform(-1, 1, (S, Hkv * D)))
    cos, sin = orc.rope_tables(10000.0, D, cap)
    q_ref, kc_ref, vc_ref = _chain_reference(q, k, v, H, Hkv, D, S, off, cap, cos, sin)
    kc = np.zeros((Hkv, cap, D), np.float16)
    vc = np.zeros((Hkv, cap, D), np.float16)
    q_rot = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, S, off, cap, rope_mode=0))
    assert np.array_equal(q_rot.view(np.uint16), q_ref.view(np.uint16))
    assert np.array_equal(kc.view(np.uint16), kc_ref.view(np.uint16))  # tests/kv_prep_fused.rs:239-244
    assert np.array_equal(vc.view(np.uint16), vc_ref.view(np.uint16))
    assert not kc[:, :off].any() and not kc[:, off + S:].any()  # untouched slots stay zero


def _deinterleave(x, D):
    """Per head: even dims first, then odd dims."""
    shp = x.shape
    xx = x.reshape(shp[0], -1, D)
    return np.concatenate([xx[..., 0::2], xx[..., 1::2]], axis=-1).reshape(shp)


def _interleave(x, D):
    shp = x.shape
    xx = x.reshape(-1, D)
    out = np.empty_like(xx)
    out[:, 0::2], out[:, 1::2] = xx[:, :D // 2], xx[:, D // 2:]
    return out.reshape(shp)


@pytest.mark.parametrize("S,off,cap,H,Hkv,D", [(1, 5, 16, 14, 2, 64), (5, 3, 16, 24, 8, 128)])
def test_kv_prep_fused_normal_is_neox_under_deinterleave(S, off, cap, H, Hkv, D):
    """`normal` pairing (kv_prep_fused.metal:66-73) has no reference test; pinned by
    normal(x) == interleave(neox(deinterleave(x))) and by the complex-rotation closed form."""
    rng = np.random.default_rng(99 + S)
    q = h16(rng.normal(size=(S, H * D)))
    k = h16(rng.normal(size=(S, Hkv * D)))
    v = h16(rng.normal(size=(S, Hkv * D)))
    cos, sin = orc.rope_tables(5e5, D, cap)
    kc_n, vc_n = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    q_n = orc.kv_prep_fused(q, k, v, kc_n, vc_n, cos, sin, orc.make_params(H, Hkv, D, S, off, cap, rope_mode=1))
    kc_x, vc_x = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    q_x = orc.kv_prep_fused(_deinterleave(q, D), _deinterleave(k, D), v, kc_x, vc_x, cos, sin,
                            orc.make_params(H, Hkv, D, S, off, cap, rope_mode=0))
    assert np.array_equal(q_n.view(np.uint16), _interleave(q_x, D).view(np.uint16))
    assert np.array_equal(kc_n.view(np.uint16), _interleave(kc_x, D).view(np.uint16))
    assert np.array_equal(vc_n.view(np.uint16), vc_x.view(np.uint16))
    # closed form
    pos = np.arange(S) + off
    q_tm = q.reshape(S, H, D)
    want = rm.rope_rotate_f64(q_tm, cos, sin, pos[:, None], "normal").transpose(1, 0, 2)
    assert np.all(np.abs(q_n.astype(np.float64) - want) <= 0.5 * rm.f16_ulp(want) + 4e-7)


def test_kv_prep_fused_nope_layer_rule():
    """apply_rope = step == 0 or (layer+1) % step != 0 (kv_prep_fused.metal:57); SmolLM3 uses step 4."""
    S, off, cap, H, Hkv, D = 2, 3, 8, 16, 4, 128
    rng = np.random.default_rng(5)
    q, k, v = (h16(rng.normal(size=(S, n * D))) for n in (H, Hkv, Hkv))
    cos, sin = orc.rope_tables(5e6, D, cap)
    plain_q = orc.kv_rearrange(q, H, H, D, S)
    plain_k = np.zeros((Hkv, cap, D), np.float16)
    orc.kv_cache_write(plain_k, orc.kv_rearrange(k, Hkv, Hkv, D, S), Hkv, D, S, off, cap)
    roped = None
    for layer in range(8):
        kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
        q_rot = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin,
                                  orc.make_params(H, Hkv, D, S, off, cap, rope_mode=1, layer_idx=layer,
                                                  no_rope_layer_step=4))
        if layer in (3, 7):
            assert np.array_equal(q_rot, plain_q) and np.array_equal(kc, plain_k)
        else:
            assert not np.array_equal(q_rot, plain_q)
            if roped is None:
                roped = (q_rot.copy(), kc.copy())
            assert np.array_equal(q_rot, roped[0]) and np.array_equal(kc, roped[1])
    kc0, vc0 = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    q0 = orc.kv_prep_fused(q, k, v, kc0, vc0, cos, sin, orc.make_params(H, Hkv, D, S, off, cap, rope_mode=1,
                                                                        layer_idx=3, no_rope_layer_step=0))
    assert np.array_equal(q0, roped[0])  # step 0 disables the rule


# ----------------------------------------------------------------------------- SDPA decode

def test_sdpa_known_answer_decode_fixture():
    g = np.load(os.path.join(GOLD, "known_answer_sdpa.npz"))
    q, k, v, want = g["oob_m1_q"], g["oob_m1_k"], g["oob_m1_v"], g["oob_m1_expected_f64"]
    H, M, D = q.shape
    N = k.shape[1]
    got = orc.sdpa_decode(q.reshape(H, D), k, v, H, H, D, N, N).reshape(H, D).astype(np.float64)
    assert np.all(np.abs(got - want[:, 0]) <= 0.5 * rm.f16_ulp(want[:, 0]) + 2e-6 * np.abs(want[:, 0]) + 1e-8)


def test_sdpa_known_answer_prefill_fixture_noncausal():
    g = np.load(os.path.join(GOLD, "known_answer_sdpa.npz"))
    q, k, v, want = (g["misaligned_m17_" + n] for n in ("q", "k", "v", "expected_f64"))
    H, M, D = q.shape
    N = k.shape[1]
    got = orc.sdpa_prefill(q, k, v, H, H, D, M, N, 0, N, causal=False)  # token-major [M, H*D]
    got = got.reshape(M, H, D).transpose(1, 0, 2).astype(np.float64)
    assert np.all(np.abs(got - want) <= 0.5 * rm.f16_ulp(want) + 4e-6 * np.abs(want) + 1e-8)


def test_lcg_stream_matches_integer_recurrence():
    # tests/flashattention_decode_parity.rs:15-30, recomputed with Python integers
    st = 1
    want = []
    for _ in range(64):
        st = (st * 1664525 + 1013904223) % (1 << 32)
        want.append(np.float32(np.float32(st >> 9) * np.float32(1.0 / (1 << 23)) * np.float32(2) - np.float32(1))
                    * np.float32(0.25))
    got, new_state = orc.lcg_fill_f16(1, 64, 0.25)
    assert new_state == st
    assert np.array_equal(got, np.array(want, np.float32).astype(np.float16))


@pytest.mark.parametrize("seed,H,D,N", [(1, 14, 64, 128), (7, 14, 64, 257), (42, 8, 128, 300)])
def test_sdpa_decode_reference_test_inputs_vs_f64(seed, H, D, N):
    """The reference's decode parity inputs (LCG, +-0.25), MHA cache [H, N, D]
    (tests/flashattention_decode_parity.rs:117-200); expected from float64 softmax."""
    st = seed
    q, st = orc.lcg_fill_f16(st, H * D, 0.25)
    k, st = orc.lcg_fill_f16(st, H * N * D, 0.25)
    v, st = orc.lcg_fill_f16(st, H * N * D, 0.25)
    k, v = k.reshape(H, N, D), v.reshape(H, N, D)
    want = rm.gqa_decode_f64(q, k, v, H, H, D, N)
    for block, warps in [(512, 16), (128, 8), (1, 1), (37, 5)]:
        got = orc.sdpa_decode(q, k, v, H, H, D, N, N, block_keys=block, warps=warps).reshape(H, D)
        assert np.max(np.abs(got.astype(np.float64) - want)) < 2.5e-4  # half an f16 ulp at |x| < 0.25 + f32 noise
    got_h = orc.sdpa_decode(q, k, v, H, H, D, N, N, block_keys=256, warps=16, tg_out_half=True).reshape(H, D)
    assert np.max(np.abs(got_h.astype(np.float64) - want)) < 3e-3  # f16 partials: the reference's looser variant


def test_sdpa_decode_invariants():
    rng = np.random.default_rng(3)
    H, Hkv, D, cap, N = 6, 2, 64, 40, 33
    q = h16(rng.normal(size=(H, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    k_same = np.broadcast_to(h16(rng.normal(size=(Hkv, 1, D))), (Hkv, cap, D)).copy()
    out = orc.sdpa_decode(q, k_same, v, H, Hkv, D, cap, N).reshape(H, D)
    for h in range(H):  # equal keys -> uniform weights -> mean of V
        want = v[h // 3, :N].astype(np.float64).mean(axis=0)
        assert np.max(np.abs(out[h].astype(np.float64) - want)) < 1e-3
    k = h16(rng.normal(size=(Hkv, cap, D)))
    out1 = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, 1).reshape(H, D)
    for h in range(H):  # a single key -> V[0]
        assert np.array_equal(out1[h], v[h // 3, 0])
    # rows beyond kv_len are never read
    k2, v2 = k.copy(), v.copy()
    k2[:, N:], v2[:, N:] = np.float16(np.nan), np.float16(np.nan)
    a = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N)
    b = orc.sdpa_decode(q, k2, v2, H, Hkv, D, cap, N)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("H,Hkv,D,N", [(14, 2, 64, 100), (24, 8, 128, 70), (16, 2, 128, 65), (16, 4, 128, 40)])
def test_sdpa_gqa_equals_mha_on_expanded_cache(H, Hkv, D, N):
    """GQA head map (flash_decode.metal:129-132) has no reference numeric test; pinned by
    GQA(compact) == MHA(repeat_kv_heads(compact)) and by float64 per-head attention."""
    rng = np.random.default_rng(H + N)
    cap = N + 5
    q = h16(rng.normal(size=(H, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    got = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N)
    k_exp = orc.repeat_kv_heads(k, Hkv, H, cap, D, cap)
    v_exp = orc.repeat_kv_heads(v, Hkv, H, cap, D, cap)
    mha = orc.sdpa_decode(q, k_exp, v_exp, H, H, D, cap, N)
    assert np.array_equal(got, mha)
    want = rm.gqa_decode_f64(q, k, v, H, Hkv, D, N)
    assert np.max(np.abs(got.reshape(H, D).astype(np.float64) - want)) < 1.5e-3


# ----------------------------------------------------------------------------- SDPA prefill

@pytest.mark.parametrize("M,prefix", [(1, 0), (2, 0), (7, 0), (16, 0), (17, 5), (26, 0), (31, 100), (32, 0), (33, 64)])
def test_sdpa_prefill_causal_vs_f64_and_decode(M, prefix):
    """m values of tests/flashattention_prefill_parity.rs:143-183; causal limit = row + query_offset
    (flash_prefill.metal:176-199)."""
    H, Hkv, D = 4, 2, 64
    N = prefix + M
    cap = N + 3
    rng = np.random.default_rng(M * 7 + prefix)
    q = h16(rng.normal(size=(H, M, D)))
    k = h16(rng.normal(size=(Hkv, cap, D)))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    got = orc.sdpa_prefill(q, k, v, H, Hkv, D, M, N, prefix, cap, causal=True, out_layout="head_major")
    want = rm.gqa_prefill_f64(q, k, v, H, Hkv, D, N, prefix, causal=True)
    assert np.max(np.abs(got.astype(np.float64) - want)) < 2e-3
    tm = orc.sdpa_prefill(q.transpose(1, 0, 2).reshape(M, H * D).copy(), k, v, H, Hkv, D, M, N, prefix, cap,
                          causal=True, q_layout="token_major", out_layout="token_major")
    assert np.array_equal(tm.reshape(M, H, D).transpose(1, 0, 2), got)  # layouts only move data
    for r in (0, M - 1):  # prefill row r == decode at kv_len = offset + r + 1
        dec = orc.sdpa_decode(q[:, r].copy(), k, v, H, Hkv, D, cap, prefix + r + 1, block_keys=32, warps=1)
        assert np.max(np.abs(dec.reshape(H, D).astype(np.float32) - got[:, r].astype(np.float32))) <= 1e-3
    if prefix == 0:
        for h in range(H):  # first row sees only key 0
            assert np.array_equal(got[h, 0], v[h // 2, 0])


def test_splitk_merge_independent_of_split_count():
    """flash_prefill.metal:452-457,843-888, including empty splits (l_s <= 0 is skipped)."""
    D, N = 64, 150
    rng = np.random.default_rng(11)
    q = h16(rng.normal(size=(D,)))
    k = h16(rng.normal(size=(N, D)))
    v = h16(rng.normal(size=(N, D)))
    want = rm.attn_f64(q[None], k[:101], v[:101], 1 / np.sqrt(D))[0]
    base = None
    for S in (1, 2, 3, 4, 8, 16):
        out, acc, m, l = orc.sdpa_row_splitk(q, k, v, D, N, 100, S)  # causal limit 100 -> later splits are empty
        assert np.max(np.abs(out.astype(np.float64) - want)) < 1e-3
        if S >= 8:
            assert np.any(l == 0) and np.all(m[l == 0] == np.float32(-1e30))
        if base is None:
            base = out
        assert np.max(np.abs(out.astype(np.float32) - base.astype(np.float32))) <= 1e-3
    tiny, _, m1, l1 = orc.sdpa_row_splitk(q, k, v, D, 5, 4, 8)  # more splits than tiles
    assert np.max(np.abs(tiny.astype(np.float64) - rm.attn_f64(q[None], k[:5], v[:5], 1 / np.sqrt(D))[0])) < 1e-3


# ----------------------------------------------------------------------------- paged cache

def test_paged_gather_scatter_roundtrip_with_permutation():
    rng = np.random.default_rng(21)
    Hkv, D, bs, N = 2, 16, 16, 75
    n_blocks = 9
    perm = rng.permutation(n_blocks)[: (N + bs - 1) // bs].astype(np.int32)
    contiguous = h16(rng.normal(size=(Hkv, N, D)))
    pool = np.full((n_blocks, Hkv, bs, D), np.float16(-7), np.float16)
    orc.paged_scatter(pool, perm, Hkv, bs, D, 0, N, contiguous)
    assert np.array_equal(orc.paged_gather(pool, perm, Hkv, bs, D, N), contiguous)
    # brute force: slot of (h, pos)
    for h, pos in [(0, 0), (1, 17), (0, 74), (1, 63)]:
        assert np.array_equal(pool[perm[pos // bs], h, pos % bs], contiguous[h, pos])
    untouched = np.setdiff1d(np.arange(n_blocks), perm)
    assert np.all(pool[untouched] == np.float16(-7))


# ----------------------------------------------------------------------------- Sage-style int8 Q/K

def test_sage_quantizer_and_decode():
    rng = np.random.default_rng(31)
    H, Hkv, D, N = 8, 2, 128, 200
    cap = 224
    k = rng.normal(size=(Hkv, cap, D))
    k += rng.normal(size=(Hkv, 1, D)) * 3  # channel bias that smoothing removes
    out_mask = rng.random(size=k.shape) < 0.01
    k = h16(np.where(out_mask, 8.0 * np.sign(k), k))
    v = h16(rng.normal(size=(Hkv, cap, D)))
    q = h16(rng.normal(size=(H, D)))
    mean = orc.sage_k_mean(k, Hkv, cap, D, N)
    assert np.max(np.abs(mean - k[:, :N].astype(np.float64).mean(axis=1))) < 1e-5
    kq, ks = orc.sage_quantize_k(k, mean, Hkv, cap, D, N)
    ksf = ks.astype(np.float64)
    centred = k[:, :N].astype(np.float32) - mean[:, None, :]
    deq = kq[:, :N].astype(np.float64) * np.repeat(ksf, 32, axis=1)[:, :N, None]
    # |x - dequant| <= scale/2 except where the f16-rounded scale clips the block maximum
    assert np.all(np.abs(deq - centred) <= 0.5 * np.repeat(ksf, 32, axis=1)[:, :N, None] * 1.002 + 1e-6 +
                  127 * np.abs(np.repeat(ksf, 32, axis=1)[:, :N, None] * 2.0 ** -11))
    assert np.all(np.abs(kq) <= 127) and not kq[:, N:].any()
    qq, qs = orc.sage_quantize_q(q, H, D)
    assert np.all(np.abs(qq.astype(np.float64) * qs[:, None] - q.astype(np.float64)) <= 0.5 * qs[:, None] + 1e-7)
    # mean smoothing leaves softmax unchanged: softmax(q (K - mu)^T) == softmax(q K^T)
    s1 = q[0].astype(np.float64) @ k[0, :N].astype(np.float64).T
    s2 = q[0].astype(np.float64) @ (k[0, :N].astype(np.float64) - mean[0].astype(np.float64)).T
    from scipy.special import softmax
    assert np.max(np.abs(softmax(s1) - softmax(s2))) < 1e-12
    got = orc.sage_decode(qq, qs, kq, ks, v, H, Hkv, D, cap, N).reshape(H, D).astype(np.float64)
    # against the int8 model evaluated in float64
    for h in range(H):
        s = (qq[h].astype(np.float64) @ kq[h // 4, :N].astype(np.float64).T) * qs[h] * \
            np.repeat(ksf[h // 4], 32)[:N] / np.sqrt(D)
        want = softmax(s) @ v[h // 4, :N].astype(np.float64)
        assert np.max(np.abs(got[h] - want)) < 1e-3
    # and the quantisation error against f16 SDPA on the unquantised tensors stays small
    full = rm.gqa_decode_f64(q, k, v, H, Hkv, D, N)
    assert np.max(np.abs(got - full)) < 5e-2


# ---------------------------------------------------------------------------------------- bf16 element mode (extension)

def test_bf16_conversions_match_an_independent_implementation():
    """orc_f32_to_bf16 / orc_bf16_to_f32 against torch's bfloat16 (round to nearest even), incl. ties, subnormals,
    infinities and NaN."""
    import torch

    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.normal(size=4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, size=4000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf, 1e-40, -1e-45], np.float32),
        (np.arange(0x3F800000, 0x3F800000 + 0x30000, 0x800, dtype=np.uint32)).view(np.float32),  # ties around 1.0
    ])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([orc.lib().orc_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    assert np.isnan(orc.lib().orc_bf16_to_f32(orc.lib().orc_f32_to_bf16(float("nan"))))
    bits = np.arange(0, 65536, 7, dtype=np.uint16)
    back = np.array([orc.lib().orc_bf16_to_f32(int(b)) for b in bits], np.float32)
    ref = (bits.astype(np.uint32) << 16).view(np.float32)
    finite = ~np.isnan(ref)  # NaN payloads do not survive the trip through a Python float
    assert np.array_equal(back.view(np.uint32)[finite], ref.view(np.uint32)[finite])
    assert np.all(np.isnan(back[~finite]))


def test_bf16_mode_attention_matches_float64_on_the_bf16_inputs():
    """In bf16 mode the same recurrences run on bf16 inputs: decode and prefill against float64 softmax of the
    (exactly representable) bf16 values, to bf16 output rounding."""
    rng = np.random.default_rng(6)
    H, Hkv, D, N, cap = 4, 2, 64, 77, 80
    q = orc.bf16_pack(rng.normal(size=(H, D)))
    k = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    v = orc.bf16_pack(rng.normal(size=(Hkv, cap, D)))
    with orc.bf16_mode():
        out = orc.sdpa_decode(q, k, v, H, Hkv, D, cap, N)
    want = rm.gqa_decode_f64(orc.bf16_unpack(q), orc.bf16_unpack(k), orc.bf16_unpack(v), H, Hkv, D, N)
    got = orc.bf16_unpack(out).reshape(H, D)
    assert np.max(np.abs(got - want)) <= 2.0 ** -8 * max(1.0, float(np.max(np.abs(want))))
    # and f16 mode is restored afterwards
    qh = rng.normal(size=(H, D)).astype(np.float16)
    kh, vh = rng.normal(size=(Hkv, cap, D)).astype(np.float16), rng.normal(size=(Hkv, cap, D)).astype(np.float16)
    assert np.max(np.abs(orc.sdpa_decode(qh, kh, vh, H, Hkv, D, cap, N).reshape(H, D).astype(np.float64)
                         - rm.gqa_decode_f64(qh, kh, vh, H, Hkv, D, N))) <= 2e-3


def test_bf16_mode_kv_prep_rotation_is_rounded_once_to_bf16():
    rng = np.random.default_rng(7)
    H, Hkv, D, T, cap, pos = 4, 2, 32, 3, 16, 5
    qf, kf, vf = (rng.normal(size=(T, n * D)).astype(np.float32) for n in (H, Hkv, Hkv))
    q, k, v = orc.bf16_pack(qf), orc.bf16_pack(kf), orc.bf16_pack(vf)
    cos, sin = orc.rope_tables(1e4, D, cap)
    kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
    with orc.bf16_mode():
        qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, T, pos, cap, rope_mode=0))
    # V is copied bit for bit; rotated values equal the float64 rotation of the bf16 inputs up to one bf16 rounding
    assert np.array_equal(vc[:, pos:pos + T].view(np.uint16),
                          v.reshape(T, Hkv, D).transpose(1, 0, 2).view(np.uint16))
    x = orc.bf16_unpack(q).reshape(T, H, D).astype(np.float64)
    c, s_ = cos[pos:pos + T].astype(np.float64), sin[pos:pos + T].astype(np.float64)
    half = D // 2
    lo = x[..., :half] * c[:, None, :] - x[..., half:] * s_[:, None, :]
    hi = x[..., half:] * c[:, None, :] + x[..., :half] * s_[:, None, :]
    want = np.concatenate([lo, hi], axis=-1).transpose(1, 0, 2)
    got = orc.bf16_unpack(qr).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2.0 ** -8 * max(1.0, float(np.max(np.abs(want))))


# ---------------------------------------------------------------- KV prefix copies and the capacity policy

def test_align_capacity_reference_vectors():
    """The reference's own vectors (src/model/context.rs:318-323)."""
    for c, want in [(0, 128), (1, 128), (127, 128), (128, 128), (129, 256), (200, 256)]:
        assert orc.align_capacity(c) == want


def test_grown_capacity_hand_worked_cases_and_invariants():
    """ensure_kv_capacity (src/model/executor.rs:2354-2382) with the default strategy (initial 2048, factor 2.0,
    src/model/context.rs:42-49), worked by hand; then invariants over a sweep."""
    assert orc.grown_capacity(2048, 2048, 8192) == 2048          # already sufficient
    assert orc.grown_capacity(2048, 2049, 8192) == 4096          # 2048 * 2
    assert orc.grown_capacity(2048, 5000, 8192) == 5120          # max(4096, 5000) = 5000 -> aligned
    assert orc.grown_capacity(4096, 4097, 6000) == 6016          # min(8192, 6000) = 6000 -> aligned past the maximum
    assert orc.grown_capacity(2048, 8193, 8192) == 0             # exceeds max_context_len: InvalidOperation
    assert orc.grown_capacity(2048, 3000, 8192, 0.0) == 8192     # FullReserve
    assert orc.grown_capacity(2048, 2100, 8192, 1.5) == 3072     # (2048 * 1.5) as usize
    assert orc.grown_capacity(1000, 1001, 8192, 1.1) == 1152     # (1000 * 1.1f32) as usize = 1100 -> 1152
    rng = np.random.default_rng(0)
    for _ in range(2000):
        alloc = int(orc.align_capacity(int(rng.integers(1, 20000))))
        mx = int(rng.integers(alloc, 70000))
        req = int(rng.integers(1, mx + 1))
        g = orc.grown_capacity(alloc, req, mx)
        if req <= alloc:
            assert g == alloc
        else:
            assert g % 128 == 0 and g >= req and g <= orc.align_capacity(mx)
            assert g >= min(2 * alloc, mx) and orc.grown_capacity(alloc, min(req + 1, mx), mx) >= g


def test_kv_prefix_copy_is_the_per_head_blit():
    """Brute force over indices: dst[h, p, :] = src[h, p, :] for p < prefix_len, everything else unchanged; and the
    snapshot -> clobber -> restore round trip (src/model/executor.rs:1195-1212, 1296-1318)."""
    rng = np.random.default_rng(1)
    for heads, cs, cd, D, n, dt in [(3, 10, 16, 6, 7, np.float16), (2, 8, 8, 4, 8, np.int8), (1, 5, 9, 3, 0, np.float32)]:
        src = rng.integers(0, 250, size=(heads, cs, D)).astype(dt)
        dst = rng.integers(0, 250, size=(heads, cd, D)).astype(dt)
        want = dst.copy()
        for h in range(heads):
            for p in range(n):
                for d in range(D):
                    want[h, p, d] = src[h, p, d]
        got = dst.copy()
        assert orc.kv_prefix_copy(src, got, n) == 0
        assert np.array_equal(got, want)
    live = rng.normal(size=(4, 32, 8)).astype(np.float16)
    snap = np.zeros((4, 20, 8), np.float16)
    assert orc.kv_prefix_copy(live, snap, 20) == 0
    assert np.array_equal(snap, live[:, :20])
    clob = rng.normal(size=(4, 32, 8)).astype(np.float16)
    cur = clob.copy()
    assert orc.kv_prefix_copy(snap, cur, 20) == 0
    assert np.array_equal(cur[:, :20], live[:, :20]) and np.array_equal(cur[:, 20:], clob[:, 20:])
    assert orc.kv_prefix_copy(live, snap, 21) == -1  # prefix_len exceeds the snapshot's capacity: nothing copied
    assert np.array_equal(snap, live[:, :20])


def test_paged_copy_blocks_index_map():
    rng = np.random.default_rng(2)
    pool = rng.normal(size=(6, 2, 16, 8)).astype(np.float16)
    want = pool.copy()
    want[5] = pool[1]
    want[0] = pool[3]
    got = pool.copy()
    orc.paged_copy_blocks(got, 2, 16, 8, [1, 3, 2, -1, 6, 4], [5, 0, 2, 1, 0, 9])
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- FusedQkv

def test_weight_index_layouts():
    """Row-major is row*K + k; the canonical layout is a bijection onto [0, N*K) that keeps each 32-feature block of a
    row contiguous and places block kb of row n at 32*(n + kb*N) (src/compound/stages/layout.rs:95-100,
    src/metals/gemv/qkv_project.metal:83-96)."""
    K, N = 96, 7
    seen = set()
    for n in range(N):
        for k in range(K):
            assert orc.weight_index(0, n, k, K, N) == n * K + k
            i = orc.weight_index(1, n, k, K, N)
            assert i == (k & 31) + (n << 5) + (k & ~31) * N  # the kernel's own fast form for weights_per_block = 32
            seen.add(i)
    assert seen == set(range(N * K))
    w = np.arange(N * K, dtype=np.float32).reshape(N, K).astype(np.float16)
    c = orc.to_canonical(w)
    assert np.array_equal(c.reshape(K // 32, N, 32)[1, 3], w[3, 32:64])


@pytest.mark.parametrize("K,N,NK,m,norm,bias", [(1024, 1024, 128, 1, True, True), (64, 40, 24, 3, True, False),
                                                 (96, 16, 8, 2, False, True)])
def test_fused_qkv_vs_float64(K, N, NK, m, norm, bias):
    """Against float64 matrix products on the same f16-rounded normalised input, with the reference test's data
    distributions (tests/qkv_parity_f16.rs:100-118); both layouts give the same bits."""
    rng = np.random.default_rng(K + m)
    x = rng.uniform(-1, 1, (m, K)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, K).astype(np.float16)
    ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
    bs = [rng.uniform(-0.1, 0.1, n).astype(np.float16) for n in (N, NK, NK)]
    got = orc.fused_qkv(x, *ws, gamma=g if norm else None, biases=bs if bias else None)
    got_c = orc.fused_qkv(x, *[orc.to_canonical(w) for w in ws], gamma=g if norm else None, biases=bs if bias else None, layout=1)
    xf = x.astype(np.float32)
    if norm:
        inv = (1.0 / np.sqrt((xf.astype(np.float64) ** 2).sum(1, keepdims=True) / K + 1e-6)).astype(np.float32)
        xn = (xf * inv * g.astype(np.float32)).astype(np.float16).astype(np.float64)
    else:
        xn = xf.astype(np.float64)
    for o, oc, w, b in zip(got, got_c, ws, bs):
        assert np.array_equal(o, oc)
        ref = xn @ w.astype(np.float64).T + (b.astype(np.float64) if bias else 0.0)
        ulp = np.maximum(np.abs(ref), 2.0 ** -10) * 2.0 ** -10
        assert np.all(np.abs(o.astype(np.float64) - ref) <= 1.5 * ulp + 1e-4)
    # identity weights: the projection returns the normalised input
    eye = np.eye(K, dtype=np.float16)
    q, _, _ = orc.fused_qkv(x, eye, eye[:8], eye[:8], gamma=g if norm else None)
    assert np.array_equal(q.astype(np.float64), xn)


@pytest.mark.parametrize("m,n,k,alpha,beta", [(1, 128, 128, 1.0, 0.0), (1, 256, 256, 0.5, 0.0), (2, 40, 96, 1.0, 1.0), (3, 16, 64, 0.25, 0.75)])
def test_matmul_gemv_vs_float64_and_linearity(m, n, k, alpha, beta):
    """alpha * x.W^T + bias + beta * residual against float64 (shapes and alpha of tests/gemv_v2_parity.rs:244-301);
    both layouts give the same bits; the residual term is linear in beta (beta = 0 drops it exactly)."""
    rng = np.random.default_rng(n + k)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    w = rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16)
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    got = orc.matmul_gemv(x, w, b, c, 0, 32, alpha, beta)
    assert np.array_equal(got, orc.matmul_gemv(x, orc.to_canonical(w), b, c, 1, 32, alpha, beta))
    ref = alpha * (x.astype(np.float64) @ w.astype(np.float64).T) + b.astype(np.float64) + beta * c.astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= 1.5 * np.maximum(np.abs(ref), 2.0 ** -10) * 2.0 ** -10 + 1e-4)
    assert np.array_equal(orc.matmul_gemv(x, w, b, c, 0, 32, alpha, 0.0), orc.matmul_gemv(x, w, b, None, 0, 32, alpha, 0.0))
    assert np.array_equal(orc.matmul_gemv(x, np.zeros_like(w), None, c, 0, 32, 1.0, 1.0), c)  # zero weights: out = residual


def test_q8_0_projections_vs_float64_on_dequantised_weights():
    """The Q8 recurrence (tests/gemv_v2_parity.rs:82-125: per 8 weights an integer-valued partial sum times the block
    scale) against float64 products with the dequantised weights w8 * scale; the quantiser's round trip error is
    within half a step of each block's scale; both layouts give the same bits."""
    rng = np.random.default_rng(9)
    m, n, k = 3, 40, 96
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    w = rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16)
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    w8, sc = orc.quantize_q8_0(w)
    deq = w8.astype(np.float64).reshape(n, k // 32, 32) * sc.astype(np.float64)[:, :, None]
    assert np.all(np.abs(deq.reshape(n, k) - w.astype(np.float64)) <= 0.5 * np.repeat(sc.astype(np.float64), 32, axis=1) + 1e-6)
    got = orc.matmul_gemv_q8(x, w8, sc, b, c, 0, 32, 0.5, 0.75)
    assert np.array_equal(got, orc.matmul_gemv_q8(x, orc.to_canonical(w8), sc, b, c, 1, 32, 0.5, 0.75))
    ref = 0.5 * (x.astype(np.float64) @ deq.reshape(n, k).T) + b.astype(np.float64) + 0.75 * c.astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= 1.5 * np.maximum(np.abs(ref), 2.0 ** -10) * 2.0 ** -10 + 1e-4)
    # unit scales and small integers: the result is the exact integer dot product
    xi = rng.integers(-3, 4, (1, 64)).astype(np.float16)
    wi = rng.integers(-5, 6, (8, 64)).astype(np.int8)
    one = np.ones((8, 2), np.float16)
    assert np.array_equal(orc.matmul_gemv_q8(xi, wi, one).astype(np.int64), xi.astype(np.int64) @ wi.astype(np.int64).T)
    # fused QKV = the same projections on the normalised input
    g = rng.uniform(0.5, 1.5, k).astype(np.float16)
    q, kk, v = orc.fused_qkv_q8(x, [w8, w8[:8], w8[8:16]], [sc, sc[:8], sc[8:16]], gamma=g)
    xf = x.astype(np.float32)
    inv = (1.0 / np.sqrt((xf.astype(np.float64) ** 2).sum(1, keepdims=True) / k + 1e-6)).astype(np.float32)
    xn = (xf * inv * g.astype(np.float32)).astype(np.float16)
    assert np.array_equal(q, orc.matmul_gemv_q8(xn, w8, sc))
    assert np.array_equal(kk, orc.matmul_gemv_q8(xn, w8[:8], sc[:8])) and np.array_equal(v, orc.matmul_gemv_q8(xn, w8[8:16], sc[8:16]))


# ---------------------------------------------------------------- Q4_0 weights

def test_q4_0_nibble_order_is_the_loaders_adjacent_pairs():
    """GGML stores weight j in the low and weight j + 16 in the high nibble of byte j of a block; the reference's loader
    (and its test helper, tests/gemm_v2_parity.rs:141-196) de-interleaves that into adjacent pairs, which is the order
    policy_q4_0.metal:70-98 reads. The transform below is that helper's loop; packing adjacent elements directly must
    give the same bytes, and the oracle's reader must return the original integers."""
    rng = np.random.default_rng(40)
    q = rng.integers(-8, 8, 32).astype(np.int8)
    u = (q + 8).astype(np.uint8)
    ggml = np.array([(u[16 + j] << 4) | u[j] for j in range(16)], np.uint8)
    block = np.zeros(16, np.uint8)
    for i in range(8):
        b0, b1 = ggml[2 * i], ggml[2 * i + 1]
        block[i] = ((b1 & 0x0F) << 4) | (b0 & 0x0F)
        block[i + 8] = (b1 & 0xF0) | (b0 >> 4)
    assert np.array_equal(block, orc.pack_q4_0(q))
    assert np.array_equal(orc.unpack_q4_0(block), q)
    assert np.array_equal(orc.unpack_q4_0(np.array([0x00, 0xFF, 0x80, 0x7F], np.uint8)),
                          np.array([-8, -8, 7, 7, -8, 0, 7, -1], np.int8))


def test_q4_0_quantiser_and_dot_against_float64():
    """scale = max|w| / 7, q = round(w / scale) in [-8, 7] (tests/gemm_v2_parity.rs:112-166); the dot product of the
    oracle (the Q8 block recurrence on the unpacked integers) equals the float64 product with the dequantised weights."""
    rng = np.random.default_rng(41)
    n, k, m = 24, 96, 3
    w = rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    q, sc = orc.quantize_q4_0(w)
    assert q.min() >= -8 and q.max() <= 7
    blocks = w.astype(np.float32).reshape(n, k // 32, 32)
    assert np.array_equal(sc, (np.abs(blocks).max(axis=2) / np.float32(7.0)).astype(np.float16))
    amax = np.abs(blocks).argmax(axis=2)  # the largest weight of a block maps to +-7
    assert np.all(np.abs(np.take_along_axis(q.reshape(n, k // 32, 32), amax[:, :, None], axis=2)) == 7)
    deq = q.reshape(n, k // 32, 32).astype(np.float64) * sc.astype(np.float64)[:, :, None]
    assert np.max(np.abs(deq.reshape(n, k) - w.astype(np.float64))) <= 0.5 * float(sc.astype(np.float64).max()) * 1.01
    for layout in (0, 1):
        stored = orc.to_canonical(q) if layout == 1 else q.reshape(-1)
        got = orc.matmul_gemv_q8(x, orc.unpack_q4_0(orc.pack_q4_0(stored)), sc, layout=layout)
        want = x.astype(np.float64) @ deq.reshape(n, k).T
        assert np.max(np.abs(got.astype(np.float64) - want)) <= 2.0 ** -10 * np.maximum(np.abs(want), 2.0 ** -10).max() + 1e-5


def test_dequantize_blocks_is_one_rounding_of_the_exact_product():
    """The GEMM form of block-quantised weights (src/metals/mma/tile_loader.metal:100-120; CPU reference of
    tests/gemm_v2_parity.rs:295-350): w = f16(q * scale). q * scale is exact in f32 and f64, so the f32 route of
    orc.dequantize_blocks must equal the float64 product rounded once - for Q8_0 and Q4_0 integers, subnormal scales
    included."""
    rng = np.random.default_rng(43)
    n, k = 8, 128
    for lo, hi in ((-127, 128), (-8, 8)):
        q = rng.integers(lo, hi, (n, k)).astype(np.int8)
        sc = rng.uniform(0, 0.02, (n, k // 32)).astype(np.float16)
        sc[0, 0], sc[1, 1], sc[2, 2] = np.float16(6e-8), np.float16(3e-5), np.float16(0)  # subnormal, near the normal edge, zero
        got = orc.dequantize_blocks(q, sc)
        want = (q.astype(np.float64).reshape(n, k // 32, 32) * sc.astype(np.float64)[:, :, None]).reshape(n, k).astype(np.float16)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
