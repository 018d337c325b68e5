"""GPU parity: FusedQkv (RMSNorm -> Q/K/V projections, F16 weights) against the oracle's restatement of the
reference test's CPU helpers (tests/qkv_parity_f16.rs:17-72). The reference accepts |diff| < 0.1 there; the bar
here is two f16 units in the last place of the expected value (f32 sums of k_dim products in another order, rounded
once), plus the f16 rounding of a normalised input that sits on a rounding boundary (rsqrt against 1/sqrt)."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, ctx

pytestmark = pytest.mark.gpu


def _data(rng, K, N, NK, m):
    # distributions of tests/qkv_parity_f16.rs:100-118
    x = rng.uniform(-1, 1, (m, K)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, K).astype(np.float16)
    ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
    bs = [rng.uniform(-0.1, 0.1, n).astype(np.float16) for n in (N, NK, NK)]
    return x, g, ws, bs


def _paths(m):
    """(GEMM threshold, GEMM variant) pairs to run a shape with: the library's defaults, plus - for a few input rows -
    the GEMM forced, - for short chunks - the passes of 16 rows over the weight stream forced, and - wherever the GEMM
    runs - each of its kernels (operand tiles through registers, straight into LDS in steps of 64 or of 32 features)."""
    if m == 1:
        return [(0, 0)]
    if m < 12:
        return [(0, 0), (1, 0), (1, 1)]
    if m <= 64:
        return [(0, 0), (0, 1), (0, 2), (0, 3), (1 << 30, 0)]
    return [(0, 0), (0, 1), (0, 2), (0, 3)]


def _gemm_runs(m, min_m):
    """Whether the library takes the GEMM for m input rows under the threshold override min_m (0 = its default of 12).
    Block-quantised weights then follow the reference GEMM's arithmetic (f16(q * scale) weights, then the F16 product,
    src/metals/mma/tile_loader.metal:100-120), the weight-stream kernel the GEMV policies' (block sums times scale)."""
    return m >= (12 if min_m == 0 else min_m)


def _close(got, want, K):
    g, w = got.astype(np.float64), want.astype(np.float64)
    ulp = np.maximum(np.abs(w), 2.0 ** -10) * 2.0 ** -10
    # the f16 rounding of the normalised input may differ in isolated elements (rsqrt vs 1/sqrt, another order of the
    # sum of squares): each moves every sum of its row by one input ulp (2^-9 for 2 <= |x| < 4) times |w| <= 0.1, and
    # with hundreds of input rows of thousands of features a row sees up to three or four of them (measured: 4.4e-4
    # over 256 x 5120 outputs, 3.1e-4 over 16 x 5120; without the norm the same shapes stay within 6e-6 of 2 ulps)
    slack = 8 * 2.0 ** -10 * 0.1
    return bool(np.all(np.abs(g - w) <= 2 * ulp + slack))


@pytest.mark.parametrize("K,N,NK,m,norm,bias,layout", [
    (1024, 1024, 128, 1, True, True, 0),      # the reference test's shape (tests/qkv_parity_f16.rs:92-95), row-major
    (1024, 1024, 128, 1, True, True, 1),      # same, canonical blocked weights
    (3072, 3072, 1024, 1, True, False, 1),    # Llama-3.2-3B decode
    (896, 896, 128, 1, True, True, 1),        # Qwen2.5-0.5B (biases)
    (2048, 2048, 256, 1, False, False, 1),    # no RMSNorm
    (3072, 3072, 1024, 5, True, False, 1),    # a few tokens
    (896, 896, 128, 32, True, True, 1),       # a default prefill chunk: split-K GEMM, and two passes of 16 input rows
    (896, 896, 128, 17, True, True, 0),
    (64, 40, 24, 3, True, True, 1),           # rows that do not fill tiles, tiles that straddle the three matrices
    (8192, 256, 64, 2, True, False, 1),       # long rows: more units than one request batch
    # many input rows: the tiled GEMM (128 x 128 output tiles, 64 features per step)
    (896, 896, 128, 64, True, True, 1),       # an input tile half empty
    (896, 896, 128, 200, True, True, 0),      # row-major weights; 896 = 7 tiles, 200 = 2 tiles of input rows, ragged
    (3072, 3072, 1024, 256, True, False, 1),  # Llama-3.2-3B, a 256-token prefill chunk
    (1056, 200, 72, 130, True, True, 1),      # k_dim = 16.5 steps; weight rows that do not fill tiles
    (1056, 200, 72, 130, False, True, 0),
    (64, 40, 20, 70, True, True, 1),          # output rows that are not multiples of 8: element-wise stores
    (2048, 2048, 256, 512, False, False, 1),  # the largest chunk the reference's prefill takes, no norm
])
def test_fused_qkv_equals_oracle(K, N, NK, m, norm, bias, layout):
    announce("fused qkv", K, N, NK, m, norm, bias, layout)
    f = ctx()
    rng = np.random.default_rng(K + N + m)
    x, g, ws, bs = _data(rng, K, N, NK, m)
    want = orc.fused_qkv(x, *ws, gamma=g if norm else None, biases=bs if bias else None, layout=0)
    dev_w = [f.array(orc.to_canonical(w) if layout == 1 else w.reshape(-1)) for w in ws]
    dx, dg = f.array(x), f.array(g)
    db = [f.array(b) for b in bs]
    outs = [f.zeros((m, n)) for n in (N, NK, NK)]
    # from 12 input rows on the library runs the GEMM; short chunks are also forced through the passes of 16 rows over
    # the weight stream, and shapes of a few rows through the GEMM
    gemm_bits = None  # the GEMM kernels share tiling, step order and split points: their outputs are bit-equal
    try:
        for min_m, variant in _paths(m):
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            for o in outs:
                o.upload(np.zeros(o.shape, np.float16))
            f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), outs[0].arg(), outs[1].arg(), outs[2].arg(),
                        K, N, NK, m, gamma=dg.arg() if norm else None, biases=[b.arg() for b in db] if bias else None, layout=layout)
            got_all = [o.download() for o in outs]
            for got, w, name in zip(got_all, want, "qkv"):
                assert np.all(np.isfinite(got)), (name, min_m, variant)
                assert _close(got, w, K), (name, min_m, variant, float(np.max(np.abs(got.astype(np.float64) - w.astype(np.float64)))))
            if _gemm_runs(m, min_m):
                bits_now = [g.view(np.uint16).copy() for g in got_all]
                if gemm_bits is None:
                    gemm_bits = bits_now
                else:
                    assert all(np.array_equal(a, b) for a, b in zip(gemm_bits, bits_now)), (min_m, variant)
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    for b in dev_w + [dx, dg] + db + outs:
        b.free()


def test_fused_qkv_feeds_kv_prep_and_decode():
    """The step before the path and the path: FusedQkv -> fused RoPE + append + decode equals the oracle's chain."""
    announce("fused qkv -> decode step")
    f = ctx()
    rng = np.random.default_rng(77)
    H, Hkv, D, K, cap, pos = 8, 2, 64, 512, 256, 100
    x, g, ws, _ = _data(rng, K, H * D, Hkv * D, 1)
    kc = rng.normal(size=(Hkv, cap, D)).astype(np.float16)
    vc = rng.normal(size=(Hkv, cap, D)).astype(np.float16)
    cos, sin = fa.rope_tables(1e4, D, cap)
    q, k, v = orc.fused_qkv(x, *ws, gamma=g)
    kc_w, vc_w = kc.copy(), vc.copy()
    qr = orc.kv_prep_fused(q, k, v, kc_w, vc_w, cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=0))
    want = orc.sdpa_decode(qr[:, 0].copy(), kc_w, vc_w, H, Hkv, D, cap, pos + 1)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dx, dg, dkc, dvc, dcos, dsin = f.array(x), f.array(g), f.array(kc), f.array(vc), f.array(cos), f.array(sin)
    dq, dk, dv, dout = f.zeros((1, H * D)), f.zeros((1, Hkv * D)), f.zeros((1, Hkv * D)), f.zeros((1, H * D))
    f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), dq.arg(), dk.arg(), dv.arg(), K, H * D, Hkv * D, 1,
                gamma=dg.arg())
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NEOX)
    f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, dkc.arg(), dvc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p)
    got = dout.download().reshape(H, D).astype(np.float64)
    assert float(np.max(np.abs(got - want.reshape(H, D).astype(np.float64)))) <= 4e-3  # projection ulps carried through
    for b in dev_w + [dx, dg, dkc, dvc, dcos, dsin, dq, dk, dv, dout]:
        b.free()


def test_fused_qkv_errors():
    announce("fused qkv errors")
    f = ctx()
    K, N, NK = 64, 32, 16
    x, wq, wk, wv = f.zeros((1, K)), f.zeros((N * K,)), f.zeros((NK * K,)), f.zeros((NK * K,))
    oq, ok, ov = f.zeros((1, N)), f.zeros((1, NK)), f.zeros((1, NK))
    args = lambda: (x.arg(), wq.arg(), wk.arg(), wv.arg(), oq.arg(), ok.arg(), ov.arg())  # noqa: E731
    f.fused_qkv(*args(), K, N, NK, 1)  # fine
    w8 = f.zeros((N * K,), np.int8)
    with pytest.raises(fa.FoundryError) as e:  # int8 (Q8_0) weights need their scales
        f.fused_qkv(x.arg(), w8.arg(), wk.arg(), wv.arg(), oq.arg(), ok.arg(), ov.arg(), K, N, NK, 1)
    assert e.value.variant == "InputNotFound"
    sc = f.zeros((N, K // 32))
    with pytest.raises(fa.FoundryError) as e:  # mixed policies: the reference falls back to three projections
        f.fused_qkv(x.arg(), w8.arg(), wk.arg(), wv.arg(), oq.arg(), ok.arg(), ov.arg(), K, N, NK, 1,
                    scales=(sc.arg(), fa.TensorArg(), fa.TensorArg()))
    assert e.value.variant == "UnsupportedDtype"
    wq4 = wq.arg(dtype=4)  # Q4_1: not built
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(x.arg(), wq4, wk.arg(), wv.arg(), oq.arg(), ok.arg(), ov.arg(), K, N, NK, 1)
    assert e.value.variant == "UnsupportedDtype"
    sc.free()
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(*args(), 48, N, NK, 1)
    assert e.value.variant in ("OperationNotSupported", "InvalidShape")
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(*args(), K, N, NK, 1, weights_per_block=64)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(*args(), K, N + 1, NK, 1)
    assert e.value.variant == "InvalidShape"
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(*args(), K, N, NK, 2)
    assert e.value.variant == "InvalidShape"
    b = f.zeros((N,))
    with pytest.raises(fa.FoundryError) as e:  # bias_q without bias_k / bias_v
        f.fused_qkv(*args(), K, N, NK, 1, biases=(b.arg(), fa.TensorArg(), fa.TensorArg()))
    assert e.value.variant == "InputNotFound"
    t = x.arg()
    t.buffer = None
    with pytest.raises(fa.FoundryError) as e:
        f.fused_qkv(t, wq.arg(), wk.arg(), wv.arg(), oq.arg(), ok.arg(), ov.arg(), K, N, NK, 1)
    assert e.value.variant == "InputNotFound"
    f.synchronize()
    for z in (x, wq, wk, wv, oq, ok, ov, w8, b):
        z.free()


@pytest.mark.parametrize("K,N,NK,m,norm,bias,layout", [
    (3072, 3072, 1024, 32, True, False, 1),   # Llama-3.2-3B, the reference's default prefill chunk
    (3072, 3072, 1024, 17, True, True, 0),    # row-major weights, a ragged second half of the input rows
    (2048, 2048, 256, 12, False, True, 1),    # no RMSNorm, the fewest rows the kernel takes by default
    (2048, 3000, 40, 31, True, True, 1),      # weight rows that do not fill the workgroups' tiles, tiles across the matrices
])
def test_fused_qkv_chunk_of_up_to_32_rows_in_one_launch(K, N, NK, m, norm, bias, layout):
    """12 to 32 input rows against F16 weights of 2048 or 3072 features run as ONE weight-stream launch (each wave keeps
    its slice of the input rows in registers); an explicit GEMM threshold sends the same call through the GEMM. Both
    against the oracle, and the profiler's launch counts say which kernel ran."""
    announce("fused qkv, chunk in one launch", K, N, NK, m, norm, bias, layout)
    f = ctx()
    rng = np.random.default_rng(K + N + m + 7)
    x, g, ws, bs = _data(rng, K, N, NK, m)
    want = orc.fused_qkv(x, *ws, gamma=g if norm else None, biases=bs if bias else None, layout=0)
    dev_w = [f.array(orc.to_canonical(w) if layout == 1 else w.reshape(-1)) for w in ws]
    dx, dg = f.array(x), f.array(g)
    db = [f.array(b) for b in bs]
    outs = [f.zeros((m, n)) for n in (N, NK, NK)]
    try:
        for min_m, kernel in ((0, "fused_qkv_rows32_kernel"), (12, "fused_qkv_gemm_kernel")):
            f.set_gemm_min_m(min_m)
            for o in outs:
                o.upload(np.zeros(o.shape, np.float16))
            f.profile_reset()
            f.profile_enable(True)
            f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), outs[0].arg(), outs[1].arg(), outs[2].arg(),
                        K, N, NK, m, gamma=dg.arg() if norm else None, biases=[b.arg() for b in db] if bias else None, layout=layout)
            f.synchronize()
            assert f.profile_query(kernel)[0] == 1, (kernel, min_m)
            f.profile_enable(False)
            for o, w, name in zip(outs, want, "qkv"):
                got = o.download()
                assert np.all(np.isfinite(got)), (name, min_m)
                assert _close(got, w, K), (name, min_m, float(np.max(np.abs(got.astype(np.float64) - w.astype(np.float64)))))
    finally:
        f.profile_enable(False)
        f.set_gemm_min_m()
    for b in dev_w + [dx, dg] + db + outs:
        b.free()


@pytest.mark.parametrize("m,n,k,canonical,bias,resid,alpha,beta", [
    (32, 3072, 3072, True, False, True, 1.0, 1.0),    # Llama-3.2-3B o_proj of a default prefill chunk
    (20, 2048, 2048, False, True, True, 0.25, 0.75),  # row-major weights, bias, scaled residual
])
def test_matmul_chunk_of_up_to_32_rows_in_one_launch(m, n, k, canonical, bias, resid, alpha, beta):
    announce("matmul, chunk in one launch", m, n, k, canonical, bias, resid, alpha, beta)
    f = ctx()
    rng = np.random.default_rng(m + n + k + 7)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    w = rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16)
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    want = orc.matmul_gemv(x, w, b if bias else None, c if resid else None, 0, 32, alpha, beta)
    dx, dw = f.array(x), f.array(orc.to_canonical(w) if canonical else w.reshape(-1))
    db, dc, out = f.array(b), f.array(c), f.zeros((m, n))
    try:
        for min_m, kernel in ((0, "matmul_rows32_kernel"), (12, None)):
            f.set_gemm_min_m(min_m)
            out.upload(np.zeros((m, n), np.float16))
            f.profile_reset()
            f.profile_enable(True)
            f.matmul(dx.arg(), dw.arg(), out.arg(), m, n, k, bias=db.arg() if bias else None, c=dc.arg() if resid else None,
                     transpose_b=not canonical, alpha=alpha, beta=beta)
            f.synchronize()
            assert f.profile_query("matmul_rows32_kernel")[0] == (1 if kernel else 0), min_m
            f.profile_enable(False)
            got = out.download()
            g, wv = got.astype(np.float64), want.astype(np.float64)
            assert np.all(np.abs(g - wv) <= 2 * np.maximum(np.abs(wv), 2.0 ** -10) * 2.0 ** -10 + 1e-4), (min_m, float(np.max(np.abs(g - wv))))
    finally:
        f.profile_enable(False)
        f.set_gemm_min_m()
    for z in (dx, dw, db, dc, out):
        z.free()


# ---------------------------------------------------------------- MatMul (the o_proj consumer of attn_out)

@pytest.mark.parametrize("m,n,k,canonical,bias,resid,alpha,beta", [
    (1, 128, 128, False, False, False, 1.0, 0.0),    # tests/gemv_v2_parity.rs:244-254
    (1, 256, 256, False, False, False, 0.5, 0.0),    # :280-289 (alpha)
    (1, 128, 512, False, True, False, 1.0, 0.0),     # :303-330 (k > n, bias)
    (1, 4096, 4096, False, False, False, 1.0, 0.0),  # :406-416
    (1, 3072, 3072, True, False, True, 1.0, 1.0),    # Llama-3.2-3B o_proj: canonical weights, residual, beta 1
    (1, 896, 896, True, True, True, 1.0, 1.0),
    (5, 3072, 3072, True, False, True, 1.0, 1.0),
    (32, 896, 896, False, False, True, 0.25, 0.75),  # a prefill chunk through the same path
    (3, 40, 64, True, True, True, 1.0, 0.5),
    # many input rows: the tiled GEMM
    (256, 3072, 3072, True, False, True, 1.0, 1.0),  # o_proj of a 256-token prefill chunk
    (100, 896, 896, False, True, True, 0.25, 0.75),
    (77, 40, 96, True, True, True, 1.0, 0.5),
])
def test_matmul_gemv_equals_oracle(m, n, k, canonical, bias, resid, alpha, beta):
    announce("matmul", m, n, k, canonical, bias, resid, alpha, beta)
    f = ctx()
    rng = np.random.default_rng(m + n + k)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    w = rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16)
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    want = orc.matmul_gemv(x, w, b if bias else None, c if resid else None, 0, 32, alpha, beta)
    dx, dw = f.array(x), f.array(orc.to_canonical(w) if canonical else w.reshape(-1))
    db, dc, out = f.array(b), f.array(c), f.zeros((m, n))
    try:
        for min_m, variant in _paths(m):  # the GEMM kernels and the passes over the weight stream, as in the FusedQkv test
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            out.upload(np.zeros((m, n), np.float16))
            f.matmul(dx.arg(), dw.arg(), out.arg(), m, n, k, bias=db.arg() if bias else None, c=dc.arg() if resid else None,
                     transpose_b=not canonical, alpha=alpha, beta=beta)
            got = out.download()
            # the reference's own bar is 1e-3 * sqrt(k) (tests/gemv_v2_parity.rs:214); here: 2 f16 ulps of the expected value
            g, wv = got.astype(np.float64), want.astype(np.float64)
            assert np.all(np.abs(g - wv) <= 2 * np.maximum(np.abs(wv), 2.0 ** -10) * 2.0 ** -10 + 1e-4), (min_m, variant, float(np.max(np.abs(g - wv))))
            assert float(np.max(np.abs(g - wv))) <= 1e-3 * np.sqrt(k)
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    for z in (dx, dw, db, dc, out):
        z.free()


def test_matmul_errors():
    announce("matmul errors")
    f = ctx()
    a, b, o = f.zeros((1, 64)), f.zeros((32 * 64,)), f.zeros((1, 32))
    f.matmul(a.arg(), b.arg(), o.arg(), 1, 32, 64)
    with pytest.raises(fa.FoundryError) as e:
        f.matmul(a.arg(), b.arg(), o.arg(), 1, 32, 64, transpose_a=True)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:
        f.matmul(a.arg(), b.arg(), o.arg(), 1, 32, 64, activation=1)
    assert e.value.variant == "OperationNotSupported"
    with pytest.raises(fa.FoundryError) as e:
        f.matmul(a.arg(), b.arg(), o.arg(), 1, 33, 64)
    assert e.value.variant == "InvalidShape"
    b8 = f.zeros((32 * 64,), np.int8)
    with pytest.raises(fa.FoundryError) as e:  # Q8_0 weights without scales
        f.matmul(a.arg(), b8.arg(), o.arg(), 1, 32, 64)
    assert e.value.variant == "InputNotFound"
    with pytest.raises(fa.FoundryError) as e:  # Q4_1: not built
        f.matmul(a.arg(), b.arg(dtype=4), o.arg(), 1, 32, 64)
    assert e.value.variant == "UnsupportedDtype"
    f.synchronize()
    for z in (a, b, o, b8):
        z.free()


# ---------------------------------------------------------------- Q8_0 weights

@pytest.mark.parametrize("K,N,NK,m,norm,bias,layout", [
    (1024, 1024, 128, 1, True, True, 1),
    (3072, 3072, 1024, 1, True, False, 1),   # Llama-3.2-3B decode
    (896, 896, 128, 5, True, True, 1),
    (896, 896, 128, 20, False, True, 0),     # row-major; the split-K GEMM, and two passes of input rows
    (64, 40, 24, 3, True, True, 1),
    (896, 896, 128, 32, True, True, 1),      # a default prefill chunk
    (3072, 3072, 1024, 200, True, False, 1), # Llama-3.2-3B, ragged input tiles
    (1056, 200, 72, 130, True, True, 0),     # k_dim = 16.5 steps, weight rows that do not fill tiles, row-major
    (1056, 200, 72, 130, False, True, 1),
    (64, 40, 20, 70, True, True, 1),         # element-wise stores
])
def test_fused_qkv_q8_equals_oracle(K, N, NK, m, norm, bias, layout):
    announce("fused qkv q8", K, N, NK, m, norm, bias, layout)
    f = ctx()
    rng = np.random.default_rng(K + N + m + 1)
    x, g, ws, bs = _data(rng, K, N, NK, m)
    q8 = [orc.quantize_q8_0(w) for w in ws]
    want_stream = orc.fused_qkv_q8(x, [q for q, _ in q8], [s for _, s in q8], gamma=g if norm else None, biases=bs if bias else None)
    want_gemm = orc.fused_qkv(x, *[orc.dequantize_blocks(q, s) for q, s in q8], gamma=g if norm else None,
                              biases=bs if bias else None, layout=0)
    dev_w = [f.array(orc.to_canonical(q) if layout == 1 else q.reshape(-1)) for q, _ in q8]
    dev_s = [f.array(s) for _, s in q8]
    dx, dg = f.array(x), f.array(g)
    db = [f.array(b) for b in bs]
    outs = [f.zeros((m, n)) for n in (N, NK, NK)]
    try:
        for min_m, variant in _paths(m):
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            for o in outs:
                o.upload(np.zeros(o.shape, np.float16))
            f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), outs[0].arg(), outs[1].arg(), outs[2].arg(),
                        K, N, NK, m, gamma=dg.arg() if norm else None, biases=[b.arg() for b in db] if bias else None, layout=layout,
                        scales=[s.arg() for s in dev_s])
            for o, w, name in zip(outs, want_gemm if _gemm_runs(m, min_m) else want_stream, "qkv"):
                got = o.download()
                assert np.all(np.isfinite(got)), (name, min_m, variant)
                assert _close(got, w, K), (name, min_m, variant, float(np.max(np.abs(got.astype(np.float64) - w.astype(np.float64)))))
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    for b in dev_w + dev_s + [dx, dg] + db + outs:
        b.free()


@pytest.mark.parametrize("m,n,k,canonical,bias,resid,alpha,beta", [
    (1, 128, 128, False, False, False, 1.0, 0.0),
    (1, 3072, 3072, True, False, True, 1.0, 1.0),   # o_proj
    (1, 256, 256, True, True, False, 0.5, 0.0),
    (7, 896, 896, True, True, True, 1.0, 0.5),
    (40, 896, 896, False, True, True, 0.25, 0.75),   # the split-K GEMM, and passes of 16 rows
    (256, 3072, 3072, True, False, True, 1.0, 1.0),  # o_proj of a 256-token prefill chunk
])
def test_matmul_q8_equals_oracle(m, n, k, canonical, bias, resid, alpha, beta):
    announce("matmul q8", m, n, k, canonical, bias, resid, alpha, beta)
    f = ctx()
    rng = np.random.default_rng(m + n + k + 2)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    w8, sc = orc.quantize_q8_0(rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16))
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    want_stream = orc.matmul_gemv_q8(x, w8, sc, b if bias else None, c if resid else None, 0, 32, alpha, beta)
    want_gemm = orc.matmul_gemv(x, orc.dequantize_blocks(w8, sc), b if bias else None, c if resid else None, 0, 32, alpha, beta)
    dx, dw, ds = f.array(x), f.array(orc.to_canonical(w8) if canonical else w8.reshape(-1)), f.array(sc)
    db, dc, out = f.array(b), f.array(c), f.zeros((m, n))
    try:
        for min_m, variant in _paths(m):
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            out.upload(np.zeros((m, n), np.float16))
            f.matmul(dx.arg(), dw.arg(), out.arg(), m, n, k, bias=db.arg() if bias else None, c=dc.arg() if resid else None,
                     transpose_b=not canonical, alpha=alpha, beta=beta, b_scales=ds.arg())
            g, wv = out.download().astype(np.float64), (want_gemm if _gemm_runs(m, min_m) else want_stream).astype(np.float64)
            assert np.all(np.abs(g - wv) <= 2 * np.maximum(np.abs(wv), 2.0 ** -10) * 2.0 ** -10 + 1e-4), (min_m, variant, float(np.max(np.abs(g - wv))))
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    with pytest.raises(fa.FoundryError) as e:  # Q8_0 weights without their scales
        f.matmul(dx.arg(), dw.arg(), out.arg(), m, n, k, transpose_b=not canonical)
    assert e.value.variant == "InputNotFound"
    f.synchronize()
    for z in (dx, dw, ds, db, dc, out):
        z.free()


# ---------------------------------------------------------------- Q4_0 weights

@pytest.mark.parametrize("K,N,NK,m,norm,bias,layout", [
    (1024, 1024, 128, 1, True, True, 1),
    (3072, 3072, 1024, 1, True, False, 1),   # Llama-3.2-3B decode
    (896, 896, 128, 5, True, True, 0),       # row-major bytes
    (64, 40, 24, 3, True, True, 1),
    (896, 896, 128, 20, False, True, 1),     # the split-K GEMM, and two passes of input rows
    (896, 896, 128, 32, True, True, 0),      # a default prefill chunk, row-major bytes
    (3072, 3072, 1024, 200, True, False, 1), # Llama-3.2-3B, ragged input tiles
    (1056, 200, 72, 130, True, True, 0),     # k_dim = 16.5 steps, weight rows that do not fill tiles
    (1056, 200, 72, 130, False, True, 1),
])
def test_fused_qkv_q4_0_equals_oracle(K, N, NK, m, norm, bias, layout):
    """Q4_0 weights (policy_q4_0.metal): the GPU reads the packed bytes, the oracle the integers its own reader makes of
    the same bytes, through the Q8 block recurrence."""
    announce("fused qkv q4_0", K, N, NK, m, norm, bias, layout)
    f = ctx()
    rng = np.random.default_rng(K + N + m + 4)
    x, g, ws, bs = _data(rng, K, N, NK, m)
    q4 = [orc.quantize_q4_0(w) for w in ws]
    packed = [orc.pack_q4_0(orc.to_canonical(q) if layout == 1 else q.reshape(-1)) for q, _ in q4]
    want_stream = orc.fused_qkv_q8(x, [orc.unpack_q4_0(p) for p in packed], [s for _, s in q4], gamma=g if norm else None,
                                   biases=bs if bias else None, layout=layout)
    want_gemm = orc.fused_qkv(x, *[orc.dequantize_blocks(q, s) for q, s in q4], gamma=g if norm else None,
                              biases=bs if bias else None, layout=0)
    dev_w = [f.array(p) for p in packed]
    dev_s = [f.array(s) for _, s in q4]
    dx, dg = f.array(x), f.array(g)
    db = [f.array(b) for b in bs]
    outs = [f.zeros((m, n)) for n in (N, NK, NK)]
    wargs = [w.arg(dims=(n, K), dtype=fa.DTYPE_Q4_0) for w, n in zip(dev_w, (N, NK, NK))]
    try:
        for min_m, variant in _paths(m):
            f.set_gemm_min_m(min_m)
            f.set_gemm_variant(variant)
            for o in outs:
                o.upload(np.zeros(o.shape, np.float16))
            f.fused_qkv(dx.arg(), wargs[0], wargs[1], wargs[2], outs[0].arg(), outs[1].arg(), outs[2].arg(),
                        K, N, NK, m, gamma=dg.arg() if norm else None, biases=[b.arg() for b in db] if bias else None, layout=layout,
                        scales=[s.arg() for s in dev_s])
            for o, w, name in zip(outs, want_gemm if _gemm_runs(m, min_m) else want_stream, "qkv"):
                got = o.download()
                assert np.all(np.isfinite(got)), (name, min_m, variant)
                assert _close(got, w, K), (name, min_m, variant, float(np.max(np.abs(got.astype(np.float64) - w.astype(np.float64)))))
    finally:
        f.set_gemm_min_m()
        f.set_gemm_variant()
    for b in dev_w + dev_s + [dx, dg] + db + outs:
        b.free()


@pytest.mark.parametrize("m,n,k,canonical,bias,resid,alpha,beta", [
    (1, 128, 128, False, False, False, 1.0, 0.0),
    (1, 3072, 3072, True, False, True, 1.0, 1.0),   # o_proj
    (7, 896, 896, True, True, True, 0.5, 0.5),
    (40, 896, 896, False, True, True, 0.25, 0.75),   # the split-K GEMM
    (256, 3072, 3072, True, False, True, 1.0, 1.0),  # o_proj of a 256-token prefill chunk
])
def test_matmul_q4_0_equals_oracle(m, n, k, canonical, bias, resid, alpha, beta):
    announce("matmul q4_0", m, n, k, canonical, bias, resid, alpha, beta)
    f = ctx()
    rng = np.random.default_rng(m + n + k + 5)
    x = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    q, sc = orc.quantize_q4_0(rng.uniform(-0.1, 0.1, (n, k)).astype(np.float16))
    b = rng.uniform(-0.1, 0.1, n).astype(np.float16)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    packed = orc.pack_q4_0(orc.to_canonical(q) if canonical else q.reshape(-1))
    if m >= 12:  # the GEMM's arithmetic
        want = orc.matmul_gemv(x, orc.dequantize_blocks(q, sc), b if bias else None, c if resid else None, 0, 32, alpha, beta)
    else:
        want = orc.matmul_gemv_q8(x, orc.unpack_q4_0(packed), sc, b if bias else None, c if resid else None,
                                  1 if canonical else 0, 32, alpha, beta)
    dx, dw, ds = f.array(x), f.array(packed), f.array(sc)
    db, dc, out = f.array(b), f.array(c), f.zeros((m, n))
    f.matmul(dx.arg(), dw.arg(dims=(n, k), dtype=fa.DTYPE_Q4_0), out.arg(), m, n, k, bias=db.arg() if bias else None,
             c=dc.arg() if resid else None, transpose_b=not canonical, alpha=alpha, beta=beta, b_scales=ds.arg())
    g, wv = out.download().astype(np.float64), want.astype(np.float64)
    assert np.all(np.abs(g - wv) <= 2 * np.maximum(np.abs(wv), 2.0 ** -10) * 2.0 ** -10 + 1e-4), float(np.max(np.abs(g - wv)))
    for z in (dx, dw, ds, db, dc, out):
        z.free()


def test_gemm_path_replays_in_a_graph_with_new_inputs():
    """FusedQkv (split-K GEMM with the norm kernel in front and the finish kernel behind) followed by the o_proj MatMul
    (GEMM with residual), captured once and replayed with other inputs in the same buffers: every replay equals the
    eager result bit for bit (the partial tiles are added in split order) and the oracle to the bar above. The workspace
    for the normalised input and the partial tiles is sized by the eager call before the capture."""
    announce("gemm graph replay")
    f = ctx()
    K, N, NK, m = 512, 512, 128, 40
    rng = np.random.default_rng(99)
    _, g, ws, bs = _data(rng, K, N, NK, m)
    wo = rng.uniform(-0.1, 0.1, (K, N)).astype(np.float16)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dwo, dg = f.array(orc.to_canonical(wo)), f.array(g)
    dx = f.zeros((m, K))
    outs = [f.zeros((m, n)) for n in (N, NK, NK)]
    dproj = f.zeros((m, K))

    def enqueue():
        f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), outs[0].arg(), outs[1].arg(), outs[2].arg(),
                    K, N, NK, m, gamma=dg.arg(), layout=1)
        f.matmul(outs[0].arg(), dwo.arg(), dproj.arg(), m, K, N, c=dx.arg(), transpose_b=False, alpha=1.0, beta=1.0)

    xs = [rng.uniform(-1, 1, (m, K)).astype(np.float16) for _ in range(3)]
    dx.upload(xs[0])
    enqueue()  # eager: sizes the workspace
    f.synchronize()
    f.start_capture()
    enqueue()
    graph = f.end_capture()
    for x in xs:
        dx.upload(x)
        enqueue()
        f.synchronize()
        eager = [o.download().copy() for o in outs] + [dproj.download().copy()]
        for o in outs + [dproj]:
            o.upload(np.zeros(o.shape, np.float16))
        graph.launch()
        f.synchronize()
        got = [o.download() for o in outs] + [dproj.download()]
        for a, b in zip(got, eager):
            assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
        want = orc.fused_qkv(x, *ws, gamma=g, layout=0)
        for a, w in zip(got[:3], want):
            assert _close(a, w, K)
        want_o = orc.matmul_gemv(got[0], wo, None, x, 0, 32, 1.0, 1.0)
        gv, wv = got[3].astype(np.float64), want_o.astype(np.float64)
        assert np.all(np.abs(gv - wv) <= 2 * np.maximum(np.abs(wv), 2.0 ** -10) * 2.0 ** -10 + 1e-4)
    graph.destroy()
    for b in dev_w + [dwo, dg, dx, dproj] + outs:
        b.free()


def test_gemm_workspace_must_be_reserved_before_a_capture():
    """The GEMM form keeps the normalised input (and split-K partial tiles) in the context's workspace; inside a capture
    the workspace cannot grow, so a call that needs more than is reserved fails with a message naming
    fa_ctx_reserve_workspace; after one eager call of the same shape (or that reservation) the capture works."""
    announce("gemm workspace under capture")
    f = fa.Foundry()  # a context of its own: the shared one may already hold a large workspace
    try:
        K, N, NK, m = 8192, 128, 64, 4608  # normalised input: 75.5 MB, more than a new context's 64 MB
        rng = np.random.default_rng(5)
        x = rng.uniform(-1, 1, (m, K)).astype(np.float16)
        g = rng.uniform(0.5, 1.5, K).astype(np.float16)
        ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
        dev_w = [f.array(orc.to_canonical(w)) for w in ws]
        dx, dg = f.array(x), f.array(g)
        outs = [f.zeros((m, n)) for n in (N, NK, NK)]

        def call():
            f.fused_qkv(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), outs[0].arg(), outs[1].arg(), outs[2].arg(),
                        K, N, NK, m, gamma=dg.arg(), layout=1)

        f.start_capture()
        with pytest.raises(fa.FoundryError) as e:
            call()
        assert "fa_ctx_reserve_workspace" in str(e.value)
        f.end_capture().destroy()
        call()  # eagerly, the call sizes the workspace itself (fa_ctx_reserve_workspace with the byte count does the same)
        f.synchronize()
        for o in outs:
            o.upload(np.zeros(o.shape, np.float16))
        f.start_capture()
        call()
        graph = f.end_capture()
        graph.launch()
        f.synchronize()
        rows = slice(m - 24, m)  # the oracle on the last rows
        want = orc.fused_qkv(x[rows], *ws, gamma=g, layout=0)
        for o, w in zip(outs, want):
            assert _close(o.download()[rows], w, K)
        graph.destroy()
    finally:
        f.close()
