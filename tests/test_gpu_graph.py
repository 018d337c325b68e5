"""GPU: captured decode steps (fa_start_capture / fa_end_capture / fa_graph_launch) replay correctly with the
position read from device memory, and per-kernel profiling reports the launches."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, bits, ctx, h16, max_abs

pytestmark = pytest.mark.gpu


def test_captured_decode_steps_replay():
    announce("graph replay")
    f = ctx()
    rng = np.random.default_rng(8)
    H, Hkv, D, cap, layers, start = 24, 8, 128, 512, 3, 300
    steps = 6
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    kc = [h16(rng.normal(size=(Hkv, cap, D))) for _ in range(layers)]
    vc = [h16(rng.normal(size=(Hkv, cap, D))) for _ in range(layers)]
    dkc, dvc = [f.array(x) for x in kc], [f.array(x) for x in vc]
    q, k, v = (h16(rng.normal(size=(layers, n * D))) for n in (H, Hkv, Hkv))
    dq, dk, dv = f.array(q), f.array(k), f.array(v)
    dqr, dout = f.zeros((layers, H * D)), f.zeros((layers, H * D))
    dpos = f.array(np.array([start], np.uint32))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, fa.ROPE_NORMAL)

    def row(buf, i, n):
        return buf.arg((1, n), offset=i * n * 2)

    def enqueue_step():
        for i in range(layers):
            f.kv_prep_fused(row(dq, i, H * D), row(dk, i, Hkv * D), row(dv, i, Hkv * D), row(dqr, i, H * D),
                            dkc[i].arg(), dvc[i].arg(), dcos.arg(), dsin.arg(), p, d_position=dpos)
            f.flash_decode_dyn(row(dqr, i, H * D), dkc[i].arg(), dvc[i].arg(), row(dout, i, H * D), H, D, dpos, 1, cap)
        f.u32_add(dpos, 1, 1)

    f.start_capture()
    with pytest.raises(fa.FoundryError):
        f.start_capture()  # "Capture already active" (src/lib.rs:95-97)
    enqueue_step()
    graph = f.end_capture()
    with pytest.raises(fa.FoundryError):
        f.end_capture()  # "No active capture"
    okc, ovc = [x.copy() for x in kc], [x.copy() for x in vc]
    for t in range(steps):
        graph.launch()
        f.synchronize()  # eager host work between replays
        got = dout.download().reshape(layers, H, D)
        for i in range(layers):
            qr = orc.kv_prep_fused(q[i:i + 1], k[i:i + 1], v[i:i + 1], okc[i], ovc[i], cos, sin,
                                   orc.make_params(H, Hkv, D, 1, start + t, cap, rope_mode=1))
            want = orc.sdpa_decode(qr[:, 0].copy(), okc[i], ovc[i], H, Hkv, D, cap, start + t + 1).reshape(H, D)
            assert max_abs(got[i], want) <= 2e-3, (t, i)
        assert int(dpos.download()[0]) == start + t + 1
    for i in range(layers):
        assert np.array_equal(bits(dkc[i].download()), bits(okc[i]))
    graph.destroy()


def test_per_kernel_profiling_counts_launches():
    announce("profiling")
    f = ctx()
    H, Hkv, D, cap, N = 8, 2, 128, 4096, 4000
    dq, dk, dv, do = f.zeros((1, H * D)), f.zeros((Hkv, cap, D)), f.zeros((Hkv, cap, D)), f.zeros((1, H * D))
    f.profile_reset()
    f.profile_enable(True)
    try:
        for _ in range(5):
            f.flash_attention(dq.arg(), dk.arg(), dv.arg(), do.arg(), True, N - 1, H, D, N, 1)
        n, ms = f.profile_query("flash_decode_mfma")
        assert n == 5 and 0.0 < ms < 50.0
        with pytest.raises(fa.FoundryError):
            f.start_capture()
    finally:
        f.profile_enable(False)
        f.profile_reset()


def _split_decode_state(f, rng, H, Hkv, D, cap, start):
    cos, sin = fa.rope_tables(5e5, D, cap)
    kc, vc = h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    q, k, v = (h16(rng.normal(size=(1, n * D))) for n in (H, Hkv, Hkv))
    dev = dict(cos=f.array(cos), sin=f.array(sin), kc=f.array(kc), vc=f.array(vc), q=f.array(q), k=f.array(k),
               v=f.array(v), out=f.zeros((1, H * D)), pos=f.array(np.array([start], np.uint32)))
    return (cos, sin, kc, vc, q, k, v), dev


@pytest.mark.parametrize("merge", [1, 0, 2], ids=["merge_kernel", "merge_in_kernel", "merge_polled"])
def test_graph_survives_workspace_growth(merge):
    """A recorded split decode addresses the workspace (and the arrival counters) it was captured against. Growing the
    workspace afterwards must leave that buffer alive for the graph: replays before and after the growth equal the
    oracle, and so does an eager call on the new workspace."""
    announce("graph replay after the workspace has grown, merge", merge)
    f = fa.Foundry(0)  # a context of its own: its workspace is the initial 64 MiB
    rng = np.random.default_rng(81 + merge)
    H, Hkv, D, cap, start = 24, 8, 128, 4096, 3000
    (cos, sin, kc, vc, q, k, v), d = _split_decode_state(f, rng, H, Hkv, D, cap, start)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, fa.ROPE_NORMAL)
    f.set_decode_variant(0, merge)
    try:
        def step():
            f.decode_step_fused(d["q"].arg(), d["k"].arg(), d["v"].arg(), None, d["kc"].arg(), d["vc"].arg(),
                                d["cos"].arg(), d["sin"].arg(), d["out"].arg(), p, d_position=d["pos"], kv_len_bound=cap)
            f.u32_add(d["pos"], 1, 1)

        f.start_capture()
        step()
        graph = f.end_capture()
        ok, ov = kc.copy(), vc.copy()

        def expect(t):
            qr = orc.kv_prep_fused(q, k, v, ok, ov, cos, sin, orc.make_params(H, Hkv, D, 1, start + t, cap, rope_mode=1))
            return orc.sdpa_decode(qr[:, 0].copy(), ok, ov, H, Hkv, D, cap, start + t + 1).reshape(-1)

        graph.launch()
        f.synchronize()
        assert max_abs(d["out"].download().reshape(-1), expect(0)) <= 2e-3
        # outgrow the workspace (64 MiB at first) while the graph is alive, then use the new one eagerly
        grown = 160 << 20
        f.reserve_workspace(grown)
        step()
        f.synchronize()
        assert max_abs(d["out"].download().reshape(-1), expect(1)) <= 2e-3
        for t in (2, 3):
            graph.launch()
            f.synchronize()
            assert max_abs(d["out"].download().reshape(-1), expect(t)) <= 2e-3, t
        assert np.array_equal(bits(d["kc"].download()), bits(ok))
        f.reserve_workspace(grown + (64 << 20))  # a second retirement while the same graph lives
        graph.launch()
        f.synchronize()
        assert max_abs(d["out"].download().reshape(-1), expect(4)) <= 2e-3
        graph.destroy()  # frees the retired buffers
        step()
        f.synchronize()
        assert max_abs(d["out"].download().reshape(-1), expect(5)) <= 2e-3
    finally:
        for b in d.values():
            b.free()
        f.close()


def test_stream_waiting_calls_are_refused_during_capture():
    announce("capture guards")
    f = ctx()
    buf = f.zeros((16,))
    f.start_capture()
    try:
        for call in (lambda: buf.download(), lambda: buf.upload(np.zeros(16, np.float16)), lambda: f.synchronize(),
                     lambda: f.profile_reset(), lambda: f.profile_query("x"), lambda: buf.free()):
            with pytest.raises(fa.FoundryError) as e:
                call()
            assert e.value.variant == "OperationFailed" and "capture" in str(e.value)
        f.u32_add(buf, 1, 0)  # the capture is still valid: record something and finish it
    finally:
        graph = f.end_capture()
    graph.launch()
    f.synchronize()
    graph.destroy()
    buf.free()


def test_fused_step_past_its_bound_is_reported():
    """A replayed fused step whose device position has moved past kv_len_bound (still inside the capacity) drops the
    token; the next synchronize says so, once."""
    announce("fused step beyond kv_len_bound")
    f = ctx()
    rng = np.random.default_rng(5)
    H, Hkv, D, cap, start = 8, 2, 128, 512, 100
    (cos, sin, kc, vc, q, k, v), d = _split_decode_state(f, rng, H, Hkv, D, cap, start)
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, fa.ROPE_NEOX)
    bound = start + 2  # room for positions start and start + 1

    def step():
        f.decode_step_fused(d["q"].arg(), d["k"].arg(), d["v"].arg(), None, d["kc"].arg(), d["vc"].arg(), d["cos"].arg(),
                            d["sin"].arg(), d["out"].arg(), p, d_position=d["pos"], kv_len_bound=bound)
        f.u32_add(d["pos"], 1, 1)

    step()
    step()
    f.synchronize()  # both inside the bound
    step()           # position start + 2: kv_len start + 3 > bound
    with pytest.raises(fa.FoundryError) as e:
        f.synchronize()
    assert e.value.variant == "InvalidOperation" and "kv_len_bound" in str(e.value)
    f.synchronize()  # reported once
    got_k = d["kc"].download()
    assert np.array_equal(bits(got_k[:, start + 2]), bits(kc[:, start + 2])), "the dropped token must not be stored"
    for b in d.values():
        b.free()


def test_stream_timer_and_compute_units():
    announce("stream timer")
    f = ctx()
    assert f.n_cus() >= 1
    with pytest.raises(fa.FoundryError) as e:
        f.timer_stop()  # nothing started
    assert e.value.variant == "InvalidOperation"
    word = f.array(np.zeros(4, np.uint32))
    f.start_capture()
    with pytest.raises(fa.FoundryError):
        f.timer_start()  # not during a capture
    for _ in range(64):
        f.u32_add(word, 1, 1)
    g = f.end_capture()
    f.timer_start()
    for _ in range(4):
        g.launch()
    ms = f.timer_stop()
    assert 0.0 < ms < 100.0
    assert int(word.download()[0]) == 256
    g.destroy()
    word.free()


def test_captured_prefill_chunks_with_the_fused_qkv_write_stage_replay():
    """A prefill chunk of one layer as a captured graph - FusedQkv with KvPrepFused as its write stage (norm kernel, split-K
    GEMM, finish kernel), then the chunk's attention over the cache (split-K prefill + merge) - replayed several times
    with eager work and synchronisations between the replays; every replay must reproduce the eager result bit for bit."""
    announce("graph replay, fused qkv + kv prep + prefill chunk")
    f = ctx()
    rng = np.random.default_rng(21)
    H, Hkv, D, K, m, prefix, cap = 24, 8, 128, 1024, 32, 1000, 1280
    N, NK = H * D, Hkv * D
    x = rng.uniform(-1, 1, (m, K)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, K).astype(np.float16)
    ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
    kc0, vc0 = h16(rng.normal(size=(Hkv, cap, D))), h16(rng.normal(size=(Hkv, cap, D)))
    cos, sin = fa.rope_tables(5e5, D, cap)
    dev_w = [f.array(orc.to_canonical(w)) for w in ws]
    dx, dg, dcos, dsin = f.array(x), f.array(g), f.array(cos), f.array(sin)
    dkc, dvc = f.array(kc0), f.array(vc0)
    dqr, dout = f.zeros((H, m, D)), f.zeros((m, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, prefix, cap, fa.ROPE_NORMAL)

    def enqueue():
        f.fused_qkv_kv_prep(dx.arg(), dev_w[0].arg(), dev_w[1].arg(), dev_w[2].arg(), K, dqr.arg(), dcos.arg(), dsin.arg(), p,
                            k_cache=dkc.arg(), v_cache=dvc.arg(), gamma=dg.arg())
        f.flash_attention(dqr.arg(), dkc.arg(), dvc.arg(), dout.arg(), True, prefix, H, D, prefix + m, m)

    enqueue()  # eager: the reference result, and the workspace at its final size before the capture
    f.synchronize()
    want_out, want_k, want_qr = bits(dout.download()), bits(dkc.download()), bits(dqr.download())
    f.start_capture()
    enqueue()
    graph = f.end_capture()
    scratch = f.zeros((64, 64))
    for t in range(4):
        for d, src in ((dkc, kc0), (dvc, vc0)):
            d.upload(src)
        dout.upload(np.zeros((m, H * D), np.float16))
        dqr.upload(np.zeros((H, m, D), np.float16))
        graph.launch()
        f.synchronize()
        assert np.array_equal(bits(dout.download()), want_out), t
        assert np.array_equal(bits(dkc.download()), want_k), t
        assert np.array_equal(bits(dqr.download()), want_qr), t
        scratch.upload(np.full((64, 64), t, np.float16))  # eager work between the replays
        f.synchronize()
    graph.destroy()
    for b in dev_w + [dx, dg, dcos, dsin, dkc, dvc, dqr, dout, scratch]:
        b.free()
