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
