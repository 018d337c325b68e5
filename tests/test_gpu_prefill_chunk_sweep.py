"""GPU: the short-chunk prefill kernel against the tiled prefill kernel over a sweep of shapes (its fixed cases run with the
rest of the prefill suite, once per prefill variant, in test_gpu_prefill.py)."""
import numpy as np
import pytest

import foundry_attn as fa
import orc
from gpu_util import announce, ctx, h16, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-3


def test_prefill_chunk_kernel_agrees_with_the_tiled_kernel_on_random_shapes():
    """A sweep over shapes the fixed cases do not name: group sizes 1 to 8 (1 to 16 column blocks: one and two groups of
    column blocks, full and partial), head_dim 64 and 128, 1 to 64 rows, prefixes from nothing to a few thousand tokens,
    causal or not, f16 or bf16 - the short-chunk kernel forced (variant 3) against the tiled kernel (variant 2) on the same
    device tensors, cache rows past kv_len poisoned with NaN. The two sum a row's weights in different orders: one f16
    ulp, taken here as 2e-3 on values of order 1; some shapes are checked against the oracle as well."""
    announce("prefill chunk kernel, random shapes")
    rng = np.random.default_rng(20240611)
    f = ctx()
    try:
        for case in range(48):
            D = int(rng.choice([64, 128]))
            G = int(rng.choice([1, 2, 3, 4, 5, 7, 8]))
            Hkv = int(rng.choice([1, 2, 4, 8]))
            H = G * Hkv
            M = int(rng.integers(1, 65))
            prefix = int(rng.choice([0, 1, 31, 100, 257, 1000, 2049, 3000, 5000]))
            causal = bool(rng.random() < 0.8)
            bf16 = bool(rng.random() < 0.25)
            N = prefix + M
            cap = N + int(rng.integers(0, 40))
            print("[case]", case, dict(D=D, G=G, Hkv=Hkv, M=M, prefix=prefix, causal=causal, bf16=bf16), flush=True)
            q = rng.normal(size=(H, M, D)).astype(np.float32)
            k = rng.normal(size=(Hkv, cap, D)).astype(np.float32)
            v = rng.normal(size=(Hkv, cap, D)).astype(np.float32)
            k[:, N:], v[:, N:] = np.nan, np.nan
            if bf16:
                conv = lambda x: (x.view(np.uint32) >> 16).astype(np.uint16)  # truncation is as good as rounding here
                dq, dk, dv = (fa.DevBuf(f, x.shape, np.uint16).upload(conv(x)) for x in (q, k, v))
                dt = fa.DTYPE_BF16
            else:
                dq, dk, dv = f.array(h16(q)), f.array(h16(k)), f.array(h16(v))
                dt = None
            outs = []
            for variant in (2, 3):
                f.set_prefill_variant(variant)
                do = fa.DevBuf(f, (M, H * D), np.uint16).upload(np.zeros((M, H * D), np.uint16))
                edt = fa.DTYPE_BF16 if bf16 else fa.DTYPE_F16
                args = [b.arg(dtype=edt) for b in (dq, dk, dv, do)]
                f.flash_attention(args[0], args[1], args[2], args[3], causal, prefix, H, D, N, M)
                f.synchronize()
                raw = do.download()
                outs.append((raw.astype(np.uint32) << 16).view(np.float32) if bf16 else raw.view(np.float16).astype(np.float32))
                do.free()
            assert np.all(np.isfinite(outs[1])), case
            tol = 2e-2 if bf16 else TOL
            assert float(np.max(np.abs(outs[0] - outs[1]))) <= tol, (case, float(np.max(np.abs(outs[0] - outs[1]))))
            if not bf16 and case % 6 == 0:
                want = orc.sdpa_prefill(h16(q), h16(k), h16(v), H, Hkv, D, M, N, prefix, cap, causal=causal, out_layout="token_major",
                                        n_threads=8)
                assert max_abs(outs[1].reshape(M, H * D), want.reshape(M, H * D)) <= TOL, case
            for b in (dq, dk, dv):
                b.free()
    finally:
        f.set_prefill_variant(0)
