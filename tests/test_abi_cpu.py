"""No-GPU checks of the C ABI: the library loads, exports every symbol the header declares, its host-only
entry points work, and errors follow the documented convention."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import foundry_attn as fa
import orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "foundry_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = fa.load()
    names = _declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), "symbol %s declared in foundry_attn.h is not exported" % n
    # and the binding declares a prototype for each of them
    assert set(names) == set(fa.PROTOTYPES), set(names) ^ set(fa.PROTOTYPES)


def test_struct_layouts_match_the_reference_abi():
    # KvPrepFusedParamsResolved is 13 x u32 = 52 bytes (src/metals/kv_prep/mod.rs:79-114)
    assert C.sizeof(fa.KvPrepFusedParams) == 52
    assert [f[0] for f in fa.KvPrepFusedParams._fields_] == [
        "d_model", "kv_dim", "head_dim", "n_heads", "n_kv_heads", "group_size", "seq_len", "position_offset",
        "max_seq_len", "total_elements", "rope_mode", "layer_idx", "no_rope_layer_step"]
    assert C.sizeof(fa.TensorArg) == 8 + 8 + 4 + 4 + 32 + 32


def test_status_names():
    lib = fa.load()
    for code, name in fa.STATUS_NAMES.items():
        assert lib.fa_status_name(code).decode() == name
    assert lib.fa_version().decode().startswith("foundry_attn")


@pytest.mark.parametrize("base,D,P,ff", [(1e6, 64, 1100, False), (5e5, 128, 8500, False), (5e6, 128, 300, True)])
def test_host_rope_tables_equal_oracle(base, D, P, ff):
    factors = np.linspace(1, 4, D // 2).astype(np.float32) if ff else None
    cos, sin = fa.rope_tables(base, D, P, factors)
    ocos, osin = orc.rope_tables(base, D, P, factors)
    assert np.array_equal(cos.view(np.uint16), ocos.view(np.uint16))
    assert np.array_equal(sin.view(np.uint16), osin.view(np.uint16))
    wc, ws = fa.rope_tables(base, D, P, factors, pos_begin=P - 10)
    assert np.array_equal(wc, cos[P - 10:]) and np.array_equal(ws, sin[P - 10:])


def test_host_errors_without_a_device():
    lib = fa.load()
    with pytest.raises(fa.FoundryError) as e:
        fa.rope_tables(1e4, 63, 4)
    assert e.value.variant == "InvalidShape"
    assert lib.fa_ctx_create(0, None) == 2  # NullPointer
    h = C.c_void_p()
    st = lib.fa_ctx_create(4096, C.byref(h))  # no such device anywhere
    assert st == 1 and "Device not found" in lib.fa_last_error_string().decode()
    assert lib.fa_synchronize(None) == 2
    assert lib.fa_graph_destroy(None) == 0 and lib.fa_ctx_destroy(None) == 0


def test_capacity_policy_equals_oracle():
    """fa_align_capacity / fa_grown_capacity are host arithmetic: same values as the oracle's restatement of
    src/model/context.rs:213-219 and src/model/executor.rs:2354-2382 over a sweep."""
    for c in list(range(0, 400)) + [2047, 2048, 2049, 65535, 65536, 1 << 20]:
        assert fa.align_capacity(c) == orc.align_capacity(c)
    rng = np.random.default_rng(7)
    for _ in range(3000):
        alloc = int(rng.integers(0, 40000))
        mx = int(rng.integers(1, 140000))
        req = int(rng.integers(0, 150000))
        gf = float(rng.choice([0.0, 1.1, 1.5, 2.0, 3.0]))
        assert fa.grown_capacity(alloc, req, mx, gf) == orc.grown_capacity(alloc, req, mx, gf), (alloc, req, mx, gf)


def test_header_is_plain_c99_and_links_from_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 (pedantic) and a C program must link against the library
    and call its host-only entry points."""
    import subprocess
    src = tmp_path / "abi.c"
    src.write_text('#include <stdio.h>\n#include "foundry_attn.h"\n'
                   'int main(void) {\n'
                   '    fa_fused_qkv_params q; fa_matmul_params m; fa_kv_prep_fused_params k; fa_tensor_arg t; fa_paged_kv pg;\n'
                   '    (void)q; (void)m; (void)k; (void)t; (void)pg;\n'
                   '    if (fa_align_capacity(129) != 256) return 1;\n'
                   '    if (fa_grown_capacity(2048, 2049, 8192, 2.0f) != 4096) return 2;\n'
                   '    printf("%s %s\\n", fa_version(), fa_status_name(FA_ERR_INVALID_SHAPE));\n'
                   '    return 0;\n}\n')
    exe = tmp_path / "abi"
    libdir = os.path.join(ROOT, "test-burn_amd")
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                           str(src), "-o", str(exe), "-L", libdir, "-lfoundry_attn", "-Wl,-rpath," + libdir])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "InvalidShape" in out.stdout
