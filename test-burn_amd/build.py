"""Builds libfoundry_attn.so (HIP, gfx950 only) next to this file.

    python test-burn_amd/build.py            # incremental: recompiles sources newer than their objects
    python test-burn_amd/build.py --force    # recompile everything

hipcc cross-compiles without a GPU. Packed-FP32 code generation is disabled for all device code.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
# FOUNDRY_ATTN_BUILD_FLAGS (extra hipcc flags) and FOUNDRY_ATTN_BUILD_TAG (suffix of the object directory and of the
# library name) make a second, differently configured library next to the product one, e.g. a development build with
# -DFA_DECODE_TRACE; foundry_attn.py loads it when FOUNDRY_ATTN_LIB names it.
TAG = os.environ.get("FOUNDRY_ATTN_BUILD_TAG", "")
OBJ = os.path.join(HERE, "build" + TAG)
LIB = os.path.join(HERE, "libfoundry_attn%s.so" % TAG)
SOURCES = ["fa_api.hip", "fa_kvprep.hip", "fa_decode.hip", "fa_decode_d64.hip", "fa_decode_d128.hip", "fa_decode_d64_w4.hip", "fa_decode_d128_w4.hip", "fa_prefill.hip", "fa_chunk.hip",
           "fa_sage.hip", "fa_kvcopy.hip", "fa_qkv.hip", "fa_gemm.hip", "fa_legacy.hip", "fa_probe.hip"]
HEADERS = [os.path.join(CSRC, "fa_internal.h"), os.path.join(CSRC, "fa_decode_impl.h"), os.path.join(CSRC, "fa_qkv_rope.h"), os.path.join(CSRC, "fa_lds_dma.h"), os.path.join(CSRC, "fa_sage_quant.h"),
           os.path.join(HERE, "..", "include", "foundry_attn.h")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + os.environ.get("FOUNDRY_ATTN_BUILD_FLAGS", "").split()


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(p) > t for p in [src] + HEADERS)


def _compile(name, force):
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ, name.replace(".hip", ".o"))
    if force or _stale(src, obj):
        # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless, filtered out
        r = subprocess.run([HIPCC] + FLAGS + ["-c", src, "-o", obj], stderr=subprocess.PIPE, text=True)
        err = "\n".join(ln for ln in r.stderr.splitlines() if "packed-fp32-ops" not in ln)
        if err.strip():
            sys.stderr.write(err + "\n")
        if r.returncode != 0:
            raise subprocess.CalledProcessError(r.returncode, r.args)
        return True
    return False


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        changed = list(ex.map(lambda n: _compile(n, force), SOURCES))
    objs = [os.path.join(OBJ, n.replace(".hip", ".o")) for n in SOURCES]
    if any(changed) or not os.path.exists(LIB):
        subprocess.check_call([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
