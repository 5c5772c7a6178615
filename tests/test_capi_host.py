"""CPU-side checks of the C-ABI library: it loads, exports every symbol the
header declares, and rejects calls made before llama2_init -- no GPU work."""
import ctypes as C
import os
import re

from managedllama2_amd import capi, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "llama2_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llama2_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_functions()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), n
    assert names == capi.EXPORTS  # the binding types exactly what the header declares


def test_calls_before_init_fail_loudly():
    # a fresh process has not called llama2_init: every entry point must refuse
    import subprocess
    import sys
    code = (
        "import ctypes as C, sys; sys.path.insert(0, %r)\n"
        "from managedllama2_amd import capi\n"
        "p = C.c_void_p()\n"
        "assert capi.raw('llama2_malloc', C.byref(p), 16) == capi.ERR_NOT_INITIALIZED\n"
        "assert 'llama2_init' in capi.last_error()\n"
        "assert capi.raw('llama2_rmsnorm', None, None, None, 4, 1e-5) == capi.ERR_NOT_INITIALIZED\n"
        "assert capi.raw('llama2_sync') == capi.ERR_NOT_INITIALIZED\n"
        "assert capi.load().llama2_stream() is None\n"
        "print('ok')\n" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "ok" in out.stdout, out.stderr


def test_config_struct_is_the_32_byte_header():
    assert C.sizeof(capi.Config) == 32  # src/Config.cs:6-19


def test_algorithmic_byte_counts():
    b = synth.layer_matvec_set_bytes(4096, 11008)
    assert synth.qweight_bytes(4096, 4096) == 8716288
    assert synth.qweight_bytes(11008, 4096) == 23429120  # zeros padded to 11 words per row
    assert (b["qkv"], b["o"], b["swiglu"], b["down"]) == (26181632, 8740864, 46880256, 23467520)
    assert b["total"] == 105270272
    assert synth.layer_matvec_set_bytes(5120, 13824)["total"] == 164960256
