"""The CPU-side C and C++ code under AddressSanitizer and UndefinedBehaviorSanitizer
(host code only; no GPU is touched).

1. oracle/oracle.c, the checker every parity test trusts: built as
   liboracle_asan.so and driven through the oracle's own test files in a child
   process (the sanitizer runtime has to be loaded before the interpreter
   starts).  An out-of-bounds read in the oracle would otherwise pass silently
   and be compared against.
2. The C++ host layer's model-file checks (llama2_host.hpp: Config::LoadConfig,
   TransformerWeights::ExpectedBytes, MappedFile): built as
   libllama2_host_asan.so and fed good, truncated, oversized, header-only,
   shorter-than-header and corrupt-header files.  Every bad file must be
   refused with the reference's exception, never crash or trip the sanitizer.
"""
import os
import struct
import subprocess
import sys

import pytest

from managedllama2_amd import modelfile, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CFG = dict(dim=256, hidden_dim=640, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=300, seq_len=32, rope_theta=10000.0)


def sanitizer_env(**extra):
    asan = subprocess.check_output(["gcc", "-print-file-name=libasan.so"], text=True).strip()
    if not os.path.isabs(asan) or not os.path.exists(asan):
        pytest.skip("gcc has no libasan.so in this image")
    env = dict(os.environ)
    # The C++ runtime has to be there when the sanitizer runtime looks up __cxa_throw (the
    # interpreter itself does not link it).  The harness may preload a library of its own:
    # keep it, behind the sanitizer runtime.
    cxx = subprocess.check_output(["g++", "-print-file-name=libstdc++.so.6"], text=True).strip()
    env["LD_PRELOAD"] = " ".join(x for x in (asan, cxx if os.path.isabs(cxx) else "", os.environ.get("LD_PRELOAD", "")) if x)
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1:verify_asan_link_order=0"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    env["OMP_NUM_THREADS"] = "4"
    env.update(extra)
    return env


def test_oracle_under_address_and_ub_sanitizers():
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "liboracle_asan.so"])
    lib = os.path.join(ROOT, "oracle", "liboracle_asan.so")
    env = sanitizer_env(LLAMA2_ORACLE_LIB=lib)
    which = subprocess.run([sys.executable, "-c", "from oracle import oracle; print(oracle.lib()._name)"], env=env, cwd=ROOT,
                           capture_output=True, text=True, timeout=120)
    assert which.returncode == 0 and which.stdout.strip().endswith("liboracle_asan.so"), which.stdout + which.stderr
    files = [os.path.join(ROOT, "tests", f) for f in ("test_oracle_qweight.py", "test_oracle_ops.py",
                                                      "test_oracle_sampler.py", "test_oracle_repack.py")]
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", "-m", "not gpu"] + files,
                       env=env, cwd=ROOT, capture_output=True, text=True, timeout=900)
    tail = (r.stdout + r.stderr)[-3000:]
    assert r.returncode == 0, tail
    assert "passed" in r.stdout and "AddressSanitizer" not in tail and "runtime error" not in tail, tail


HOST_SCRIPT = r"""
import sys
from managedllama2_amd import hostlib
for path in sys.argv[1:]:
    try:
        hostlib.check_model_file(path)
        print("OK", path)
    except hostlib.HostError as e:
        print("ERR", e.code, path, str(e)[:60])
"""


def test_host_model_file_checks_under_sanitizers(tmp_path):
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "managedllama2_amd", "host"), "../libllama2_host_asan.so"])
    lib = os.path.join(ROOT, "managedllama2_amd", "libllama2_host_asan.so")
    good = str(tmp_path / "good.bin")
    modelfile.write_model(good, CFG, synth.random_model(CFG, seed=21))
    data = open(good, "rb").read()

    def header(**fields):
        c = dict(CFG, **fields)
        return struct.pack("<7if", c["dim"], c["hidden_dim"], c["n_layers"], c["n_heads"], c["n_kv_heads"], c["vocab_size"],
                           c["seq_len"], c["rope_theta"]) + data[32:]

    cases = {
        "good": (data, "OK"),
        "short": (data[:-10], "ERR 1"),
        "long": (data + b"\0" * 6, "ERR 1"),
        "header_only": (data[:32], "ERR 1"),
        "half_header": (data[:16], "ERR 1"),
        "one_byte": (b"\x01", "ERR 1"),
        "zero_heads": (header(n_heads=0), "ERR 1"),          # kvDim would divide by it
        "negative_heads": (header(n_heads=-2), "ERR 1"),
        "zero_kv_heads": (header(n_kv_heads=0), "ERR 1"),
        "negative_dim": (header(dim=-256), "ERR 1"),
        "huge_dim": (header(dim=2**31 - 1, n_heads=1, n_kv_heads=1), "ERR 1"),  # sizes would overflow
        "huge_vocab": (header(vocab_size=2**31 - 1), "ERR 1"),
        "zero_layers": (header(n_layers=0), "ERR 1"),
        "heads_do_not_divide": (header(n_heads=3, n_kv_heads=3), "ERR 1"),
        "gqa": (header(n_kv_heads=1), "ERR 2"),
    }
    paths = []
    for name, (blob, _) in cases.items():
        p = str(tmp_path / (name + ".bin"))
        open(p, "wb").write(blob)
        paths.append(p)
    r = subprocess.run([sys.executable, "-c", HOST_SCRIPT] + paths, env=sanitizer_env(LLAMA2_HOST_LIB=lib), cwd=ROOT,
                       capture_output=True, text=True, timeout=300)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out[-3000:]
    assert "AddressSanitizer" not in out and "runtime error" not in out, out[-3000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith(("OK", "ERR"))]
    assert len(lines) == len(cases), out[-3000:]
    for line, (name, (_, want)) in zip(lines, cases.items()):
        assert line.startswith(want), (name, line)
    # the Python reader refuses the same headers
    for name, (_, want) in cases.items():
        if want == "ERR 1" and name not in ("short", "long", "header_only"):
            with pytest.raises(modelfile.ModelFileError):
                modelfile.read_config(str(tmp_path / (name + ".bin")))
