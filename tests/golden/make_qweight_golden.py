"""Transcribe the numeric data of the reference's golden known-answer test
(test/QWeightTestData.cs:11-175, used by test/QWeightTests.cs:29-48) into
qweight_golden.json.  The C# file is read as text; nothing is executed.

Run once in a container where the reference checkout is mounted:
    python tests/golden/make_qweight_golden.py [/root/reference]
The JSON it writes is committed, the reference is not needed afterwards.
"""
import json
import os
import re
import sys


def _block(text, name):
    m = re.search(name + r"\s*=\s*new\s+\w+\[\d*\]\s*\{(.*?)\};", text, re.S)
    if not m:
        raise SystemExit("array %r not found" % name)
    return [int(tok.rstrip("u"), 0) for tok in re.findall(r"0x[0-9a-fA-F]+|\d+u?", m.group(1))]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    text = open(os.path.join(ref, "test", "QWeightTestData.cs")).read()
    zero = int(re.search(r"zero\s*=\s*(\d+)\s*;", text).group(1))
    data = {
        "source": "test/QWeightTestData.cs:11-175",
        "zero_word": zero,
        "zeros": _block(text, r"\bzeros"),
        "scales_f32_bits": _block(text, r"var scales"),
        "weights": _block(text, r"\bweights"),
        "checks_f32_bits": _block(text, r"var checks"),
    }
    assert len(data["zeros"]) == 8 and len(data["scales_f32_bits"]) == 8
    assert len(data["weights"]) == 128 and len(data["checks_f32_bits"]) == 1024
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qweight_golden.json")
    with open(out, "w") as f:
        json.dump(data, f, separators=(",", ":"))
        f.write("\n")
    print("wrote", out)


if __name__ == "__main__":
    main()
