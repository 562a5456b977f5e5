"""C++ host layer on the GPU: HipBackend buffers, HipCompute, the registered
ScaledDotProductAttention operator (including the reference's attention
known-answer test, tests/test_vulkan.cpp:353-482) and the KV classes, each
checked against the CPU oracle inside the C++ program
(granite_amd/host/tests/host_gpu_test.cpp)."""
import json
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
BIN = ROOT / "granite_amd" / "bin" / "host_gpu_test"
SRC = ROOT / "granite_amd" / "host" / "tests" / "host_gpu_test.cpp"


def test_known_answer_constants_match_fixture():
    """The expected values compiled into the C++ test are the committed fixture's."""
    doc = json.loads((Path(__file__).parent / "golden" / "vulkan_attention_kat.json").read_text())
    text = SRC.read_text()
    for row in doc["expected"]:
        for value in row:
            assert repr(value) in text, value
    assert doc["scale"] == 0.5 and re.search(r'attrs\.set\("scale", 0\.5\)', text)


@pytest.mark.gpu
def test_host_layer_gpu_cases():
    if not BIN.exists():
        pytest.fail(f"{BIN} is missing: run `python -m granite_amd.build` first")
    res = subprocess.run([str(BIN)], capture_output=True, text=True, timeout=300)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode != 77, "host_gpu_test found no usable gfx950 GPU"
    assert res.returncode == 0, res.stdout[-3000:]
    assert "0 failed checks" in res.stdout
    assert res.stdout.count("[  OK  ]") >= 6
