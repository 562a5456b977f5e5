"""Writes tests/golden/vulkan_attention_kat.json: the inputs of the reference's
only attention known-answer test (tests/test_vulkan.cpp:353-482: Sq=2, Skv=3,
D=4, non-causal, Q[i]=i+1, K stored transposed [D,T] with K[i]=(i+1)/2,
V[i]=(i+1)/4, scale 1/sqrt(D), tolerance 1e-4) and the expected output
evaluated in float64 from the softmax definition.  Run from the repo root."""
import json
from pathlib import Path

import numpy as np

seq_q, seq_kv, d = 2, 3, 4
q = (np.arange(seq_q * d, dtype=np.float64) + 1).reshape(seq_q, d)
k_t = ((np.arange(d * seq_kv, dtype=np.float64) + 1) * 0.5).reshape(d, seq_kv)
v = ((np.arange(seq_kv * d, dtype=np.float64) + 1) * 0.25).reshape(seq_kv, d)
scale = 1.0 / np.sqrt(d)
s = q @ k_t * scale
p = np.exp(s - s.max(axis=1, keepdims=True))
p /= p.sum(axis=1, keepdims=True)
out = p @ v
doc = {
    "source": "reference tests/test_vulkan.cpp:353-482",
    "seq_q": seq_q, "seq_kv": seq_kv, "head_dim": d, "scale": scale, "tolerance": 1e-4,
    "q": q.tolist(), "k_transposed": k_t.tolist(), "v": v.tolist(), "expected": out.tolist(),
}
Path(__file__).with_name("vulkan_attention_kat.json").write_text(json.dumps(doc, indent=1))
print(out)
