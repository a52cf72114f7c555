"""A MoE layer read from a GGUF file (tests/golden/make_tiny_gguf.py writes it) and run on the GPU: router + experts + combine,
bit for bit the oracle on the file's own bytes."""
import os
import sys

import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import bits, dev

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_tiny_gguf as mk

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("gate_type,down_type,hidden,ffn,experts,K,T", [
    (mk.GGML_Q4_K, mk.GGML_Q4_K, 512, 256, 6, 2, 3),
    (mk.GGML_Q5_K, mk.GGML_Q8_0, 1024, 512, 16, 4, 8),
    (mk.GGML_Q4_K, mk.GGML_Q6_K, 2048, 768, 32, 8, 2),
    (mk.GGML_Q4_K, mk.GGML_Q5_1, 1024, 384, 8, 2, 5)])
def test_moe_layer_from_a_gguf_file(strix, tmp_path, gate_type, down_type, hidden, ffn, experts, K, T):
    path = str(tmp_path / "layer.gguf")
    _, _, arrays, _, _ = mk.tiny_moe_file(path, seed=hidden + T, hidden=hidden, ffn=ffn, experts=experts, layers=2, gate_type=gate_type, down_type=down_type)
    g = strix.GgufFile(path)
    layer = 1
    moe, router, norm, m = g.load_moe_layer(layer, K, T, intermediates=True)
    assert (m.hidden, m.ffn, m.experts, m.gate_type, m.down_type) == (hidden, ffn, experts, gate_type, down_type)
    a = arrays[layer]
    assert np.array_equal(bits(router.cpu().numpy()), bits(a["router"])) and np.array_equal(bits(norm.cpu().numpy()), bits(a["norm"]))
    rng = np.random.default_rng(7)
    x = rng.standard_normal((T, hidden)).astype(np.float16)
    y, ids, wts, _ = moe.run_layer(dev(x), router)
    ids_ref, w_ref, _, _ = orc.route(x.astype(np.float32), a["router"], K)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), ids_ref) and np.array_equal(bits(wts.cpu().numpy()), bits(w_ref))
    c, d, s, _ = orc.quantize_a8(x.astype(np.float32))
    ref = orc.routed_experts(hidden, ffn, K, a["gate"], a["up"], a["down"], down_type, c, d, s, ids_ref, gate_type=gate_type)
    assert np.array_equal(bits(moe.rawdots[:T].cpu().numpy()), bits(ref.rawdots))
    assert np.array_equal(bits(y.cpu().numpy()), bits(orc.combine(0, w_ref, ids_ref, ref.rawdots)))
    g.close()
