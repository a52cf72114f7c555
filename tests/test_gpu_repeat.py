"""Launch-after-launch determinism of every sweep that streams weights through LDS copy rings.

A copy into a ring slot is written to LDS when its data arrives, whatever LDS reads of that slot the wave still has queued; the
kernels therefore wait for their LDS reads before they issue a copy into a slot they have read. A
missing wait of that kind shows as a few wrong rows in a few launches of a hundred, never in a single parity run - so each
ring is launched a few hundred times here on full-entropy blocks and every launch must leave the bits of the first. (The
first launch's bits against the oracle are the other GPU tests' business.)"""
import numpy as np
import pytest
import torch

import orc
from test_gpu_parity import dev, make_layer, random_q4k

pytestmark = pytest.mark.gpu


def repeat(fn, snapshot, launches):
    fn()
    first = [t.clone() for t in snapshot()]
    bad = torch.zeros((), dtype=torch.int64, device=first[0].device)
    for _ in range(launches):
        fn()
        for got, want in zip(snapshot(), first):
            bad += (got.reshape(-1).view(torch.uint8) != want.reshape(-1).view(torch.uint8)).sum()
    return int(bad)


# rows 1 / 4: the 16-rows-per-wave rings; 8: the early-routes front launch + contiguous down stages; 12: the same with more rows
# per compute unit; 24: the staged 64-row rings of a batch past the fused sizes
@pytest.mark.parametrize("E,H,I,K,T", [(128, 2048, 768, 8, 1), (128, 2048, 768, 8, 4), (128, 2048, 768, 8, 8), (64, 1024, 512, 4, 12), (32, 2048, 768, 4, 24)])
def test_layer_entry_repeats_its_bits(strix, E, H, I, K, T):
    rng = np.random.default_rng(1000 + E + T)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    n = T * K
    snap = lambda: (layer.output[:T], layer.rawdots[:T], layer.down_codes[:n], layer.down_deltas[:n], layer.down_sums[:n])
    assert repeat(lambda: layer.run_layer(x, wr), snap, 300) == 0
    assert int(layer.status[:T].sum()) == 0


# the staged entry points on their own (router outside): the 64-row projection and down rings with shared items
@pytest.mark.parametrize("E,H,I,K,T", [(16, 2048, 768, 8, 8), (8, 1536, 1024, 2, 16)])
def test_staged_entry_points_repeat_their_bits(strix, E, H, I, K, T):
    rng = np.random.default_rng(2000 + E + T)
    gate, up, down = make_layer(rng, H, I, E, full_entropy=True)
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    ids, wts, _ = strix.route(x, wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T)
    n = T * K
    snap = lambda: (layer.output[:T], layer.rawdots[:T], layer.down_codes[:n])
    assert repeat(lambda: layer.run(x, ids, wts), snap, 300) == 0


# the dense matrices of an FFN (one expert, top-1): the pair / quad rings and, from five rows on, the matrix-core sweep
@pytest.mark.parametrize("T", [1, 4, 8])
def test_dense_ffn_repeats_its_bits(strix, T):
    H, I = 1280, 1792
    rng = np.random.default_rng(3000 + T)
    gate, up, down = random_q4k(rng, (1, I), H), random_q4k(rng, (1, I), H), random_q4k(rng, (1, H), I)
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    ids = torch.zeros((T, 1), dtype=torch.int32, device=x.device)
    ones = torch.ones((T, 1), dtype=torch.float32, device=x.device)
    layer = strix.MoeLayer(H, I, 1, 1, dev(gate), dev(up), dev(down), T)
    snap = lambda: (layer.output[:T], layer.down_codes[:T])
    assert repeat(lambda: layer.run(x, ids, ones), snap, 300) == 0


# down rows in the host executor's formats (their own rings) through the layer entry
@pytest.mark.parametrize("down_type", [orc.Q8_0, orc.Q5_1, orc.Q6_K])
def test_other_down_formats_repeat_their_bits(strix, down_type):
    E, H, I, K, T = 16, 1024, 512, 4, 8
    rng = np.random.default_rng(4000 + int(down_type))
    gate, up = random_q4k(rng, (E, I), H), random_q4k(rng, (E, I), H)
    down = orc.quantize_rows(down_type, (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32))
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down.reshape(E, H, -1)), T, down_type=down_type)
    snap = lambda: (layer.output[:T], layer.rawdots[:T])
    assert repeat(lambda: layer.run_layer(x, wr), snap, 300) == 0


# the matrix-core prefill (workgroup-shared rings between loader and multiplier waves, a barrier per step)
@pytest.mark.parametrize("H,I,E,K,T", [(1024, 512, 12, 4, 300), (768, 1280, 5, 2, 150)])
def test_prefill_f16_repeats_its_bits(strix, H, I, E, K, T):
    rng = np.random.default_rng(5000 + T)
    gate, up, down = make_layer(rng, H, I, E)
    wr = dev((rng.standard_normal((E, H)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((T, H)).astype(np.float16))
    ids, wts, _ = strix.route(x, wr, K)
    layer = strix.MoeLayer(H, I, E, K, dev(gate), dev(up), dev(down), T, prefill_f16=True)
    out = {}

    def run():
        out["y"] = layer.run_prefill_f16(x, ids, wts)
    assert repeat(run, lambda: (out["y"], layer.rawdots[:T]), 100) == 0
    assert int(layer.status[:T].sum()) == 0
