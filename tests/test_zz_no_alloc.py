"""The allocation-free layer entry (mi355_moe_enqueue_layer_static) against mi355_moe_enqueue_layer: same bits, on two calls in
a row, the second with a smaller input; and its size limits are refused before anything runs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _layer(strix, H, I, E, K, T, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = lambda shape: strix.quantize_weight_rows(strix.TYPE_Q4_K, torch.randn(shape, generator=g, device="cuda") * 0.02)
    gate, up, down = q((E, I, H)), q((E, I, H)), q((E, H, I))
    wr = torch.randn((E, H), generator=g, device="cuda") * 0.02
    x = torch.randn((T, H), generator=g, device="cuda").to(torch.float16)
    return strix.MoeLayer(H, I, E, K, gate, up, down, T), wr, x


@pytest.mark.parametrize("H,I,E,K,T,T2", [(2048, 768, 128, 8, 8, 3), (1024, 512, 16, 4, 16, 1), (6144, 1280, 160, 8, 16, 5)])
def test_static_workspace_layer_equals_the_caller_workspace_layer(strix, H, I, E, K, T, T2):
    layer, wr, x = _layer(strix, H, I, E, K, T, seed=H + T)
    for rows in (T, T2):                       # two calls in a row, the second with fewer rows
        xs = x[:rows].contiguous()
        want, ids, wts, _ = layer.run_layer(xs, wr)
        want, ids, wts = want.clone(), ids.clone(), wts.clone()
        want_status = layer.status[:rows].clone()
        ids2 = torch.full((rows, K), -1, dtype=torch.int32, device="cuda")
        wts2 = torch.full((rows, K), -1.0, dtype=torch.float32, device="cuda")
        status2 = torch.full((rows,), 77, dtype=torch.int32, device="cuda")
        out2 = torch.full((rows, H), -7.0, dtype=torch.float32, device="cuda")
        got = layer.run_layer_static(xs, wr, ids2, wts2, status2, out2)
        torch.cuda.synchronize()
        assert torch.equal(ids2, ids)
        assert np.array_equal(wts2.cpu().numpy().view(np.uint32), wts.cpu().numpy().view(np.uint32))
        assert torch.equal(status2, want_status) and int(status2.sum()) == 0
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.cpu().numpy().view(np.uint32))


def test_static_workspace_layer_refuses_sizes_beyond_its_limits(strix):
    layer, wr, x = _layer(strix, 1024, 512, 16, 4, 17, seed=5)
    ids = torch.zeros((17, 4), dtype=torch.int32, device="cuda")
    wts = torch.zeros((17, 4), dtype=torch.float32, device="cuda")
    status = torch.zeros(17, dtype=torch.int32, device="cuda")
    out = torch.full((17, 1024), -7.0, dtype=torch.float32, device="cuda")
    with pytest.raises(strix.StrixError) as err:
        layer.run_layer_static(x, wr, ids, wts, status, out)
    assert err.value.code == strix.E_INVALID_ARGUMENT and "1..16" in str(err.value)
    torch.cuda.synchronize()
    assert bool((out == -7.0).all())


def test_static_workspace_layer_inside_a_captured_graph(strix):
    """The entry point is for callers under stream capture: after mi355_static_workspace_prepare (the symbol look-up, outside
    capture) the call is captured into a HIP graph and replayed with eager calls of the library in between; every replay
    gives the eager result's bits. Nothing in the sequence allocates or records a memset node."""
    H, I, E, K, T = 2048, 768, 128, 8, 8
    layer, wr, x = _layer(strix, H, I, E, K, T, seed=91)
    strix.check(strix.lib().mi355_static_workspace_prepare(None))
    want, ids, wts, _ = layer.run_layer(x, wr)
    want, ids = want.clone(), ids.clone()
    ids2 = torch.zeros((T, K), dtype=torch.int32, device="cuda")
    wts2 = torch.zeros((T, K), dtype=torch.float32, device="cuda")
    status2 = torch.zeros((T,), dtype=torch.int32, device="cuda")
    out2 = torch.zeros((T, H), dtype=torch.float32, device="cuda")
    layer.run_layer_static(x, wr, ids2, wts2, status2, out2)          # warm call outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.run_layer_static(x, wr, ids2, wts2, status2, out2)
    for replay in range(4):
        out2.fill_(-3.0); ids2.fill_(-1); status2.fill_(55)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ids2, ids) and int(status2.sum()) == 0, replay
        assert np.array_equal(out2.cpu().numpy().view(np.uint32), want.cpu().numpy().view(np.uint32)), replay
        # eager work of the same library between the replays: another shape through the same built-in workspace
        other, _, _, _ = layer.run_layer(x[:3].contiguous(), wr)
        o3 = torch.zeros((3, H), dtype=torch.float32, device="cuda")
        layer.run_layer_static(x[:3].contiguous(), wr, ids2[:3].clone(), wts2[:3].clone(), status2[:3].clone(), o3)
        torch.cuda.synchronize()
        assert np.array_equal(o3.cpu().numpy().view(np.uint32), other.cpu().numpy().view(np.uint32)), replay
