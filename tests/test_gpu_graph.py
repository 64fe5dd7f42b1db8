"""A decode step (append of one token per sequence + fused attention) captured in a HIP graph: every replay equals
the same step launched eagerly on a twin cache."""
import pytest
import torch

from tests.helpers import DT, kv_input

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


@pytest.mark.parametrize("med3x,dn,S,b_r", [(True, "bf16", 24, 3), (False, "fp16", 96, 4)])
def test_graph_replays_equal_eager_steps(med3x, dn, S, b_r):
    """Six replays with eager work and synchronisations between them; after each one the output and every plane of
    the cache equal those of the eagerly driven twin (the captured step holds no memset node: counters and flags are
    cleared by kernels)."""
    import hqmq
    dt = DT[dn]
    B, Hq, Hkv, d_h, T0, steps = 4, 8, 2, 128, 300, 6
    cap = T0 + steps + 2
    inner = hqmq.HQMQ(n_layers=1, n_heads=Hkv, secondary_size=S, radius_bits=b_r, device=DEV)
    w = hqmq.with_outlier_extraction(inner) if med3x else inner
    make = lambda: w.new_cache(B, cap, d_h, dt, 0, sideband_frac=0.5) if med3x else w.new_cache(B, cap, d_h, dt, 0)
    k0 = kv_input((B, Hkv, T0, d_h), dt, seed=1, outlier_p=0.03).to(DEV)
    v0 = kv_input((B, Hkv, T0, d_h), dt, seed=2, outlier_p=0.01).to(DEV)
    start = torch.tensor([T0, T0 - 17, T0 - 130, 5], dtype=torch.int32, device=DEV)       # ragged contexts
    caches = []
    for _ in range(2):
        c = make()
        w.append(c, k0, v0, 0)
        c.crop_(start)
        caches.append(c)
    graph_cache, eager_cache = caches
    news = kv_input((B, Hkv, 2 * (steps + 1), d_h), dt, seed=3, outlier_p=0.05).to(DEV)
    qs = torch.randn(steps + 1, B, Hq, 1, d_h, generator=torch.Generator().manual_seed(4)).to(dt).to(DEV)

    k_buf, v_buf, q_buf = news[:, :, 0:1].clone(), news[:, :, 1:2].clone(), qs[0].clone()
    pos_g, lens_g, out_g = start.clone(), start.clone(), torch.empty_like(q_buf)

    def step(cache, k, v, q, pos, lens, out):
        w.append(cache, k, v, 0, pos=pos)
        lens.copy_(pos)
        lens.add_(1)
        hqmq.fused_attention_packed(q, cache, kv_lens=lens, T_kv=cap, out=out)
        pos.add_(1)

    # warm-up on a side stream (workspaces are allocated here, outside the capture), on a scratch cache
    scratch = make()
    w.append(scratch, k0, v0, 0)
    scratch.crop_(start)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        p, l = start.clone(), start.clone()
        step(scratch, k_buf, v_buf, q_buf, p, l, torch.empty_like(q_buf))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(graph_cache, k_buf, v_buf, q_buf, pos_g, lens_g, out_g)
    # the capture launched nothing: the graph cache is still in its start state
    pos_e, lens_e, out_e = start.clone(), start.clone(), torch.empty_like(q_buf)
    names = ["main", "aux", "scale"] + (["flags", "sideband", "sb_tile_off", "sb_count", "sb_coord"] if med3x else [])
    for i in range(steps):
        k_buf.copy_(news[:, :, 2 * i + 2:2 * i + 3])          # eager work between the replays
        v_buf.copy_(news[:, :, 2 * i + 3:2 * i + 4])
        q_buf.copy_(qs[i + 1])
        graph.replay()
        torch.cuda.synchronize()
        step(eager_cache, k_buf.clone(), v_buf.clone(), q_buf.clone(), pos_e, lens_e, out_e)
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.int16), out_e.view(torch.int16)), f"replay {i}: output"
        assert torch.equal(pos_g, pos_e)
        for a, b in ((graph_cache.K, eager_cache.K), (graph_cache.V, eager_cache.V)):
            for name in names:
                x, y = getattr(a, name), getattr(b, name)
                if x is not None:
                    assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), f"replay {i}: {name}"
