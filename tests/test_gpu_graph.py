"""The launches are graph-capturable (GPU): no allocation, memset or synchronisation inside the library;
the fused forward's hand-off counters carry a per-launch tag, which a replay repeats.  Each captured call
is replayed several times with new inputs and eager work between the replays, and every replay is
compared with the eager result."""
import pytest
import torch

import rwkv_ops_amd
from rwkv_ops_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu


def _static(xs, device):
    return [x.to(device).clone() for x in xs]


# two-kernel form; fused form with three chunks and with two (the second is then each counter's only reader)
@pytest.mark.parametrize("B,T,H", [(2, 200, 3), (4, 130, 32), (4, 100, 32), (3, 640, 40)])
def test_forward_under_graph_replay(device, B, T, H):
    sets = [make_inputs(B, T, H, 64, seed=40 + i, dtype=torch.bfloat16) for i in range(3)]
    stat = _static(sets[0], device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                        # warm-up on the capture stream
        for _ in range(2):
            rwkv_ops_amd.generalized_delta_rule(*stat[:6], initial_state=stat[6])
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, s_g = rwkv_ops_amd.generalized_delta_rule(*stat[:6], initial_state=stat[6])
    for xs in sets + sets[:1]:
        for dst, src in zip(stat, xs):
            dst.copy_(src.to(device))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_s = o_g.clone(), s_g.clone()
        o_e, s_e = rwkv_ops_amd.generalized_delta_rule(*stat[:6], initial_state=stat[6])   # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got_o, o_e) and torch.equal(got_s, s_e)


def test_decode_under_graph_replay(device):
    B, H, steps = 6, 4, 4
    xs = make_inputs(B, steps, H, 64, seed=50, dtype=torch.bfloat16)
    seq = [x.to(device) for x in xs[:6]]
    state_g = xs[6].to(device).clone()
    state_e = state_g.clone()
    stat = [s[:, 0].contiguous().clone() for s in seq]
    rwkv_ops_amd.rwkv7_decode_step(*stat, state_g.clone())              # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    snapshot = state_g.clone()
    with torch.cuda.graph(graph):
        o_g = rwkv_ops_amd.rwkv7_decode_step(*stat, state_g)
    state_g.copy_(snapshot)                                              # capture does not execute, but be explicit
    for t in range(steps):
        for dst, s in zip(stat, seq):
            dst.copy_(s[:, t])
        graph.replay()
        torch.cuda.synchronize()
        o_e = rwkv_ops_amd.rwkv7_decode_step(*[s[:, t].contiguous() for s in seq], state_e)
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(state_g, state_e)


def test_decode_pool_under_graph_replay(device):
    """A decode step over a pool of states with the slot table on the device: nothing in the call reads the
    table back (a read-back cannot be captured), the replays follow the table's current contents, and every
    replay equals the eager call and the CPU oracle on the gathered states."""
    from oracle import native_c
    from rwkv_ops_amd.synthetic import rel_l2
    B, H, steps, n_state = 5, 4, 3, 9
    xs = make_inputs(B, steps, H, 64, seed=51, dtype=torch.bfloat16)
    seq = [x.to(device) for x in xs[:6]]
    g = torch.Generator().manual_seed(52)
    pool_cpu = 0.1 * torch.randn(n_state, H, 64, 64, generator=g)
    pool_g, pool_e = pool_cpu.to(device), pool_cpu.to(device)
    maps = [[8, 0, 3, 5, 1], [2, 7, 3, 0, 6], [4, 5, 6, 7, 8]]
    smap = torch.tensor(maps[0], dtype=torch.int32, device=device)
    stat = [s[:, 0].contiguous().clone() for s in seq]
    rwkv_ops_amd.rwkv7_decode_step(*stat, pool_g.clone(), state_map=smap)            # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g = rwkv_ops_amd.rwkv7_decode_step(*stat, pool_g, state_map=smap)
    pool_g.copy_(pool_cpu)
    for t in range(steps):
        for dst, s in zip(stat, seq):
            dst.copy_(s[:, t])
        smap.copy_(torch.tensor(maps[t], dtype=torch.int32))
        before = pool_e.cpu()
        graph.replay()
        torch.cuda.synchronize()
        o_e = rwkv_ops_amd.rwkv7_decode_step(*[s[:, t].contiguous() for s in seq], pool_e, state_map=maps[t])
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(pool_g, pool_e)
        o_ref, s_ref = native_c.run(*[x[:, t:t + 1] for x in xs[:6]], before[maps[t]])
        assert rel_l2(o_g[:, None], o_ref) < 5e-3 and rel_l2(pool_g[maps[t]], s_ref) < 5e-3
        untouched = [i for i in range(n_state) if i not in maps[t]]
        assert torch.equal(pool_g[untouched].cpu(), before[untouched])


def test_forward_with_a_device_state_map_under_graph_replay(device):
    B, T, H, n_state = 4, 130, 32, 6
    xs = make_inputs(B, T, H, 64, seed=53, dtype=torch.bfloat16)
    dev = [x.to(device) for x in xs[:6]]
    pool = (0.1 * torch.randn(n_state, H, 64, 64, generator=torch.Generator().manual_seed(54))).to(device)
    smap = torch.tensor([5, 0, 0, 2], dtype=torch.int32, device=device)
    rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=pool, state_map=smap)    # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, s_g = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=pool, state_map=smap)
    for m in ([1, 1, 4, 3], [0, 5, 2, 2]):
        smap.copy_(torch.tensor(m, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        o_e, s_e = rwkv_ops_amd.generalized_delta_rule(*dev, initial_state=pool, state_map=m)
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(s_g, s_e)


def test_backward_under_graph_replay(device):
    B, T, H = 2, 200, 3
    sets = [make_inputs(B, T, H, 64, seed=60 + i, dtype=torch.bfloat16) for i in range(2)]
    stat = _static(sets[0], device)
    g = torch.Generator().manual_seed(1)
    d_o = torch.randn(B, T, H, 64, generator=g).to(torch.bfloat16).to(device)
    d_s = (0.1 * torch.randn(B, H, 64, 64, generator=g)).to(device)
    op = torch.ops.rwkv_ops_amd.rwkv7_bwd
    op(*stat, d_o, d_s)                                                  # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        grads_g = op(*stat, d_o, d_s)
    for xs in sets + sets[:1]:
        for dst, src in zip(stat, xs):
            dst.copy_(src.to(device))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in grads_g]
        ref = op(*stat, d_o, d_s)
        torch.cuda.synchronize()
        for a_, b_ in zip(got, ref):
            assert torch.equal(a_, b_)


def test_float32_backward_under_graph_replay(device):
    """The chunked float32 backward (four launches) captured once; the replays see ordinary decays, then decays too
    strong for the chunk form (the token-by-token kernel takes the call inside the same graph), then ordinary ones
    again: every replay equals the eager call on the same inputs."""
    B, T, H = 2, 100, 2
    sets = [list(make_inputs(B, T, H, 64, seed=70 + i, dtype=torch.float32)) for i in range(3)]
    sets[1][1] = 2.0 + torch.randn(B, T, H, 64, generator=torch.Generator().manual_seed(3))
    stat = _static(sets[0], device)
    g = torch.Generator().manual_seed(1)
    d_o = torch.randn(B, T, H, 64, generator=g).to(device)
    d_s = (0.1 * torch.randn(B, H, 64, 64, generator=g)).to(device)
    op = torch.ops.rwkv_ops_amd.rwkv7_bwd
    op(*stat, d_o, d_s)                                                  # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        grads_g = op(*stat, d_o, d_s)
    for xs in sets + sets[:1]:
        for dst, src in zip(stat, xs):
            dst.copy_(src.to(device))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in grads_g]
        ref = op(*stat, d_o, d_s)
        torch.cuda.synchronize()
        for a_, b_ in zip(got, ref):
            assert torch.isfinite(a_).all() and torch.equal(a_, b_)


def test_calls_overlapping_on_two_streams(device):
    """Forward calls in flight at once on two streams (one-kernel form: workgroups of both launches wait for
    their predecessors while sharing the CUs), each with its own workspace, give the results of the same
    calls made one after the other."""
    xa = [x.to(device) for x in make_inputs(4, 700, 32, 64, seed=31, dtype=torch.bfloat16)]
    xb = [x.to(device) for x in make_inputs(2, 900, 64, 64, seed=32, dtype=torch.bfloat16)]
    with torch.no_grad():
        ref_a = rwkv_ops_amd.generalized_delta_rule(*xa[:6], initial_state=xa[6])
        ref_b = rwkv_ops_amd.generalized_delta_rule(*xb[:6], initial_state=xb[6])
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    with torch.no_grad():
        for _ in range(6):
            with torch.cuda.stream(s1):
                outs_a.append(rwkv_ops_amd.generalized_delta_rule(*xa[:6], initial_state=xa[6]))
            with torch.cuda.stream(s2):
                outs_b.append(rwkv_ops_amd.generalized_delta_rule(*xb[:6], initial_state=xb[6]))
    torch.cuda.synchronize()
    for o, s in outs_a:
        assert torch.equal(o, ref_a[0]) and torch.equal(s, ref_a[1])
    for o, s in outs_b:
        assert torch.equal(o, ref_b[0]) and torch.equal(s, ref_b[1])
