"""The whole hot path captured in a HIP graph (through torch.cuda.CUDAGraph) and replayed: every replay must give
bit for bit what the same calls give when run eagerly on the same inputs, with eager work between the replays.
No entry point of the path synchronises the host or enqueues a memset, which is what makes it capturable."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_hot_path_replays_in_a_graph():
    from mole_amd import hip_ops as H
    S, M, E, k, Fd = 1024, 256, 8, 2, 512
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(7)
    rnd = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc)
    x = rnd(S, M).to(dt).cuda()
    dy = rnd(S, M, sc=1e-2).to(dt).cuda()
    wg = rnd(E, M, sc=0.05).cuda()
    w1, b1 = rnd(E, Fd, M, sc=0.05).to(dt).cuda(), rnd(E, Fd, sc=0.05).to(dt).cuda()
    w2, b2 = rnd(E, Fd, M, sc=0.05).to(dt).cuda(), rnd(E, M, sc=0.05).to(dt).cuda()
    gw1, gb1 = torch.empty_like(w1), torch.empty_like(b1)
    gw2, gb2 = torch.empty_like(w2), torch.empty_like(b2)

    def step():
        scores = H.gate_fwd(x, wg)
        r = H.route(scores, k, 1.0)
        xd = H.dispatch_fwd(x, r.row, S * k)                      # S*k rows bound the kept rows: no host sync
        out, h, a = H.ffn_fwd(xd, r.offsets, r.kept_rows, w1, b1, w2, b2)
        y = H.combine_fwd(out, r.row, r.gates)
        d_o, dgates = H.combine_bwd(dy, out, r.row, r.gates)
        gx = H.ffn_bwd(d_o, xd, h, a, r.offsets, r.kept_rows, w1, w2, gw1, gb1, gw2, gb2)
        dlogits = H.gate_bwd(dgates, scores, r.idx, True)
        dx = H.dispatch_bwd(gx, r.row, dlogits, wg)
        dwg = H.gate_wgrad(dlogits, x)
        return [y, dx, dwg, gw1, gb1, gw2, gb2, r.row, r.l_aux]

    want0 = [t.clone() for t in step()]                            # also warms up every kernel before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(4):
        if rep:                                                    # new inputs in the captured buffers
            x.copy_(rnd(S, M).to(dt))
            dy.copy_(rnd(S, M, sc=1e-2).to(dt))
        want = want0 if rep == 0 else [t.clone() for t in step()]  # eager work between the replays
        torch.cuda.synchronize()
        for t in (gw1, gb1, gw2, gb2):
            t.fill_(7.0)                                           # the replay must rewrite them
        graph.replay()
        torch.cuda.synchronize()
        for i, (got, exp) in enumerate(zip(outs, want)):
            assert torch.equal(got, exp), f"replay {rep}, output {i}"
