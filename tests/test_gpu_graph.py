"""The whole MoE step (route sort -> layer0 -> layer1 -> gather-reduce -> quantisation) captured in a HIP graph.
Every entry point is asynchronous, allocates nothing and never synchronises, so the step is capturable; replays
must reproduce the eager result bit for bit, also with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

from oracle import configs

pytestmark = pytest.mark.gpu


def test_step_in_hip_graph_replays_bit_exact():
    from flux_amd import capi
    wl = configs.make_workload("C1")
    dev = "cuda"
    x, w1, w2 = (wl.tensors[k].to(dev) for k in ("x", "w1", "w2"))
    choosed = wl.choosed.to(dev)
    row_w = wl.row_weight.to(dev)
    m, t, k, e = wl.rows, wl.tokens, wl.topk, wl.experts
    y = torch.empty(m, wl.ffn, dtype=torch.bfloat16, device=dev)
    z = torch.empty(m, wl.hidden, dtype=torch.float32, device=dev)
    out = torch.empty(t, wl.hidden, dtype=torch.bfloat16, device=dev)

    def step():
        splits, _off, scatter, gather, _tki = capi.route_sort(choosed, e)
        capi.grouped_gemm(x, w1, splits, out=y, gather_a=gather)
        capi.grouped_gemm(y, w2, splits, out=z, row_scale=row_w)
        capi.topk_gather_reduce(z, scatter.reshape(-1), k, out=out)
        q, s = capi.quant_e4m3(out)
        return q, s

    q_eager, s_eager = step()          # also performs the one-time kernel attribute set-up outside the capture
    torch.cuda.synchronize()
    out_eager = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        q_g, s_g = step()
    for rep in range(4):
        out.fill_(0)
        y.fill_(0)
        z.fill_(0)
        # eager work of the program between the replays
        _ = (x.float() @ x.float().t()).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, out_eager), f"replay {rep}: output differs from the eager step"
        assert torch.equal(q_g.view(torch.uint8), q_eager.view(torch.uint8)) and torch.equal(s_g, s_eager)


def test_no_alloc_step_with_fused_reduce_in_hip_graph():
    """The step built from the entry points that bring their own scratch: the route sort over the library's static
    scratch array (nothing is allocated inside the capture, by torch or by the library) and layer1 with the top-k
    reduction in the GEMM's epilogue (its fp32 accumulator is cleared by a fill kernel, not a memset node).  Replays
    must give the eager bits (top-2: the two additions commute)."""
    from flux_amd import capi
    wl = configs.make_workload("C1")
    dev = "cuda"
    x, w1, w2 = (wl.tensors[k].to(dev) for k in ("x", "w1", "w2"))
    choosed = wl.choosed.to(dev)
    row_w = wl.row_weight.to(dev)
    m, t, k, e = wl.rows, wl.tokens, wl.topk, wl.experts
    i32 = dict(dtype=torch.int32, device=dev)
    sort_out = (torch.empty(e, **i32), torch.empty(e + 1, **i32), torch.empty(t, k, **i32), torch.empty(m, **i32),
                torch.empty(m, **i32))
    y = torch.empty(m, wl.ffn, dtype=torch.bfloat16, device=dev)
    out = torch.empty(t, wl.hidden, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(t * wl.hidden * 4, dtype=torch.uint8, device=dev)

    def step():
        splits, _off, _scatter, gather, _tki = capi.route_sort_static(choosed, e, sort_out)
        capi.grouped_gemm(x, w1, splits, out=y, gather_a=gather)
        capi.grouped_gemm_topk_reduce(y, w2, splits, gather, t, out=out, workspace=ws, row_scale=row_w)

    step()
    torch.cuda.synchronize()
    out_eager = out.clone()
    assert np.array_equal(sort_out[2].cpu().numpy(), wl.scatter_index)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(4):
        out.fill_(0)
        y.fill_(0)
        ws.fill_(7)
        for o in sort_out:
            o.fill_(-1)
        _ = (x.float() @ x.float().t()).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, out_eager), f"replay {rep}: output differs from the eager step"
        assert np.array_equal(sort_out[3].cpu().numpy(), wl.gather_index)
