"""GPU test of the entry point that allocates nothing, fluxmi_moe_route_sort_static: through the C-ABI its
outputs must equal fluxmi_moe_route_sort's bit for bit, on two calls in a row of which the second is smaller
(the static scratch keeps the first call's contents), and sizes beyond the static array must be rejected."""
import numpy as np
import pytest
import torch

from oracle import configs, routing

pytestmark = pytest.mark.gpu


def _outputs(tokens, topk, experts, dev):
    m = tokens * topk
    i32 = dict(dtype=torch.int32, device=dev)
    return (torch.full((experts,), -7, **i32), torch.full((experts + 1,), -7, **i32), torch.full((tokens, topk), -7, **i32),
            torch.full((m,), -7, **i32), torch.full((m,), -7, **i32))


def test_static_scratch_route_sort_equals_workspace_route_sort_twice():
    from flux_amd import capi
    dev = torch.device("cuda:0")
    assert capi.load().fluxmi_moe_route_sort_static_init() == 0  # the set-up a caller does ahead of a capture
    first = True
    # a large three-kernel case, then smaller ones (two-kernel and single-workgroup paths) on the same scratch
    for name, tokens in (("C4", 40000), ("C4", None), ("C3", None), ("C5", 300), ("C1", None)):
        wl, _ = configs.make_routing(name, tokens=tokens)
        print(f"[case] route_sort_static {name} tokens={wl.tokens} topk={wl.topk} experts={wl.experts}", flush=True)
        choosed = wl.choosed.to(dev)
        out = _outputs(wl.tokens, wl.topk, wl.experts, dev)
        torch.cuda.synchronize()
        # torch's allocator only sees torch's own requests; the device's free memory (hipMemGetInfo) also sees a
        # hipMalloc / hipFree made inside the library
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        capi.route_sort_static(choosed, wl.experts, out)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory changed hands during the call"
        ref = capi.route_sort(choosed, wl.experts)
        for got, want, nm in zip(out, ref, ("splits", "offsets", "scatter_index", "gather_index", "topk_index")):
            assert torch.equal(got, want), f"{name}: {nm} differs from fluxmi_moe_route_sort"
        assert np.array_equal(out[0].cpu().numpy(), wl.splits)
        assert np.array_equal(out[2].cpu().numpy(), wl.scatter_index)
        assert np.array_equal(out[3].cpu().numpy(), wl.gather_index)
        if first:
            # dropped pairs (ids out of range) on the same scratch
            c2 = choosed.clone()
            c2[::7, 0] = wl.experts + 3
            out2 = _outputs(wl.tokens, wl.topk, wl.experts, dev)
            capi.route_sort_static(c2, wl.experts, out2)
            ref2 = capi.route_sort(c2, wl.experts)
            for got, want in zip(out2[:3], ref2[:3]):
                assert torch.equal(got, want)
            first = False


def test_static_scratch_rejects_sizes_beyond_the_array():
    from flux_amd import capi
    lib = capi.load()
    assert lib.fluxmi_moe_route_sort_static_max_bytes() == 4 << 20
    dev = torch.device("cuda:0")
    tokens, topk, experts = 1 << 20, 2, 1024          # (4096 + 1) * 1024 * 4 bytes = 16 MiB of histograms
    assert lib.fluxmi_moe_route_sort_workspace_bytes(tokens, topk, experts) > (4 << 20)
    choosed = torch.zeros(tokens, topk, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="static"):
        capi.route_sort_static(choosed, experts, _outputs(tokens, topk, experts, dev))
