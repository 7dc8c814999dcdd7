"""The layer under HIP graph capture: the library allocates nothing, clears nothing with memset and keeps no
state between calls, so a captured forward pass must replay to the same bits as the eager one -- also after
other work has run in between, and with new inputs written into the captured buffers."""
import pytest
import torch

from tests.gpu_util import DEV, announce, gpu_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,H,I", [(1, 512, 1024), (64, 512, 1024), (300, 512, 1024), (1024, 512, 1024)])
def test_captured_layer_replays_bit_exact(T, H, I):
    from electrock_infer_amd.layers.moe.fused_moe import fused_experts, get_workspace
    announce(f"graph capture T={T}")
    E = 8
    x, lg, w13, w2 = gpu_inputs(T, H, I, E, seed=T)
    ws = get_workspace(x.device, T, H, I, E, 2)
    eager = fused_experts(x, w13, w2, lg, topk=2, workspace=ws).clone()     # also warms up one-time setup calls
    static_x, static_lg = x.clone(), lg.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fused_experts(static_x, w13, w2, static_lg, topk=2, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = fused_experts(static_x, w13, w2, static_lg, topk=2, workspace=ws)
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, eager), f"replay {rep}"
        # eager work of the program between replays, on the same workspace
        other = fused_experts(x.flip(0).contiguous(), w13, w2, lg.flip(0).contiguous(), topk=2, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(other.flip(0), eager)
    # new inputs through the captured buffers
    x2, lg2, _, _ = gpu_inputs(T, H, I, E, seed=T + 1)
    static_x.copy_(x2)
    static_lg.copy_(lg2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(static_out, fused_experts(x2, w13, w2, lg2, topk=2, workspace=ws))


def test_captured_decoder_tail_replays_bit_exact():
    from electrock_infer_amd.layers.moe.fused_moe import fused_experts_normed, get_workspace
    announce("graph capture, norm + gate + experts")
    T, H, I, E = 48, 512, 1024, 8
    x, _, w13, w2 = gpu_inputs(T, H, I, E, seed=5)
    g = torch.Generator(device=DEV).manual_seed(5)
    r = torch.randn(T, H, generator=g, device=DEV).to(torch.bfloat16)
    nw = (1.0 + 0.1 * torch.randn(H, generator=g, device=DEV)).to(torch.bfloat16)
    gw = (torch.randn(E, H, generator=g, device=DEV) * 0.05).to(torch.bfloat16)
    ws = get_workspace(x.device, T, H, I, E, 2)
    out_e, res_e = fused_experts_normed(x, r, nw, 1e-5, gw, w13, w2, topk=2, workspace=ws)
    out_e, res_e = out_e.clone(), res_e.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, res_g = fused_experts_normed(x, r, nw, 1e-5, gw, w13, w2, topk=2, workspace=ws)
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e) and torch.equal(res_g, res_e), f"replay {rep}"
        fused_experts_normed(x, r, nw, 1e-5, gw, w13, w2, topk=2, workspace=ws)
        torch.cuda.synchronize()


def test_graphs_of_two_batch_sizes_through_the_module_share_the_workspace():
    """The usual capture pattern of an engine: eager warm-up and capture at one batch size, then at a larger one,
    through FusedMoE.forward (which takes no workspace argument and uses the device's shared one).  The larger batch
    makes the shared buffer grow; the first graph still holds the old address, so that buffer must stay alive: the
    first graph, replayed after the second was captured and run, has to give its eager result -- also after other
    allocations had the chance to land on freed memory."""
    from electrock_infer_amd import FusedMoE
    from electrock_infer_amd.layers.moe import fused_moe
    announce("graph capture of two batch sizes through FusedMoE.forward")
    H, I, E = 512, 1024, 8
    fused_moe.release_workspaces(DEV)          # start from an empty cache so that the second size does grow it
    x, lg, w13, w2 = gpu_inputs(96, H, I, E, seed=21)
    layer = FusedMoE(E, 2, H, I, tp_size=1, params_dtype=torch.bfloat16).to(DEV)
    layer.w13_weight.data, layer.w2_weight.data = w13, w2
    graphs = []
    for T in (8, 96):
        xs, ls = x[:T].clone(), lg[:T].clone()
        eager = layer(xs.clone(), ls).clone()
        buf = xs.clone()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = layer(buf, ls)                # in place: out is buf
        graphs.append((g, buf, xs, eager))
    assert len(fused_moe._retired.get(torch.device(DEV).index, [])) >= 1     # the buffer did grow in between
    junk = [torch.randn(1 << 20, device=DEV) for _ in range(8)]              # would reuse a freed workspace
    for rep in range(2):
        for g, buf, xs, eager in graphs:
            buf.copy_(xs)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(buf, eager), f"replay {rep}"
    del junk


def test_shared_workspace_refuses_to_grow_under_capture():
    """A batch size the shared workspace has not seen, first met under capture: the buffer would be allocated from
    the graph's private pool and then serve eager calls too, so the layer raises instead and names the remedy."""
    from electrock_infer_amd.layers.moe import fused_moe
    announce("graph capture, workspace growth refused")
    H, I, E = 512, 1024, 8
    fused_moe.release_workspaces(DEV)
    x, lg, w13, w2 = gpu_inputs(128, H, I, E, seed=9)
    fused_moe.fused_experts(x[:8].contiguous(), w13, w2, lg[:8].contiguous(), topk=2)      # sizes the buffer for 8 tokens
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="reserve_workspace"):
        with torch.cuda.graph(g):
            fused_moe.fused_experts(x, w13, w2, lg, topk=2)
    torch.cuda.synchronize()
    fused_moe.reserve_workspace(DEV, 128, H, I, E, 2)
    eager = fused_moe.fused_experts(x, w13, w2, lg, topk=2).clone()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        out = fused_moe.fused_experts(x, w13, w2, lg, topk=2)
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
