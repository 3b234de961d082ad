"""The layer under HIP graph capture: forward + backward of ``MoELayer`` (router, plan, FP8 dispatch, grouped GEMMs with the
split last round, combine, shared expert on the second stream) captured once with ``torch.cuda.graph`` and replayed on new
inputs.  Nothing in the path synchronises with the host, allocates outside torch's allocator or clears memory with a memset
node, so every replay must reproduce the eager result on the same inputs bit for bit -- replayed several times, with eager
work and synchronisations in between."""

import types

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fp8_dispatch,shared", [(False, 1), (True, 0), (True, 1)])
def test_layer_forward_backward_replays_in_a_hip_graph(gpu, fp8_dispatch, shared):
    from picotron_amd.expert_parallel.expert_parallel import MoELayer

    T, H, I, E, k = 300, 256, 128, 4, 2
    cfg = types.SimpleNamespace(hidden_size=H, intermediate_size=I, num_experts=E, num_experts_per_tok=k, num_shared_experts=shared,
                                norm_topk_prob=True, ep_fp8_dispatch=fp8_dispatch)
    torch.manual_seed(1)
    moe = MoELayer(cfg).cuda().bfloat16()
    with torch.no_grad():
        for p in moe.parameters():
            p.copy_(torch.randn_like(p) * 0.05)
    params = list(moe.parameters())
    g = torch.Generator().manual_seed(2)
    inputs = [(torch.randn(1, T, H, generator=g).bfloat16(), torch.randn(1, T, H, generator=g).bfloat16()) for _ in range(4)]

    def eager(x, up):
        moe.zero_grad(set_to_none=True)
        xin = x.cuda().requires_grad_(True)
        out = moe(xin)
        out.backward(up.cuda())
        return [out.detach().clone(), xin.grad.clone()] + [p.grad.clone() for p in params]

    want = [eager(x, up) for x, up in inputs]

    static_x = inputs[0][0].cuda().requires_grad_(True)
    static_up = inputs[0][1].cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up on the capture's side of the fence: workspaces, weight stacks
        for _ in range(2):
            moe.zero_grad(set_to_none=True)
            static_x.grad = None
            moe(static_x).backward(static_up)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    moe.zero_grad(set_to_none=True)
    static_x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = moe(static_x)
        static_out.backward(static_up)
    static_grads = [static_x.grad] + [p.grad for p in params]
    assert all(t is not None for t in static_grads)
    for i in (1, 2, 3, 0):
        x, up = inputs[i]
        with torch.no_grad():
            static_x.copy_(x.cuda())
            static_up.copy_(up.cuda())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [static_out.detach()] + static_grads
        for a, b in zip(got, want[i]):
            assert torch.equal(a, b), i
        # eager work between the replays, on memory of the ordinary pool
        scratch = torch.randn(1 << 20, device=gpu)
        assert torch.isfinite(scratch.sum())
