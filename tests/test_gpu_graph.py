"""The expert block's forward captured in a HIP graph: the library allocates nothing, clears
nothing with memsets and never synchronises, and the default path keeps the group sizes on the
device, so the whole of forward_stage3 (index kernels, quantisations, grouped GEMMs, scattered
store) can be recorded once and replayed.  Every replay, with the program's own eager work and
synchronisations in between, must equal the eager result bit for bit."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_forward_stage3_replays_from_a_graph_bit_for_bit():
    from oracle import moe as OM
    from pith_train_amd.dualpipe_utils import FP8WeightCacheControl
    from pith_train_amd.modules import experts as X

    E, H, I, T, k = 16, 512, 256, 512, 4
    g = torch.Generator().manual_seed(11)
    mod = X.Qwen35MoeExperts(H, I, E).cuda().to(torch.bfloat16)
    with torch.no_grad():
        mod.gate_up_proj.weight.copy_((torch.randn((E, 2 * I, H), generator=g) * 0.02).bfloat16())
        mod.down_proj.weight.copy_((torch.randn((E, H, I), generator=g) * 0.02).bfloat16())
    FP8WeightCacheControl.step()
    inputs = [(torch.randn((T * k, H), generator=g).bfloat16().cuda(),
               OM.make_routing(T, E, k, seed=s).reshape(-1).cuda()) for s in range(4)]

    def run(tokens, eidx):
        with torch.no_grad():
            return X.forward_stage3(mod, tokens, eidx, E)

    eager = [run(t, e).clone() for t, e in inputs]  # also the warm-up: one-time kernel attributes, weight cache
    torch.cuda.synchronize()

    static_tok, static_idx = inputs[0][0].clone(), inputs[0][1].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # a few runs on the capture stream first, as graph capture wants
        for _ in range(2):
            run(static_tok, static_idx)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = run(static_tok, static_idx)

    for n, (tokens, eidx) in enumerate(inputs + inputs[:2]):
        static_tok.copy_(tokens)
        static_idx.copy_(eidx)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, eager[n % len(inputs)]), f"replay {n} differs from the eager result"
        # the program's own eager work between replays
        again = run(tokens, eidx)
        torch.cuda.synchronize()
        assert torch.equal(again, eager[n % len(inputs)])
