"""The host loops under HIP graph capture: the library allocates nothing, never synchronises
and clears its scratches with kernels, so a forward + backward pass can be recorded once and
replayed.  Every replay, with other work and a synchronisation in between, must reproduce
the eager results."""
import pytest
import torch

from oracle import lvx_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("batched", [False, True])
def test_forward_backward_replays_from_a_graph(batched):
    import lv_xattn as lvx
    from lv_xattn import _lib
    _lib.load()
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    q, k, v, do = (t[n].to(DEV) for n in ("q", "k", "v", "do"))

    def run():
        _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds, batched=batched)
        dq, dk, dv = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash",
                                        rounds=w.rounds, batched=batched)
        return o, L, dq, dk, dv

    eager = [x.clone() for x in run()]           # also fills the host layer's workspace cache
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run()
    for _ in range(3):
        for x in outs:
            x.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want, what in zip(outs[:3], eager[:3], ("O", "LSE", "dQ")):
            assert torch.equal(got, want), what
        for got, want, what in zip(outs[3:], eager[3:], ("dK", "dV")):
            scale = want.float().abs().max().item()
            assert (got.float() - want.float()).abs().max().item() <= 2e-2 * scale, what
