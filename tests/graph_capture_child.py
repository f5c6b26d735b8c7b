"""Run by test_graph_capture.py in a process of its own: captures forward + backward of the MoE layer into a device
graph, replays it for several inputs with eager work and synchronisations between the replays, and compares every
replay with an eager run of a second layer holding the same parameters.  Prints "identical" on success."""

import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch

import flash_model_architectures_amd as xma


def main() -> int:
    torch.manual_seed(0)
    dtype = torch.bfloat16
    E, k, H, I, T = 8, 2, 256, 128, 512
    moe = xma.MoE(E, k, H, I, xma.swiglu_packed, True, False, 0.02).to(dtype).cuda()
    static_x = torch.randn(T, H, device="cuda").to(dtype).requires_grad_()
    d_y = torch.randn(T, H, device="cuda").to(dtype)
    inputs = [torch.randn(T, H, device="cuda").to(dtype) for _ in range(3)]

    def step():
        y, _ = moe(static_x)
        y.backward(d_y)
        return y

    # warm-up on a side stream, as torch asks for before a capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            static_x.grad = None
            moe.zero_grad(set_to_none=True)
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    static_x.grad = None
    moe.zero_grad(set_to_none=True)
    with torch.cuda.graph(graph):
        static_y = step()

    replays = []
    for _ in range(2):
        for inp in inputs:
            with torch.no_grad():
                static_x.copy_(inp)
            graph.replay()
            # the program's own eager work and a synchronisation between replays
            (torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")).sum().item()
            replays.append([t.detach().clone() for t in (static_y, static_x.grad, moe.c_fc.weight.grad,
                                                         moe.c_proj.weight.grad, moe.gate.weight.grad)])

    eager = xma.MoE(E, k, H, I, xma.swiglu_packed, True, False, 0.02).to(dtype).cuda()
    eager.load_state_dict(moe.state_dict())
    for j, got in enumerate(replays):
        x = inputs[j % len(inputs)].clone().requires_grad_()
        eager.zero_grad(set_to_none=True)
        y, _ = eager(x)
        y.backward(d_y)
        want = (y, x.grad, eager.c_fc.weight.grad, eager.c_proj.weight.grad, eager.gate.weight.grad)
        for name, a, b in zip(("y", "dX", "dW up", "dW down", "dW gate"), got, want):
            if not torch.equal(a, b):
                print(f"replay {j}: {name} differs from the eager run by {(a.float() - b.float()).abs().max().item():.3e}")
                return 1
    print("identical")
    return 0


if __name__ == "__main__":
    sys.exit(main())
