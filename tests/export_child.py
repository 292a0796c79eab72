"""Child process of tests/test_export_portable_gpu.py: loads an exported program that this process did
not trace (nothing of the module that was exported exists here), runs it on the saved inputs and writes
the outputs. Usage: python export_child.py <program.pt2> <inputs.pt> <outputs.pt>"""

import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    program, inputs_path, outputs_path = sys.argv[1:4]
    import torch

    import openequivariance_amd  # noqa: F401  (registers the oeq_amd ops the program refers to)
    from openequivariance_amd._torch import ops

    assert not ops._registry, "a fresh process: no kernel set is registered before the program runs"
    ep = torch.export.load(program)
    inputs = torch.load(inputs_path, weights_only=True)
    inputs = tuple(t.cuda() for t in inputs)
    module = ep.module()
    out = module(*inputs)
    assert len(ops._registry) == 1, "the kernel set was rebuilt from the description in the graph"
    # gradients through the loaded program as well (the backward ops receive the same description)
    leaves = tuple(t.detach().clone().requires_grad_(t.is_floating_point()) for t in inputs)
    module(*leaves).sum().backward()
    grads = tuple(t.grad.cpu() for t in leaves if t.is_floating_point())
    torch.save((out.cpu(),) + grads, outputs_path)
    print("child ok", tuple(out.shape))


if __name__ == "__main__":
    main()
