"""Drop-in training wrapper (reference: monet/monet_wrapper.py:7-44).

    model = MONeTWrapper(model, solution_file, input_shape).cuda()
    loss = criterion(model(x), target); loss.backward(); optimizer.step()

The forward and backward of `model` are replaced by the compiled schedule in
`solution_file`; everything outside (loss, optimizer) stays ordinary PyTorch:
an autograd Function bridges the two, handing the gradient of the model output
to `Schedule.backward`, which leaves parameter gradients in `.grad`.
"""
import torch

from .schedule import create_schedule
from .solver import Solution  # noqa: F401  (solution files refer to it)


class MONeTWrapperF(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, schedule, state_dict):
        ctx.schedule = schedule
        output = schedule.forward(input_.detach(), *state_dict)
        return output.requires_grad_(True)

    @staticmethod
    def backward(ctx, grad_output):
        ctx.schedule.backward(grad_output)
        return None, None, None


class MONeTWrapper(torch.nn.Module):
    def __init__(self, model, sol_file, input_shape):
        super().__init__()
        if model._get_name() == 'MobileNetV2':
            model = torch.nn.Sequential(
                model.features, torch.nn.AdaptiveAvgPool2d((1, 1)), torch.nn.Flatten(start_dim=1),
                model.classifier[0], model.classifier[1])
        self.model = model
        self.sol_file = sol_file
        self.input_shape = input_shape
        # in a list so that nn.Module does not try to register it
        self.schedule = [create_schedule(model, sol_file, input_shape)]

    def train(self, mode=True):
        self.model.train(mode)
        return self

    def forward(self, x):
        # the Function's output only joins the autograd graph if an input requires grad
        x.requires_grad_(True)
        state = self.state_dict(keep_vars=True)
        return MONeTWrapperF.apply(x, self.schedule[0], list(state.values()))


def reserve_pool(expected_bytes, device=None):
    """Make the caching allocator hold one block of `expected_bytes` before training starts
    and hand it back to the allocator's free list, so that the schedule's tensors are carved
    out of that block instead of out of many smaller segments (the step the reference's
    README.md:60-65 asks its users to do by hand with `torch.zeros(expected_memory / 4)`).
    The block is left uninitialised: only the reservation matters."""
    pool = torch.empty(int(expected_bytes), dtype=torch.uint8,
                       device=device if device is not None else torch.device("cuda"))
    del pool
