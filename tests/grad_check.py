"""Gradient parity of a whole training step, measured the way that works for deep fp32
networks: float64 autograd on the GPU is the truth, stock fp32 autograd on the same weights
and batch is the yardstick.  Two fp32 evaluations of a deep randomly initialised network
differ from each other by far more than 1e-5 (different summation orders are amplified
layer by layer), so "equal to stock fp32 within 1e-5" is not a property any implementation
has; "no further from the float64 gradient than stock fp32 is" is, and it is what these
helpers assert for EVERY parameter.  (The protocol of the reference's --check_diff,
monet/schedule.py:446-478, prints mean differences against stock fp32 and asserts nothing.)
"""
import copy

import torch


def stock_gradients(model, x, loss_fn, dtype):
    """{name: gradient as float64} and the loss of stock autograd on a copy of `model` in
    `dtype` (training mode: batch statistics)."""
    m = copy.deepcopy(model).to(dtype).train()
    m.zero_grad(set_to_none=True)
    loss = loss_fn(m(x.to(dtype)))
    loss.backward()
    grads = {n: p.grad.detach().double() for n, p in m.named_parameters()}
    value = float(loss.detach())
    del m, loss
    torch.cuda.empty_cache()
    return grads, value


def relative_errors(got, truth):
    """{name: max|got - truth| / max|truth|} (a parameter whose true gradient is all zero -
    e.g. a bias in front of a BatchNorm - is measured against the largest gradient of the
    model instead, since both sides then hold rounding noise only)."""
    top = max(float(t.abs().max()) for t in truth.values())
    out = {}
    for n, t in truth.items():
        scale = float(t.abs().max())
        if scale < 1e-6 * top:
            scale = top
        out[n] = float((got[n].double() - t).abs().max()) / scale
    return out


def assert_no_worse_than_stock(got, g32, g64, label, factor=4.0, slack=1e-5):
    """Every parameter: err(got) <= factor * err(stock fp32) + slack, errors relative to the
    float64 gradient's largest entry.  Prints what was achieved."""
    ours, stock = relative_errors(got, g64), relative_errors(g32, g64)
    worst = max(ours, key=lambda n: ours[n] / (factor * stock[n] + slack))
    print("%s: %d parameters; largest relative error against float64: ours %.3e, stock fp32 "
          "%.3e; median ours %.3e, stock %.3e; tightest parameter %s (ours %.3e, stock %.3e)" % (
              label, len(ours), max(ours.values()), max(stock.values()),
              sorted(ours.values())[len(ours) // 2], sorted(stock.values())[len(stock) // 2],
              worst, ours[worst], stock[worst]), flush=True)
    bad = [(n, ours[n], stock[n]) for n in ours if not ours[n] <= factor * stock[n] + slack]
    assert not bad, "%s: %d parameters further from float64 than stock fp32 allows: %s" % (
        label, len(bad), bad[:5])
    return ours, stock
