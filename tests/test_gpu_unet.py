"""The UNet configuration end to end on the GPU: `UNet(3, 2, 416, 608)`, batch 11, per-pixel
labels, softmax cross entropy over the class dimension, forward + backward through
`MONeTWrapper` under the committed 10 GB and 6 GB schedules.  This is where channel
concatenation, the replicating "upsample" (adaptive average pooling to a multiple of the
input size), 2x2 max pooling with indices, convolutions with bias and the spatial
cross-entropy meet a solver-made schedule.  Reference: models/unet/unet_model.py:8-37,
unet_parts.py:8-63, monet/schedule.py:391, monet/lm_ops/cat.py:5-29."""
import os

import pytest
import torch

from grad_check import (assert_no_worse_than_stock, assert_same_as_unconstrained, run_schedule,
                        schedule_choices, stock_gradients)

pytestmark = pytest.mark.gpu

DATA = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "data")
BS = 11


@pytest.fixture(scope="module")
def unet_case(cuda):
    """Model, batch, labels, and the float64 / stock-fp32 gradients every schedule is
    measured against."""
    from monet_amd.models import build_model
    torch.manual_seed(0)
    model, shape, _ = build_model("unet")
    assert model.n_classes == 2 and tuple(shape) == (3, 416, 608)
    model = model.to(cuda).train()
    gen = torch.Generator(device=cuda).manual_seed(21)
    x = torch.randn((BS,) + tuple(shape), device=cuda, generator=gen)
    labels = torch.randint(0, 2, (BS, shape[1], shape[2]), device=cuda, generator=gen)
    loss_fn = lambda out: torch.nn.functional.cross_entropy(out, labels)
    g64, l64 = stock_gradients(model, x, loss_fn, torch.float64)
    g32, l32 = stock_gradients(model, x, loss_fn, torch.float32)
    print("UNet bs%d loss: float64 %.9f, stock fp32 %.9f" % (BS, l64, l32), flush=True)
    return model, shape, x, labels, loss_fn, g64, g32, l64


_UNCONSTRAINED = {}   # mode -> (gradients, loss, output, choices) of the 100 GB schedule


@pytest.mark.parametrize("budget", [10, 6])
@pytest.mark.parametrize("mode", ["inplace_conv_multiway_newnode",
                                  "fused_inplace_conv_multiway_newnode"])
def test_unet_batch_11_under_the_committed_schedules(cuda, unet_case, mode, budget):
    from monet_amd.graph import ComputeNode
    model, shape, x, labels, loss_fn, g64, g32, l64 = unet_case
    if mode not in _UNCONSTRAINED:
        w0, g0, l0, _, o0 = run_schedule(cuda, model, x, loss_fn, os.path.join(
            DATA, "solution_unet_%d_%s_100.00.pkl" % (BS, mode)), tuple(shape))
        _UNCONSTRAINED[mode] = ({k: v.cpu() for k, v in g0.items()}, l0, o0, schedule_choices(w0))
        del w0, g0
    sol = os.path.join(DATA, "solution_unet_%d_%s_%d.00.pkl" % (BS, mode, budget))
    # weights + batch + activations + workspaces + parameter gradients + the loss's own tensors
    wrapped, got, loss, peak_mb, out = run_schedule(cuda, model, x, loss_fn, sol, tuple(shape))
    ops = {n.op for n in wrapped.schedule[0].nodes if isinstance(n, ComputeNode)}
    assert {"aten::cat", "aten::adaptive_avg_pool2d", "aten::max_pool2d"} <= ops
    assert wrapped.schedule[0].solution.r[1:].sum() > 0 or budget == 10  # 6 GB recomputes
    print("UNet %s %d GB: peak %.1f MiB, loss %.9f" % (mode, budget, peak_mb, loss), flush=True)
    assert peak_mb <= budget * 1024, peak_mb
    assert abs(loss - l64) < 1e-5 * max(1.0, abs(l64))
    assert set(got) == set(g64) and all(bool(torch.isfinite(g).all()) for g in got.values())
    assert_no_worse_than_stock(got, g32, g64, "UNet %s %d GB" % (mode, budget))
    ref_got, ref_loss, ref_out, ref_choices = _UNCONSTRAINED[mode]
    assert_same_as_unconstrained(
        (got, loss, out, schedule_choices(wrapped)),
        ({k: v.to(cuda) for k, v in ref_got.items()}, ref_loss, ref_out, ref_choices), g64,
        "UNet %s %d GB" % (mode, budget))
