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
    # and over all parameters together: the typical parameter is no further than 1.5 times stock
    med_ours = sorted(ours.values())[len(ours) // 2]
    med_stock = sorted(stock.values())[len(stock) // 2]
    assert med_ours <= 1.5 * med_stock + slack, (label, med_ours, med_stock)
    return ours, stock


def run_schedule(cuda, model, x, loss_fn, sol, shape):
    """One forward + backward of `model` (a copy) through MONeTWrapper under the solution file
    `sol`: (wrapper, {name: gradient}, loss, peak MiB of the step without what the caller's
    fixtures hold on the device, model output on the host)."""
    from monet_amd.monet_wrapper import MONeTWrapper
    wrapped = MONeTWrapper(copy.deepcopy(model), sol, shape).to(cuda)
    wrapped.train()
    own = sum(t.numel() * t.element_size() for t in wrapped.state_dict().values()) + \
        x.numel() * x.element_size()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    others = torch.cuda.memory_allocated() - own     # what the fixtures keep on the device
    torch.cuda.reset_peak_memory_stats()
    out = wrapped(x)
    loss = loss_fn(out)
    loss.backward()
    torch.cuda.synchronize()
    peak_mb = (torch.cuda.max_memory_allocated() - others) / 2 ** 20
    got = {k: p.grad.detach().clone() for k, p in wrapped.model.named_parameters()}
    return wrapped, got, float(loss.detach()), peak_mb, out.detach().cpu()


def schedule_choices(wrapped):
    """Signature of what a solution decides about the forward pass besides storing and
    recomputing: per operator its implementation, convolution variant and whether it runs in
    place.  Two schedules with equal signatures run the same forward kernels on the same values
    (every forward kernel is reproducible), with different lifetimes, and must give a
    bit-identical model output."""
    sched = wrapped.schedule[0]
    sol, si = sched.solution, sched.si

    def variant(t, j):
        if not (si.select_conv_algo and j in si.conv_list):
            return -1
        on = [c for c in range(sol.rf.shape[2]) if sol.rf[t, si.conv_list[j], c]]
        return on[0] if on else -1
    return tuple((j, sched._implementation(sol, 0, j), variant(0, j),
                  bool(si.do_inplace and j in si.inplace_list and sol.ip[0][j]))
                 for j in range(si.loss) if sol.r[0][j] and si.solver_to_graph[j] >= 0)


def assert_same_as_unconstrained(run, ref, g64, label):
    """A budgeted schedule against the unconstrained one of the same operator set, same weights
    and batch; `run` and `ref` are (gradients, loss, model output, schedule_choices).  Equal
    forward signatures: the model output bit for bit.  Gradients cannot be held to that: the
    backward convolution kernels that split their reduction add the slices with atomics, so two
    runs of ONE schedule already differ in the last bits, kernel variants and backward
    formulations differ between the schedules, and a deep network amplifies either like any
    other rounding difference.  So each parameter is required to be as close to the float64
    gradient as the unconstrained run is (within a factor 2, plus 1e-5 of the gradient's
    largest entry)."""
    (got, loss, out, fwd), (ref_got, ref_loss, ref_out, ref_fwd) = run, ref
    if fwd == ref_fwd:
        # (the loss itself is torch's: its reduction over a label map adds with atomics, so two
        # evaluations of the same output may differ in the last digit)
        assert torch.equal(out, ref_out), (label, float((out - ref_out).abs().max()))
        assert abs(loss - ref_loss) <= 1e-6 * abs(ref_loss), (label, loss, ref_loss)
    same = sum(1 for n in got if torch.equal(got[n], ref_got[n]))
    a, b = relative_errors(got, g64), relative_errors(ref_got, g64)
    bad = [(n, a[n], b[n]) for n in a if not a[n] <= 2.0 * b[n] + 1e-5]
    print("%s: forward choices %s the unconstrained schedule's; %d of %d gradients bit-identical; "
          "largest error against float64 %.3e (unconstrained %.3e)" % (
              label, "equal (output bit-identical)" if fwd == ref_fwd else "differ from", same,
              len(got), max(a.values()), max(b.values())), flush=True)
    assert not bad, "%s: %d parameters further from float64 than the unconstrained run: %s" % (
        label, len(bad), bad[:5])
