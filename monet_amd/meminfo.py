"""Per-operator workspace memory and run time, measured on the GPU (reference:
monet/meminfo.py).  These numbers are what the schedule solver trades against
recomputation, so they are taken exactly the way the executor will run the
operator: through the op classes, with the caching allocator's statistics.

  meminfo(...)     -> (fwd MB, bwd MB, fwd-recompute MB)   workspace = peak
                      allocation during the call minus the bytes of what the
                      call returns (meminfo.py:230-243, 366-384)
  computeinfo(...) -> (fwd ms, bwd ms, fwd-recompute ms)   mean of 20 runs
                      between device synchronisations (meminfo.py:42-50)

Each returns one entry per kernel variant for convolutions in "conv" modes
(a variant that fails records run time -1 / memory 0, meminfo.py:52-55,
245-248), an (out-of-place, in-place) pair for operators with an `inplace`
switch in "inplace" modes, first-forward and recompute-forward entries for
BatchNorm, and a single entry otherwise.
"""
import gc
from time import time

import numpy as np
import torch

from . import lm_ops
from .graph import ComputeNode, Param, is_batch_norm, two_step_backward

RUNTIME_SAMPLES = 20


def _concrete(shape, bs):
    return [d if d != -1 else bs for d in list(shape)]


def _build_args(n, graph, bs, bwd_op, params):
    """Operator arguments as the executor would pass them, plus, per argument,
    what is needed to re-create a stand-in later: [shape, requires_grad, device]."""
    device = torch.device("cuda", torch.cuda.current_device())
    split = two_step_backward(n)
    args, meta = [], []
    for a in n.args:
        if isinstance(a, ComputeNode.V):
            args.append(a.value)
            meta.append(a.value)
            continue
        if isinstance(graph.nodes[a.index], Param):
            p = params[a.index]
            if split:
                p = p.requires_grad_(bwd_op == "param_grad")
            args.append(p)
            meta.append([p.shape, p.requires_grad, p.device])
        else:
            shape = _concrete(graph.nodes[a.index].shape, bs)
            grad = a.requires_grad and not (split and bwd_op == "param_grad")
            args.append(torch.randn(shape, device=device).requires_grad_(grad))
            meta.append([shape, grad, device])
    return args, meta


def _storage_list(op):
    s = op.backward_storage
    return s if isinstance(s, list) else [s]


def _required_storage(op, meta, outs):
    req = []
    for storage in _storage_list(op):
        if isinstance(storage, lm_ops.InputStorage):
            req.extend(meta[i] for i in storage.ids)
        elif isinstance(storage, lm_ops.OutputStorage):
            req.append([outs[0].shape, outs[0].requires_grad, outs[0].device, outs[0].dtype])
        elif isinstance(storage, lm_ops.IntermediateStorage):
            assert len(outs) > 1
            req.append([outs[-1].shape, outs[-1].requires_grad, outs[-1].device, outs[-1].dtype])
    return req


def _materialise(required):
    out = []
    for r in required:
        if isinstance(r, list):
            dtype = r[3] if len(r) > 3 else torch.float
            t = torch.ones(list(r[0]), device=r[2], dtype=dtype)
            out.append(t.requires_grad_(r[1]) if dtype.is_floating_point else t)
        else:
            out.append(r)
    return out


def _as_list(outs):
    return list(outs) if isinstance(outs, (tuple, list)) else [outs]


def _bytes(tensors):
    return sum(t.numel() * t.element_size() for t in tensors if t is not None)


def _timed(fn, samples=RUNTIME_SAMPLES, rounds=3):
    """Seconds per call: one untimed call (the allocator fetches what the call needs), then
    the smallest mean of `rounds` batches of `samples` calls.  One slow batch - another
    process's burst, a clock ramp - would otherwise put milliseconds on one operator of the
    profile and send the solver around it (the reference takes one mean of 20,
    monet/meminfo.py:46-60)."""
    torch.cuda.empty_cache()
    fn()
    best = None
    for _ in range(rounds):
        torch.cuda.synchronize()
        t0 = time()
        for _ in range(samples):
            fn()
        torch.cuda.synchronize()
        dt = (time() - t0) / samples
        best = dt if best is None else min(best, dt)
    return best


def _peak_over_outputs(fn):
    """(workspace bytes, outputs) of one call: allocator peak minus returned bytes."""
    gc.collect()   # garbage that is only freed during the call would be taken off its peak
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_stats()['allocated_bytes.all.peak']
    outs = fn()
    torch.cuda.empty_cache()
    peak = torch.cuda.memory_stats()['allocated_bytes.all.peak'] - before
    outs = _as_list(outs)
    return peak - _bytes(outs), outs


def _backward_setup(n, op, meta, outs, bwd_op):
    required = _required_storage(op, meta, outs)
    if bwd_op == "ip_grad" and two_step_backward(n):
        required[0] = None  # the input-gradient step runs without the stored input
    return required, outs[0].shape, outs[0].device


def computeinfo(n, op, graph, bs, bwd_op, conv_mode, inplace_mode, *params):
    """Run times in ms: (forward, backward, recompute-forward)."""
    args, meta = _build_args(n, graph, bs, bwd_op, params)
    if n.is_depthwise:
        op.is_depthwise = True
    runtime_fwd, runtime_fwd_recompute, runtime_bwd = [], [], []
    conv_sweep = conv_mode and n.op == "aten::_convolution" and not n.is_depthwise

    if conv_sweep:
        for alg in range(op.n_fwd_algos()):
            op.algorithm = alg
            try:
                runtime_fwd.append(_timed(lambda: op.forward(*args)))
                if op.algorithm != alg:   # refused for this shape: the operator fell back
                    runtime_fwd[-1] = -1
            except Exception as e:
                print("C: Failed fwd algo", alg, e)
                runtime_fwd.append(-1)
            torch.cuda.empty_cache()
        op.algorithm = 0
        outs = op.forward(*args)
    elif inplace_mode and hasattr(op, 'inplace'):
        for flag in (False, True):
            op.inplace = flag
            runtime_fwd.append(_timed(lambda: op.forward(*args)))
        op.inplace = False
        outs = op.forward(*args)
    elif is_batch_norm(n.op):
        def first_forward():
            op.params = None
            return op.forward(*args)
        runtime_fwd.append(_timed(first_forward))
        op.params = None
        outs = op.forward(*args)  # seeds the saved statistics
        runtime_fwd_recompute.append(_timed(lambda: op.forward(*args)))
    else:
        runtime_fwd.append(_timed(lambda: op.forward(*args)))
        outs = op.forward(*args)

    if bwd_op is not None:
        outs = _as_list(outs)
        required, shape, device = _backward_setup(n, op, meta, outs, bwd_op)
        saved_params = getattr(op, 'params', None)
        del outs, args
        stored = _materialise(required)
        gradin = torch.ones(shape, device=device)
        if hasattr(op, 'params'):
            op.params = saved_params
        step = 10 if bwd_op == "ip_grad" else 0
        if conv_sweep:
            count = op.n_bwd_ip_algos() if bwd_op == "ip_grad" else op.n_bwd_wt_algos()
            for alg in range(count):
                op.algorithm = step + alg
                try:
                    runtime_bwd.append(_timed(lambda: op.backward(gradin, stored, nodel=True)))
                    if op.algorithm != step + alg:   # refused: the operator fell back
                        runtime_bwd[-1] = -1
                except Exception as e:
                    print("C: Failed bwd algo", alg, e)
                    runtime_bwd.append(-1)
                    torch.cuda.empty_cache()
        else:
            if two_step_backward(n):
                op.algorithm = step
            runtime_bwd.append(_timed(lambda: op.backward(gradin, stored, nodel=True)))

    to_ms = lambda v: np.array(v, dtype='f4') * 1000.
    return to_ms(runtime_fwd), to_ms(runtime_bwd), to_ms(runtime_fwd_recompute)


def meminfo(n, op, graph, bs, bwd_op, conv_mode, inplace_mode, *params):
    """Workspace in MB: (forward, backward, recompute-forward)."""
    args, meta = _build_args(n, graph, bs, bwd_op, params)
    if n.is_depthwise:
        op.is_depthwise = True
    fwd_mem, fwd_mem_recompute, bwd_mem = [], [], []
    conv_sweep = conv_mode and n.op == "aten::_convolution" and not n.is_depthwise
    outs = None

    if conv_sweep:
        for alg in range(op.n_fwd_algos()):
            op.algorithm = alg
            try:
                ws, outs = _peak_over_outputs(lambda: op.forward(*args))
                fwd_mem.append(ws)
            except Exception as e:
                print("M: Failed fwd algo", alg, e)
                fwd_mem.append(0)
                torch.cuda.empty_cache()
        if outs is None:
            outs = [torch.zeros(_concrete(n.shape, bs), device=args[0].device)]
    elif inplace_mode and hasattr(op, 'inplace'):
        for flag in (False, True):
            op.inplace = flag
            outs = None
            ws, outs = _peak_over_outputs(lambda: op.forward(*args))
            fwd_mem.append(ws)
    elif is_batch_norm(n.op):
        ws, outs = _peak_over_outputs(lambda: op.forward(*args))       # first forward
        fwd_mem.append(ws)
        outs = None
        ws, outs = _peak_over_outputs(lambda: op.forward(*args))       # same op again: recompute
        fwd_mem_recompute.append(ws)
    else:
        ws, outs = _peak_over_outputs(lambda: op.forward(*args))
        fwd_mem.append(ws)

    if bwd_op is not None:
        required, shape, device = _backward_setup(n, op, meta, outs, bwd_op)
        del outs, args
        split = two_step_backward(n)
        step = -1
        if split:
            step = 10 if bwd_op == "ip_grad" else 0
        count = 1
        if conv_sweep:
            count = op.n_bwd_ip_algos() if bwd_op == "ip_grad" else op.n_bwd_wt_algos()
        for alg in range(count):
            try:
                stored = _materialise(required)
                gradin = torch.ones(shape, device=device)
                if step != -1:
                    op.algorithm = step + alg
                torch.cuda.empty_cache()
                torch.cuda.reset_peak_memory_stats()
                before = torch.cuda.memory_stats()['allocated_bytes.all.peak']
                # the op frees the stored tensors as it consumes them; that belongs to the measure
                grads = op.backward(gradin, stored)
                peak = torch.cuda.memory_stats()['allocated_bytes.all.peak'] - before
                torch.cuda.empty_cache()
                bwd_mem.append(peak - _bytes(_as_list(grads)))
                del gradin, grads
            except Exception as e:
                print("M: Failed bwd algo", alg, e)
                if count == 1:
                    raise RuntimeError("an operator with a single implementation must run") from e
                bwd_mem.append(0)

    to_mb = lambda v: np.array(v, dtype='f8') / 1024. / 1024.
    return to_mb(fwd_mem), to_mb(bwd_mem), to_mb(fwd_mem_recompute)
