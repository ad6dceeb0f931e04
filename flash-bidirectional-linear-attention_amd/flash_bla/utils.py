"""Helpers shared by the operator wrappers (counterpart of flash_bla/utils.py:9-15,45-67)."""
import functools
import warnings

import torch


def contiguous(fn):
    """Make every tensor argument of an autograd forward/backward contiguous
    (flash_bla/utils.py:9-15)."""
    @functools.wraps(fn)
    def wrapper(ctx, *args, **kwargs):
        args = tuple(a.contiguous() if isinstance(a, torch.Tensor) else a for a in args)
        kwargs = {n: (a.contiguous() if isinstance(a, torch.Tensor) else a) for n, a in kwargs.items()}
        return fn(ctx, *args, **kwargs)
    return wrapper


def _rms(t):
    return t.detach().double().flatten().pow(2).mean().sqrt().item()


def get_abs_err(x, y):
    """Largest absolute difference between two tensors (name kept from flash_bla/utils.py:45)."""
    return torch.max(torch.abs(x.detach() - y.detach())).item() if x.numel() else 0.0


def get_err_ratio(x, y):
    """RMS of the difference relative to the RMS of `x`, guarded against a zero `x` by 1e-8
    (name kept from flash_bla/utils.py:49)."""
    return _rms(x.detach() - y.detach()) / (_rms(x) + 1e-8)


def get_max_rel_err(ref, x):
    """max|x - ref| / max|ref|: the parity figure used for the HIP kernels."""
    ref = ref.detach().double()
    x = x.detach().double()
    return ((x - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def assert_close(prefix, ref, tri, ratio, warning=False, err_atol=1e-6):
    """Acceptance rule of the layers' self-tests (flash_bla/utils.py:55-67), as a decision table:

      largest difference <= err_atol                        pass, returns that difference
      RMS ratio < ratio                                     pass, returns the ratio
      RMS ratio >= ratio, and `warning` or the result is
        close in either sense (ratio < 1 %, diff <= 0.3)    pass with a warning, returns the ratio
      otherwise                                             AssertionError
    """
    worst = get_abs_err(ref, tri)
    if worst <= err_atol:
        return worst
    rel = get_err_ratio(ref, tri)
    report = f"{prefix:>8} diff: {worst:.6f} ratio: {rel:.6f}"
    tolerated = warning or rel < 0.01 or worst <= 0.3
    if rel > ratio and tolerated:
        warnings.warn(report)
    elif not tolerated:
        assert rel < ratio, report
    return rel


class CapturedForward:
    """An inference forward of `module` recorded once into a HIP graph and replayed per call.

    The blocks around the operators (projections, norms, activations) are a few dozen short
    kernels; at the LinFusion shapes their launch overhead is most of the block's time.  The
    operators enqueue on the current stream, allocate through torch and never synchronise, so
    torch's graph capture records them like any other kernel.  Inputs are copied into the
    recorded input tensors, the result is the recorded output tensor (overwritten by the next
    call).  Shapes, dtypes and keyword arguments are fixed at construction."""

    def __init__(self, module, *example_inputs, warmup=3, **kwargs):
        self._static_in = [t.clone() for t in example_inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(side):
            for _ in range(warmup):  # lazy initialisation (LDS attributes, caches) happens here
                module(*self._static_in, **kwargs)
        torch.cuda.current_stream().wait_stream(side)
        self._graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self._graph):
            self._static_out = module(*self._static_in, **kwargs)

    def __call__(self, *inputs):
        for dst, src in zip(self._static_in, inputs):
            dst.copy_(src)
        self._graph.replay()
        return self._static_out


class CapturedStep:
    """Forward and backward of `fn` recorded once into one HIP graph and replayed per call.

    For short sequences a training step of an operator is six short kernels whose launches,
    together with the autograd bookkeeping around them, can take the host longer than the GPU
    needs to run them; a replay is one launch.  `fn(*inputs)` must return one tensor.  Inputs
    and the output gradient are copied into recorded tensors; the call returns the recorded
    output and the recorded gradients of the inputs that require them (None for the others),
    all overwritten by the next call.  Shapes and dtypes are fixed at construction."""

    def __init__(self, fn, example_inputs, example_grad_output, warmup=3):
        self._static_in = [t.detach().clone().requires_grad_(t.requires_grad) for t in example_inputs]
        self._static_gout = example_grad_output.detach().clone()
        self._leaves = [t for t in self._static_in if t.requires_grad]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):  # lazy initialisation (LDS attributes, caches) happens here
                torch.autograd.grad(fn(*self._static_in), self._leaves, self._static_gout)
        torch.cuda.current_stream().wait_stream(side)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._static_out = fn(*self._static_in)
            grads = torch.autograd.grad(self._static_out, self._leaves, self._static_gout)
        grads = iter(grads)
        self._static_grads = [next(grads) if t.requires_grad else None for t in self._static_in]

    def __call__(self, inputs, grad_output):
        with torch.no_grad():
            for dst, src in zip(self._static_in, inputs):
                dst.copy_(src)
            self._static_gout.copy_(grad_output)
        self._graph.replay()
        return self._static_out, self._static_grads

    def replay(self):
        """Replays the step on the recorded tensors as they are (no copies)."""
        self._graph.replay()
        return self._static_out, self._static_grads
