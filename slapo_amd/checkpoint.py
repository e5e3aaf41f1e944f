"""Activation checkpointing that replays the random streams the HIP dropout kernels draw from.

Interface of the reference's slapo/checkpoint.py (`CheckpointFunctionWithRNGTracker`,
`checkpoint`; reference lines 15-124).  The HIP ops take one (seed, offset) pair per launch from
the device's default generator (`slapo_amd.random.draw_philox`) and keep no mask tensor, so a
recompute yields the same masks exactly when the generator -- and the named streams of the
`CudaRNGStatesTracker`, which `fork()` swaps into that generator -- are put back to where they
stood when the block first ran.  That is all this module does on top of the usual reentrant
checkpoint: `_RngSnapshot` captures the host generator, the device generator and the tracker's
streams; the backward replays the block under the forward's snapshot and then returns every
stream to where the backward found it, so that the recompute leaves no trace in the surrounding
random sequence.
"""
from __future__ import annotations

import contextlib

import torch
from torch.utils.checkpoint import checkpoint as _torch_checkpoint

from .random import get_cuda_rng_tracker, is_random_seed_set


class _RngSnapshot:
    """Host generator state, device generator state and the tracker's named streams at one point
    in time.  The device state goes through the tracker's backend, which sets it without cloning
    (reference slapo/random.py:18-46) and lets the state machine run on a machine without a GPU."""

    __slots__ = ("host", "device", "streams")

    def __init__(self):
        tracker = get_cuda_rng_tracker()
        self.host = torch.get_rng_state()
        self.device = tracker.backend.get_state()
        self.streams = tracker.get_states()

    def restore(self):
        tracker = get_cuda_rng_tracker()
        torch.set_rng_state(self.host)
        tracker.backend.set_state(self.device)
        tracker.set_states(self.streams)

    @contextlib.contextmanager
    def replayed(self):
        """Run a block under this snapshot, then put every stream back where it was."""
        outer = _RngSnapshot()
        self.restore()
        try:
            yield
        finally:
            outer.restore()


class CheckpointFunctionWithRNGTracker(torch.autograd.Function):
    """Reentrant checkpoint of `run_function(*args)`: forward runs without a graph and keeps only
    the tensor arguments; backward runs the function again under the forward's random streams
    and differentiates that second run (reference slapo/checkpoint.py:15-108)."""

    @staticmethod
    def forward(ctx, run_function, *args):
        ctx.run_function = run_function
        ctx.rng = _RngSnapshot()
        with torch.no_grad():
            outputs = run_function(*args)
        # Non-tensor arguments stay in the context; tensors go through save_for_backward as
        # detached aliases, which keeps their storage alive even if the caller (a pipeline
        # engine, say) drops its own reference before the backward.
        ctx.is_tensor = [torch.is_tensor(a) for a in args]
        ctx.plain_args = [None if t else a for a, t in zip(args, ctx.is_tensor)]
        ctx.save_for_backward(*[a.detach() for a in args if torch.is_tensor(a)])
        ctx.needs_grad = [torch.is_tensor(a) and a.requires_grad for a in args]
        return outputs

    @staticmethod
    def backward(ctx, *grad_outputs):
        if not torch.autograd._is_checkpoint_valid():
            raise RuntimeError(
                "Checkpointing is not compatible with .grad(), please use .backward() if possible"
            )
        saved = iter(ctx.saved_tensors)
        inputs = []
        for plain, is_tensor, needs in zip(ctx.plain_args, ctx.is_tensor, ctx.needs_grad):
            if is_tensor:
                t = next(saved).detach()
                t.requires_grad = needs
                inputs.append(t)
            else:
                inputs.append(plain)
        with ctx.rng.replayed(), torch.enable_grad():
            outputs = ctx.run_function(*inputs)
        if torch.is_tensor(outputs):
            outputs = (outputs,)
        pairs = [(o, g) for o, g in zip(outputs, grad_outputs)
                 if torch.is_tensor(o) and o.requires_grad]
        if pairs:
            torch.autograd.backward([o for o, _ in pairs], [g for _, g in pairs])
        return (None,) + tuple(x.grad if torch.is_tensor(x) else None for x in inputs)


def checkpoint(function, *args, use_reentrant=True, **kwargs):
    """Checkpoint `function(*args)`.  Once `set_random_seed` has set up the tracked streams the
    stream-replaying function above is used; before that this is torch's own checkpoint with
    the given arguments (reference slapo/checkpoint.py:111-124)."""
    if not is_random_seed_set():
        return _torch_checkpoint(function, *args, use_reentrant=use_reentrant, **kwargs)
    return CheckpointFunctionWithRNGTracker.apply(function, *args)
