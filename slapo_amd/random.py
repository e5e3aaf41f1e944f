"""Seed and generator-state management for the HIP dropout kernels.

Mirrors the interface of the reference's slapo/random.py (`CudaRNGStatesTracker`,
`get_cuda_rng_tracker`, `model_parallel_cuda_manual_seed`, `set_random_seed`,
`is_random_seed_set`; reference lines 49-228) and adds `draw_philox`, the one place where a HIP
kernel's (seed, offset) pair is taken from -- and the offset advanced on -- the device's default
generator.  Because the kernels read the very generator that `fork()` swaps in and out, they are
compatible with `.fork_rng()` schedules and with RNG-restoring activation checkpointing without
further plumbing.

The tracker talks to the generator through a small backend object so that its state machine can
be exercised on a machine without a GPU.
"""
from __future__ import annotations

import contextlib
import random as _py_random

import numpy as np
import torch

_MODEL_PARALLEL_RNG_TRACKER_NAME = "model-parallel-rng"


class DeviceGeneratorBackend:
    """The current device's default generator (what torch.nn.functional.dropout draws from)."""

    @staticmethod
    def _gen(device=None):
        idx = torch.cuda.current_device() if device is None else torch.device(device).index
        if idx is None:
            idx = torch.cuda.current_device()
        torch.cuda.init()
        return torch.cuda.default_generators[idx]

    def get_state(self):
        return self._gen().get_state()

    def set_state(self, state):
        # No clone of `state` (reference slapo/random.py:18-46 avoids it for speed).
        self._gen().set_state(state)

    def manual_seed(self, seed):
        torch.cuda.manual_seed(seed)


class CudaRNGStatesTracker:
    """Named snapshots of the device generator state.

    `add(name, seed)` records the state the generator would have right after seeding with
    `seed`; `fork(name)` runs a block under that state and stores the advanced state back, so
    successive forks continue the named stream while the surrounding stream is untouched
    (reference slapo/random.py:49-119).
    """

    def __init__(self, backend=None):
        self.backend = backend if backend is not None else DeviceGeneratorBackend()
        self.states_ = {}
        self.seeds_ = set()

    def reset(self):
        self.states_ = {}
        self.seeds_ = set()

    def get_states(self):
        return dict(self.states_)

    def set_states(self, states):
        self.states_ = states

    def add(self, name, seed):
        if seed in self.seeds_:
            raise Exception(f"seed {seed} already exists")
        if name in self.states_:
            raise Exception(f"cuda rng state {name} already exists")
        self.seeds_.add(seed)
        outer = self.backend.get_state()
        self.backend.manual_seed(seed)
        self.states_[name] = self.backend.get_state()
        self.backend.set_state(outer)

    @contextlib.contextmanager
    def fork(self, name=_MODEL_PARALLEL_RNG_TRACKER_NAME):
        if name not in self.states_:
            raise RuntimeError(
                f"cuda rng state {name} is not added. Did you call 'set_random_seed'?"
            )
        outer = self.backend.get_state()
        self.backend.set_state(self.states_[name])
        try:
            yield
        finally:
            self.states_[name] = self.backend.get_state()
            self.backend.set_state(outer)


_CUDA_RNG_STATE_TRACKER = CudaRNGStatesTracker()


def get_cuda_rng_tracker():
    return _CUDA_RNG_STATE_TRACKER


def model_parallel_cuda_manual_seed(seed, tp_rank, always_enable_tp_seed):
    """Default stream <- `seed` (or the TP seed under sequence parallelism); tracked
    "model-parallel-rng" stream <- seed + 2718 + tp_rank (reference slapo/random.py:131-176)."""
    tp_seed = seed + 2718 + tp_rank
    _CUDA_RNG_STATE_TRACKER.reset()
    torch.cuda.manual_seed(tp_seed if always_enable_tp_seed else seed)
    _CUDA_RNG_STATE_TRACKER.add(_MODEL_PARALLEL_RNG_TRACKER_NAME, tp_seed)
    return tp_seed


def is_random_seed_set():
    return bool(_CUDA_RNG_STATE_TRACKER.get_states())


def set_random_seed(seed=2013, dp_rank=None, pp_rank=None, tp_rank=None,
                    always_enable_tp_seed=False):
    """Per-rank seed arithmetic of the reference (slapo/random.py:184-228): +100 per pipeline
    stage, +10 per data-parallel rank; python / numpy / torch are seeded with the result and,
    when a device is present and tp_rank is given, the device streams are set up."""
    if pp_rank is not None:
        seed += 100 * pp_rank
    if dp_rank is not None:
        seed += 10 * dp_rank
    _py_random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.device_count() > 0 and tp_rank is not None:
        model_parallel_cuda_manual_seed(seed, tp_rank, always_enable_tp_seed)
    return seed


def draw_philox(offset_increment: int, device=None):
    """Take (seed, offset) for one kernel launch from the device's default generator and advance
    its offset by `offset_increment` (a multiple of 4), exactly as an ATen random kernel would.
    Must be called from forward only; backward re-uses the pair saved in the autograd context."""
    if offset_increment % 4 != 0:
        raise ValueError("Philox offset increments are multiples of 4")
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        # The pair is read on the host and baked into the launch: a captured graph would replay
        # one and the same mask.  `draw_philox_state` is the capturable form.
        raise RuntimeError(
            "slapo_amd: draw_philox reads (seed, offset) from the device generator on the host "
            "and cannot be captured into a graph; use draw_philox_state"
        )
    gen = DeviceGeneratorBackend._gen(device)
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + offset_increment)
    return seed, offset


def draw_philox_state(offset_increment: int, device=None):
    """`draw_philox` for the ops of this package: (seed, offset, state).

    Outside a graph capture `state` is None and (seed, offset) are `draw_philox`'s.  While the
    current stream is being captured the pair cannot travel by value (every replay would draw one
    and the same mask), so it lives in device memory instead: `state` is a tensor of two 64-bit
    integers written by a torch random kernel that is captured with the launch and draws from the
    device's default generator, which torch re-seeds for every replay of the graph.  The kernels
    of the op (forward and backward) read {seed, offset} from it when they run; the by-value
    seed and offset are 0 and unused.  A replay's mask is then a function of the generator's
    state at that replay -- fresh per replay, repeatable after `torch.cuda.manual_seed` -- though
    not the mask an eager call would draw from the same state."""
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        if offset_increment % 4 != 0:
            raise ValueError("Philox offset increments are multiples of 4")
        dev = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        state = torch.randint(0, 2 ** 62, (2,), dtype=torch.int64, device=dev)
        return 0, 0, state
    seed, offset = draw_philox(offset_increment, device)
    return seed, offset, None
