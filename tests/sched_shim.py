"""A stand-in for the schedule primitives through which the reference installs this package's
modules: trace (flattening decomposed linears), find a functional pattern, replace the matched
subgraph by a module under the reference's arity rule, replace a whole submodule, fork_rng.
torch.fx only; nothing here is product code.  Behaviour follows the reference's
slapo/primitives/replace.py:48-88 (required arguments of the new module must equal the external
inputs of the matched subgraph), slapo/primitives/fuse.py (the match is handed to `replace`),
slapo/primitives/tensor_parallel.py:183-194 (forward under `tracker.fork()`, `traceable = False`).
"""
import functools
import inspect

import torch
from torch import fx, nn
from torch.fx.passes.utils.matcher_utils import SubgraphMatcher

from slapo_amd import get_cuda_rng_tracker
from slapo_amd.op import LinearWithSeparateBias


def decompose(root: nn.Module, path: str):
    """`.decompose()`: an nn.Linear becomes GEMM + separate bias add (weights shared)."""
    lin = root.get_submodule(path)
    new = LinearWithSeparateBias(lin.in_features, lin.out_features, device=lin.weight.device,
                                 dtype=lin.weight.dtype)
    new.weight, new.bias = lin.weight, lin.bias
    replace_module(root, path, new)
    return new


class _FlattenTracer(fx.Tracer):
    def is_leaf_module(self, m, qualname):
        if isinstance(m, LinearWithSeparateBias):
            return False  # `.trace(flatten=True)`: the bias add shows up in the parent graph
        if getattr(m, "traceable", True) is False:
            return True
        return super().is_leaf_module(m, qualname)


def trace(root: nn.Module) -> fx.GraphModule:
    return fx.GraphModule(root, _FlattenTracer().trace(root))


def find(gm: fx.GraphModule, pattern):
    """Matches of the traced `pattern` function: a list of node lists in graph order."""
    pgraph = fx.symbolic_trace(pattern).graph
    matcher = SubgraphMatcher(pgraph, match_output=False, match_placeholder=False,
                              remove_overlapping_matches=True)
    order = {n: i for i, n in enumerate(gm.graph.nodes)}
    found = []
    for m in matcher.match(gm.graph):
        ops = [n for pn, n in m.nodes_map.items() if pn.op not in ("placeholder", "output")]
        found.append(sorted(ops, key=order.get))
    return found


def required_args(new_mod: nn.Module, ops, concrete_args=None):
    """The arity rule of replace.py:48-88."""
    sig = inspect.signature(new_mod.forward)
    need = [k for k, v in sig.parameters.items()
            if v.default is inspect.Parameter.empty and v.kind is not inspect.Parameter.VAR_POSITIONAL]
    concrete_args = concrete_args or {}
    subgraph_args = []
    for node in ops:
        for arg in node.args:
            if isinstance(arg, fx.Node) and arg not in ops and arg not in subgraph_args:
                subgraph_args.append(arg)
    if len(subgraph_args) + len(concrete_args) != len(need):
        raise ValueError(
            "The number of arguments (w/o default values) of the "
            f"new module ({len(need)}) does not match "
            "the number of arguments of the original subgraph "
            f"({len(subgraph_args)}). Please use `concrete_args` to "
            "specify the arguments."
        )
    return subgraph_args, dict(concrete_args)


def replace_subgraph(gm: fx.GraphModule, ops, new_mod: nn.Module, name: str, concrete_args=None):
    """`.replace(new_mod, subgraph)` / `.fuse(subgraph)`: one call_module node takes the place of
    the matched nodes; its positional arguments are the subgraph's external inputs in order."""
    args, kwargs = required_args(new_mod, ops, concrete_args)
    idx, unique = 0, f"{name}_0"
    while hasattr(gm, unique):
        idx += 1
        unique = f"{name}_{idx}"
    gm.add_module(unique, new_mod)
    last = ops[-1]
    with gm.graph.inserting_after(last):
        node = gm.graph.call_module(unique, tuple(args), kwargs)
    last.replace_all_uses_with(node)
    for n in reversed(ops):
        gm.graph.erase_node(n)
    gm.graph.lint()
    gm.recompile()
    return unique


def replace_module(root: nn.Module, path: str, new_mod: nn.Module):
    """`sch[path].replace(new_mod)` for a whole submodule."""
    parent_path, _, leaf = path.rpartition(".")
    setattr(root.get_submodule(parent_path) if parent_path else root, leaf, new_mod)
    return new_mod


def fork_rng(mod: nn.Module):
    """`sch.fork_rng()`: tensor_parallel.py:183-194."""
    def decorator(func):
        @functools.wraps(func)
        def wrapper(*args, **kwargs):
            with get_cuda_rng_tracker().fork():
                return func(*args, **kwargs)
        return wrapper

    mod.forward = decorator(mod.forward)
    mod.traceable = False
    return mod
