"""Glue between AOT autograd and the passes: the joint forward/backward graph
is optimised as one graph, then split.

Same surface as the reference's python/gtl/helper/aot_helper.py:24-33
(`partition_func(joint_module, joint_inputs, joint_compiler, **kwargs)`,
`compiler_fn(fx_module, _)`), used as in its model tests
(unittest/fx_passes/xmlcnn.py:48-62, 82-89):

    model = aot_module(model, compiler_fn, compiler_fn,
                       partial(partition_func, joint_compiler=joint_optimization))
"""
from __future__ import annotations

import logging
from functools import partial
from typing import Callable

import torch
import torch.fx as fx
from functorch.compile import aot_module, make_boxed_func
from torch._functorch.partitioners import default_partition

from .passes import GTLFrontend, pass_cse, pass_decomposition, pass_fusion


def partition_func(joint_module: fx.GraphModule, joint_inputs, joint_compiler: Callable, **kwargs):
    """Runs `joint_compiler` on the joint graph in place, then splits it where
    the original forward ended."""
    joint_compiler(joint_module)
    fw, bw = default_partition(joint_module, joint_inputs, **kwargs)
    for gm in (fw, bw):
        _drop_unused_random(gm)
    return fw, bw


def _drop_unused_random(gm: fx.GraphModule) -> None:
    """torch.fx never removes random ops as dead code, so the split leaves a
    copy of every `rand_like` the forward graph still runs eagerly in the
    backward graph as well, its result unused (the backward reads the saved
    mask).  An unused draw only costs time: remove it, and what it kept alive."""
    changed = False
    for node in reversed(list(gm.graph.nodes)):
        if node.op == "call_function" and not node.users and "rand" in getattr(node.target, "__name__", str(node.target)):
            gm.graph.erase_node(node)
            changed = True
    if changed:
        gm.graph.eliminate_dead_code()
        gm.recompile()


def compiler_fn(fx_module: fx.GraphModule, _):
    """Forward / backward 'compiler': the graphs already hold the fused
    kernels, so they run as they are."""
    logging.debug("============Optimized Source Code============")
    logging.debug(fx_module.code)
    return make_boxed_func(fx_module)


def joint_optimization(joint_module: fx.GraphModule) -> fx.GraphModule:
    """The pass pipeline of the reference's model tests, without the passes
    that belong to other anchors: frontend -> decomposition -> CSE -> fusion."""
    joint_module, _ = GTLFrontend()(joint_module)
    pass_decomposition(joint_module, joint_module.graph)
    pass_cse(joint_module, joint_module.graph)
    pass_fusion(joint_module, joint_module.graph)
    return joint_module


def aot_optimize(model: torch.nn.Module, joint_compiler: Callable = joint_optimization) -> torch.nn.Module:
    """`model` with forward and backward traced by AOT autograd and every
    mm / bmm of the joint graph fused with its epilogue."""
    return aot_module(model, compiler_fn, compiler_fn, partial(partition_func, joint_compiler=joint_compiler))


def evt_backend(gm: fx.GraphModule, example_inputs):
    """Backend for `torch.compile(model, backend=evt_backend)`: Dynamo's graph
    goes through AOT autograd with the same joint pipeline as `aot_optimize`."""
    from torch._dynamo.backends.common import aot_autograd
    return aot_autograd(fw_compiler=compiler_fn, bw_compiler=compiler_fn,
                        partition_fn=partial(partition_func, joint_compiler=joint_optimization))(gm, example_inputs)


class _Captured(Exception):
    pass


def aot_capture(model: torch.nn.Module, example_inputs, joint_compiler: Callable = joint_optimization) -> dict:
    """Trace, optimise and split `model` as `aot_optimize` does, but stop
    before anything runs: returns {"joint", "fw", "bw"} graph modules.  Works
    without a GPU (the fused kernels are only built or launched when called)."""
    box: dict = {}

    def capture(joint_module, joint_inputs, **kwargs):
        fw, bw = partition_func(joint_module, joint_inputs, joint_compiler, **kwargs)
        box.update(joint=joint_module, fw=fw, bw=bw)
        raise _Captured()

    try:
        aot_module(model, compiler_fn, compiler_fn, capture)(*example_inputs)
    except _Captured:
        pass
    return box
