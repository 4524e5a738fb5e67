"""HIP-graph capture / replay of the decode forward, in place of the reference's ACL graph wrapper
(src/omni_npu/compilation/acl_graph.py:69-272).

Same dispatch rules: the wrapper trusts ``batch_descriptor`` and ``cudagraph_runtime_mode`` from the forward context,
passes straight through when the mode is NONE or differs from its own, captures on the first call per descriptor and
replays afterwards, and (debug) checks that the input addresses did not move.  What is different on this hardware: the
kernels read sequence lengths, query offsets, block tables and slots from device tensors, so a replay needs no
post-replay host update (the reference pushes padded host lists with ``aclgraph.update``, acl_graph.py:243-262);
``_pad_list`` is kept for callers that still build such lists.  torch.cuda.CUDAGraph is a hipGraph on ROCm.
"""
from __future__ import annotations

import copy
import dataclasses
import logging
import os
from contextlib import ExitStack
from typing import Any, Callable, Optional
from unittest.mock import patch

import torch

from .._vllm_compat import BatchDescriptor, CUDAGraphMode, get_forward_context, weak_ref_tensors

logger = logging.getLogger(__name__)


@dataclasses.dataclass
class HIPGraphEntry:
    batch_descriptor: BatchDescriptor
    graph: Optional[Any] = None
    output: Optional[Any] = None
    input_addresses: Optional[list] = None


@dataclasses.dataclass
class HIPGraphOptions:
    """The reference's options (acl_graph.py:190-222), acted on the same way: ``debug_log_enable`` logs each capture,
    ``gc_disable`` turns ``gc.collect`` and ``torch.cuda.empty_cache`` into no-ops for the duration of a capture (a
    piecewise model captures one graph per layer), ``weak_ref_output`` lets go of the strong reference to the output
    inside the capture (safe for the last graph of a forward only)."""
    debug_log_enable: bool = True
    gc_disable: bool = False
    weak_ref_output: bool = True


class HIPGraphWrapper:
    def __init__(self, runnable: Callable, vllm_config: Any, runtime_mode: CUDAGraphMode, graph_pool: Any = None,
                 cudagraph_options: Optional[HIPGraphOptions] = None):
        self.runnable = runnable
        self.vllm_config = vllm_config
        self.graph_pool = graph_pool
        self.runtime_mode = runtime_mode
        self.compilation_config = getattr(vllm_config, "compilation_config", None)
        self.first_run_finished = False
        self.is_debugging_mode = os.environ.get("VLLM_LOGGING_LEVEL", "INFO") == "DEBUG"
        assert self.runtime_mode != CUDAGraphMode.NONE
        self.graph_options = cudagraph_options or HIPGraphOptions()
        self.concrete_graph_entries: dict = {}

    def __getattr__(self, key: str):
        if hasattr(self.runnable, key):
            return getattr(self.runnable, key)
        raise AttributeError(f"Attribute {key} not exists in the runnable of graph wrapper: {self.runnable}")

    def unwrap(self) -> Callable:
        return self.runnable

    def __call__(self, *args, **kwargs):
        forward_context = get_forward_context()
        batch_descriptor = forward_context.batch_descriptor
        runtime_mode = forward_context.cudagraph_runtime_mode
        if runtime_mode == CUDAGraphMode.NONE or runtime_mode != self.runtime_mode:
            # profile run, warm-up, or a wrapper of another mode is responsible: run eagerly
            return self.runnable(*args, **kwargs)

        entry = self.concrete_graph_entries.get(batch_descriptor)
        if entry is None:
            entry = self.concrete_graph_entries[batch_descriptor] = HIPGraphEntry(batch_descriptor=batch_descriptor)

        if entry.graph is None:
            if self.graph_options.debug_log_enable:
                logger.debug("Capturing a hipGraph on (%s,%s)", self.runtime_mode.name, entry.batch_descriptor)
            entry.input_addresses = [x.data_ptr() for x in args if isinstance(x, torch.Tensor)]
            graph = torch.cuda.CUDAGraph()
            with ExitStack() as stack:
                if self.graph_options.gc_disable:
                    stack.enter_context(patch("gc.collect", lambda: None))
                    stack.enter_context(patch("torch.cuda.empty_cache", lambda: None))
                forward_context.capturing = True
                try:
                    with torch.cuda.graph(graph, pool=self.graph_pool):
                        output = self.runnable(*args, **kwargs)
                        if self.graph_options.weak_ref_output:
                            output = weak_ref_tensors(output)
                finally:
                    forward_context.capturing = False
            # the entry never holds a strong reference: the graph's memory pool owns the bytes
            entry.output = weak_ref_tensors(output)
            entry.graph = graph
            return output

        if self.is_debugging_mode:
            new_input_addresses = [x.data_ptr() for x in args if isinstance(x, torch.Tensor)]
            assert new_input_addresses == entry.input_addresses, (
                f"Input addresses for graphs are different during replay. Expected {entry.input_addresses}, "
                f"got {new_input_addresses}")
        entry.graph.replay()
        return entry.output

    def _pad_list(self, lst, n, v=None):
        if not lst or len(lst) == n:
            return copy.deepcopy(lst)
        if v is None:
            v = lst[-1]
        return (lst + [v] * (n - len(lst))) if len(lst) < n else lst[:n]


ACLGraphWrapper = HIPGraphWrapper      # the reference's class name, for callers that import it
