"""``torch.compile`` backend that routes a traced model through the manager.

Packaged form of the hook every integration of the reference writes by hand
(examples/ae/scripts/bench_hf_transformers.py:17-58; examples/ae/patch/
vllm.patch:33-64): graphs without a symbolic size are returned untouched, the
scheduler class is loaded from ``config.scheduler_path`` (``"file.py:Class"`` or
``"package.module:Class"``) and constructed as ``Class(config)``, the manager is
initialised inside the backend call and its synchronous callable is returned.

Usage::

    manager = DynaFlowManager()
    backend = make_backend(manager, config)
    torch._dynamo.mark_dynamic(x, 0)
    compiled = torch.compile(model, backend=backend, fullgraph=True)
    manager.prepare(batch_size, num_tokens)      # before EVERY call
    y = compiled(x)
"""
from __future__ import annotations

import importlib
import importlib.util
from collections.abc import Callable
from typing import Any

import torch

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.interface import OpSchedulerBase
from dynaflow_amd.manager import DynaFlowManager


def load_scheduler_class(path: str) -> type[OpSchedulerBase]:
    """Resolve ``"file.py:Class"`` or ``"pkg.module:Class"`` to the class."""
    where, _, cls_name = path.partition(":")
    if not cls_name:
        raise ValueError(f"scheduler_path must look like 'file.py:Class', got {path!r}")
    if where.endswith(".py"):
        spec = importlib.util.spec_from_file_location("_dynaflow_scheduler", where)
        if spec is None or spec.loader is None:
            raise ImportError(f"cannot load scheduler file {where}")
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
    else:
        module = importlib.import_module(where)
    return getattr(module, cls_name)


def make_backend(
    manager: DynaFlowManager,
    config: DynaFlowConfig,
    scheduler: OpSchedulerBase | None = None,
) -> Callable[[torch.fx.GraphModule, list[Any]], Callable]:
    """Build the backend callable for ``torch.compile(..., backend=...)``."""

    def backend(gm: torch.fx.GraphModule, example_inputs: list[Any]) -> Callable:
        if not any(isinstance(v, torch.SymInt) for v in example_inputs):
            return gm
        policy = scheduler if scheduler is not None else load_scheduler_class(config.scheduler_path)(config)
        manager.initialize(
            graph_module=gm,
            config=config,
            scheduler=policy,
            example_inputs=list(example_inputs),
        )
        return manager.get_callable()

    return backend
