"""Per-sub-graph backend objects and the pass that installs them.

* ``SubgraphBackend`` (dynaflow/executor/compiler.py:19-85) is the callable
  stored in ``split_gm.__dict__["submod_<id>"]``.  Calling it dispatches on the
  token count found at ``args[shape_arg_index]``: sizes listed in
  ``compile_sizes`` get their own callable (built lazily, only during a
  dry-run), everything else goes to the dynamic callable.
* ``SubgraphCompiler`` (dynaflow/executor/compiler.py:88-150) interprets the
  split graph once under the ambient fake-tensor mode and wraps every
  sub-module it passes.  It therefore has to run inside the ``torch.compile``
  backend call that produced the graph.

Where the reference compiles a sub-graph with TorchInductor, this build lowers
it onto the HIP operators (``hip_lowering.lower_to_hip``); where it wraps with
CUDA graphs, this build wraps with hipGraphs (``hipgraph.CUDAGraphWrapper``).
"""
from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch
import torch.fx as fx

from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
from dynaflow_amd.executor.hipgraph import CUDAGraphWrapper
from dynaflow_amd.interface import OperatorHandle
from dynaflow_amd.runtime.env import get_op_handle


class SubgraphBackend:
    """Backend wrapper of one FX sub-graph."""

    def __init__(
        self,
        subgraph_gm: fx.GraphModule,
        shape_arg_index: int,
        inductor_config: InductorConfig,
        cudagraph_config: CUDAGraphConfig,
        *,
        use_inductor: bool,
        use_cudagraph: bool,
        lowering_options: dict | None = None,
    ) -> None:
        assert not use_inductor or inductor_config.enabled
        assert not use_cudagraph or cudagraph_config.enabled
        self.gm = subgraph_gm
        tag = getattr(subgraph_gm, "tag", set())
        assert isinstance(tag, set)
        self.tag = tag
        self.shape_arg_index = shape_arg_index
        self.inductor_config = inductor_config
        self.cudagraph_config = cudagraph_config
        self.use_inductor = use_inductor
        self.use_cudagraph = use_cudagraph
        self.callable_dynamic: Callable[..., Any] | None = None
        self.callables_per_size: dict[int, Callable[..., Any]] = {}
        self.lowering_stats: dict[str, int] = {}
        self.lowering_options = dict(lowering_options or {})

    def compile(self, example_inputs: list[Any], runtime_shape: int | None = None) -> Callable[..., Any]:
        """Build the callable for the dynamic shape or for one fixed size."""
        shape = example_inputs[self.shape_arg_index]
        assert (isinstance(shape, torch.SymInt) and runtime_shape is None) or int(shape) == runtime_shape
        fn: Callable[..., Any] = self.gm
        if self.use_inductor:
            from dynaflow_amd.executor.hip_lowering import lower_to_hip

            fn, self.lowering_stats = lower_to_hip(self.gm, **self.lowering_options)
        if self.use_cudagraph:
            fn = CUDAGraphWrapper(fn, self.cudagraph_config)
        return fn

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        assert self.shape_arg_index < len(args)
        size = int(args[self.shape_arg_index])
        sizes = self.inductor_config.compile_sizes
        if sizes is not None and size in sizes:
            fn = self.callables_per_size.get(size)
            if fn is None:
                handle = get_op_handle()
                assert isinstance(handle, OperatorHandle) and handle._is_dryrun, (
                    "a callable for a listed size is built only inside a dry-run (one operator handle in flight)"
                )
                fn = self.callables_per_size[size] = self.compile(list(args), size)
            return fn(*args, **kwargs)
        assert self.callable_dynamic is not None
        return self.callable_dynamic(*args, **kwargs)


class SubgraphCompiler(fx.Interpreter):
    """Walks the split graph in fake mode and installs a backend per sub-module."""

    def __init__(
        self,
        module: fx.GraphModule,
        config: DynaFlowConfig,
        *,
        inductor_compile_targets: list[str],
        cudagraph_targets: list[str],
    ) -> None:
        super().__init__(module)
        from torch._guards import detect_fake_mode

        self.config = config
        self.inductor_compile_targets = set(inductor_compile_targets)
        self.cudagraph_targets = set(cudagraph_targets)
        self.fake_mode = detect_fake_mode()

    def run(self, *args: Any, initial_env: dict[fx.Node, Any] | None = None,
            enable_io_processing: bool = True) -> Any:
        assert self.fake_mode is not None, "SubgraphCompiler must run inside a torch.compile backend call"
        from torch._dispatch.python import enable_python_dispatcher

        fake_args = [
            self.fake_mode.from_tensor(a) if isinstance(a, torch.Tensor) else a for a in args
        ]
        with self.fake_mode, enable_python_dispatcher():
            return super().run(*fake_args)

    def call_module(self, target: Any, args: tuple, kwargs: dict) -> Any:
        assert isinstance(target, str)
        out = super().call_module(target, args, kwargs)
        submod = self.fetch_attr(target)
        assert isinstance(submod, fx.GraphModule)
        # the token count reaches every sub-graph as a symbolic integer argument;
        # the first one found is the size the backend dispatches on
        symbolic = [i for i, a in enumerate(args) if isinstance(a, torch.SymInt)]
        assert len(symbolic) > 0, f"{target} has no symbolic size argument"
        backend = SubgraphBackend(
            submod,
            symbolic[0],
            self.config.inductor_config,
            self.config.cudagraph_config,
            use_inductor=target in self.inductor_compile_targets,
            use_cudagraph=target in self.cudagraph_targets,
            lowering_options={"fuse_silu_epilogue": bool(self.config.knob("fuse_silu_epilogue", False)),
                              "stack_projections": bool(self.config.knob("stack_projections", True))},
        )
        backend.callable_dynamic = backend.compile(list(args))
        self.module.__dict__[target] = backend
        return out
