"""MI355X-native implementation of DynaFlow's intra-device overlap path.

Public surface (same module layout as the reference package):

    dynaflow_amd.config      DynaFlowConfig, InductorConfig, CUDAGraphConfig
    dynaflow_amd.interface   InputInfo, SplitConfig, OperatorHandle,
                             ExecutionContext, OpSchedulerBase
    dynaflow_amd.matching    Op, Mod, MatchingRule, split_graph, tag_graph
    dynaflow_amd.manager     DynaFlowManager
    dynaflow_amd.utils       pack_tokens

The kernels live in ``libdynaflow_hip.so`` (sources in ``csrc/``, C ABI in
``include/dynaflow_hip.h``) and are reached through ``dynaflow_amd.ops``.
"""
from dynaflow_amd import config as config
from dynaflow_amd import interface as interface
from dynaflow_amd import manager as manager

__version__ = "0.1.0"


def install_as_dynaflow() -> None:
    """Make ``import dynaflow...`` resolve to this package, so that a scheduler or host file written against the
    reference package (``from dynaflow.interface import OpSchedulerBase`` ...) runs without an edit.

    Registers ``dynaflow`` and the reference's sub-module names in ``sys.modules`` (``dynaflow.executor.cudagraph``
    maps to the graph wrapper of this build); refuses if another package of that name is already imported.
    """
    import importlib
    import sys

    own = sys.modules[__name__]
    present = sys.modules.get("dynaflow")
    if present is not None and present is not own:
        raise RuntimeError("another package named 'dynaflow' is already imported")
    names = {
        "dynaflow": __name__,
        "dynaflow.config": f"{__name__}.config",
        "dynaflow.interface": f"{__name__}.interface",
        "dynaflow.manager": f"{__name__}.manager",
        "dynaflow.matching": f"{__name__}.matching",
        "dynaflow.utils": f"{__name__}.utils",
        "dynaflow.runtime": f"{__name__}.runtime",
        "dynaflow.runtime.engine": f"{__name__}.runtime.engine",
        "dynaflow.runtime.env": f"{__name__}.runtime.env",
        "dynaflow.executor": f"{__name__}.executor",
        "dynaflow.executor.compiler": f"{__name__}.executor.compiler",
        "dynaflow.executor.cudagraph": f"{__name__}.executor.hipgraph",
    }
    for alias, target in names.items():
        sys.modules[alias] = importlib.import_module(target)
    # ``import dynaflow.executor.cudagraph`` also looks the sub-module up as an attribute of its parent
    sys.modules["dynaflow.executor"].cudagraph = sys.modules["dynaflow.executor.cudagraph"]
