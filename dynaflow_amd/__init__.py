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
