"""Execution backends of a sub-graph: HIP kernel lowering and hipGraph replay."""
from dynaflow_amd.executor.compiler import SubgraphBackend, SubgraphCompiler  # noqa: F401
