"""Configuration records of the scheduling layer.

Field names, order and defaults follow the reference records
(dynaflow/config.py:6-29) so that a scheduler file written against them is
constructed with the same keyword arguments.  Two of the records keep their
historical names although the machinery behind them is different here:

* ``InductorConfig`` selects the *kernel backend* of a sub-graph.  When it is
  enabled the sub-graph is lowered onto the hand-written HIP kernels of this
  package (there is no TorchInductor / Triton code path).
* ``CUDAGraphConfig`` drives hipGraph capture (``torch.cuda.CUDAGraph`` is a
  hipGraph on ROCm).

HIP-specific knobs live in ``DynaFlowConfig.additional_config``:

``hip_backend``        bool, default True: lower matched aten nodes to HIP ops
``gate_up_fusion``     bool, default True: one GEMM for gate and up projection
``whole_graph``        bool, default False: capture the whole multi-stream
                       schedule as ONE hipGraph and replay it per forward
``max_tokens``         rows of the static input buffers used under graphs
``min_nano_split_tokens`` / ``num_nano_batches``  scheduler policy knobs
"""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class CUDAGraphConfig:
    # (dynaflow/config.py:6-11)
    enabled: bool
    capture_sizes: list[int]
    weak_ref_output: bool = True
    check_ptr_consistency: bool = True


#: hipGraph is what actually runs on MI355X; same record under the native name.
HIPGraphConfig = CUDAGraphConfig


@dataclass
class InductorConfig:
    # (dynaflow/config.py:14-20)
    enabled: bool
    compile_sizes: set[int] | None = None
    options: dict | None = None
    disable_remote_cache: bool = True
    disable_autograd_cache: bool = True


#: Native name of the same record: the slot is taken by the HIP kernel backend.
KernelBackendConfig = InductorConfig


@dataclass
class DynaFlowConfig:
    # (dynaflow/config.py:23-29)
    scheduler_path: str
    max_num_splits: int
    inductor_config: InductorConfig
    cudagraph_config: CUDAGraphConfig
    additional_config: dict = field(default_factory=dict)

    def knob(self, name: str, default=None):
        """Read one entry of ``additional_config`` (``None``-safe)."""
        extra = self.additional_config or {}
        return extra.get(name, default)
