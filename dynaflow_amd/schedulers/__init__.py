"""Scheduling policies shipped with the package."""
from dynaflow_amd.schedulers.nanoflow import NanoFlowScheduler  # noqa: F401
from dynaflow_amd.schedulers.staggered import StaggeredScheduler  # noqa: F401
from dynaflow_amd.schedulers.mlp_overlap import MLPOverlapScheduler  # noqa: F401
from dynaflow_amd.schedulers.decoder_overlap import DecoderOverlapScheduler  # noqa: F401
