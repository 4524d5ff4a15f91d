"""FlexTensor-compatible kernel generation and tuning backend for AMD Instinct
MI355X (gfx950).

Public surface (same names as the reference package):

    from flextensor_amd.task import Task, register_task, TASK_TABLE
    from flextensor_amd.scheduler import schedule, schedule_with_config
    from flextensor_amd.utils import Config
    from flextensor_amd import build          # stands in for tvm.build

Importing the package touches neither torch nor the GPU.
"""
from .plan import build  # noqa: F401

__version__ = "0.1.0"
