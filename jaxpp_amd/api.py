"""Public names, as exported by the reference's ``jaxpp.api``
(src/jaxpp/api.py:19-45), for the part of the system this package builds."""
# ruff: noqa: F401
from jaxpp_amd import __version__, nn, optim
from jaxpp_amd.core import (collect_task_times_ms, mpmd_jit_with_loop, order_tasks,
                            validate_schedule, value_and_grad)
from jaxpp_amd.mesh import DeviceMesh, MpmdMesh
from jaxpp_amd.pipelining import mark_stage_end, pipeline_enter_stage
from jaxpp_amd.schedules import (BaseSchedule, DualPipeV, Eager1F1B, Interleaved1F1B, KimiK2,
                                 Std1F1B, ZeroBubble)
from jaxpp_amd.training import Add, Concat, Max, take, treduce, treduce_i
