"""MI355X-native stage executor behind the JaxPP pipeline-parallel API.

``import jaxpp_amd as jaxpp`` gives ``mark_stage_end``, ``treduce``,
``mpmd_jit_with_loop``, ``MpmdMesh`` and the schedule classes under the
reference's names (see jaxpp_amd/api.py)."""
__version__ = "0.1.0"

_API = ("nn", "optim", "take", "collect_task_times_ms", "mpmd_jit_with_loop", "order_tasks", "validate_schedule",
        "value_and_grad", "DeviceMesh", "MpmdMesh", "mark_stage_end", "pipeline_enter_stage",
        "BaseSchedule", "DualPipeV", "Eager1F1B", "Interleaved1F1B", "KimiK2", "Std1F1B",
        "ZeroBubble", "Add", "Concat", "Max", "treduce", "treduce_i")


def __getattr__(name):
    if name in _API:
        from jaxpp_amd import api
        return getattr(api, name)
    raise AttributeError(f"module 'jaxpp_amd' has no attribute {name!r}")
