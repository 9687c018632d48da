"""Schedule options and scheduler dispatch (reference:
python/ditto/auto_schedule/schedulers/dispatch.py:17-152, schedulers/common.py:34-42,
schedule.py:82-104).

Only the ``"chimera"`` scheduler exists here: it covers the layers that run as fused chains.
Tasks bound to ``"ansor"`` (the reference's generic auto-scheduler for everything else) are outside
this package and are rejected unless that group is empty.
"""
from collections import OrderedDict

from ... import hardware as hw
from .chimera_integrate import auto_schedule_build_tasks as auto_schedule_build_tasks_chimera
from .chimera_integrate import auto_schedule_tasks as auto_schedule_tasks_chimera


class ScheduleOption(object):
    """Same fields and defaults as the reference's (dispatch.py:43-78); ``builder`` / ``runner`` /
    ``target_host`` are kept for call compatibility and not used."""

    def __init__(self, target, target_host="llvm", trials=100, task_name="", log_file="tmp.log", builder="local",
                 runner="local", scheduler=None, verbose=2, device_name=None, dtype="float32",
                 mma_in_dtype="float16", mma_acc_dtype="float32", mma_MI=16, mma_NI=16, mma_KI=16):
        self.target = target
        self.target_host = target_host
        self.trials = trials
        self.task_name = task_name
        self.log_file = log_file
        self.builder = builder
        self.runner = runner
        self.scheduler = scheduler
        self.verbose = verbose
        self.device = hw.query_hw_param(device_name) if device_name is not None else None
        self.dtype = dtype
        self.mma_in_dtype = mma_in_dtype
        self.mma_acc_dtype = mma_acc_dtype
        self.mma_MI = mma_MI
        self.mma_NI = mma_NI
        self.mma_KI = mma_KI


def extract_tasks_from_graph(graph):
    """OrderedDict[layer fingerprint, [layers]] in graph order (common.py:34-42)."""
    tasks = OrderedDict()
    for layer in graph.get_all_layers():
        tasks.setdefault(layer.fingerprint, []).append(layer)
    return tasks


def get_tasks_scheduler_builder(scheduler_name):
    if scheduler_name == "chimera":
        return (auto_schedule_tasks_chimera, auto_schedule_build_tasks_chimera)
    if scheduler_name in (None, "ansor"):
        raise NotImplementedError("the generic (ansor) scheduler is outside this package: only layers that run "
                                  "as fused chains can be scheduled")
    raise ValueError("Scheduler not known: %s.\n" % scheduler_name)


def _bound(bound_tasks):
    for scheduler_name, tasks in bound_tasks.items():
        if len(tasks) == 0:
            continue  # an empty group needs no scheduler
        yield scheduler_name, tasks


def auto_schedule_bound_tasks(bound_tasks, schedule_option):
    """Tune, then build: {workload key: (schedule, schedule_tensors)} (schedule.py:82-104)."""
    ret = {}
    for scheduler_name, tasks in _bound(bound_tasks):
        scheduler, builder = get_tasks_scheduler_builder(scheduler_name)
        scheduler(tasks, schedule_option)
        for k, v in builder(tasks, schedule_option).items():
            assert k not in ret, "The same workload assigned to different schedulers!"
            ret[k] = v
    return ret


def retrieve_schedule_bound_tasks(bound_tasks, schedule_option):
    """Build from the log without measuring (dispatch.py:137-152)."""
    schedules = {}
    for scheduler_name, tasks in _bound(bound_tasks):
        _, builder = get_tasks_scheduler_builder(scheduler_name)
        schedules.update(builder(tasks, schedule_option))
    return schedules
