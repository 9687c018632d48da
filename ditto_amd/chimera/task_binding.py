"""Assign a scheduler to every task (reference: python/ditto/chimera/task_binding.py:6-20)."""
from collections import OrderedDict

from ..auto_compute.nn.module import is_self_attention_layer


def task_binding(tasks):
    """``tasks``: OrderedDict[workload key, [layers]] -> OrderedDict[scheduler, tasks]: attention
    layers go to ``"chimera"`` (the fused chain), everything else to ``"ansor"``."""
    ret = OrderedDict()
    ret["chimera"] = OrderedDict()
    ret["ansor"] = OrderedDict()
    for k, lst in tasks.items():
        if is_self_attention_layer(lst[0]):
            ret["chimera"][k] = lst
        else:
            ret["ansor"][k] = lst
    return ret
