"""Tile-variant choice by measurement, with the reference's tuning-log format, and the
task-level entry points of python/ditto/auto_schedule (``ScheduleOption``,
``extract_tasks_from_graph``, ``auto_schedule_bound_tasks``, ``retrieve_schedule_bound_tasks``)."""
from . import schedulers
from .schedulers import chimera_integrate
from .schedulers.dispatch import (ScheduleOption, auto_schedule_bound_tasks, extract_tasks_from_graph,
                                  get_tasks_scheduler_builder, retrieve_schedule_bound_tasks)
