"""Tile-variant choice by measurement, with the reference's tuning-log format
(reference: python/ditto/auto_schedule)."""
from . import schedulers
from .schedulers import chimera_integrate
