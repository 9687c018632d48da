"""Operator builders and the layer wrapper (reference: python/ditto/auto_compute)."""
from . import nn
from .graph import Layer, layer
