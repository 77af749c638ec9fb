"""Rows per token that one layer of a step leaves for later layers of the same step.

A model names such a part among its shared parts (ModelSpec.positions, the named parts that mixers are handed
when they are built); the layer that makes the rows calls put(step, rows), the later ones get(step). Nothing is
kept from one step to the next: rows left in another step are refused.
"""
from __future__ import annotations

from .registry import register_part


class TokenRows:
    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self._step = None
        self._rows = None

    def put(self, step, rows):
        self._step, self._rows = step, rows

    def get(self, step):
        if self._step is not step or self._rows is None:
            raise ValueError("no layer of this step has left its rows yet (the layer that makes them must run first)")
        return self._rows


register_part("position", "token_rows", TokenRows)
