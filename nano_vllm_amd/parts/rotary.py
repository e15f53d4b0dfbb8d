"""Position encodings.

A position encoding part offers two things to a mixer:
  rotary_table()   a float32 table [positions, head_dim] (cosines, then sines) when the
                   encoding is a rotation of the pairs (i, i + head_dim/2), which the mixer's
                   fused kernel applies itself; None otherwise
  apply(q, k, positions, num_heads, num_kv_heads, head_dim)
                   encodes q [T, heads*head_dim] and k [T, kv_heads*head_dim] in place; the
                   mixer calls it when there is no table

"rotary_neox": nanovllm/layers/rotary_embedding.py:17-48 - inv_freq_i = 1 / theta^(2i/D) and
angle = position * inv_freq_i in float32 whatever the model's element type, pairs (i, i+D/2).
The reference rotates the whole head (qwen3.py:49-54 passes rotary_dim = head_dim); with a
smaller rotary_dim R the table is R wide and the first R channels of a head are rotated, in
pairs (i, i + R/2), the others left as they are.
With scaling_factor every frequency is divided by that constant (positions stretched linearly).
A mixer whose model names no longest sequence asks for step_table(batch) instead of the table of all
positions: the cosines and sines of the step's own tokens, [tokens, R], made once per step by a
kernel that reads the positions on the device (so a captured step makes it anew at every replay) and
shared by all the layers that rotate alike.
"rotary_interleaved": the same angles, the pairs being the neighbours (2i, 2i + 1) of the first R channels.
"none": no encoding.
"""
from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import BuildContext, Part
from .registry import register_part


class RotaryNeox(Part):
    """params: head_dim, theta, max_position (rows of the table), rotary_dim (channels of a head
    that are rotated; default all), scaling_factor (default 1)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.max_position = int(params.get("max_position", build.max_position))
        rotary_dim = params.get("rotary_dim")
        self.rotary_dim = self.head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_neox: {self.rotary_dim} rotated channels of a head of {self.head_dim}: "
                             f"the number must be even and at most the head's")
        # The reference's own float32 expression (rotary_embedding.py:29), evaluated on the host:
        # the angles' rounding is part of the model.
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float) / self.rotary_dim))
        self.scaling_factor = float(params.get("scaling_factor", 1.0))
        if not self.scaling_factor > 0:
            raise ValueError(f"rotary_neox: the scaling factor must be positive, got {self.scaling_factor}")
        if self.scaling_factor != 1.0:
            inv_freq = inv_freq / self.scaling_factor
        self.inv_freq = inv_freq
        self._device = build.device
        self._table = None
        self._inv_freq_dev = None

    def step_table(self, batch) -> torch.Tensor:
        """float32 [tokens, rotary_dim]: cosines, then sines, of the step's tokens at their positions."""
        kept = getattr(batch, "step_cache", None)
        if kept is None:
            kept = batch.step_cache = {}
        key = ("rotary_step", self.rotary_dim, self.theta, self.scaling_factor)
        if key not in kept:
            if self._inv_freq_dev is None:
                self._inv_freq_dev = self.inv_freq.to(self._device)
            kept[key] = self.kernels.rotary_step_table(self._inv_freq_dev, batch.positions)
        return kept[key]

    def rotary_table(self) -> Optional[torch.Tensor]:
        if self._table is None:            # made on first use: building a part touches no device
            self._table = self.kernels.rotary_table(self.inv_freq.to(self._device), self.max_position)
        return self._table

    def apply(self, q, k, positions, num_heads, num_kv_heads, head_dim):
        raise NotImplementedError("rotary_neox is applied through its table")


class RotaryInterleaved(RotaryNeox):
    """The same angles p * theta^(-2i/R), i < R/2, over the first R channels of a head, but the pair that turns by
    angle i is the neighbours (2i, 2i + 1).  Offered through step_table only (the cosines and sines of the step's
    tokens, R/2 cosines and then R/2 sines a row): the mixers' preparation kernels pair the channels."""
    interleaved = True

    def rotary_table(self):
        return None


class NoPositionEncoding(Part):
    def rotary_table(self):
        return None

    def apply(self, q, k, positions, num_heads, num_kv_heads, head_dim):
        return None


register_part("position_encoding", "rotary_neox", RotaryNeox)
register_part("position_encoding", "rotary_interleaved", RotaryInterleaved)
register_part("position_encoding", "none", NoPositionEncoding)
