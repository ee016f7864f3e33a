"""Mamba-2 style state-space mixer over the engine's per-sequence state slots.

A mixer layer owns two tensors with one row per state slot (``engine.block_manager.StateSlotPool``
hands a slot to each running sequence): the last ``conv - 1`` inputs of the short convolution and
the f32 recurrent state.  A step's sequences -- prefill chunks of any length and one-token decode
rows alike -- are described by ``AttnMeta.seq_cu`` / ``state_slots``; a sequence whose first row
sits at position 0 starts from a zero state, whatever an earlier owner left in the slot.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import ops


@dataclass
class Mamba2Spec:
    heads: int
    vdim: int          # P: columns of a head's state
    state: int         # N: rows of a head's state
    groups: int        # B / C groups (head h reads group h // (heads / groups))
    conv: int          # taps of the causal convolution over [x | B | C]
    norm_groups: int   # equal parts of the gated output normalised separately

    @classmethod
    def from_dict(cls, m: dict) -> "Mamba2Spec":
        s = cls(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)), int(m.get("conv", 4)),
                int(m.get("norm_groups", 1)))
        if s.heads % s.groups or s.inner % s.norm_groups or not 1 <= s.conv <= 8 or s.state > 256:
            raise ValueError(f"unsupported Mamba-2 sizes {m}")
        return s

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def proj_out(self) -> int:
        """Rows of the input projection: [z | x B C | dt]."""
        return self.inner + self.conv_channels + self.heads

    def make_state(self, slots: int, dtype, device):
        """(conv state [slots, conv - 1, C] in the activation dtype, SSM state f32 [slots, heads, P, N])."""
        return (torch.zeros(slots, max(self.conv - 1, 1), self.conv_channels, dtype=dtype, device=device),
                torch.zeros(slots, self.heads, self.vdim, self.state, dtype=torch.float32, device=device))

    def state_bytes(self, dtype) -> int:
        esz = torch.tensor([], dtype=dtype).element_size()
        return max(self.conv - 1, 1) * self.conv_channels * esz + self.heads * self.vdim * self.state * 4


def mamba2_mixer(h, w_in, conv_w, conv_b, dt_bias, A_log, D, norm_w, w_out, spec: Mamba2Spec, eps: float, state, meta):
    """h [T, W] -> [T, W]: input projection, causal conv + SiLU over [x | B | C], the selective scan
    with an f32 state, gate, grouped RMS norm, output projection.  ``state`` = (conv, ssm) of this
    layer run; dt, the decay and the recurrence are f32."""
    conv_state, ssm_state = state
    u = ops.linear(h, w_in)
    inner, C = spec.inner, spec.conv_channels
    xbc = ops.conv_silu(u, inner, C, conv_w, conv_b, conv_state, meta.seq_cu, meta.state_slots, meta.positions,
                        meta.max_seq_len)
    y = ops.ssm_scan(xbc, u[:, inner + C:inner + C + spec.heads], spec.heads, spec.vdim, spec.state, spec.groups, dt_bias, A_log, D,
                     ssm_state, meta.seq_cu, meta.state_slots, meta.positions, max_len=meta.max_seq_len)
    g = ops.gated_group_rmsnorm(y, u[:, :inner], norm_w, spec.norm_groups, eps)
    return ops.linear(g, w_out)
