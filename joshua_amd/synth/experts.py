"""Stacks of synthetic experts with distinct bytes, cheap to make at full model size.

A DeepSeek-V3-shaped layer holds 257 experts of 11 to 23 MB each: quantising that many
normal matrices takes minutes, and repeating one expert makes every expert's bytes equal,
which hides a kernel that reads the wrong expert.  Here one expert is quantised from
N(0, sigma) and expert e is that template with the packed quants of every block rotated
by e bytes (and, once the rotations repeat, moved on by seven blocks): the scales stay
where they are (so the weights keep their magnitude), every byte pattern is a valid
block, and no two experts hold the same bytes.  The host side
builds single experts on demand (for the CPU check of the routed ones), the device side
the whole stack.
"""
from __future__ import annotations

import numpy as np

# (block bytes, first and one-past-last byte of the packed quants that are rotated)
_PAYLOAD = {
    8: (34, 2, 34),       # Q8_0:    d | qs[32]
    10: (84, 16, 80),     # Q2_K:    scales[16] | qs[64] | d | dmin
    12: (144, 16, 144),   # Q4_K:    d | dmin | scales[12] | qs[128]
    14: (210, 0, 192),    # Q6_K:    ql[128] | qh[64] | scales[16] | d
    16: (66, 2, 66),      # IQ2_XXS: d | 8 x (codes, signs + scale)
    39: (17, 1, 17),      # MXFP4:   e | qs[16]
}


class RolledExperts:
    """`n_expert` experts of `template.size` bytes each; expert 0 is the template."""

    def __init__(self, qtype: int, template: np.ndarray, n_expert: int):
        self.block_bytes, self.lo, self.hi = _PAYLOAD[qtype]
        self.template = np.ascontiguousarray(template, dtype=np.uint8).reshape(-1, self.block_bytes)
        self.n_expert, self.per = n_expert, self.template.size

    @property
    def size(self) -> int:
        return self.per * self.n_expert

    def _shifts(self, e: int) -> tuple[int, int]:
        span = self.hi - self.lo
        return (7 * (e // span)) % self.template.shape[0], e % span

    def expert(self, e: int) -> np.ndarray:
        out = self.template.copy()
        out[:, self.lo:self.hi] = np.roll(self.template[:, self.lo:self.hi], self._shifts(e), axis=(0, 1))
        return out.reshape(-1)

    def __getitem__(self, sl: slice) -> np.ndarray:
        """The bytes of one expert, addressed as the slice of the stack that holds it."""
        e, rem = divmod(sl.start, self.per)
        if rem or sl.stop - sl.start != self.per:
            raise IndexError("RolledExperts serves whole experts only")
        return self.expert(e)

    def device_stack(self, torch, device):
        """uint8 tensor [n_expert * per] on `device`, built there from the template."""
        t = torch.from_numpy(self.template).to(device)
        out = torch.empty((self.n_expert, self.template.shape[0], self.block_bytes), dtype=torch.uint8, device=device)
        out[:] = t
        for e in range(1, self.n_expert):
            out[e, :, self.lo:self.hi] = torch.roll(t[:, self.lo:self.hi], self._shifts(e), dims=(0, 1))
        return out.reshape(-1)
