"""Append-in-place full-precision KV window.

The reference grows its residual cache with `torch.cat` on every decode step
(patch_internvl.py:264-266), an O(R) copy per layer per token.  This buffer
keeps capacity ahead of the length and hands out views `(B, H, R, D)`; the
caller still receives and returns plain tensors, so the HF-style
`past_key_value` tuple contract is unchanged."""
from __future__ import annotations

from typing import Optional, Tuple

import torch


class GrowingKV:
    def __init__(self):
        self.k: Optional[torch.Tensor] = None
        self.v: Optional[torch.Tensor] = None
        self.len = 0

    def _owns(self, past) -> bool:
        return (self.k is not None and past is not None and past[0].data_ptr() == self.k.data_ptr()
                and past[0].shape[2] == self.len and past[0].shape[:2] == self.k.shape[:2]
                and past[0].stride() == self.k.stride())

    def reserve(self, past: Optional[Tuple[torch.Tensor, torch.Tensor]], need: int, like: torch.Tensor,
                shape_bh: Tuple[int, int], D: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """Make the buffers hold `past` (None, or a (B, H, R, D) pair) with room for `need` rows in
        all, and return the whole buffers (B, H, capacity, D); rows beyond R are for the caller to fill."""
        R = 0 if past is None else past[0].shape[2]
        if not self._owns(past) or need > self.k.shape[2]:
            B, H = shape_bh
            cap = need + max(256, need // 8)
            k = torch.empty((B, H, cap, D), dtype=like.dtype, device=like.device)
            v = torch.empty_like(k)
            if R:
                k[:, :, :R] = past[0]
                v[:, :, :R] = past[1]
            self.k, self.v = k, v
            self.len = R
        return self.k, self.v

    def append(self, past: Optional[Tuple[torch.Tensor, torch.Tensor]], k_new: torch.Tensor,
               v_new: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """past: None or the (K, V) pair returned earlier (or any (B, H, R, D) pair);
        k_new, v_new: (B, H, n, D).  Returns views of length R + n."""
        B, H, n, D = k_new.shape
        R = 0 if past is None else past[0].shape[2]
        need = R + n
        self.reserve(past, need, k_new, (B, H), D)
        self.k[:, :, R:need] = k_new
        self.v[:, :, R:need] = v_new
        self.len = need
        return self.k[:, :, :need], self.v[:, :, :need]

    def extended(self, need: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """Views of the first `need` rows after the caller filled rows [len, need) in place."""
        self.len = need
        return self.k[:, :, :need], self.v[:, :, :need]
