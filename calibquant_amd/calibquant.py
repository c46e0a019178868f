"""Operator surface of the reference's `calibquant.py`, backed by HIP kernels.

Same names, argument order, shapes and return dtypes as the reference
(`quant` calibquant.py:24, `fused_kernel` :104, `encode` :115,
`fused_kernel_wv` :269, constants :8-20), so code written as
`from calibquant import quant, fused_kernel, fused_kernel_wv, encode`
(patch_internvl.py:10) runs unchanged against this module.  Every operator
launches hand-written gfx950 kernels through the C-ABI library; there is no
Triton, no torch.compile and no CPU path.

The fused decode path (`calibquant_amd.ops.decode_attn`) does not go through
these four operators; they exist for callers that keep the unfused sequence.
"""
from __future__ import annotations

import torch

from . import ops
from ._lib import CalibQuantError

DATA_TYPE = torch.float16      # dtype of fused_kernel / fused_kernel_wv outputs (calibquant.py:8)
DEVICE = "cuda"                # calibquant.py:11

BITS_KV = 1                    # calibquant.py:13

if BITS_KV == 1:               # calibquant.py:15-20
    SCALE_V = 0.3
    SCALE_K = 0.5
else:
    SCALE_V = 1
    SCALE_K = 1


def quant(x, bits, per_channel=False, scale=1, post_scale=False):
    """b-bit min-max quantiser (calibquant.py:24-42).

    x: (B, T, H, D) bf16 / fp16 GPU tensor (any strides with a contiguous last
    axis).  `per_channel=True` reduces over dim 1, one scale / zero-point per
    (batch, head, channel), shaped (B, 1, H, D); this is the mode the attention
    path uses (patch_internvl.py:181,187).  `per_channel=False` takes one
    minimum and maximum over the whole tensor (calibquant.py:29-31); scale and
    zero_point are then 0-d tensors.
    Returns `(x_q, scale, zero_point)` when `post_scale` is set, else
    `(dequantised x, scale, zero_point)`.
    Arithmetic rounds to x.dtype after every step, as the reference's chain of
    torch ops does."""
    if bits not in (1, 2):
        raise CalibQuantError(f"quant: {bits}-bit codes are not supported (1 or 2)")
    if per_channel:
        x_q, s, z = ops.quant_codes(x, int(bits), float(scale))
    else:
        x_q, s, z = ops.quant_codes_tensor(x, int(bits), float(scale))
    if post_scale:
        return x_q, s, z
    return s * (x_q - z), s, z          # calibquant.py:38, same two torch ops


def encode(X: torch.Tensor, bits=BITS_KV, datum_per_elem=int(8 / BITS_KV)):
    """Pack integer indices along the last axis, `datum_per_elem` per byte,
    first index in the most significant bits (calibquant.py:114-137).
    X: (B, H, T, D) integer tensor (int64 in the reference) -> uint8 (B, H, T, D*bits/8)."""
    if datum_per_elem != 8 // bits:
        raise CalibQuantError("encode: datum_per_elem must equal 8 // bits")
    return ops.encode_indices(X, int(bits))


def fused_kernel(unique_values: torch.Tensor, weights: torch.Tensor, features_enc: torch.Tensor,
                 BITS=BITS_KV, DATUM_PER_ELM=int(8 / BITS_KV)):
    """c[b,h,0,t] = sum_d weights[b,h,0,d] * unique_values[code[b,h,t,d]] (calibquant.py:54-111).
    weights (B, H, 1, D); features_enc uint8 (B, H, T, D*BITS/8) -> fp16 (B, H, 1, T)."""
    B, H = features_enc.shape[0], features_enc.shape[1]
    T = features_enc.shape[-2]
    D = features_enc.shape[-1] * DATUM_PER_ELM
    out = ops.lut_vecmat("qk", unique_values, weights.reshape(B * H, D), features_enc.reshape(B * H, T, -1), int(BITS))
    return out.view(weights.shape[0], weights.shape[1], 1, T)


def fused_kernel_wv(unique_values: torch.Tensor, weights: torch.Tensor, features_enc: torch.Tensor,
                    BITS=BITS_KV, DATUM_PER_ELM=int(8 / BITS_KV)):
    """c[b,h,0,d] = sum_t weights[b,h,0,t] * unique_values[code[b,h,t,d]] (calibquant.py:192-276).
    weights (B, H, 1, T); features_enc uint8 (B, H, T, D*BITS/8) -> fp16 (B, H, 1, D)."""
    B, H = features_enc.shape[0], features_enc.shape[1]
    T = features_enc.shape[-2]
    D = features_enc.shape[-1] * DATUM_PER_ELM
    out = ops.lut_vecmat("pv", unique_values, weights.reshape(B * H, T), features_enc.reshape(B * H, T, -1), int(BITS))
    return out.view(weights.shape[0], weights.shape[1], 1, D)
