"""Helpers shared by the GPU parity tests: oracle arrays <-> torch tensors."""
import numpy as np
import torch

from oracle import cq_oracle as O

TDT = {"bf16": torch.bfloat16, "fp16": torch.float16}
CLIPS = {1: (0.5, 0.3), 2: (1.0, 1.0)}   # (SCALE_K, SCALE_V) of the reference per bit width


def to_gpu(a, dtype):
    """float32 ndarray of storage-dtype-representable values -> GPU tensor of that dtype (exact)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(TDT[dtype]).cuda()


def to_np(t):
    return t.detach().float().cpu().numpy()


def same_bits(a, b):
    """Equality of two float arrays treating NaN == NaN and +0 == -0 as in value comparison."""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    return bool(np.all((a == b) | (np.isnan(a) & np.isnan(b))))


def make_case(B, Hq, Hkv, D, T, R, bits, dtype, seed, outlier_kind="x10"):
    """Seeded decode-attention case: oracle-side arrays (numpy) of one layer."""
    k, v = O.synth_kv(B, T, Hkv, D, dtype, seed, outlier_kind=outlier_kind)
    ck_, cv_ = CLIPS[bits]
    ck, sk, zk = O.quantize_pack(k, bits, ck_, dtype)
    cv, sv, zv = O.quantize_pack(v, bits, cv_, dtype)
    rng = np.random.default_rng(seed + 1000)
    q = O.round_to(rng.standard_normal((B, Hq, D), dtype=np.float32), dtype)
    kr = O.round_to(rng.standard_normal((B, Hkv, R, D), dtype=np.float32), dtype)
    vr = O.round_to(rng.standard_normal((B, Hkv, R, D), dtype=np.float32), dtype)
    return dict(q=q, ck=ck, cv=cv, sk=sk, zk=zk, sv=sv, zv=zv, kr=kr, vr=vr, k=k, v=v)


def case_to_gpu(c, dtype):
    g = {}
    for n in ("q", "sk", "zk", "sv", "zv", "kr", "vr"):
        g[n] = to_gpu(c[n], dtype)
    g["ck"] = torch.from_numpy(c["ck"]).cuda()
    g["cv"] = torch.from_numpy(c["cv"]).cuda()
    return g


def reference_rope_sequence(x, cos, sin):
    """The torch ops that run at patch_internvl.py:125-128 of the reference (with its rotate_half,
    :110-115, which negates the upper half of its argument in place), on a private copy of x:
    `copy_().mul_(cos)`, in-place `rotate_half`, `addcmul_(tmp, sin)`.  cos / sin broadcast against x."""
    x = x.clone()
    e = torch.empty_like(x)
    e.copy_(x).mul_(cos)
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    x2.neg_()
    tmp = torch.cat((x2, x1), dim=-1)
    e.addcmul_(tmp, sin)
    return e
