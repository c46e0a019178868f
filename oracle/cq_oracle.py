"""CPU oracle for CalibQuant's quantized-KV decode path (numpy).

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP kernels are
compared against.  Only the test-suite, the smoke entry and the CPU-baseline
leg of the benchmark may import it; the shipped package never does.

Every function restates one piece of the reference algorithm and cites the
reference lines it follows (paths are relative to the reference checkout).

Number representation
---------------------
The reference runs in a 16-bit storage dtype (bf16 for the model, fp16 for
the Triton outputs).  Each torch elementwise op computes in fp32 and rounds
its result to the storage dtype, so a chain of ops rounds after *every* op.
Here a "storage-dtype tensor" is a float32 ndarray whose values are all
exactly representable in that dtype; `round_to` performs the rounding step.

Pinning status (what each function is checked against in tests/):
  round_to              torch CPU casts (library)                      pinned
  quant                 torch CPU eager bf16/fp16 op chain, threshold
                        identity, dequant levels, idempotence, hand case  pinned
  lut_indices           property lut[idx] == x_q                        pinned
  encode / unpack       numpy.packbits (b=1), loop (b=2), round trip    pinned
  lut_vecmat_qk / _pv   einsum over unpacked codes                      pinned
  calibrate             min/max/affine invariants, brute force          pinned
  decode_attention      textbook softmax attention over dequantised
                        K/V when the calibration offsets are (0, 0);
                        partition identity; fp64 post-scale identity    pinned
  quant(per_channel=False)   torch CPU eager chain with x.min() / x.max()  pinned
  rope                  torch CPU running the reference's op sequence
                        (copy_().mul_(), in-place rotate_half, addcmul_);
                        differs from the two-rounding form in ~25 % of
                        the elements, which the test also checks        pinned
  kivi_quantize_pack / kivi_pv   torch CPU eager chain of new_pack.py:64-72
                        (levels_division="true"), closed form + little-endian
                        word packing (numpy.packbits bitorder='little' at
                        b=1), group min / range, midpoint rule           pinned
  decode_attention(v_token_group)   python-loop brute force on explicitly
                        dequantised scale*code + minimum values          pinned
"""
from __future__ import annotations

import math

import numpy as np

DTYPES = ("bf16", "fp16", "fp32")


# --------------------------------------------------------------------------
# storage-dtype rounding
# --------------------------------------------------------------------------
def round_to(x, dtype: str) -> np.ndarray:
    """Round float32 values to `dtype` (round-to-nearest-even), return float32.

    Models the implicit cast at the end of every torch elementwise op on a
    16-bit tensor (reference: every op in calibquant.py:27-36 runs on the
    model dtype set at infer.py:266)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "fp32":
        return x
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        u = x.view(np.uint32).astype(np.uint64)
        nan = np.isnan(x)
        lsb = (u >> 16) & 1
        r = ((u + 0x7FFF + lsb) >> 16) << 16
        out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).copy()
        out = np.asarray(out, dtype=np.float32)
        if nan.any():
            out = np.where(nan, np.float32(np.nan), out)
        return out.reshape(x.shape)
    raise ValueError(f"unknown dtype {dtype!r}")


def _f32(x):
    return np.asarray(x, dtype=np.float32)


# --------------------------------------------------------------------------
# a1: quant  (calibquant.py:24-42)
# --------------------------------------------------------------------------
def quant(x, bits: int, clip: float = 1.0, dtype: str = "bf16",
          levels_division: str = "reciprocal", per_channel: bool = True):
    """Per-channel b-bit min-max quantiser, `post_scale=True` branch.

    x: (B, T, H, D) storage-dtype values (float32 container).  The reduction
    runs over axis 1, as `per_channel=True` does (calibquant.py:26-28) on the
    (B, T_img, H_kv, D) views passed at patch_internvl.py:292,297.

    Returns (x_q, scale, zero): x_q has x's shape and holds the integer codes
    as storage-dtype numbers (NaN where the reference produces NaN); scale and
    zero have shape (B, 1, H, D).

    Rounding: one `round_to` per torch op.
      calibquant.py:27-28  amin/amax (exact) then `* scale`
      calibquant.py:33     `(x_max - x_min)` then `/ quant_levels`
      calibquant.py:34     `-x_min` (exact) then `/ scale`
      calibquant.py:36     `x / scale`, `+ zero_point`, clamp, round-half-even

    levels_division: torch's GPU kernel for `tensor / python_scalar` multiplies
    by the fp32 reciprocal of the scalar ("reciprocal", the behaviour on the
    device the reference hard-wires at calibquant.py:11); torch's CPU kernel
    divides ("true").  They coincide for 1-bit (levels == 1).

    per_channel=False: one minimum and one maximum over the whole tensor
    (`x.min() * scale`, `x.max() * scale`, calibquant.py:29-31); scale and
    zero are then 0-d arrays."""
    x = _f32(x)
    levels = float(2 ** bits - 1)
    c = np.float32(clip)
    with np.errstate(all="ignore"):
        if per_channel:
            x_min = round_to(x.min(axis=1, keepdims=True) * c, dtype)
            x_max = round_to(x.max(axis=1, keepdims=True) * c, dtype)
        else:
            x_min = round_to(x.min() * c, dtype)
            x_max = round_to(x.max() * c, dtype)
        # numpy min/max propagate NaN like torch.amin/amax
        diff = round_to(x_max - x_min, dtype)
        if levels_division == "reciprocal":
            inv = np.float32(1.0) / np.float32(levels)
            scale = round_to(diff * inv, dtype)
        elif levels_division == "true":
            scale = round_to(diff / np.float32(levels), dtype)
        else:
            raise ValueError(levels_division)
        zero = round_to((-x_min) / scale, dtype)
        y = round_to(x / scale, dtype)
        y = round_to(y + zero, dtype)
        y = np.where(np.isnan(y), y, np.clip(y, np.float32(0), np.float32(levels)))
        x_q = np.rint(y).astype(np.float32)  # rint = half-to-even, like torch.round
    return x_q, scale, zero


def dequant(x_q, scale, zero, dtype: str = "fp32"):
    """`scale * (x_q - zero_point)` (calibquant.py:38), rounded per op."""
    with np.errstate(all="ignore"):
        return round_to(_f32(scale) * round_to(_f32(x_q) - _f32(zero), dtype), dtype)


# --------------------------------------------------------------------------
# a2: LUT + index build  (patch_internvl.py:318-329)
# --------------------------------------------------------------------------
def lut_indices(x_q, bits: int):
    """Index of each code in the look-up table of distinct code values.

    The reference takes `unique` of the first 10 000 codes as the table and
    the position of the first match as the index; an element that matches no
    table entry (NaN) gets index 0 because `max` over an all-False mask
    returns position 0.  With the table in ascending order (what torch's
    device `unique` returns) the table is {0, .., 2^bits-1} and the index
    equals the code, which is what this function returns, together with that
    table."""
    x_q = _f32(x_q)
    lut = np.arange(2 ** bits, dtype=np.float32)
    idx = np.where(np.isnan(x_q), 0, x_q).astype(np.int64)
    return lut, idx


# --------------------------------------------------------------------------
# a3: encode  (calibquant.py:114-137)
# --------------------------------------------------------------------------
def encode(idx, bits: int) -> np.ndarray:
    """Pack 8/bits indices per byte along the last axis, first index in the
    most significant bits: byte[j] = sum_i idx[j*dpe+i] << bits*(dpe-1-i)."""
    idx = np.asarray(idx).astype(np.int64)
    dpe = 8 // bits
    *lead, d = idx.shape
    assert d % dpe == 0
    y = idx.reshape(*lead, d // dpe, dpe)
    shift = bits * (dpe - 1 - np.arange(dpe))
    return (y << shift).sum(axis=-1).astype(np.uint8)


def unpack(enc, bits: int) -> np.ndarray:
    """Inverse of `encode`, as both Triton kernels unpack
    (calibquant.py:96-98, 253-258): (byte >> shift) & (2^bits - 1)."""
    enc = np.asarray(enc, dtype=np.uint8)
    dpe = 8 // bits
    shift = (bits * (dpe - 1 - np.arange(dpe))).astype(np.uint8)
    out = (enc[..., None] >> shift) & np.uint8((1 << bits) - 1)
    return out.reshape(*enc.shape[:-1], enc.shape[-1] * dpe)


def quantize_pack(x, bits: int, clip: float, dtype: str,
                  levels_division: str = "reciprocal"):
    """Prefill quantise-and-pack of one tensor, patch_internvl.py:288-341:
    quant (a1) -> transpose to (B, H, T, D) -> indices (a2) -> encode (a3).

    x: (B, T, H, D).  Returns codes uint8 (B, H, T, D*bits/8) and scale, zero
    of shape (B, H, D) (the reference keeps them as (B, H, 1, D) before
    `repeat_kv`, patch_internvl.py:300-309)."""
    x_q, s, z = quant(x, bits, clip, dtype, levels_division)
    _, idx = lut_indices(np.transpose(x_q, (0, 2, 1, 3)), bits)
    codes = encode(idx, bits)
    return codes, s[:, 0], z[:, 0]


# --------------------------------------------------------------------------
# a4 / a8: the two LUT vec-mat kernels  (calibquant.py:54-111, 192-276)
# --------------------------------------------------------------------------
def lut_vecmat_qk(lut, a, enc, bits: int) -> np.ndarray:
    """c[m, n] = sum_k a[m, k] * lut[code[m, n, k]], fp32 accumulate, fp16 out.

    a: (B, H, 1, D); enc: (B, H, T, D*bits/8) -> (B, H, 1, T)
    (wrapper shapes calibquant.py:104-111, kernel :78-102)."""
    lut = _f32(lut)
    vals = lut[unpack(enc, bits).astype(np.int64)]            # (B,H,T,D)
    c = np.einsum("bhd,bhtd->bht", _f32(a)[:, :, 0, :], vals, dtype=np.float32)
    return round_to(c, "fp16")[:, :, None, :]


def lut_vecmat_pv(lut, a, enc, bits: int) -> np.ndarray:
    """c[m, n] = sum_k a[m, k] * lut[code[m, k, n]], fp32 accumulate, fp16 out.

    a: (B, H, 1, T); enc: (B, H, T, D*bits/8) -> (B, H, 1, D)
    (wrapper shapes calibquant.py:269-276, kernel :220-266)."""
    lut = _f32(lut)
    vals = lut[unpack(enc, bits).astype(np.int64)]            # (B,H,T,D)
    c = np.einsum("bht,bhtd->bhd", _f32(a)[:, :, 0, :], vals, dtype=np.float32)
    return round_to(c, "fp16")[:, :, None, :]


# --------------------------------------------------------------------------
# a6: calibration  (patch_internvl.py:376-385)
# --------------------------------------------------------------------------
def calibrate(w, off_max: float = -3.0, off_min: float = 0.0,
              ftype=np.float32) -> np.ndarray:
    """Affine re-mapping of the image logits of every (batch, q-head) row from
    [min, max] to [min + off_min, max + off_max].  w: (..., T); the reduction
    runs over the last axis (the reference reduces dims (2, 3) of a
    (B, Hq, 1, T) tensor)."""
    w = np.asarray(w, dtype=ftype)
    cur_max = w.max(axis=-1, keepdims=True)
    cur_min = w.min(axis=-1, keepdims=True)
    tgt_max = cur_max + ftype(off_max)
    tgt_min = cur_min + ftype(off_min)
    normalized = (w - cur_min) / (cur_max - cur_min + ftype(1e-8))
    return normalized * (tgt_max - tgt_min) + tgt_min


# --------------------------------------------------------------------------
# a4-a9: decode attention  (patch_internvl.py:344-436)
# --------------------------------------------------------------------------
def repeat_kv(x, n_rep: int) -> np.ndarray:
    """(B, Hkv, ...) -> (B, Hkv*n_rep, ...), each kv head repeated n_rep times
    consecutively (patch_internvl.py:97-107)."""
    return np.repeat(np.asarray(x), n_rep, axis=1)


def decode_attention(q, codes_k, codes_v, k_scale, k_zero, v_scale, v_zero,
                     k_res, v_res, sprompt_len: int, bits: int,
                     off_max: float = -3.0, off_min: float = 0.0,
                     calibrate_logits: bool = True, mask=None,
                     ftype=np.float32, v_token_group: int = 0) -> np.ndarray:
    """Dequant-attention oracle for one decode step, computed in `ftype` from
    the packed codes and the stored scales / zero-points.

    q: (B, Hq, D); codes_*: (B, Hkv, T, D*bits/8) uint8; *_scale, *_zero:
    (B, Hkv, D); k_res, v_res: (B, Hkv, R, D) full-precision residual window
    whose first `sprompt_len` rows precede the image block; mask: optional
    additive (B, S + T + R - S) over the [sys | image | text] order.

    Follows the decode branch: residual logits q.K/sqrt(D)
    (patch_internvl.py:365-366); image logits
    q.(s_k (code - z_k))/sqrt(D) (:369-373, post-scaling folded back);
    calibration of the image logits only (:376-385); concatenation
    [sys | image | text] (:388); additive mask (:404-410); softmax (:413);
    image output s_v (sum p code) - s_v z_v sum p (:418-425); residual
    outputs (:428-434); sum (:434).  Returns (B, Hq, D) in `ftype`.

    `v_token_group` > 0: the values are in the per-token layout of
    `kivi_quantize_pack` instead (codes_v int32 words, v_scale / v_zero the
    (B, Hkv, T, D/group) scale and minimum) and dequantise as
    scale*code + minimum (quantization.cu:116-117)."""
    q = np.asarray(q, dtype=ftype)
    B, Hq, D = q.shape
    Hkv = codes_k.shape[1]
    G = Hq // Hkv
    T = codes_k.shape[2]
    R = 0 if k_res is None else k_res.shape[2]
    S = sprompt_len
    assert 0 <= S <= R
    inv = ftype(1.0 / math.sqrt(D))
    with np.errstate(all="ignore"):
        if T:
            ck = unpack(codes_k, bits).astype(ftype)
            khat = np.asarray(k_scale, ftype)[:, :, None, :] * (ck - np.asarray(k_zero, ftype)[:, :, None, :])
            if v_token_group:
                cv = kivi_unpack(codes_v, bits).astype(ftype)
                vhat = (np.repeat(np.asarray(v_scale, ftype), v_token_group, axis=-1) * cv
                        + np.repeat(np.asarray(v_zero, ftype), v_token_group, axis=-1))
            else:
                cv = unpack(codes_v, bits).astype(ftype)
                vhat = np.asarray(v_scale, ftype)[:, :, None, :] * (cv - np.asarray(v_zero, ftype)[:, :, None, :])
            w_img = np.einsum("bhd,bhtd->bht", q, repeat_kv(khat, G)) * inv
            if calibrate_logits:
                w_img = calibrate(w_img, off_max, off_min, ftype)
        else:
            w_img = np.zeros((B, Hq, 0), ftype)
            vhat = np.zeros((B, Hkv, 0, D), ftype)
        if R:
            kr = repeat_kv(np.asarray(k_res, ftype), G)
            vr = repeat_kv(np.asarray(v_res, ftype), G)
            w_res = np.einsum("bhd,bhrd->bhr", q, kr) * inv
        else:
            w_res = np.zeros((B, Hq, 0), ftype)
            vr = np.zeros((B, Hq, 0, D), ftype)
        w = np.concatenate([w_res[:, :, :S], w_img, w_res[:, :, S:]], axis=-1)
        if mask is not None:
            w = w + np.asarray(mask, ftype)[:, None, :]
        w = w - w.max(axis=-1, keepdims=True)
        e = np.exp(w)
        p = e / e.sum(axis=-1, keepdims=True)
        vall = np.concatenate([vr[:, :, :S], repeat_kv(vhat, G), vr[:, :, S:]], axis=2)
        return np.einsum("bht,bhtd->bhd", p, vall).astype(ftype)


# --------------------------------------------------------------------------
# a12: KIVI-style per-token value quantiser  (qjl/new_pack.py:53-82) and its
# consumer (qjl/csrc/quantization.cu:67-132)
# --------------------------------------------------------------------------
def kivi_quantize_pack(v, group_size: int, bits: int, dtype: str = "bf16",
                       levels_division: str = "reciprocal"):
    """Per-token, per-group-of-channels min-max quantiser with 32/bits codes
    per int32 word, first code in the LEAST significant bits.

    v: (B, H, T, D).  For every token and every group of `group_size`
    consecutive channels: mn, mx (new_pack.py:32-50); scale = (mx - mn)/L
    (:69, GPU reciprocal rule for the python scalar); code =
    round(clamp((v - mn)/scale, 0, L)) with one rounding per op (:70-72);
    word = OR_i code[i] << i*bits (:7-28).  Returns (words int32
    (B, H, T, D*bits/32), scale (B, H, T, D/group), mn (B, H, T, D/group))."""
    v = _f32(v)
    B, H, T, D = v.shape
    L = float(2 ** bits - 1)
    ng = D // group_size
    g = v.reshape(B, H, T, ng, group_size)
    with np.errstate(all="ignore"):
        mn = g.min(-1)
        mx = g.max(-1)
        if levels_division == "reciprocal":   # torch's device kernel for tensor / python scalar
            scale = round_to(round_to(mx - mn, dtype) * (np.float32(1.0) / np.float32(L)), dtype)
        else:                                  # torch's CPU kernel divides
            scale = round_to(round_to(mx - mn, dtype) / np.float32(L), dtype)
        y = round_to(g - mn[..., None], dtype)
        y = round_to(y / scale[..., None], dtype)
        y = np.where(np.isnan(y), y, np.clip(y, 0, L))
        code = np.rint(y)
    code = np.where(np.isnan(code), 0, code).astype(np.int64).reshape(B, H, T, D)
    fpi = 32 // bits
    c = code.reshape(B, H, T, D // fpi, fpi)
    shifts = (np.arange(fpi) * bits).astype(np.int64)
    words = (c << shifts).sum(-1).astype(np.uint32).view(np.int32)
    return words, scale, mn


def kivi_unpack(words, bits: int) -> np.ndarray:
    w = np.asarray(words).view(np.uint32)
    fpi = 32 // bits
    shifts = (np.arange(fpi) * bits).astype(np.uint32)
    out = (w[..., None] >> shifts) & np.uint32((1 << bits) - 1)
    return out.reshape(*w.shape[:-1], w.shape[-1] * fpi).astype(np.int64)


def kivi_pv(p, words, scale, mn, group_size: int, bits: int) -> np.ndarray:
    """out[b,h,d] = sum_t p[b,h,t] * (scale[t,g(d)] * code[t,d] + mn[t,g(d)])
    with fp32 accumulation (quantization.cu:116-119).  p: (B, H, T);
    words/scale/mn as returned by `kivi_quantize_pack` (already repeated to
    the q-head count by the caller, patch_internvl.py:575-577)."""
    code = kivi_unpack(words, bits).astype(np.float32)
    s = np.repeat(_f32(scale), group_size, axis=-1)
    m = np.repeat(_f32(mn), group_size, axis=-1)
    return np.einsum("bht,bhtd->bhd", _f32(p), s * code + m, dtype=np.float32)


# --------------------------------------------------------------------------
# rotary position embedding  (patch_internvl.py:110-138)
# --------------------------------------------------------------------------
def rope(x, cos, sin, dtype: str = "bf16") -> np.ndarray:
    """Rotary embedding with the rounding of the ops that run in the reference.

    x: (..., D) storage-dtype values; cos, sin broadcastable to x (already
    gathered by position id).  The reference computes (patch_internvl.py:125-128)
        e = empty_like(x); e.copy_(x).mul_(cos)      -> rnd(x * cos)
        tmp = rotate_half(x)                         -> (-x2, x1), exact
        e.addcmul_(tmp, sin)                         -> rnd(e + tmp * sin)
    where addcmul works in fp32 and rounds once: the product tmp * sin of two
    16-bit values is exact in fp32, the fp32 sum is rounded to fp32 and then
    to the storage dtype - the arithmetic of the device kernel the reference
    ran (`a + alpha * (b * c)` in fp32, then the cast) and of torch's CPU
    kernel.  (The commented-out line :123 would round the second product to
    the storage dtype as well.)"""
    x = _f32(x)
    cos, sin = _f32(cos), _f32(sin)
    h = x.shape[-1] // 2
    rot = np.concatenate([-x[..., h:], x[..., :h]], axis=-1)
    first = round_to(x * cos, dtype)
    return round_to((first + rot * sin).astype(np.float32), dtype)


# --------------------------------------------------------------------------
# synthetic inputs shared by tests, smoke and the benchmark's CPU leg
# --------------------------------------------------------------------------
def synth_kv(B, T, Hkv, D, dtype: str, seed: int, outliers: int = 4,
             outlier_kind: str = "x10"):
    """K, V ~ N(0,1) of shape (B, T, Hkv, D) rounded to `dtype`; per kv-head
    `outliers` random key channels are scaled: "x10" multiplies by 10,
    "student" multiplies by |t3| + 1 with t3 ~ Student-t(nu=3)."""
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
    v = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
    for h in range(Hkv):
        ch = rng.permutation(D)[:outliers]
        if outlier_kind == "x10":
            k[:, :, h, ch] *= 10.0
        else:
            k[:, :, h, ch] *= (np.abs(rng.standard_t(3, size=outliers)) + 1.0).astype(np.float32)
    return round_to(k, dtype), round_to(v, dtype)
