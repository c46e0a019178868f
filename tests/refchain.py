"""The reference's own mixed-precision rounding sequence of the decode step, restated for information: how far
the reference's bf16 / fp16 chain sits from the fp32 dequant-attention oracle.  Not part of the oracle and not
a parity bar: no reference-held vector covers this chain and nothing pins it beyond the brackets in the tests
that use it (parity unpinned)."""
import math

import numpy as np

from oracle.cq_oracle import _f32, calibrate, lut_vecmat_pv, lut_vecmat_qk, repeat_kv, round_to


def decode_attention_refchain(q, codes_k, codes_v, k_scale, k_zero, v_scale,
                              v_zero, k_res, v_res, sprompt_len: int, bits: int,
                              dtype: str = "bf16", off_max: float = -3.0,
                              off_min: float = 0.0, mask=None) -> np.ndarray:
    """The same step with the reference's own rounding sequence, for
    information (how far the reference sits from the fp32 oracle).

    Rounding points, in order: `q * scale_key` -> model dtype
    (patch_internvl.py:373); vec-mat -> fp16 (calibquant.py:109); `/ sqrt(D)`
    -> fp16; `scale*zero*q`, its sum, `/ sqrt(D)` -> model dtype (:369-370);
    fp16 - model dtype promotes to fp32 (:373); calibration in fp32;
    residual logits -> model dtype (:365-366); softmax in fp32 -> model
    dtype (:413); p -> fp16, vec-mat -> fp16 (:418, calibquant.py:274);
    `* scale_value`, bias, subtraction (:420-425, fp16 x model dtype promotes
    to fp32 when the model dtype is bf16); residual matmuls -> model dtype
    (:432-433); final cast to bf16 (:436).  Parity unpinned: no
    reference-held vector covers this chain."""
    r = lambda a: round_to(a, dtype)  # noqa: E731
    h = lambda a: round_to(a, "fp16")  # noqa: E731
    q = _f32(q)
    B, Hq, D = q.shape
    Hkv = codes_k.shape[1]
    G = Hq // Hkv
    T = codes_k.shape[2]
    S = sprompt_len
    sq = np.float32(math.sqrt(D))
    sk, zk = repeat_kv(_f32(k_scale), G), repeat_kv(_f32(k_zero), G)
    sv, zv = repeat_kv(_f32(v_scale), G), repeat_kv(_f32(v_zero), G)
    lut = np.arange(2 ** bits, dtype=np.float32)
    enc_k, enc_v = repeat_kv(codes_k, G), repeat_kv(codes_v, G)
    kr, vr = repeat_kv(_f32(k_res), G), repeat_kv(_f32(v_res), G)
    with np.errstate(all="ignore"):
        w_s = r(r(np.einsum("bhd,bhrd->bhr", q, kr[:, :, :S])) / sq)
        w_t = r(r(np.einsum("bhd,bhrd->bhr", q, kr[:, :, S:])) / sq)
        bias = r(r(sk * zk) * q)
        bias = r(r(bias.sum(-1, keepdims=True)) / sq)
        raw = lut_vecmat_qk(lut, r(q * sk)[:, :, None, :], enc_k, bits)[:, :, 0, :]
        w_v = h(raw / sq) - bias            # fp16 - bf16 -> fp32
        if dtype == "fp16":
            w_v = h(w_v)
        w_v = calibrate(w_v, off_max, off_min, np.float32)
        w = np.concatenate([w_s, w_v, w_t], axis=-1)
        if mask is not None:
            w = w + _f32(mask)[:, None, :]
        w = w - w.max(-1, keepdims=True)
        e = np.exp(w)
        p = r(e / e.sum(-1, keepdims=True))
        p_img = p[:, :, S:S + T]
        acc = lut_vecmat_pv(lut, h(p_img)[:, :, None, :], enc_v, bits)[:, :, 0, :]
        mixed = (lambda a: a) if dtype == "bf16" else h
        out_v = mixed(acc * sv)
        bias_v = r(r(sv * zv) * r(p_img.sum(-1, keepdims=True)))
        out_v = mixed(out_v - bias_v)
        out_s = r(np.einsum("bhr,bhrd->bhd", p[:, :, :S], vr[:, :, :S]))
        out_t = r(np.einsum("bhr,bhrd->bhd", p[:, :, S + T:], vr[:, :, S:]))
        out = mixed(mixed(out_v + out_s) + out_t)
        return round_to(out, "bf16")
