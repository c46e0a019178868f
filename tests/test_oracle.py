"""Pins for the numpy oracle: library routines, closed forms, invariants and
brute force on tiny inputs.  None of these retype the oracle's formulas."""
import math

import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import reference_rope_sequence

TDT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _t(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(TDT[dtype])


# ---------------------------------------------------------------- round_to
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_round_to_matches_torch_cast(dtype):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65520.0, 1e38, 3.4e38, 1e-40, 5.9e-8], np.float32),
        # exact ties between neighbouring bf16 values
        (np.arange(0x3F800000, 0x3F800000 + 0x80000, 0x8000, dtype=np.uint32)).view(np.float32),
    ])
    got = O.round_to(x, dtype)
    want = torch.from_numpy(x).to(TDT[dtype]).float().numpy()
    assert np.array_equal(got, want)
    assert np.isnan(O.round_to(np.array([np.nan], np.float32), dtype)).all()


# ------------------------------------------------------------------- quant
def _torch_chain(x, bits, clip, dtype):
    """The quantiser written with torch's own elementwise ops on a real 16-bit
    tensor: the library decides every rounding (CPU kernels divide by the
    python scalar, hence levels_division='true' on the oracle side)."""
    xt = _t(x, dtype)
    L = 2 ** bits - 1
    mn = xt.amin(dim=1, keepdim=True) * clip
    mx = xt.amax(dim=1, keepdim=True) * clip
    s = (mx - mn) / L
    z = -mn / s
    xq = torch.round(torch.clamp(xt / s + z, 0, L))
    return xq.float().numpy(), s.float().numpy(), z.float().numpy()


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("bits,clip", [(1, 0.5), (1, 0.3), (2, 1), (2, 1.0)])
def test_quant_matches_torch_eager_chain(dtype, bits, clip):
    k, v = O.synth_kv(2, 257, 3, 64, dtype, seed=11)
    for x in (k, v):
        xq, s, z = O.quant(x, bits, clip, dtype, levels_division="true")
        xq_t, s_t, z_t = _torch_chain(x, bits, clip, dtype)
        assert np.array_equal(s, s_t)
        assert np.array_equal(z, z_t)
        assert np.array_equal(xq, xq_t)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits,clip", [(1, 0.5), (2, 1)])
def test_quant_whole_tensor_matches_torch_eager_chain(dtype, bits, clip):
    """per_channel=False (calibquant.py:29-31): x.min() / x.max() over the whole tensor."""
    k, _ = O.synth_kv(2, 65, 3, 64, dtype, seed=12)
    xq, s, z = O.quant(k, bits, clip, dtype, levels_division="true", per_channel=False)
    xt = _t(k, dtype)
    L = 2 ** bits - 1
    mn, mx = xt.min() * clip, xt.max() * clip
    st = (mx - mn) / L
    zt = -mn / st
    xq_t = torch.round(torch.clamp(xt / st + zt, 0, L))
    assert s.shape == () and float(s) == float(st) and float(z) == float(zt)
    assert np.array_equal(xq, xq_t.float().numpy())
    assert len(np.unique(xq)) == L + 1


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_rope_matches_the_reference_op_sequence_on_torch_cpu(dtype):
    rng = np.random.default_rng(3)
    x = O.round_to(rng.standard_normal((2, 5, 7, 128)).astype(np.float32) * 3, dtype)
    ang = rng.uniform(0, 6.3, size=(2, 1, 7, 64)).astype(np.float32)
    ang = np.concatenate([ang, ang], -1)
    cos, sin = O.round_to(np.cos(ang), dtype), O.round_to(np.sin(ang), dtype)
    got = O.rope(x, cos, sin, dtype)
    want = reference_rope_sequence(_t(x, dtype), _t(cos, dtype), _t(sin, dtype)).float().numpy()
    assert np.array_equal(got, want)
    # the two-rounding form (x*cos) + (rotate_half(x)*sin) is a different function: a restatement
    # that rounded the second product would fail the comparison above
    xt, ct, st_ = _t(x, dtype), _t(cos, dtype), _t(sin, dtype)
    two = (xt * ct + torch.cat((-xt[..., 64:], xt[..., :64]), -1) * st_).float().numpy()
    frac = np.mean(two != want)
    assert 0.02 < frac < 0.6, frac
    # rotation by angle 0 is the identity, by pi/2 it is rotate_half (cos, sin exactly 1 / 0)
    one, zero = np.ones_like(cos), np.zeros_like(cos)
    assert np.array_equal(O.rope(x, one, zero, dtype), x)
    assert np.array_equal(O.rope(x, zero, one, dtype), np.concatenate([-x[..., 64:], x[..., :64]], -1))


def test_quant_reciprocal_rule_differs_only_by_rounding():
    k, _ = O.synth_kv(2, 300, 4, 128, "bf16", seed=5)
    a = O.quant(k, 2, 1.0, "bf16", "reciprocal")
    b = O.quant(k, 2, 1.0, "bf16", "true")
    # same for 1-bit by construction; for 2-bit the scales agree to 1 bf16 ulp
    assert np.all(np.abs(a[1] - b[1]) <= np.abs(b[1]) * 2 ** -7)
    a1 = O.quant(k, 1, 0.5, "bf16", "reciprocal")
    b1 = O.quant(k, 1, 0.5, "bf16", "true")
    for u, w in zip(a1, b1):
        assert np.array_equal(u, w)


def test_quant_one_bit_threshold_and_levels_fp32():
    """In (near-)exact arithmetic the 1-bit code is 1 iff x > (min+max)/2 * c
    ... i.e. x/s + z > 0.5 with s = c(max-min), z = -c*min/s; and the two
    dequantised levels are c*min and c*max."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 500, 2, 16)).astype(np.float32)
    c = 0.5
    xq, s, z = O.quant(x, 1, c, "fp32")
    mn, mx = x.min(1, keepdims=True), x.max(1, keepdims=True)
    thr = 0.5 * c * (mx - mn) + c * mn          # x/s + z > 1/2
    margin = np.abs(x - thr) > 1e-4
    assert np.array_equal((x > thr)[margin], (xq == 1)[margin])
    deq = O.dequant(xq, s, z, "fp32")
    lo = np.broadcast_to(c * mn, x.shape)
    hi = np.broadcast_to(c * mx, x.shape)
    assert np.allclose(deq[xq == 0], lo[xq == 0], atol=1e-5)
    assert np.allclose(deq[xq == 1], hi[xq == 1], atol=1e-5)


@pytest.mark.parametrize("bits", [1, 2])
def test_quant_idempotent_on_dequantised_data(bits):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, 64, 2, 8)).astype(np.float32)
    xq, s, z = O.quant(x, bits, 1.0, "fp32")
    deq = O.dequant(xq, s, z, "fp32")
    # min and max are kept (clip 1), so requantising reproduces the codes
    xq2, s2, z2 = O.quant(deq, bits, 1.0, "fp32")
    assert np.array_equal(xq, xq2)
    assert np.allclose(s, s2, rtol=1e-5)


def test_quant_hand_case_two_bit():
    # one channel, values chosen so every step is exact in bf16:
    # min 0, max 3 -> s = 1, z = 0 -> codes = round-half-even(x)
    x = np.array([0.0, 0.5, 1.0, 1.5, 2.5, 3.0, 2.0, 0.25], np.float32).reshape(1, 8, 1, 1)
    xq, s, z = O.quant(x, 2, 1.0, "bf16", "true")
    assert s.item() == 1.0 and z.item() == 0.0
    assert xq.ravel().tolist() == [0, 0, 1, 2, 2, 3, 2, 0]
    # shifted: min -1, max 2 -> s = 1, z = 1
    xq, s, z = O.quant(x - 1, 2, 1.0, "bf16", "true")
    assert s.item() == 1.0 and z.item() == 1.0
    assert xq.ravel().tolist() == [0, 0, 1, 2, 2, 3, 2, 0]


def test_quant_constant_channel_follows_ieee():
    x = np.ones((1, 8, 1, 2), np.float32)
    x[0, :, 0, 1] = np.arange(8)
    xq, s, z = O.quant(x, 1, 0.5, "bf16")
    assert s[0, 0, 0, 0] == 0 and np.isinf(z[0, 0, 0, 0]) and z[0, 0, 0, 0] < 0
    assert np.isnan(xq[0, :, 0, 0]).all()
    _, idx = O.lut_indices(xq, 1)
    assert (idx[0, :, 0, 0] == 0).all()


# ------------------------------------------------------------ LUT / encode
@pytest.mark.parametrize("bits", [1, 2])
def test_lut_is_identity(bits):
    k, _ = O.synth_kv(1, 64, 2, 32, "bf16", 1)
    xq, _, _ = O.quant(k, bits, 1.0, "bf16")
    lut, idx = O.lut_indices(xq, bits)
    assert np.array_equal(lut[idx], xq)
    assert sorted(np.unique(xq).tolist()) == list(range(2 ** bits))


def test_encode_one_bit_is_packbits_big():
    rng = np.random.default_rng(0)
    idx = rng.integers(0, 2, size=(2, 3, 17, 128))
    assert np.array_equal(O.encode(idx, 1), np.packbits(idx.astype(np.uint8), axis=-1, bitorder="big"))


def test_encode_two_bit_loop_and_roundtrip():
    rng = np.random.default_rng(1)
    idx = rng.integers(0, 4, size=(1, 2, 5, 16))
    enc = O.encode(idx, 2)
    for t in range(5):
        for j in range(4):
            c = idx[0, 1, t, 4 * j:4 * j + 4]
            assert enc[0, 1, t, j] == (c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3]
    assert np.array_equal(O.unpack(enc, 2), idx)
    idx1 = rng.integers(0, 2, size=(1, 2, 5, 16))
    assert np.array_equal(O.unpack(O.encode(idx1, 1), 1), idx1)


# ------------------------------------------------------------ LUT vec-mat
@pytest.mark.parametrize("bits", [1, 2])
def test_lut_vecmat_is_einsum_over_unpacked(bits):
    rng = np.random.default_rng(2)
    B, H, T, D = 2, 3, 37, 32
    idx = rng.integers(0, 2 ** bits, size=(B, H, T, D))
    enc = O.encode(idx, bits)
    lut = np.array([0.5, -1.25, 2.0, 3.0][: 2 ** bits], np.float32)   # not the identity
    a = rng.standard_normal((B, H, 1, D)).astype(np.float32)
    p = rng.random((B, H, 1, T)).astype(np.float32)
    dense = lut[idx].astype(np.float64)
    qk = (a[:, :, 0, None, :].astype(np.float64) * dense).sum(-1)
    pv = (p[:, :, 0, :, None].astype(np.float64) * dense).sum(2)
    assert np.allclose(O.lut_vecmat_qk(lut, a, enc, bits)[:, :, 0], qk, atol=2e-2, rtol=2e-3)
    assert np.allclose(O.lut_vecmat_pv(lut, p, enc, bits)[:, :, 0], pv, atol=2e-2, rtol=2e-3)
    # outputs are fp16 numbers
    out = O.lut_vecmat_qk(lut, a, enc, bits)
    assert np.array_equal(out, out.astype(np.float16).astype(np.float32))


# ------------------------------------------------------------- calibration
def test_calibration_invariants():
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((3, 4, 200)) * 4).astype(np.float64)
    c = O.calibrate(w, -3.0, 0.0, np.float64)
    assert np.allclose(c.min(-1), w.min(-1))
    assert np.allclose(c.max(-1), w.max(-1) - 3.0, atol=1e-6)
    # affine in w: second differences of (sorted) pairs vanish
    i = np.argsort(w, -1)
    ws, cs = np.take_along_axis(w, i, -1), np.take_along_axis(c, i, -1)
    slope = (cs[..., -1:] - cs[..., :1]) / (ws[..., -1:] - ws[..., :1])
    assert np.allclose(cs, cs[..., :1] + slope * (ws - ws[..., :1]), atol=1e-9)
    # range below 3 reverses the order
    w2 = rng.random((1, 1, 50))
    c2 = O.calibrate(w2, -3.0, 0.0, np.float64)
    assert np.array_equal(np.argsort(w2, -1), np.argsort(-c2, -1))
    # offsets (0, 0) leave the logits (almost) unchanged
    assert np.allclose(O.calibrate(w, 0.0, 0.0, np.float64), w, atol=1e-6)


# -------------------------------------------------------- decode attention
def _case(B=2, Hq=8, Hkv=2, D=32, T=96, R=24, bits=1, dtype="bf16", seed=0):
    k, v = O.synth_kv(B, T, Hkv, D, dtype, seed)
    clip_k, clip_v = (0.5, 0.3) if bits == 1 else (1.0, 1.0)
    ck, sk, zk = O.quantize_pack(k, bits, clip_k, dtype)
    cv, sv, zv = O.quantize_pack(v, bits, clip_v, dtype)
    rng = np.random.default_rng(seed + 100)
    q = O.round_to(rng.standard_normal((B, Hq, D)), dtype)
    kr = O.round_to(rng.standard_normal((B, Hkv, R, D)), dtype)
    vr = O.round_to(rng.standard_normal((B, Hkv, R, D)), dtype)
    return q, ck, cv, sk, zk, sv, zv, kr, vr


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("S", [0, 7, 24])
def test_decode_attention_reduces_to_textbook_softmax(bits, S):
    """Without calibration the step is ordinary attention over the
    concatenation [K_res[:S] | dequant(K_img) | K_res[S:]]; checked against
    torch's softmax/matmul in fp64."""
    q, ck, cv, sk, zk, sv, zv, kr, vr = _case(bits=bits)
    G = q.shape[1] // ck.shape[1]
    out = O.decode_attention(q, ck, cv, sk, zk, sv, zv, kr, vr, S, bits,
                             calibrate_logits=False, ftype=np.float64)
    kd = sk[:, :, None, :].astype(np.float64) * (O.unpack(ck, bits) - zk[:, :, None, :].astype(np.float64))
    vd = sv[:, :, None, :].astype(np.float64) * (O.unpack(cv, bits) - zv[:, :, None, :].astype(np.float64))
    K = torch.from_numpy(np.concatenate([kr[:, :, :S], kd, kr[:, :, S:]], 2)).double().repeat_interleave(G, 1)
    V = torch.from_numpy(np.concatenate([vr[:, :, :S], vd, vr[:, :, S:]], 2)).double().repeat_interleave(G, 1)
    Q = torch.from_numpy(q).double()[:, :, None, :]
    want = torch.softmax(Q @ K.transpose(2, 3) / math.sqrt(q.shape[-1]), -1) @ V
    assert np.allclose(out, want[:, :, 0].numpy(), atol=1e-10)
    # offsets (0,0) with calibration switched on is the same thing up to 1e-8
    out0 = O.decode_attention(q, ck, cv, sk, zk, sv, zv, kr, vr, S, bits,
                              off_max=0.0, off_min=0.0, ftype=np.float64)
    assert np.allclose(out0, out, atol=1e-6)


def test_decode_attention_post_scale_identity_fp64():
    """raw/sqrt(D) - bias == q.(s(code - z))/sqrt(D)  (patch_internvl.py:369-373)."""
    q, ck, cv, sk, zk, *_ = _case(bits=2)
    G = q.shape[1] // ck.shape[1]
    D = q.shape[-1]
    skr, zkr = O.repeat_kv(sk, G).astype(np.float64), O.repeat_kv(zk, G).astype(np.float64)
    code = O.repeat_kv(O.unpack(ck, 2), G).astype(np.float64)
    raw = np.einsum("bhd,bhtd->bht", q * skr, code)
    bias = (skr * zkr * q).sum(-1, keepdims=True) / math.sqrt(D)
    lhs = raw / math.sqrt(D) - bias
    rhs = np.einsum("bhd,bhtd->bht", q.astype(np.float64), skr[:, :, None] * (code - zkr[:, :, None])) / math.sqrt(D)
    assert np.allclose(lhs, rhs, atol=1e-9)


def test_decode_attention_calibrated_brute_force_and_mask():
    """Tiny case recomputed with python loops, including the additive mask."""
    q, ck, cv, sk, zk, sv, zv, kr, vr = _case(B=1, Hq=2, Hkv=1, D=8, T=5, R=3, bits=2, dtype="fp16", seed=3)
    S = 1
    rng = np.random.default_rng(9)
    mask = np.where(rng.random((1, 8)) < 0.3, -1e4, 0.0)
    out = O.decode_attention(q, ck, cv, sk, zk, sv, zv, kr, vr, S, 2, mask=mask, ftype=np.float64)
    ukc, uvc = O.unpack(ck, 2), O.unpack(cv, 2)
    for h in range(2):
        wi = []
        for t in range(5):
            wi.append(sum(float(q[0, h, d]) * float(sk[0, 0, d]) * (int(ukc[0, 0, t, d]) - float(zk[0, 0, d])) for d in range(8)) / math.sqrt(8))
        mx, mn = max(wi), min(wi)
        wi = [(w - mn) / (mx - mn + 1e-8) * ((mx - 3) - mn) + mn for w in wi]
        wr = [sum(float(q[0, h, d]) * float(kr[0, 0, r, d]) for d in range(8)) / math.sqrt(8) for r in range(3)]
        logits = wr[:S] + wi + wr[S:]
        logits = [l + float(mask[0, i]) for i, l in enumerate(logits)]
        m = max(logits)
        e = [math.exp(l - m) for l in logits]
        p = [x / sum(e) for x in e]
        for d in range(8):
            vals = [float(vr[0, 0, r, d]) for r in range(S)]
            vals += [float(sv[0, 0, d]) * (int(uvc[0, 0, t, d]) - float(zv[0, 0, d])) for t in range(5)]
            vals += [float(vr[0, 0, r, d]) for r in range(S, 3)]
            want = sum(pp * vv for pp, vv in zip(p, vals))
            assert abs(out[0, h, d] - want) < 1e-9


def test_decode_attention_no_image_or_no_residual():
    q, ck, cv, sk, zk, sv, zv, kr, vr = _case()
    a = O.decode_attention(q, ck[:, :, :0], cv[:, :, :0], sk, zk, sv, zv, kr, vr, 0, 1, ftype=np.float64)
    G = q.shape[1] // kr.shape[1]
    K = torch.from_numpy(kr).double().repeat_interleave(G, 1)
    V = torch.from_numpy(vr).double().repeat_interleave(G, 1)
    want = torch.softmax(torch.from_numpy(q).double()[:, :, None] @ K.transpose(2, 3) / math.sqrt(q.shape[-1]), -1) @ V
    assert np.allclose(a, want[:, :, 0].numpy(), atol=1e-10)
    b = O.decode_attention(q, ck, cv, sk, zk, sv, zv, None, None, 0, 1, ftype=np.float64)
    assert b.shape == q.shape and np.isfinite(b).all()


def test_refchain_is_close_to_fp32_oracle():
    q, ck, cv, sk, zk, sv, zv, kr, vr = _case(T=512, R=32, D=64)
    a = O.decode_attention(q, ck, cv, sk, zk, sv, zv, kr, vr, 8, 1)
    from tests.refchain import decode_attention_refchain
    b = decode_attention_refchain(q, ck, cv, sk, zk, sv, zv, kr, vr, 8, 1, "bf16")
    assert np.abs(a - b).max() < 5e-2 and np.abs(a - b).mean() < 1e-2


# -------------------------------------------------------------------- KIVI
@pytest.mark.parametrize("bits", [2, 4])
def test_kivi_pack_little_endian_and_pv(bits):
    rng = np.random.default_rng(0)
    v = O.round_to(rng.standard_normal((1, 2, 9, 64)), "fp16")
    words, s, mn = O.kivi_quantize_pack(v, 32, bits, "fp16")
    codes = O.kivi_unpack(words, bits)
    # word layout: code i sits at bit i*bits
    w0 = int(np.asarray(words).view(np.uint32)[0, 0, 0, 0])
    fpi = 32 // bits
    assert [(w0 >> (i * bits)) & (2 ** bits - 1) for i in range(fpi)] == codes[0, 0, 0, :fpi].tolist()
    # dequantised values bracket the data within one step
    deq = np.repeat(s, 32, -1) * codes + np.repeat(mn, 32, -1)
    assert np.all(np.abs(deq - v) <= np.repeat(s, 32, -1) * 0.51 + 1e-3)
    # each group attains code 0 and code L
    g = codes.reshape(1, 2, 9, 2, 32)
    assert (g.min(-1) == 0).all() and (g.max(-1) == 2 ** bits - 1).all()
    p = rng.random((1, 2, 9)).astype(np.float32)
    out = O.kivi_pv(p, words, s, mn, 32, bits)
    assert np.allclose(out, np.einsum("bht,bhtd->bhd", p, deq), atol=1e-5)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
def test_kivi_quantiser_matches_torch_eager_chain(bits, dtype):
    """The per-token quantiser against the torch ops of qjl/new_pack.py:64-72 on a real 16-bit CPU
    tensor (min / max per group, `(mx - mn) / L`, `data - mn`, `div_`, `clamp_`, `round_`); the
    CPU kernel divides by the python scalar, hence levels_division="true" on the oracle side."""
    rng = np.random.default_rng(21)
    v = O.round_to(rng.standard_normal((2, 3, 37, 128)).astype(np.float32) * 2, dtype)
    words, s, mn = O.kivi_quantize_pack(v, 32, bits, dtype, levels_division="true")
    vt = _t(v, dtype).reshape(2 * 3 * 37, 4, 32)
    mn_t, mx_t = vt.amin(-1), vt.amax(-1)
    L = 2 ** bits - 1
    sc_t = (mx_t - mn_t) / L
    d = vt - mn_t.unsqueeze(-1)
    d.div_(sc_t.unsqueeze(-1))
    d = d.clamp_(0, L).round_().to(torch.int32)
    assert np.array_equal(s.reshape(-1, 4), sc_t.float().numpy())
    assert np.array_equal(mn.reshape(-1, 4), mn_t.float().numpy())
    assert np.array_equal(O.kivi_unpack(words, bits).reshape(-1, 4, 32), d.numpy())


def test_kivi_one_bit_words_are_packbits_little():
    """1-bit per-token codes: the int32 words equal numpy's little-bit-order packing of the codes
    (library routine), and every group's codes are the comparison with the group midpoint."""
    rng = np.random.default_rng(5)
    v = O.round_to(rng.standard_normal((2, 1, 7, 128)), "bf16")
    words, s, mn = O.kivi_quantize_pack(v, 32, 1, "bf16")
    codes = O.kivi_unpack(words, 1)
    packed = np.packbits(codes.astype(np.uint8), axis=-1, bitorder="little")
    assert np.array_equal(packed.reshape(2, 1, 7, 4, 4).view(np.uint32)[..., 0].view(np.int32), words)
    g = v.reshape(2, 1, 7, 4, 32)
    assert np.array_equal(mn, g.min(-1)) and np.array_equal(s, O.round_to(g.max(-1) - g.min(-1), "bf16"))
    # away from the midpoint the code is just "above the middle of the group's range"
    mid = (g.max(-1, keepdims=True) + g.min(-1, keepdims=True)) / 2
    clear = np.abs(g - mid) > 0.02 * (g.max(-1, keepdims=True) - g.min(-1, keepdims=True))
    assert np.array_equal(codes.reshape(g.shape)[clear], (g > mid)[clear].astype(np.int64))


def test_decode_attention_per_token_values_brute_force():
    """The per-token value branch of the oracle against python loops on explicitly dequantised
    values scale*code + minimum (quantization.cu:116-117)."""
    q, ck, _cv, sk, zk, _sv, _zv, kr, vr = _case(B=1, Hq=2, Hkv=1, D=32, T=6, R=2, bits=2, dtype="fp16", seed=11)
    rng = np.random.default_rng(12)
    v = O.round_to(rng.standard_normal((1, 1, 6, 32)), "fp16")
    words, s, mn = O.kivi_quantize_pack(v, 32, 2, "fp16")
    out = O.decode_attention(q, ck, words, sk, zk, s, mn, kr, vr, 1, 2, ftype=np.float64, v_token_group=32)
    codes = O.kivi_unpack(words, 2)
    ukc = O.unpack(ck, 2)
    for h in range(2):
        wi = [sum(float(q[0, h, d]) * float(sk[0, 0, d]) * (int(ukc[0, 0, t, d]) - float(zk[0, 0, d])) for d in range(32))
              / math.sqrt(32) for t in range(6)]
        mx, mi = max(wi), min(wi)
        wi = [(w - mi) / (mx - mi + 1e-8) * ((mx - 3) - mi) + mi for w in wi]
        wr = [sum(float(q[0, h, d]) * float(kr[0, 0, r, d]) for d in range(32)) / math.sqrt(32) for r in range(2)]
        logits = wr[:1] + wi + wr[1:]
        m = max(logits)
        e = [math.exp(l - m) for l in logits]
        p = [x / sum(e) for x in e]
        for d in range(32):
            vals = [float(vr[0, 0, 0, d])]
            vals += [float(s[0, 0, t, 0]) * int(codes[0, 0, t, d]) + float(mn[0, 0, t, 0]) for t in range(6)]
            vals += [float(vr[0, 0, 1, d])]
            assert abs(out[0, h, d] - sum(pp * vv for pp, vv in zip(p, vals))) < 1e-9


def test_oracle_results_are_frozen_by_the_committed_digests():
    """The oracle's own results on three small seeded cases equal the committed digests
    (tests/golden/oracle_vectors.json, written by tests/golden/make_vectors.py): an edit that
    changes the oracle's numbers fails here.  These are not reference outputs."""
    import importlib.util
    import json
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(here, "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = json.load(open(os.path.join(here, "oracle_vectors.json")))
    got = mod.vectors()
    assert sorted(got) == sorted(want)
    for name, w in want.items():
        g = got[name]
        for key in ("codes_k", "codes_v", "k_scale", "k_zero", "v_scale", "v_zero"):
            assert g[key] == w[key], (name, key)
        assert np.allclose(g["out_head0"], w["out_head0"], atol=2e-6), name
        assert abs(g["out_sum"] - w["out_sum"]) < 1e-3, name


def test_chunk_partials_merge_like_the_unchunked_softmax():
    """The arithmetic of the chunked step's merge, on the CPU: every chunk leaves (m, l, acc) = (its maximum
    logit, the sum of exp(w - m), the exp-weighted value sum); combining them eight at a time with a running
    (m, numerator, denominator) - the order the merging workgroup uses, with chunks that are masked out
    entirely (m = -inf) and a residual partial among them - gives the softmax-weighted sum over all
    positions, whatever the chunking."""
    rng = np.random.default_rng(3)
    for nchunk, T, D in ((1, 50, 8), (8, 400, 16), (9, 333, 8), (19, 1000, 4)):
        w = rng.standard_normal(T) * 5
        w[rng.random(T) < 0.1] = -np.inf
        v = rng.standard_normal((T, D))
        bounds = np.linspace(0, T, nchunk + 1).astype(int)
        if nchunk > 2:
            w[bounds[1]:bounds[2]] = -np.inf            # a chunk with every position masked
        parts = []
        for c in range(nchunk):
            ws, vs = w[bounds[c]:bounds[c + 1]], v[bounds[c]:bounds[c + 1]]
            m = ws.max() if ws.size else -np.inf
            e = np.zeros_like(ws) if m == -np.inf else np.exp(ws - m)
            parts.append((m, e.sum(), e @ vs))
        m, num, den = -np.inf, np.zeros(D), 0.0
        for s0 in range(0, nchunk, 8):
            blk = parts[s0:s0 + 8]
            mb = max([m] + [p_[0] for p_ in blk])
            keep = 0.0 if m == -np.inf else np.exp(m - mb)
            num, den = num * keep, den * keep
            for pm, pl, pa in blk:
                wgt = 0.0 if pm == -np.inf else np.exp(pm - mb)
                den += pl * wgt
                num = num + pa * wgt
            m = mb
        ok = np.isfinite(w)
        p_full = np.exp(w[ok] - w[ok].max())
        want = (p_full / p_full.sum()) @ v[ok]
        assert np.allclose(num / den, want, rtol=1e-12, atol=1e-12)
