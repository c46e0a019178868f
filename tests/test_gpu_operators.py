"""GPU parity of the four operators of the reference's `calibquant.py` surface
(quant, encode, fused_kernel, fused_kernel_wv) against the oracle, and of the
unfused call sequence of the reference's decode branch assembled from them."""
import math

import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import CLIPS, make_case, case_to_gpu, reference_rope_sequence, same_bits, to_gpu, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cq():
    from calibquant_amd import calibquant
    return calibquant


@pytest.mark.parametrize("bits", [1, 2])
def test_quant_then_encode_like_the_reference_prefill(cq, bits):
    """quant -> transpose -> (identity LUT) indices -> encode, patch_internvl.py:290-339."""
    k, _ = O.synth_kv(2, 300, 4, 128, "bf16", seed=1)
    x = to_gpu(k, "bf16")
    x_q, s, z = cq.quant(x, bits=bits, per_channel=True, scale=CLIPS[bits][0], post_scale=True)
    assert x_q.shape == x.shape and s.shape == (2, 1, 4, 128)
    oxq, os_, oz = O.quant(k, bits, CLIPS[bits][0], "bf16")
    assert same_bits(to_np(x_q), oxq) and same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
    idx = x_q.transpose(1, 2).long()                      # the reference's inverse_indices are int64
    enc = cq.encode(idx, bits, 8 // bits)
    assert enc.dtype == torch.uint8 and enc.shape == (2, 4, 300, 128 * bits // 8)
    assert np.array_equal(enc.cpu().numpy(), O.encode(np.transpose(oxq, (0, 2, 1, 3)).astype(np.int64), bits))
    deq, _, _ = cq.quant(x, bits=bits, per_channel=True, scale=CLIPS[bits][0], post_scale=False)
    assert same_bits(to_np(deq), O.dequant(oxq, os_, oz, "bf16"))


@pytest.mark.parametrize("bits", [1, 2])
def test_fused_kernels_honour_an_arbitrary_table(cq, bits):
    rng = np.random.default_rng(0)
    B, H, T, D = 2, 8, 333, 128
    idx = rng.integers(0, 2 ** bits, size=(B, H, T, D))
    enc = O.encode(idx, bits)
    lut = np.array([0.25, -1.5, 2.0, 3.0][: 2 ** bits], np.float32)
    a = O.round_to(rng.standard_normal((B, H, 1, D)), "bf16")
    p = O.round_to(rng.random((B, H, 1, T)) / T, "fp16")
    enc_g = torch.from_numpy(enc).cuda()
    qk = cq.fused_kernel(to_gpu(lut, "bf16"), to_gpu(a, "bf16"), enc_g, bits, 8 // bits)
    pv = cq.fused_kernel_wv(to_gpu(lut, "fp16"), to_gpu(p, "fp16"), enc_g, bits, 8 // bits)
    assert qk.dtype == torch.float16 and qk.shape == (B, H, 1, T) and pv.shape == (B, H, 1, D)
    want_qk, want_pv = O.lut_vecmat_qk(lut, a, enc, bits), O.lut_vecmat_pv(lut, p, enc, bits)
    # fp32 accumulation order differs from numpy's: allow one fp16 ulp
    assert np.allclose(to_np(qk), want_qk, rtol=2e-3, atol=2e-3)
    assert np.allclose(to_np(pv), want_pv, rtol=2e-3, atol=1e-4)


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_quant_whole_tensor_mode(cq, bits, dtype):
    """quant(per_channel=False) (calibquant.py:29-31): one min / max over the whole tensor; bit-exact
    against the oracle and against torch-ROCm running the reference's op chain on the device."""
    k, _ = O.synth_kv(3, 700, 4, 128, dtype, seed=4)
    x = to_gpu(k, dtype)[:, :, 1:, :]                      # a strided view: heads 1..3
    clip = CLIPS[bits][0]
    x_q, s, z = cq.quant(x, bits=bits, per_channel=False, scale=clip, post_scale=True)
    assert x_q.shape == x.shape and s.dim() == 0 and z.dim() == 0
    oxq, os_, oz = O.quant(k[:, :, 1:, :], bits, clip, dtype, per_channel=False)
    assert float(s) == float(os_) and float(z) == float(oz)
    assert same_bits(to_np(x_q), oxq)
    L = 2 ** bits - 1
    mn, mx = x.min() * clip, x.max() * clip
    st = (mx - mn) / L
    zt = -mn / st
    xq_t = torch.round(torch.clamp(x / st + zt, 0, L))
    assert torch.equal(s, st) and torch.equal(z, zt) and torch.equal(x_q, xq_t)
    deq, _, _ = cq.quant(x, bits=bits, per_channel=False, scale=clip, post_scale=False)
    assert torch.equal(deq, st * (xq_t - zt))
    # any shape ending in the channel axis
    flat = to_gpu(k, dtype).reshape(-1, 128)
    fq, fs, fz = cq.quant(flat, bits=bits, per_channel=False, scale=clip, post_scale=True)
    o2 = O.quant(k, bits, clip, dtype, per_channel=False)
    assert fq.shape == flat.shape and same_bits(to_np(fq), o2[0].reshape(-1, 128)) and float(fs) == float(o2[1])


def test_fused_kernels_with_a_table_shorter_than_the_code_range(cq):
    """The reference builds its table from the levels seen in the first 10 000 codes
    (patch_internvl.py:318-329), so it can hold fewer than 2^bits entries: a code without an
    entry contributes 0 and nothing past the table is read."""
    rng = np.random.default_rng(1)
    B, H, T, D, bits = 1, 2, 100, 128, 2
    idx = rng.integers(0, 4, size=(B, H, T, D))
    enc = O.encode(idx, bits)
    a = O.round_to(rng.standard_normal((B, H, 1, D)), "bf16")
    p = O.round_to(rng.random((B, H, 1, T)) / T, "fp16")
    enc_g = torch.from_numpy(enc).cuda()
    for n in (1, 3):
        short = np.array([0.5, -1.0, 2.0][:n], np.float32)
        full = np.concatenate([short, np.zeros(4 - n, np.float32)])
        # the table sits at the very end of its allocation's used part: entries past it would be foreign memory
        qk = cq.fused_kernel(to_gpu(short, "bf16"), to_gpu(a, "bf16"), enc_g, bits, 4)
        pv = cq.fused_kernel_wv(to_gpu(short, "fp16"), to_gpu(p, "fp16"), enc_g, bits, 4)
        assert np.allclose(to_np(qk), O.lut_vecmat_qk(full, a, enc, bits), rtol=2e-3, atol=2e-3)
        assert np.allclose(to_np(pv), O.lut_vecmat_pv(full, p, enc, bits), rtol=2e-3, atol=1e-4)


def test_unfused_reference_sequence_agrees_with_the_fused_kernel(cq):
    """The decode branch written as the reference writes it (patch_internvl.py:352-436), on top of
    the four operators, lands within the reference's own mixed-precision noise of the fused kernel."""
    from calibquant_amd import ops
    from calibquant_amd.patch_internvl import repeat_kv
    B, Hq, Hkv, T, R, S, bits = 2, 32, 8, 1024, 64, 41, 1
    c = make_case(B, Hq, Hkv, 128, T, R, bits, "bf16", seed=3)
    g = case_to_gpu(c, "bf16")
    G = Hq // Hkv
    q = g["q"][:, :, None, :]
    key_states, value_states = repeat_kv(g["kr"], G), repeat_kv(g["vr"], G)
    scale_key, zero_key = repeat_kv(g["sk"][:, :, None], G), repeat_kv(g["zk"][:, :, None], G)
    scale_val, zero_val = repeat_kv(g["sv"][:, :, None], G), repeat_kv(g["zv"][:, :, None], G)
    lut = torch.arange(2, device="cuda", dtype=torch.bfloat16)
    enc_k, enc_v = repeat_kv(g["ck"], G), repeat_kv(g["cv"], G)
    w_s = torch.matmul(q, key_states[:, :, :S].transpose(2, 3)) / math.sqrt(128)
    w_t = torch.matmul(q, key_states[:, :, S:].transpose(2, 3)) / math.sqrt(128)
    bias_k = torch.sum(scale_key * zero_key * q, dim=-1, keepdim=True) / math.sqrt(128)
    w_v = cq.fused_kernel(lut, q * scale_key, enc_k) / math.sqrt(128) - bias_k
    cur_max, cur_min = w_v.amax(dim=(2, 3), keepdim=True), w_v.amin(dim=(2, 3), keepdim=True)
    w_v = (w_v - cur_min) / (cur_max - cur_min + 1e-8) * ((cur_max - 3) - cur_min) + cur_min
    p = torch.softmax(torch.cat([w_s, w_v, w_t], dim=-1), dim=-1, dtype=torch.float32).to(q.dtype)
    out_v = cq.fused_kernel_wv(lut.half(), p[..., S:S + T].half(), enc_v) * scale_val
    out_v = out_v - scale_val * zero_val * torch.sum(p[..., S:S + T], dim=-1, keepdim=True)
    out = out_v + torch.matmul(p[..., :S], value_states[:, :, :S]) + torch.matmul(p[..., S + T:], value_states[:, :, S:])
    fused = ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"],
                            sprompt_len=S, bits=bits)
    err = (out[:, :, 0].float() - fused.float()).abs()
    assert err.max().item() < 5e-2 and err.mean().item() < 1e-2
    # and the restatement of that mixed-precision chain (tests/refchain.py, informational) tracks the torch sequence closely
    from tests.refchain import decode_attention_refchain
    chain = decode_attention_refchain(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                                        c["kr"], c["vr"], S, bits, "bf16")
    assert np.abs(chain - to_np(out[:, :, 0])).mean() < 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads", [(32, 8), (48, 8), (8, 8)])
def test_rope_append_equals_the_torch_op_chain_bit_for_bit(dtype, heads):
    """Split of the fused projection, rotary embedding and window append in one launch against
    the reference's chain of torch ops (patch_internvl.py:119-138, 219-234, 264-266)."""
    from calibquant_amd import ops, patch_internvl as pi
    Hq, Hkv = heads
    G, D, B, cap, rows = Hq // Hkv, 128, 3, 40, 300
    torch.manual_seed(4)
    qkv = torch.randn(B, 1, (Hq + 2 * Hkv) * D, device="cuda").to(dtype)
    t = torch.arange(rows, device="cuda", dtype=torch.float32)
    inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, device="cuda").float() / D))
    emb = torch.cat([torch.outer(t, inv)] * 2, dim=-1)
    cos, sin = emb.cos().to(dtype), emb.sin().to(dtype)
    pos = torch.tensor([[7], [250], [0]], device="cuda", dtype=torch.long)
    row = torch.tensor([17], device="cuda", dtype=torch.long)
    kwin = torch.zeros(B, Hkv, cap, D, device="cuda", dtype=dtype)
    vwin = torch.zeros_like(kwin)
    q_out = torch.empty(B, Hq, D, device="cuda", dtype=dtype)
    ops.RopeAppendCall(qkv, cos, sin, pos, q_out, kwin, vwin, row).run()
    torch.cuda.synchronize()
    v5 = qkv.view(B, 1, Hkv, 2 + G, D)
    q = v5[..., :G, :].reshape(B, 1, Hq, D).transpose(1, 2)
    k = v5[..., -2, :].transpose(1, 2)
    v = v5[..., -1, :].transpose(1, 2)
    # (1) the oracle, (2) the package's Python helper, (3) torch-ROCm running the reference's own op
    # sequence on the device.  (1) and (2) agree with the kernel bit for bit.  (3) does so in bf16; in
    # fp16 torch-ROCm's addcmul on strided operands rounds the exact sum once where the kernel the
    # reference ran rounds the fp32 sum (about 7 elements in a million sit on such a tie).
    c1, s1 = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
    name = "bf16" if dtype == torch.bfloat16 else "fp16"
    assert np.array_equal(to_np(q_out), O.rope(to_np(q[:, :, 0]), to_np(c1[:, 0]), to_np(s1[:, 0]), name))
    assert np.array_equal(to_np(kwin[:, :, 17]), O.rope(to_np(k[:, :, 0]), to_np(c1[:, 0]), to_np(s1[:, 0]), name))
    assert torch.equal(vwin[:, :, 17], v[:, :, 0])
    qh, kh = pi.apply_rotary_pos_emb(q, k, cos, sin, pos)
    assert torch.equal(qh[:, :, 0], q_out) and torch.equal(kh[:, :, 0], kwin[:, :, 17])
    qr, kr = reference_rope_sequence(q, c1, s1), reference_rope_sequence(k, c1, s1)
    if dtype == torch.bfloat16:
        assert torch.equal(q_out, qr[:, :, 0]) and torch.equal(kwin[:, :, 17], kr[:, :, 0])
    else:
        assert (q_out != qr[:, :, 0]).float().mean().item() < 1e-3
        assert torch.allclose(q_out.float(), qr[:, :, 0].float(), rtol=2e-3, atol=0)
    two = q * c1 + pi.rotate_half(q) * s1              # the two-rounding form is a different function
    assert (two != qr).float().mean().item() > 0.02
    kwin[:, :, 17] = 0
    vwin[:, :, 17] = 0
    assert not kwin.any() and not vwin.any()          # nothing else was written
    row.fill_(cap)                                     # a row outside the window: keys / values are dropped
    ops.RopeAppendCall(qkv, cos, sin, pos, q_out, kwin, vwin, row).run()
    torch.cuda.synchronize()
    assert not kwin.any() and not vwin.any()


def test_rope_append_full_batch_and_replay_by_device_counters():
    """Batch 64 at the 8B head layout: the launch prepared once follows the device-side row and
    position counters, as a recorded decode step needs."""
    from calibquant_amd import ops, patch_internvl as pi
    Hq, Hkv, G, D, B, cap, rows = 32, 8, 4, 128, 64, 8, 4000
    torch.manual_seed(6)
    t = torch.arange(rows, device="cuda", dtype=torch.float32)
    inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, device="cuda").float() / D))
    emb = torch.cat([torch.outer(t, inv)] * 2, dim=-1)
    cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
    qkv = torch.empty(B, (Hq + 2 * Hkv) * D, device="cuda", dtype=torch.bfloat16)
    pos = torch.full((B, 1), 3392, device="cuda", dtype=torch.long)
    row = torch.zeros(1, device="cuda", dtype=torch.long)
    kwin = torch.zeros(B, Hkv, cap, D, device="cuda", dtype=torch.bfloat16)
    vwin = torch.zeros_like(kwin)
    q_out = torch.empty(B, Hq, D, device="cuda", dtype=torch.bfloat16)
    call = ops.RopeAppendCall(qkv, cos, sin, pos, q_out, kwin, vwin, row)
    for step in range(3):
        qkv.copy_(torch.randn_like(qkv))
        call.run()
        v5 = qkv.view(B, 1, Hkv, 2 + G, D)
        q = v5[..., :G, :].reshape(B, 1, Hq, D).transpose(1, 2)
        c1, s1 = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
        qr, kr = reference_rope_sequence(q, c1, s1), reference_rope_sequence(v5[..., -2, :].transpose(1, 2), c1, s1)
        assert torch.equal(q_out, qr[:, :, 0]) and torch.equal(kwin[:, :, step], kr[:, :, 0])     # bf16
        assert np.array_equal(to_np(q_out), O.rope(to_np(q[:, :, 0]), to_np(c1[:, 0]), to_np(s1[:, 0]), "bf16"))
        assert torch.equal(vwin[:, :, step], v5[:, 0, :, -1, :])
        pos.add_(1)
        row.add_(1)
    assert not kwin[:, :, 3:].any()
