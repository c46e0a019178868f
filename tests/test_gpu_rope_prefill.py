"""Prefill rotary embedding in HIP: `rope_rows` (queries, keys outside the image block) and
`rope_quantize_pack` (image block of the keys: rotation fused into the quantise-and-pack pass).
Bit-exact against the oracle (`O.rope` then `O.quantize_pack`), against the same arithmetic
written as separate torch ops on the device, and against the two-step HIP path."""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import CLIPS, TDT, same_bits, to_gpu, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from calibquant_amd import ops as o
    return o


def _tables(rows, D, dtype):
    t = torch.arange(rows, device="cuda", dtype=torch.float32)
    inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, device="cuda").float() / D))
    emb = torch.cat([torch.outer(t, inv)] * 2, dim=-1)
    return emb.cos().to(TDT[dtype]).contiguous(), emb.sin().to(TDT[dtype]).contiguous()


def _torch_rope(x, cos, sin, pos):
    """x (B, T, H, D), pos (B, T): rnd(rnd(x*cos) + rotate_half(x)*sin) as separate fp32 torch ops."""
    c, s = cos[pos].unsqueeze(2), sin[pos].unsqueeze(2)
    h = x.shape[-1] // 2
    rot = torch.cat((-x[..., h:], x[..., :h]), dim=-1)
    return torch.add((x * c).float(), rot.float() * s.float()).to(x.dtype)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_rope_rows_is_bit_exact(ops, dtype):
    B, N, Hkv, G, D = 2, 333, 4, 3, 128
    torch.manual_seed(1)
    proj = (torch.randn(B, N, Hkv, G + 2, D, device="cuda") * 2).to(TDT[dtype])
    cos, sin = _tables(5000, D, dtype)
    pos = torch.randint(0, 5000, (B, N), device="cuda")
    for sl in (proj[..., 0, :], proj[..., -2, :], proj[:, 7:200, :, 1, :]):
        p = pos[:, :sl.shape[1]]
        got = ops.rope_rows(sl, cos, sin, p)
        assert torch.equal(got, _torch_rope(sl, cos, sin, p))
        want = O.rope(to_np(sl), to_np(cos[p].unsqueeze(2)), to_np(sin[p].unsqueeze(2)), dtype)
        assert np.array_equal(to_np(got), want)
    # positions given as the start of an arange, output into a strided slice of a larger buffer
    big = torch.zeros(B, N + 5, Hkv, D, device="cuda", dtype=TDT[dtype])
    ar = (torch.arange(N, device="cuda") + 41)[None].expand(B, N)
    ops.rope_rows(proj[..., -2, :], cos, sin, 41, out=big[:, 5:])
    assert torch.equal(big[:, 5:], _torch_rope(proj[..., -2, :], cos, sin, ar)) and not big[:, :5].any()
    assert torch.equal(ops.rope_rows(proj[..., -2, :], cos, sin, ar), big[:, 5:])      # expanded (stride 0) position ids


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("T", [1, 300, 1024, 2048, 3328])
def test_rope_quantize_pack_is_bit_exact(ops, T, bits, dtype):
    B, Hkv, G, D, S = 2, 4, 2, 128, 9
    N = S + T + 4
    k, _ = O.synth_kv(B, N, Hkv * (G + 2), D, dtype, seed=T + bits, outlier_kind="student")
    proj = to_gpu(k, dtype).view(B, N, Hkv, G + 2, D)
    k_raw = proj[..., -2, :]
    cos, sin = _tables(N + 100, D, dtype)
    pos = (torch.arange(N, device="cuda")[None] + torch.tensor([[0], [57]], device="cuda")).contiguous()
    clip = CLIPS[bits][0]
    k_rot = torch.zeros(B, N, Hkv, D, device="cuda", dtype=TDT[dtype])
    ck, sk, zk = ops.rope_quantize_pack(k_raw[:, S:S + T], cos, sin, pos[:, S:S + T], k_rot[:, S:S + T], bits, clip)
    torch.cuda.synchronize()
    # rotated rows: the separate kernel, the torch ops, nothing outside the slice
    two = ops.rope_rows(k_raw[:, S:S + T], cos, sin, pos[:, S:S + T])
    assert torch.equal(k_rot[:, S:S + T], two) and torch.equal(two, _torch_rope(k_raw[:, S:S + T], cos, sin, pos[:, S:S + T]))
    assert not k_rot[:, :S].any() and not k_rot[:, S + T:].any()
    # packed state: the two-step HIP path and the oracle on the oracle's own rotation
    ck2, sk2, zk2 = ops.quantize_pack(two, bits, clip)
    assert torch.equal(ck, ck2) and same_bits(to_np(sk), to_np(sk2)) and same_bits(to_np(zk), to_np(zk2))
    kr = O.rope(to_np(k_raw[:, S:S + T]), to_np(cos[pos[:, S:S + T]].unsqueeze(2)), to_np(sin[pos[:, S:S + T]].unsqueeze(2)), dtype)
    ock, osk, ozk = O.quantize_pack(kr, bits, clip, dtype)
    assert np.array_equal(ck.cpu().numpy(), ock) and same_bits(to_np(sk), osk) and same_bits(to_np(zk), ozk)


def test_rope_quantize_pack_full_size_equals_the_two_step_path(ops):
    """(64, 3328, 8, 128) key block of a fused projection output, bf16, arange positions from 41."""
    B, T, Hkv, G, D = 64, 3328, 8, 4, 128
    torch.manual_seed(2)
    proj = torch.randn(B, T, Hkv, G + 2, D, device="cuda", dtype=torch.bfloat16)
    cos, sin = _tables(T + 41, D, "bf16")
    k_rot = torch.empty(B, T, Hkv, D, device="cuda", dtype=torch.bfloat16)
    ck, sk, zk = ops.rope_quantize_pack(proj[..., -2, :], cos, sin, 41, k_rot, 1, 0.5)
    two = ops.rope_rows(proj[..., -2, :], cos, sin, 41)
    ck2, sk2, zk2 = ops.quantize_pack(two, 1, 0.5)
    assert torch.equal(k_rot, two) and torch.equal(ck, ck2) and torch.equal(sk, sk2) and torch.equal(zk, zk2)
    rows = two[:2, :, :2]
    ar = (torch.arange(T, device="cuda") + 41)[None].expand(2, T)
    assert torch.equal(rows, _torch_rope(proj[:2, :, :2, -2, :], cos, sin, ar))


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_rope_rows_grouped_equals_one_launch_per_query_head(ops, dtype):
    """All G query heads of every kv head of a fused projection output in one launch: the bits of the
    per-head launches (which are pinned to the oracle and to torch's op sequence above)."""
    B, N, Hkv, G, D = 2, 77, 4, 6, 128
    k, _ = O.synth_kv(B, N, Hkv * (G + 2), D, dtype, seed=5, outlier_kind="student")
    proj = to_gpu(k, dtype).view(B, N, Hkv, G + 2, D)
    cos, sin = _tables(N + 100, D, dtype)
    pos = (torch.arange(N, device="cuda")[None] + torch.tensor([[0], [57]], device="cuda")).contiguous()
    out = torch.zeros(B, N, Hkv, G, D, device="cuda", dtype=TDT[dtype])
    got = ops.rope_rows_grouped(proj[..., :G, :], cos, sin, pos, out=out)
    torch.cuda.synchronize()
    assert got is out
    for gq in range(G):
        assert torch.equal(out[..., gq, :], ops.rope_rows(proj[..., gq, :], cos, sin, pos))
    assert torch.equal(ops.rope_rows_grouped(proj[..., :G, :], cos, sin, 3), torch.stack(
        [ops.rope_rows(proj[..., gq, :], cos, sin, 3) for gq in range(G)], dim=3))


def test_rope_quantize_pack_refuses_what_the_one_pass_kernel_cannot_hold(ops):
    from calibquant_amd._lib import CalibQuantError
    x = torch.randn(1, 4000, 2, 128, device="cuda", dtype=torch.bfloat16)
    cos, sin = _tables(4100, 128, "bf16")
    with pytest.raises(CalibQuantError):
        ops.rope_quantize_pack(x, cos, sin, 0, torch.empty_like(x), 1, 0.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_prefill_same_state_through_every_rotary_path(dtype):
    """The patched attention's prefill with the rotary embedding (a) in `cq_rope_rows` followed by the
    quantiser (the default), (b) fused into the quantiser (`cq_fused_rope`), (c) as the chain of torch ops
    (forced by int32 position ids): the packed codes, statistics and window rows are the same bits; the
    attention output of (a) and (b) is identical."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    cfg = InternLM2Config.tiny()
    B, S, T, TXT = 2, 5, 700, 11
    N = S + T + TXT
    got = []
    for mode in ("rows", "fused", "torch"):
        torch.manual_seed(21)
        att = InternLM2Attention(cfg).cuda().to(dtype)
        att.cq_sprompt_len, att.cq_image_token_num = S, T
        att.cq_fused_rope = mode == "fused"
        x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=dtype)
        pos = torch.arange(N, device="cuda")[None].expand(B, N)
        with torch.no_grad():
            out, _, past = pi.forward_internlm2_calibquant(att, x, None, pos.int() if mode == "torch" else pos, None,
                                                           False, True)
        got.append((att.encoded_features_k.clone(), att.encoded_features_v.clone(), [t.clone() for t in att._cq_stats],
                    past[0].clone(), past[1].clone(), out.clone()))
    for other in (1, 2):
        assert torch.equal(got[0][0], got[other][0]) and torch.equal(got[0][1], got[other][1])
        for a, b in zip(got[0][2], got[other][2]):
            assert torch.equal(a, b)
        if dtype == torch.bfloat16 or other == 1:   # (torch's fp16 addcmul rounds once: window rows may differ in the last bit)
            assert torch.equal(got[0][3], got[other][3]) and torch.equal(got[0][4], got[other][4])
    assert torch.equal(got[0][5], got[1][5])
