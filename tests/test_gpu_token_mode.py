"""Per-token value layout (`v_mode = token`, the reference's qjl/new_pack.py:53-82 quantiser and
its consumer quantization.cu:67-132): bit-exact words / scales / minima against the oracle, and the
fused decode kernel reading that layout against the fp32 dequant-attention oracle
(1e-2 max-abs, 1e-3 mean-abs)."""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import case_to_gpu, make_case, same_bits, to_gpu, to_np

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1e-2, 1e-3


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
def test_quantize_pack_token_is_bit_exact(bits, dtype):
    from calibquant_amd import ops
    B, T, H, D = 2, 333, 3, 128
    k, v = O.synth_kv(B, T, H, D, dtype, seed=31)
    v[0, 5, 1, 32:64] = v[0, 5, 1, 32]            # a constant group: scale 0, codes from NaN -> 0
    # a strided view, as the value block of a fused projection output is
    wide = torch.zeros((B, T, H, 3, D), dtype=to_gpu(v, dtype).dtype, device="cuda")
    wide[:, :, :, 2] = to_gpu(v, dtype)
    words, scale, mins = ops.quantize_pack_token(wide[:, :, :, 2], bits)
    torch.cuda.synchronize()
    w_ref, s_ref, m_ref = O.kivi_quantize_pack(np.transpose(v, (0, 2, 1, 3)), 32, bits, dtype)
    assert words.shape == (B, H, T, D * bits // 32) and words.dtype == torch.int32
    assert np.array_equal(words.cpu().numpy(), w_ref)
    assert same_bits(to_np(scale), s_ref) and same_bits(to_np(mins), m_ref)


def _token_case(B, Hq, Hkv, T, R, bits, dtype, seed):
    c = make_case(B, Hq, Hkv, 128, T, R, bits, dtype, seed)
    words, scale, mins = O.kivi_quantize_pack(np.transpose(c["v"], (0, 2, 1, 3)), 32, bits, dtype)
    c["cv"], c["sv"], c["zv"] = words, scale, mins
    return c


CASES = [
    # B, Hq, Hkv, T, R, S
    (2, 32, 8, 3328, 128, 0),      # InternVL2.5-8B layer shape, small batch (one chunk of tokens)
    (2, 32, 8, 777, 60, 41),       # ragged T, system prompt rows
    (1, 48, 8, 1000, 33, 0),       # six q heads per kv head
    (1, 8, 8, 130, 0, 0),          # one q head per kv head, no residual
    (12, 56, 8, 700, 20, 3),       # seven q heads per kv head: padded units (four heads at 1 bit, two at 2 bits)
]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("case", CASES)
def test_decode_attn_token_values_match_oracle(case, bits, dtype):
    from calibquant_amd import ops
    B, Hq, Hkv, T, R, S = case
    c = _token_case(B, Hq, Hkv, T, R, bits, dtype, seed=40 + T)
    g = case_to_gpu(c, dtype)
    out = ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"],
                          g["kr"] if R else None, g["vr"] if R else None, sprompt_len=S, bits=bits, v_mode="token")
    torch.cuda.synchronize()
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                              c["kr"] if R else None, c["vr"] if R else None, S, bits, v_token_group=32)
    err = np.abs(to_np(out) - want)
    assert np.isfinite(to_np(out)).all()
    assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, (err.max(), err.mean())


@pytest.mark.parametrize("bits", [1, 2])
def test_decode_attn_token_values_split_path(bits):
    """The chunked path (min/max launch, partials, merge) with per-token values."""
    from calibquant_amd import ops
    B, Hq, Hkv, T, R, S = 1, 32, 8, 5000, 70, 3
    c = _token_case(B, Hq, Hkv, T, R, bits, "bf16", seed=77)
    g = case_to_gpu(c, "bf16")
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], S, bits,
                              v_token_group=32)
    for splits in (0, 3):
        out = ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"],
                              sprompt_len=S, bits=bits, v_mode="token", force_splits=splits)
        torch.cuda.synchronize()
        err = np.abs(to_np(out) - want)
        assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, (splits, err.max(), err.mean())


@pytest.mark.parametrize("bits", [1, 2])
def test_token_quantiser_full_size_matches_the_torch_device_op_chain(bits):
    """Benchmark layer shape (64 x 3328 x 8 x 128, bf16): the kernel's words / scales / minima equal what
    the reference's sequence of torch ops (qjl/new_pack.py:64-72) gives on this GPU, and the words
    unpack to codes in range that reach 0 and L in every group."""
    from calibquant_amd import ops
    B, T, H, D, L = 64, 3328, 8, 128, 2 ** bits - 1
    torch.manual_seed(3)
    x = torch.randn(B, T, H, D, device="cuda").to(torch.bfloat16)
    words, scale, mins = ops.quantize_pack_token(x, bits)
    g = x.permute(0, 2, 1, 3).reshape(B * H * T, D // 32, 32)
    mn = g.amin(-1)
    sc = (g.amax(-1) - mn) / L
    data = g - mn.unsqueeze(-1)
    data.div_(sc.unsqueeze(-1))
    code = data.clamp_(0, L).round_().to(torch.int32)
    assert torch.equal(scale.reshape(-1, 4), sc) and torch.equal(mins.reshape(-1, 4), mn)
    shifts = torch.arange(0, 32, bits, device="cuda", dtype=torch.int64)
    got = (words.reshape(-1, 4, bits, 1).to(torch.int64) & 0xFFFFFFFF) >> shifts & L      # (rows, groups, words, codes/word)
    assert torch.equal(got.reshape(-1, 4, 32).to(torch.int32), code)
    assert (code.amin(-1) == 0).all() and (code.amax(-1) == L).all()


def test_decode_attn_token_values_full_batch_rows_are_independent():
    """Batch 64 at the layer shape: rows fed identical inputs give identical outputs, and two rows
    agree with the oracle."""
    from calibquant_amd import ops
    B, Hq, Hkv, T, R = 64, 32, 8, 3328, 128
    c = _token_case(2, Hq, Hkv, T, R, 1, "bf16", seed=91)
    g = case_to_gpu(c, "bf16")
    rep = lambda t: t.repeat(B // 2, *([1] * (t.dim() - 1)))   # noqa: E731  rows 0,1,0,1,...
    out = ops.decode_attn(rep(g["q"]), rep(g["ck"]), rep(g["cv"]), rep(g["sk"]), rep(g["zk"]), rep(g["sv"]),
                          rep(g["zv"]), rep(g["kr"]), rep(g["vr"]), bits=1, v_mode="token")
    torch.cuda.synchronize()
    assert torch.equal(out[0::2], out[0:1].expand(B // 2, -1, -1))
    assert torch.equal(out[1::2], out[1:2].expand(B // 2, -1, -1))
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], 0, 1,
                              v_token_group=32)
    err = np.abs(to_np(out[:2]) - want)
    assert err.max() < MAX_ABS and err.mean() < MEAN_ABS
