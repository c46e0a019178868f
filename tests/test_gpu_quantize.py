"""GPU parity of the prefill quantise-and-pack kernels against the oracle:
bit-exact codes, scales and zero-points (through the C-ABI library)."""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import CLIPS, TDT, same_bits, to_gpu, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from calibquant_amd import ops
    return ops


SHAPES = [(2, 257, 3, 128), (1, 1, 2, 128), (3, 63, 1, 64), (1, 1000, 2, 256), (2, 3328, 8, 128),
          (1, 1500, 1, 128), (1, 2100, 2, 128), (1, 5000, 2, 128)]   # one-pass kernel row counts; beyond its reach


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("shape", SHAPES)
def test_quantize_pack_bit_exact(ops, shape, bits, dtype):
    B, T, H, D = shape
    print(f"case quantize_pack shape={shape} bits={bits} dtype={dtype}", flush=True)
    k, v = O.synth_kv(B, T, H, D, dtype, seed=B * 1000 + T)
    for x, clip in zip((k, v), CLIPS[bits]):
        codes, s, z = ops.quantize_pack(to_gpu(x, dtype), bits, clip)
        torch.cuda.synchronize()
        oc, os_, oz = O.quantize_pack(x, bits, clip, dtype)
        assert same_bits(to_np(s), os_)
        assert same_bits(to_np(z), oz)
        assert np.array_equal(codes.cpu().numpy(), oc)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_quantize_pack_reads_the_strided_wqkv_view(ops, dtype):
    """The reference quantises views of the fused wqkv output
    (patch_internvl.py:219-234, 284, 290): token stride (Hq+2Hkv)*D, head stride (G+2)*D."""
    B, N, Hkv, G, D, S, T = 2, 300, 2, 4, 128, 41, 200
    rng = np.random.default_rng(0)
    qkv = O.round_to(rng.standard_normal((B, N, Hkv, G + 2, D), dtype=np.float32), dtype)
    t = to_gpu(qkv, dtype)
    kview = t[:, S:S + T, :, G, :]
    vview = t[:, S:S + T, :, G + 1, :]
    assert not kview.is_contiguous()
    for view, ref, clip in ((kview, qkv[:, S:S + T, :, G], 0.5), (vview, qkv[:, S:S + T, :, G + 1], 0.3)):
        codes, s, z = ops.quantize_pack(view, 1, clip)
        oc, os_, oz = O.quantize_pack(ref, 1, clip, dtype)
        assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
        assert np.array_equal(codes.cpu().numpy(), oc)


@pytest.mark.parametrize("bits", [1, 2])
def test_quantize_pack_long_context_single_sequence(ops, bits):
    """One sequence of 32 768 tokens: few (batch, head) pairs, so the statistics of a channel are
    folded from 256 chunk partials and every threshold level is searched by its own threads."""
    B, T, H, D = 1, 32768, 2, 128
    print(f"case quantize_pack long context bits={bits}", flush=True)
    k, v = O.synth_kv(B, T, H, D, "bf16", seed=77)
    for x, clip in zip((k, v), CLIPS[bits]):
        codes, s, z = ops.quantize_pack(to_gpu(x, "bf16"), bits, clip)
        torch.cuda.synchronize()
        oc, os_, oz = O.quantize_pack(x, bits, clip, "bf16")
        assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
        assert np.array_equal(codes.cpu().numpy(), oc)


def test_quantize_pack_constant_channel_matches_ieee_reference(ops):
    x = np.random.default_rng(1).standard_normal((1, 64, 2, 128)).astype(np.float32)
    x = O.round_to(x, "bf16")
    x[0, :, 1, 5] = 1.5        # scale 0, zero -inf, codes NaN -> index 0
    x[0, :, 0, 9] = -2.0       # scale 0, zero +inf
    x[0, :, 0, 17] = 0.0       # scale 0, zero NaN
    codes, s, z = ops.quantize_pack(to_gpu(x, "bf16"), 1, 0.5)
    oc, os_, oz = O.quantize_pack(x, 1, 0.5, "bf16")
    assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
    assert np.array_equal(codes.cpu().numpy(), oc)
    assert to_np(s)[0, 1, 5] == 0 and np.isinf(to_np(z)[0, 1, 5])


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
def test_quant_and_encode_operators(ops, bits, dtype):
    """The unfused pair quant() + encode() gives the same bytes as the fused kernel."""
    B, T, H, D = 2, 130, 2, 128
    k, _ = O.synth_kv(B, T, H, D, dtype, seed=3)
    x = to_gpu(k, dtype)
    clip = CLIPS[bits][0]
    xq, s, z = ops.quant_codes(x, bits, clip)
    oxq, os_, oz = O.quant(k, bits, clip, dtype)
    assert same_bits(to_np(xq), oxq) and same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
    for idx in (xq.transpose(1, 2).contiguous(), xq.transpose(1, 2).long(), xq.transpose(1, 2).to(torch.int32),
                xq.transpose(1, 2).to(torch.uint8)):
        enc = ops.encode_indices(idx, bits)
        codes, _, _ = ops.quantize_pack(x, bits, clip)
        assert torch.equal(enc, codes)


@pytest.mark.parametrize("B", [4, 64])
@pytest.mark.parametrize("bits", [1, 2])
def test_quantize_pack_matches_torch_device_op_chain(ops, bits, B):
    """torch's own device kernels, run op by op on the 16-bit tensor, are the
    primitives the reference executes (calibquant.py:27-36).  At batch 64 (the benchmark's prefill
    tensor) every workgroup of the one-pass kernel walks eight slices, the later ones with part of
    their rows staged through LDS."""
    T, H, D = 3328, 8, 128
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((B, T, H, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    clip = CLIPS[bits][0]
    L = 2 ** bits - 1
    mn = x.amin(dim=1, keepdim=True) * clip
    mx = x.amax(dim=1, keepdim=True) * clip
    s = (mx - mn) / L
    z = -mn / s
    xq = torch.round(torch.clamp(x / s + z, 0, L))
    codes, ks, kz = ops.quantize_pack(x, bits, clip)
    assert torch.equal(ks, s[:, 0]) and torch.equal(kz, z[:, 0])
    enc = ops.encode_indices(xq.transpose(1, 2).contiguous(), bits)
    assert torch.equal(enc, codes)


@pytest.mark.parametrize("bits", [1, 2])
def test_quantize_pack_full_size_properties(ops, bits):
    """Prefill tensor of the long-context configuration (1, 32768, 8, 128):
    size-independent properties.  Codes lie in range, every channel attains
    code 0 and code L when clip == 1, and dequantising then re-quantising
    reproduces the bytes."""
    B, T, H, D = 1, 32768, 8, 128
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn((B, T, H, D), generator=g, device="cuda").to(torch.bfloat16)
    codes, s, z = ops.quantize_pack(x, bits, 1.0)
    L = 2 ** bits - 1
    dpe = 8 // bits
    shifts = torch.tensor([bits * (dpe - 1 - i) for i in range(dpe)], device="cuda", dtype=torch.uint8)
    un = ((codes[..., None] >> shifts) & L).reshape(B, H, T, D)
    assert int(un.amin()) == 0 and int(un.amax()) == L
    assert torch.all(un.amin(dim=2) == 0) and torch.all(un.amax(dim=2) == L)
    # fixed point: re-quantising the dequantised tensor in fp32-exact levels keeps the codes
    deq = (s.float()[:, :, None] * (un.float() - z.float()[:, :, None])).to(torch.bfloat16)
    codes2, _, _ = ops.quantize_pack(deq.transpose(1, 2), bits, 1.0)
    un2 = ((codes2[..., None] >> shifts) & L).reshape(B, H, T, D)
    assert (un2 != un).float().mean().item() < 2e-3


# Token axes beyond what one workgroup's registers hold of a slice (3 328 rows): the one-pass kernel splits a slice
# between 2, 4, ... workgroups of its launch when a part then has more than 2 048 rows (parts x rows per part ->
# rows per thread); the other shapes take three launches.
LONG_SHAPES = [(2, 9984, 8, 128),    # 4 x 2496 -> 10: the 26B prompt's token count
               (3, 3329, 2, 128),    # just beyond one workgroup: three launches
               (4, 13000, 1, 128),   # 4 x 3250 -> 13
               (2, 40000, 2, 128),   # 16 x 2500 -> 10
               (1, 40000, 1, 128),   # a single (batch, head) pair: three launches
               (9, 5000, 8, 128),    # 2 x 2500 -> 10; 288 slices x 2 parts: more ids than workgroups, 3 steps
               (2, 7000, 8, 128)]    # three launches


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("shape", LONG_SHAPES)
def test_quantize_pack_long_token_axis_bit_exact(ops, shape, bits, dtype):
    B, T, H, D = shape
    print(f"case quantize_pack long shape={shape} bits={bits} dtype={dtype}", flush=True)
    k, _ = O.synth_kv(B, T, H, D, dtype, seed=T + bits)
    clip = CLIPS[bits][0]
    codes, s, z = ops.quantize_pack(to_gpu(k, dtype), bits, clip)
    torch.cuda.synchronize()
    oc, os_, oz = O.quantize_pack(k, bits, clip, dtype)
    assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
    assert np.array_equal(codes.cpu().numpy(), oc)


def test_quantize_pack_long_token_axis_strided_view(ops):
    B, N, Hkv, G, D, S, T = 2, 10100, 2, 4, 128, 41, 9984
    rng = np.random.default_rng(5)
    qkv = O.round_to(rng.standard_normal((B, N, Hkv, G + 2, D), dtype=np.float32), "bf16")
    t = to_gpu(qkv, "bf16")
    view = t[:, S:S + T, :, G, :]
    assert not view.is_contiguous()
    codes, s, z = ops.quantize_pack(view, 1, 0.5)
    oc, os_, oz = O.quantize_pack(qkv[:, S:S + T, :, G], 1, 0.5, "bf16")
    assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
    assert np.array_equal(codes.cpu().numpy(), oc)


def test_quantize_pack_split_slices_give_up_and_the_host_reports_it(ops):
    """The parts of a split slice wait for each other a bounded number of polls.  With the bound at zero every
    part goes on alone (the kernel ends normally; its statistics are those of single parts, i.e. not valid): the
    call returns success, the next call on the device reports the failure once, and from then on long token axes
    take the three-launch path - bit-exact - until the bound is set again."""
    from calibquant_amd import _lib
    lib = _lib.load()
    B, T, H, D = 2, 9984, 2, 128
    k, _ = O.synth_kv(B, T, H, D, "bf16", seed=31)
    x = to_gpu(k, "bf16")
    oc, os_, oz = O.quantize_pack(k, 1, 0.5, "bf16")

    def check():
        codes, s, z = ops.quantize_pack(x, 1, 0.5)
        torch.cuda.synchronize()
        assert same_bits(to_np(s), os_) and same_bits(to_np(z), oz)
        assert np.array_equal(codes.cpu().numpy(), oc)
    check()
    before = lib.cq_quantize_pack_wait_polls(0)
    try:
        ops.quantize_pack(x, 1, 0.5)          # launched; every part gives up
        torch.cuda.synchronize()
        with pytest.raises(_lib.CalibQuantError):
            ops.quantize_pack(x, 1, 0.5)      # the host finds the word set
        check()                               # three launches from here on
    finally:
        lib.cq_quantize_pack_wait_polls(before)
    check()
