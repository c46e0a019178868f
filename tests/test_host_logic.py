"""Host-side logic that needs no GPU: the C-ABI library's exports, argument
validation at the Python boundary, cache bookkeeping, RoPE / GQA helpers."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    from calibquant_amd import _lib
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "calibquant_hip.h")).read()
    declared = set(re.findall(r"\b(cq_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(_lib.SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.cq_version() >= 100
    assert b"NULL" in lib.cq_strerror(-1) and lib.cq_strerror(0) == b"ok"


def test_decode_launch_plan_is_a_function_of_the_shape():
    """`cq_decode_attn_plan` (host only): which launch a shape gets.  Two 512-thread workgroups per compute
    unit need a layout within half of the 160 KB LDS and more units of work than the 256 compute units;
    logits kept in registers only at 1 bit with four heads per unit; chunked shapes take two launches, or one
    when all their workgroups fit the device at once."""
    from calibquant_amd import _lib
    lib = _lib.load()

    def plan(B, Hq, Hkv, T, R, bits=1, v_mode=0, force_splits=0):
        a = _lib.DecodeArgs()
        a.dtype, a.D, a.B, a.Hq, a.Hkv, a.T, a.R, a.bits, a.v_mode, a.force_splits = 0, 128, B, Hq, Hkv, T, R, bits, v_mode, force_splits
        p = _lib.DecodePlan()
        assert lib.cq_decode_attn_plan(ctypes.byref(a), ctypes.byref(p)) == 0
        return {n: getattr(p, n) for n, _ in p._fields_}

    bench = plan(64, 32, 8, 3328, 128)
    assert (bench["threads"], bench["heads_per_unit"], bench["launches"], bench["register_logits"]) == (512, 4, 1, 8)
    assert bench["lds_bytes"] <= 80 * 1024 and bench["chunk_tokens"] == 3328
    small = plan(32, 32, 8, 3328, 128)                       # 256 units: one 1024-thread workgroup per compute unit
    assert (small["threads"], small["register_logits"], small["launches"]) == (1024, 0, 1)
    two_bit = plan(64, 32, 8, 3328, 128, bits=2)            # 2 bits: paired as well, K table in two passes
    assert (two_bit["threads"], two_bit["register_logits"]) == (512, 8) and two_bit["lds_bytes"] <= 80 * 1024
    assert plan(32, 32, 8, 3328, 128, bits=2)["threads"] == 1024
    assert plan(64, 32, 8, 3328, 128, v_mode=1)["threads"] == 1024
    assert plan(64, 32, 8, 3328, 128, force_splits=2) == dict(plan(64, 32, 8, 3328, 128, force_splits=2), threads=1024, launches=2)
    two = plan(128, 16, 8, 3328, 128)                        # two heads per unit: paired, fp32 logits
    assert (two["threads"], two["heads_per_unit"], two["register_logits"]) == (512, 2, 0)
    long = plan(8, 32, 8, 32768, 0)                          # chunked: the chunks are the units; all 512 resident: one launch
    assert long["launches"] == 1 and long["threads"] == 512 and long["chunks"] * long["chunk_tokens"] >= 32768
    assert long["lds_bytes"] <= 80 * 1024
    assert plan(16, 32, 8, 32768, 0)["launches"] == 2        # twice the workgroups: they cannot all wait for each other
    assert lib.cq_decode_attn_single_launch(0) == 1          # the process-wide switch
    try:
        assert plan(8, 32, 8, 32768, 0) == dict(long, launches=2)
    finally:
        assert lib.cq_decode_attn_single_launch(1) == 0
    big = plan(16, 48, 8, 9984, 64)     # six heads per kv head: two exact units of three; one launch
    assert (big["threads"], big["heads_per_unit"], big["launches"], big["register_logits"]) == (1024, 3, 1, 10)   # logits in registers
    assert plan(64, 48, 8, 3328, 128)["heads_per_unit"] == 3 and plan(64, 48, 8, 3328, 128)["threads"] == 512
    assert plan(64, 24, 8, 3328, 128, bits=2)["heads_per_unit"] == 3      # three heads per kv head: one exact unit
    assert plan(64, 40, 8, 3328, 128)["heads_per_unit"] == 4              # five: units of 4 + 1
    assert big["lds_bytes"] <= 160 * 1024
    tok = plan(16, 48, 8, 9984, 64, v_mode=1)               # per-token values: padded four-head units too, chunked (16-byte slots)
    assert (tok["heads_per_unit"], tok["threads"], tok["register_logits"]) == (4, 1024, 0) and tok["launches"] == 2
    a = _lib.DecodeArgs()
    assert lib.cq_decode_attn_plan(ctypes.byref(a), None) < 0
    assert lib.cq_decode_attn_plan(ctypes.byref(a), ctypes.byref(_lib.DecodePlan())) < 0   # all-zero arguments


def test_decode_launch_plan_invariants_over_random_shapes():
    """Whatever the shape, the plan stays inside what the kernels assume: LDS within the device's 160 KB (half of
    it for a 512-thread workgroup), chunks that cover T, register-resident logits only for chunks that fit the
    rounds a thread keeps, two launches and a workspace exactly when T is chunked."""
    from calibquant_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(11)
    for _ in range(3000):
        Hkv = int(rng.choice([1, 2, 4, 8, 16]))
        G = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16]))
        a = _lib.DecodeArgs()
        a.dtype, a.D, a.Hkv, a.Hq = int(rng.integers(0, 2)), 128, Hkv, Hkv * G
        a.B = int(rng.choice([1, 2, 3, 8, 16, 31, 32, 33, 64, 100, 256, 1000]))
        a.T = int(rng.choice([0, 1, 63, 64, 65, 1000, 3328, 3392, 4096, 4097, 4288, 5000, 9984, 10240, 10241, 32768, 100000]))
        a.R = int(rng.choice([0, 1, 64, 128, 129, 1000])) if a.T else int(rng.choice([1, 64, 500]))
        a.bits = int(rng.integers(1, 3))
        a.v_mode = int(rng.integers(0, 2))
        a.force_splits = int(rng.choice([0, 0, 0, 1, 2, 7]))
        p = _lib.DecodePlan()
        assert lib.cq_decode_attn_plan(ctypes.byref(a), ctypes.byref(p)) == 0
        shape = (a.B, a.Hq, a.Hkv, a.T, a.R, a.bits, a.v_mode, a.force_splits)
        assert p.threads in (512, 1024) and p.heads_per_unit in (1, 2, 3, 4), shape
        G_ = a.Hq // a.Hkv
        assert (p.heads_per_unit == 3) <= (G_ % 3 == 0 and G_ % 4 != 0 and a.v_mode == 0), shape   # three only for exact units
        assert 0 < p.lds_bytes <= (80 if p.threads == 512 else 160) * 1024, shape
        assert p.chunks >= 1 and p.chunks * p.chunk_tokens >= a.T, shape
        assert p.chunk_tokens % 64 == 0, shape
        assert p.register_logits == 0 or p.chunk_tokens <= p.register_logits * p.threads, shape
        assert p.launches in (1, 2) and (p.launches == 1 or p.chunks > 1), shape
        if p.launches == 1 and p.chunks > 1:      # one launch: every chunk's workgroup resident at once
            units_ = a.B * a.Hkv * -(-G_ // p.heads_per_unit)
            assert units_ * p.chunks <= 256 * (2 if p.threads == 512 else 1) and p.chunks <= 64, shape
        assert (lib.cq_decode_attn_workspace(ctypes.byref(a)) > 0) == (p.chunks > 1), shape
        if a.v_mode == 1:
            assert p.threads == 1024 and p.register_logits == 0, shape


def test_c_abi_rejects_bad_arguments_without_touching_the_gpu():
    """Validation happens before any launch, so these calls are safe without a device."""
    from calibquant_amd import _lib
    lib = _lib.load()
    a = _lib.DecodeArgs()
    assert lib.cq_decode_attn(ctypes.byref(a), None) < 0                  # dtype/shape all zero
    a.dtype, a.bits, a.D, a.B, a.Hq, a.Hkv, a.T, a.R = 0, 3, 128, 1, 32, 8, 64, 0
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -7                # 3-bit unsupported
    a.bits, a.D = 1, 64
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -7                # head_dim 64 unsupported
    a.D, a.Hq = 128, 30
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -2                # Hq not a multiple of Hkv
    a.Hq, a.T, a.R = 32, 0, 0
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -2                # nothing to attend to
    a.T = 64
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -1                # NULL pointers
    assert lib.cq_decode_attn_workspace(ctypes.byref(a)) == 0             # fits one unit: no workspace
    a.T, a.B = 32768, 8
    ws = lib.cq_decode_attn_workspace(ctypes.byref(a))
    assert ws > 0 and ws % 4 == 0                                         # chunked path needs partials
    # 8 token chunks of partial min / max, then 3 thresholds per channel, + 4 rows for the whole-tensor mode
    assert lib.cq_quantize_pack_workspace(64, 3328, 8, 128) == (64 * 8 * (8 * 2 + 3) + 4) * 128 * 4
    a.T, a.B, a.v_mode = 64, 1, 7
    assert lib.cq_decode_attn(ctypes.byref(a), None) == -7                # unknown value layout
    assert lib.cq_quantize_pack_token(None, 0, 1, 1, 1, 128, 0, 0, 0, 1, 32, None, None, None, None) == -1
    assert lib.cq_rope_append(None, 0, 1, 32, 8, 128, None, None, 1, None, 1, None, None, None, 0, 0, 0, 1, None, None) == -1
    assert lib.cq_quantize_pack(None, 0, 1, 1, 1, 128, 0, 0, 0, 1, 0.5, None, None, None, None, 0, None) == -1
    assert lib.cq_encode(None, 3, 1, 128, 1, None, None) == -1


def test_ops_refuse_cpu_tensors_and_unsupported_dtypes():
    from calibquant_amd import ops
    from calibquant_amd._lib import CalibQuantError
    x = torch.zeros((1, 4, 1, 128), dtype=torch.bfloat16)
    with pytest.raises(CalibQuantError, match="GPU"):
        ops.quantize_pack(x, 1, 0.5)
    with pytest.raises(CalibQuantError, match="GPU"):
        ops.decode_attn(torch.zeros((1, 8, 128), dtype=torch.bfloat16), None, None, None, None, None, None, x, x)
    from calibquant_amd import calibquant
    with pytest.raises(CalibQuantError):
        calibquant.quant(x, 1, per_channel=False)
    with pytest.raises(CalibQuantError):
        calibquant.quant(x, 4, per_channel=True)


def test_reference_constants_and_helpers():
    from calibquant_amd import calibquant as cq, patch_internvl as pi
    assert (cq.BITS_KV, cq.SCALE_K, cq.SCALE_V, cq.DEVICE, cq.DATA_TYPE) == (1, 0.5, 0.3, "cuda", torch.float16)
    assert (pi.BITS_KV, pi.SCALE_K, pi.SCALE_V, pi.SPROMPT_LEN, pi.CHUNK_SIZE, pi.LOW_BITS) == (1, 0.5, 0.3, 41, 1024, True)
    assert set(pi.ATTN_FORWARD_FUNCTIONS) == {"calibquant", "qjl"}
    x = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).reshape(2, 3, 4, 5)
    assert torch.equal(pi.repeat_kv(x, 3), torch.repeat_interleave(x, 3, dim=1))
    assert pi.repeat_kv(x, 1) is x
    # rotary embedding against the textbook complex rotation
    torch.manual_seed(0)
    D, N = 8, 6
    q, k = torch.randn(1, 2, N, D), torch.randn(1, 1, N, D)
    inv = 1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.outer(torch.arange(N).float(), inv)
    cos, sin = torch.cat([ang, ang], -1).cos(), torch.cat([ang, ang], -1).sin()
    pos = torch.arange(N)[None]
    qe, ke = pi.apply_rotary_pos_emb(q, k, cos, sin, pos)
    qc = torch.complex(q[..., : D // 2], q[..., D // 2:]) * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(qe, torch.cat([qc.real, qc.imag], -1), atol=1e-6)
    assert torch.allclose((qe @ ke.transpose(-1, -2))[0, 0].diagonal(), (q @ k.transpose(-1, -2))[0, 0].diagonal(),
                          atol=1e-4)   # equal positions: rotation cancels in the dot product
    with pytest.raises(Exception):
        pi.patch_model(object(), quant_method="qjl")


def test_growing_kv_appends_in_place_and_survives_foreign_tensors():
    from calibquant_amd.kvbuffer import GrowingKV
    kv = GrowingKV()
    k0, v0 = torch.randn(2, 3, 5, 4), torch.randn(2, 3, 5, 4)
    k, v = kv.append(None, k0, v0)
    assert k.shape == (2, 3, 5, 4) and torch.equal(k, k0)
    ptr = k.data_ptr()
    k1, v1 = torch.randn(2, 3, 1, 4), torch.randn(2, 3, 1, 4)
    k, v = kv.append((k, v), k1, v1)
    assert k.data_ptr() == ptr and k.shape[2] == 6                      # appended in place
    assert torch.equal(k[:, :, :5], k0) and torch.equal(k[:, :, 5:], k1) and torch.equal(v[:, :, 5:], v1)
    foreign = (torch.randn(2, 3, 9, 4), torch.randn(2, 3, 9, 4))
    k, v = kv.append(foreign, k1, v1)                                    # not ours: copied
    assert k.shape[2] == 10 and torch.equal(k[:, :, :9], foreign[0]) and torch.equal(k[:, :, 9:], k1)
    for _ in range(600):                                                 # grow past the capacity
        k, v = kv.append((k, v), k1, v1)
    assert k.shape[2] == 610 and torch.equal(k[:, :, :9], foreign[0])


def test_internlm2_wqkv_interleave_matches_the_reference_rearrange():
    """`b q (h gs d) -> b q h gs d` with gs = groups + 2: q heads, then k, then v per kv head."""
    from einops import rearrange
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    cfg = InternLM2Config.tiny()
    att = InternLM2Attention(cfg)
    x = torch.randn(2, 3, cfg.hidden_size)
    q, k, v = att.split_qkv(x)
    qkv = rearrange(att.wqkv(x), "b q (h gs d) -> b q h gs d", gs=2 + att.num_key_value_groups, d=att.head_dim)
    assert torch.equal(q, rearrange(qkv[..., : att.num_key_value_groups, :], "b q h gs d -> b q (h gs) d"))
    assert torch.equal(k, qkv[..., -2, :]) and torch.equal(v, qkv[..., -1, :])


def test_image_token_count_is_reread_from_the_environment_every_forward(monkeypatch):
    """The reference reads IMAGE_TOKEN_NUM on every forward (patch_internvl.py:189,251): a caller that
    only updates the variable between prompts must get the new count; an explicit override on the
    module wins; the attribute a forward publishes never feeds back into the next one."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd._lib import CalibQuantError

    class Att:
        pass

    att = Att()
    monkeypatch.delenv("IMAGE_TOKEN_NUM", raising=False)
    with pytest.raises(CalibQuantError):
        pi._image_token_num(att)
    monkeypatch.setenv("IMAGE_TOKEN_NUM", "3328")
    att.image_token_num = pi._image_token_num(att)        # what a forward publishes on the module
    assert att.image_token_num == 3328
    monkeypatch.setenv("IMAGE_TOKEN_NUM", "512")           # second prompt, no custom_generate in between
    assert pi._image_token_num(att) == 512
    att.cq_image_token_num = 256                            # the explicit channel (custom_generate sets it)
    assert pi._image_token_num(att) == 256


def test_host_shim_loads_and_matches_the_library():
    """`_cq_torch_step.so` (the C++ step object of the eager decode path) imports, exposes `LayerStep`
    and was built against the same library version; no GPU call is made."""
    from calibquant_amd import _lib
    shim = _lib.load_step_shim()
    assert shim.library_version() == _lib.load().cq_version()
    assert {"step", "length", "steps", "capacity"} <= set(dir(shim.LayerStep))
    import ctypes as C
    import torch
    with pytest.raises(Exception):      # CPU tensors / wrong block size are refused before any launch
        shim.LayerStep(C.addressof(_lib.DecodeArgs()), 8, torch.zeros(1), torch.zeros(1), torch.zeros(1),
                       torch.zeros(1), 0, torch.zeros(1, dtype=torch.int64))
