"""`cq_decode_attn_static`, the entry point that allocates nothing: its scratch (per-chunk logit
min / max, flash-decoding partials and - when they fit - the logits the first launch hands to the
second) is a static device buffer inside the library.  Called through the C ABI on two calls in a row, the second with a smaller input, and
compared with `cq_decode_attn` (caller-provided workspace) and with the oracle."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import case_to_gpu, make_case, to_np

pytestmark = pytest.mark.gpu


def _args(lib_mod, g, B, Hq, Hkv, T, R, S, bits, out, force_splits=0):
    for n in ("ck", "cv"):          # the oracle hands out transposed views: the C ABI takes contiguous codes
        g[n] = g[n].contiguous()
    a = lib_mod.DecodeArgs()
    a.q, a.out = g["q"].data_ptr(), out.data_ptr()
    a.codes_k, a.codes_v = g["ck"].data_ptr(), g["cv"].data_ptr()
    a.k_scale, a.k_zero, a.v_scale, a.v_zero = (g[n].data_ptr() for n in ("sk", "zk", "sv", "zv"))
    if R:
        a.k_res, a.v_res = g["kr"].data_ptr(), g["vr"].data_ptr()
        a.res_stride_b, a.res_stride_h, a.res_stride_r = g["kr"].stride(0), g["kr"].stride(1), g["kr"].stride(2)
    a.dtype, a.B, a.Hq, a.Hkv, a.D, a.T, a.R = lib_mod.CQ_BF16, B, Hq, Hkv, 128, T, R
    a.sprompt_len, a.bits, a.calibrate = S, bits, 1
    a.calib_off_max, a.calib_off_min = -3.0, 0.0
    a.force_splits = force_splits
    return a


def test_static_scratch_entry_point_two_calls_in_a_row():
    from calibquant_amd import _lib
    lib = _lib.load()
    assert lib.cq_decode_attn_static_limit() == 8 << 20
    stream = torch.cuda.current_stream().cuda_stream
    # first call: 4 x 12 000 tokens + 50 window rows (chunked: logits + min/max launch, main launch);
    # second call: a smaller input (2 x 9 000 tokens, no window) that reuses the same scratch
    for (B, T, R, S, bits, seed) in ((4, 12000, 50, 7, 1, 401), (2, 9000, 0, 0, 1, 402), (2, 5000, 30, 0, 2, 403)):
        Hq, Hkv = 32, 8
        c = make_case(B, Hq, Hkv, 128, T, max(R, 1), bits, "bf16", seed=seed, outlier_kind="student")
        g = case_to_gpu(c, "bf16")
        out_ws = torch.zeros((B, Hq, 128), dtype=torch.bfloat16, device="cuda")
        out_st = torch.zeros_like(out_ws)
        a = _args(_lib, g, B, Hq, Hkv, T, R, S, bits, out_ws)
        need = lib.cq_decode_attn_workspace(C.byref(a))
        assert 0 < need <= lib.cq_decode_attn_static_limit()          # the chunked path: it does use scratch
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
        assert lib.cq_decode_attn(C.byref(a), stream) == 0
        b = _args(_lib, g, B, Hq, Hkv, T, R, S, bits, out_st)          # no workspace at all
        before = torch.cuda.memory_allocated()
        assert lib.cq_decode_attn_static(C.byref(b), stream) == 0
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(out_ws, out_st)                              # same kernels, same bits
        want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                                  c["kr"][:, :, :R], c["vr"][:, :, :R], S, bits)
        err = np.abs(to_np(out_st) - want)
        assert err.max() < 1e-2 and err.mean() < 1e-3, (T, float(err.max()), float(err.mean()))
    # 2 x 32 768 tokens at 2 bits: the logits the first launch would hand to the second are alone beyond the
    # static buffer, so the static entry point's main launch recomputes them while the workspace entry point
    # reads them back - same bits either way
    B, Hq, Hkv, T, R, S = 2, 32, 8, 32768, 40, 5
    c = make_case(B, Hq, Hkv, 128, T, R, 2, "bf16", seed=405, outlier_kind="student")
    g = case_to_gpu(c, "bf16")
    out_ws = torch.zeros((B, Hq, 128), dtype=torch.bfloat16, device="cuda")
    out_st = torch.zeros_like(out_ws)
    single = lib.cq_decode_attn_single_launch(0)      # (two launches for the workspace entry point as well)
    try:
        a = _args(_lib, g, B, Hq, Hkv, T, R, S, 2, out_ws)
        need = lib.cq_decode_attn_workspace(C.byref(a))
        assert need > lib.cq_decode_attn_static_limit()
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
        assert lib.cq_decode_attn(C.byref(a), stream) == 0
    finally:
        lib.cq_decode_attn_single_launch(single)
    b = _args(_lib, g, B, Hq, Hkv, T, R, S, 2, out_st)
    assert lib.cq_decode_attn_static(C.byref(b), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_ws, out_st)
    # ... and the workspace entry point's single launch (the chunks exchange their min / max inside it and
    # keep their logits: a small workspace) gives the same bits again
    out_one = torch.zeros_like(out_ws)
    a = _args(_lib, g, B, Hq, Hkv, T, R, S, 2, out_one)
    need = lib.cq_decode_attn_workspace(C.byref(a))
    assert 0 < need < lib.cq_decode_attn_static_limit()
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    a.workspace, a.workspace_bytes = ws.data_ptr(), need
    assert lib.cq_decode_attn(C.byref(a), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_one, out_st)
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], S, 2)
    err = np.abs(to_np(out_st) - want)
    assert err.max() < 1e-2 and err.mean() < 1e-3, (T, float(err.max()), float(err.mean()))
    # a single-launch shape needs no scratch and works as well
    c = make_case(2, 32, 8, 128, 700, 20, 1, "bf16", seed=404)
    g = case_to_gpu(c, "bf16")
    o1, o2 = torch.zeros((2, 32, 128), dtype=torch.bfloat16, device="cuda"), torch.zeros((2, 32, 128), dtype=torch.bfloat16, device="cuda")
    a1, a2 = _args(_lib, g, 2, 32, 8, 700, 20, 3, 1, o1), _args(_lib, g, 2, 32, 8, 700, 20, 3, 1, o2)
    assert lib.cq_decode_attn(C.byref(a1), stream) == 0 and lib.cq_decode_attn_static(C.byref(a2), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)


def test_static_scratch_entry_point_rejects_what_exceeds_its_buffer():
    """A plan whose scratch exceeds the static buffer is refused with a clear error before any launch
    (pointers are never looked at)."""
    from calibquant_amd import _lib
    lib = _lib.load()
    a = _lib.DecodeArgs()
    a.dtype, a.B, a.Hq, a.Hkv, a.D, a.T, a.R, a.bits = _lib.CQ_BF16, 64, 32, 8, 128, 32768, 0, 1
    dummy = torch.zeros(64, dtype=torch.uint8, device="cuda")
    for n in ("q", "out", "codes_k", "codes_v", "k_scale", "k_zero", "v_scale", "v_zero"):
        setattr(a, n, dummy.data_ptr())
    assert lib.cq_decode_attn_workspace(C.byref(a)) > lib.cq_decode_attn_static_limit()
    rc = lib.cq_decode_attn_static(C.byref(a), None)
    assert rc == -8 and b"static" in lib.cq_strerror(rc)
