"""Fused operators of the MI355X CalibQuant path (torch tensors in, HIP out).

`quantize_pack` replaces the prefill chain quant -> LUT indices -> encode of the
reference (calibquant.py:24-42, patch_internvl.py:318-329, calibquant.py:114-137)
and `decode_attn` replaces its decode branch (patch_internvl.py:344-436).  Both
call the C-ABI library on torch's current stream; torch only owns the memory."""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib

_DT = {torch.bfloat16: _lib.CQ_BF16, torch.float16: _lib.CQ_FP16, torch.float32: _lib.CQ_FP32,
       torch.int64: _lib.CQ_I64, torch.int32: _lib.CQ_I32, torch.uint8: _lib.CQ_U8}


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise _lib.CalibQuantError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")


def _storage_dtype(t: torch.Tensor, name: str) -> int:
    if t.dtype not in (torch.bfloat16, torch.float16):
        raise _lib.CalibQuantError(f"{name}: dtype {t.dtype} not supported (bf16 / fp16 only)")
    return _DT[t.dtype]


def _workspace(nbytes: int, device) -> Optional[torch.Tensor]:
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def empty_token_rows(B: int, T: int, H: int, D: int, dtype, device) -> torch.Tensor:
    """An uninitialised (B, T, H, D) tensor for keys or values that the quantiser will read: token rows of
    H * D elements, plus 128 bytes of padding per row where rows would otherwise lie a multiple of 2 KB apart -
    the one-pass quantiser's slices then meet too few memory channels (measured at batch 64 x 3 328 tokens x 8
    heads: 129 us per tensor contiguous, 105 us padded).  The result is a view; D stays contiguous."""
    row = H * D
    pad = 64 if (row * torch.empty((), dtype=dtype).element_size()) % 2048 == 0 else 0
    return torch.empty((B, T, row + pad), dtype=dtype, device=device)[:, :, :row].unflatten(2, (H, D))


_decode_ws = {}


def _decode_workspace(nbytes: int, device) -> Optional[torch.Tensor]:
    """The workspace of a chunked decode call: one buffer per (device, stream), shared by every call made on
    that stream (the layers of a model run one after the other; calls on one stream are ordered) and grown when
    a call needs more.  A call keeps a reference to the buffer it was prepared with, so a buffer that has been
    outgrown lives as long as the calls that use it.  Nothing in it has to survive from one call to the next."""
    if nbytes == 0:
        return None
    dev = torch.device(device)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    ws = _decode_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _decode_ws[key] = ws
    return ws


def quantize_pack(x: torch.Tensor, bits: int, clip: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-channel min-max quantise and bit-pack one K or V tensor.

    x: (B, T, H, D) view (any b/t/h strides, D contiguous), bf16 or fp16.
    Returns codes uint8 (B, H, T, D*bits/8), scale (B, H, D), zero (B, H, D)."""
    _need_gpu(x, "x")
    dt = _storage_dtype(x, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, D) with a contiguous last axis")
    B, T, H, D = x.shape
    lib = _lib.load()
    codes = torch.empty((B, H, T, D * bits // 8), dtype=torch.uint8, device=x.device)
    scale = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    zero = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    ws = _workspace(lib.cq_quantize_pack_workspace(B, T, H, D), x.device)
    with torch.cuda.device(x.device):
        rc = lib.cq_quantize_pack(x.data_ptr(), dt, B, T, H, D, x.stride(0), x.stride(1), x.stride(2),
                                  bits, float(clip), codes.data_ptr(), scale.data_ptr(), zero.data_ptr(),
                                  ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
                                  _stream(x))
    _lib.check(rc, "cq_quantize_pack")
    return codes, scale, zero


def _rope_args(x, cos, sin, pos, out):
    """Common argument block of the two rotary entry points."""
    for t, n in ((cos, "cos"), (sin, "sin"), (out, "out")):
        _need_gpu(t, n)
        if t.dtype != x.dtype:
            raise _lib.CalibQuantError("rope: cos, sin and out must share x's dtype")
    if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != x.shape[3] or not (cos.is_contiguous() and sin.is_contiguous()):
        raise _lib.CalibQuantError("rope: cos / sin must be contiguous (rows, D) tables")
    if out.shape != x.shape or out.stride(3) != 1:
        raise _lib.CalibQuantError("rope: out must be shaped like x with a contiguous last axis")
    B, T = x.shape[0], x.shape[1]
    if isinstance(pos, int):
        pos_args = (None, 0, 0, int(pos))
        keep = None
    else:
        _need_gpu(pos, "pos")
        if pos.dtype != torch.int64 or pos.shape != (B, T):
            raise _lib.CalibQuantError("rope: pos must be an int64 (B, T) tensor or an int (first position of an arange)")
        pos_args = (pos.data_ptr(), pos.stride(0), pos.stride(1), 0)
        keep = pos
    return (x.data_ptr(), _storage_dtype(x, "x"), *x.shape, x.stride(0), x.stride(1), x.stride(2),
            cos.data_ptr(), sin.data_ptr(), cos.shape[0], *pos_args,
            out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)), keep


def rope_rows(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos, out: Optional[torch.Tensor] = None):
    """Rotary embedding of x (B, T, H, D) (any b/t/h strides) with the reference's rounding:
    rnd(rnd(x*cos) + rotate_half(x)*sin).  cos / sin: (rows, D) tables; pos: int64 (B, T) position
    ids (any strides) or an int p0 for positions p0 + t.  Writes `out` (shaped like x) or a new
    contiguous tensor."""
    _need_gpu(x, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, D) with a contiguous last axis")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    args, keep = _rope_args(x, cos, sin, pos, out)
    with torch.cuda.device(x.device):
        rc = _lib.load().cq_rope_rows(*args, _stream(x))
    _lib.check(rc, "cq_rope_rows")
    return out


def rope_rows_grouped(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos, out: Optional[torch.Tensor] = None):
    """`rope_rows` over x (B, T, H, G, D) (any b/t/h/g strides) in one launch: the query block of the fused
    projection output, where the G query heads of a kv head sit side by side.  `out`: shaped like x."""
    _need_gpu(x, "x")
    if x.dim() != 5 or x.stride(4) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, G, D) with a contiguous last axis")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if out.shape != x.shape or out.stride(4) != 1:
        raise _lib.CalibQuantError("rope: out must be shaped like x with a contiguous last axis")
    args, keep = _rope_args(x[:, :, :, 0], cos, sin, pos, out[:, :, :, 0])
    (xp, dt, B, T, H, D, sb, st_, sh, cp, sp, rows, pp, psb, pst, p0, op, ob, ot, oh) = args
    with torch.cuda.device(x.device):
        rc = _lib.load().cq_rope_rows_grouped(xp, dt, B, T, H, x.shape[3], D, sb, st_, sh, x.stride(3), cp, sp, rows,
                                              pp, psb, pst, p0, op, ob, ot, oh, out.stride(3), _stream(x))
    _lib.check(rc, "cq_rope_rows_grouped")
    return out


def rope_quantize_pack(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos, out: torch.Tensor,
                       bits: int, clip: float):
    """`quantize_pack(rope(x))` in one pass over x: x (B, T, H, D) is the UN-rotated key block; the
    rotated rows are written to `out` (shaped like x) and quantised from the registers.  Returns
    codes uint8 (B, H, T, D*bits/8), scale (B, H, D), zero (B, H, D), bit-identical to
    `quantize_pack(rope_rows(x, ...), bits, clip)`.  Raises `CalibQuantError` (unsupported) for shapes
    outside the one-pass path (T > 3 328 or D != 128)."""
    _need_gpu(x, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, D) with a contiguous last axis")
    B, T, H, D = x.shape
    args, keep = _rope_args(x, cos, sin, pos, out)
    lib = _lib.load()
    codes = torch.empty((B, H, T, D * bits // 8), dtype=torch.uint8, device=x.device)
    scale = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    zero = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    ws = _workspace(lib.cq_quantize_pack_workspace(B, T, H, D), x.device)
    with torch.cuda.device(x.device):
        rc = lib.cq_rope_quantize_pack(*args, int(bits), float(clip), codes.data_ptr(), scale.data_ptr(),
                                       zero.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "cq_rope_quantize_pack")
    return codes, scale, zero


ROPE_FUSED_MAX_T = 3328      # the one-pass quantiser holds a (batch, head) slice of at most this many rows


def quantize_pack_token(x: torch.Tensor, bits: int, group_size: int = 32):
    """Per-token min-max quantiser of the values (`v_mode = token`): x (B, T, H, D) view, bf16 or
    fp16, D = 128, groups of 32 channels.  Returns words int32 (B, H, T, D*bits/32) (first channel
    in the lowest bits), scale (B, H, T, D/32), mins (B, H, T, D/32); a value is scale*code + min."""
    _need_gpu(x, "x")
    dt = _storage_dtype(x, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, D) with a contiguous last axis")
    B, T, H, D = x.shape
    lib = _lib.load()
    words = torch.empty((B, H, T, D * bits // 32), dtype=torch.int32, device=x.device)
    scale = torch.empty((B, H, T, D // group_size), dtype=x.dtype, device=x.device)
    mins = torch.empty_like(scale)
    with torch.cuda.device(x.device):
        rc = lib.cq_quantize_pack_token(x.data_ptr(), dt, B, T, H, D, x.stride(0), x.stride(1), x.stride(2),
                                        int(bits), int(group_size), words.data_ptr(), scale.data_ptr(),
                                        mins.data_ptr(), _stream(x))
    _lib.check(rc, "cq_quantize_pack_token")
    return words, scale, mins


def quant_codes(x: torch.Tensor, bits: int, clip: float):
    """The unfused quantiser: x (B, T, H, D) -> (x_q (B, T, H, D) of x.dtype
    holding the integer codes, scale (B, 1, H, D), zero (B, 1, H, D))."""
    _need_gpu(x, "x")
    dt = _storage_dtype(x, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise _lib.CalibQuantError("x must be (B, T, H, D) with a contiguous last axis")
    B, T, H, D = x.shape
    lib = _lib.load()
    xq = torch.empty((B, T, H, D), dtype=x.dtype, device=x.device)
    scale = torch.empty((B, 1, H, D), dtype=x.dtype, device=x.device)
    zero = torch.empty((B, 1, H, D), dtype=x.dtype, device=x.device)
    ws = _workspace(lib.cq_quantize_pack_workspace(B, T, H, D), x.device)
    with torch.cuda.device(x.device):
        rc = lib.cq_quant(x.data_ptr(), dt, B, T, H, D, x.stride(0), x.stride(1), x.stride(2),
                          bits, float(clip), xq.data_ptr(), scale.data_ptr(), zero.data_ptr(),
                          ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream(x))
    _lib.check(rc, "cq_quant")
    return xq, scale, zero


def quant_codes_tensor(x: torch.Tensor, bits: int, clip: float):
    """The unfused quantiser with one minimum / maximum over the whole tensor (the reference's
    `per_channel=False`): x (..., D) -> (x_q shaped like x holding the integer codes, scale (), zero ())."""
    _need_gpu(x, "x")
    dt = _storage_dtype(x, "x")
    shape = x.shape
    if x.dim() == 4 and x.stride(3) == 1:
        x4 = x
    else:
        if x.dim() < 1 or shape[-1] not in (64, 128, 256):
            raise _lib.CalibQuantError("x must end in an axis of 64, 128 or 256 elements")
        x4 = x.reshape(1, -1, 1, shape[-1])
        if x4.stride(3) != 1:
            x4 = x4.contiguous()
    B, T, H, D = x4.shape
    lib = _lib.load()
    xq = torch.empty((B, T, H, D), dtype=x.dtype, device=x.device)
    stats = torch.empty(16, dtype=x.dtype, device=x.device)        # scale at [0], zero-point at [8]
    ws = _workspace(lib.cq_quantize_pack_workspace(B, T, H, D), x.device)
    with torch.cuda.device(x.device):
        rc = lib.cq_quant_tensor(x4.data_ptr(), dt, B, T, H, D, x4.stride(0), x4.stride(1), x4.stride(2),
                                 bits, float(clip), xq.data_ptr(), stats[0:].data_ptr(), stats[8:].data_ptr(),
                                 ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "cq_quant_tensor")
    return xq.view(shape), stats[0], stats[8]


def encode_indices(idx: torch.Tensor, bits: int) -> torch.Tensor:
    """Pack integer indices (..., D) into uint8 (..., D*bits/8), first index in the high bits."""
    _need_gpu(idx, "idx")
    if idx.dtype not in _DT or idx.dtype == torch.float32:
        raise _lib.CalibQuantError(f"encode: dtype {idx.dtype} not supported")
    idx = idx.contiguous()
    D = idx.shape[-1]
    rows = idx.numel() // D if D else 0
    out = torch.empty((*idx.shape[:-1], D * bits // 8), dtype=torch.uint8, device=idx.device)
    with torch.cuda.device(idx.device):
        rc = _lib.load().cq_encode(idx.data_ptr(), _DT[idx.dtype], rows, D, bits, out.data_ptr(), _stream(idx))
    _lib.check(rc, "cq_encode")
    return out


def lut_vecmat(kind: str, lut: torch.Tensor, a: torch.Tensor, enc: torch.Tensor, bits: int) -> torch.Tensor:
    """kind 'qk': a (M, D), enc (M, T, D*bits/8) -> (M, T) fp16;
    kind 'pv': a (M, T), enc (M, T, D*bits/8) -> (M, D) fp16.
    `lut` may hold fewer than 2**bits entries: a code without an entry contributes 0."""
    if lut.numel() < 1:
        raise _lib.CalibQuantError("lut must hold at least one entry")
    for t, n in ((lut, "lut"), (a, "a"), (enc, "enc")):
        _need_gpu(t, n)
    lut, a, enc = lut.contiguous(), a.contiguous(), enc.contiguous()
    M, T, nb = enc.shape
    D = nb * 8 // bits
    out = torch.empty((M, T if kind == "qk" else D), dtype=torch.float16, device=a.device)
    fn = _lib.load().cq_lut_vecmat_qk if kind == "qk" else _lib.load().cq_lut_vecmat_pv
    with torch.cuda.device(a.device):
        rc = fn(lut.data_ptr(), _DT[lut.dtype], lut.numel(), a.data_ptr(), _DT[a.dtype], enc.data_ptr(), M, T, D, bits,
                out.data_ptr(), _stream(a))
    _lib.check(rc, f"cq_lut_vecmat_{kind}")
    return out


class DecodeCall:
    """A prepared `cq_decode_attn` call: argument block, workspace and output are
    set up once and `run()` only enqueues the launch(es) on torch's current
    stream.  The tensors it was built from are kept alive by the object."""

    def __init__(self, q, codes_k, codes_v, k_scale, k_zero, v_scale, v_zero, k_res, v_res,
                 sprompt_len=0, bits=1, calibrate=True, calib_off_max=-3.0, calib_off_min=0.0,
                 mask=None, out=None, force_splits=0, r_dev=None, v_mode="channel", static_scratch=False):
        _need_gpu(q, "q")
        dt = _storage_dtype(q, "q")
        if q.dim() != 3:
            raise _lib.CalibQuantError("q must be (B, Hq, D)")
        q = q.contiguous()
        B, Hq, D = q.shape
        a = _lib.DecodeArgs()
        T = 0
        Hkv = None
        keep = [q]
        if codes_k is not None and codes_k.shape[2] > 0:
            for t in (codes_k, codes_v, k_scale, k_zero, v_scale, v_zero):
                _need_gpu(t, "packed state")
            codes_k, codes_v = codes_k.contiguous(), codes_v.contiguous()
            k_scale, k_zero = k_scale.contiguous(), k_zero.contiguous()
            v_scale, v_zero = v_scale.contiguous(), v_zero.contiguous()
            for t in (k_scale, k_zero, v_scale, v_zero):
                if t.dtype != q.dtype:
                    raise _lib.CalibQuantError("scale / zero-point dtype must match q")
            Hkv, T = codes_k.shape[1], codes_k.shape[2]
            if v_mode == "token":
                # values in the per-token layout of quantize_pack_token: int32 words, (T, D/32) scale and minimum
                if codes_v.dtype != torch.int32 or codes_v.shape != (B, Hkv, T, D * int(bits) // 32):
                    raise _lib.CalibQuantError("v_mode='token': codes_v must be int32 (B, Hkv, T, D*bits/32)")
                if v_scale.shape != (B, Hkv, T, D // 32) or v_zero.shape != v_scale.shape:
                    raise _lib.CalibQuantError("v_mode='token': v_scale / v_zero must be (B, Hkv, T, D/32)")
            a.codes_k, a.codes_v = codes_k.data_ptr(), codes_v.data_ptr()
            a.k_scale, a.k_zero = k_scale.data_ptr(), k_zero.data_ptr()
            a.v_scale, a.v_zero = v_scale.data_ptr(), v_zero.data_ptr()
            keep += [codes_k, codes_v, k_scale, k_zero, v_scale, v_zero]
        R = 0
        if k_res is not None and k_res.shape[2] > 0:
            _need_gpu(k_res, "k_res")
            if k_res.dtype != q.dtype or v_res.dtype != q.dtype:
                raise _lib.CalibQuantError("residual dtype must match q")
            if k_res.stride(3) != 1 or v_res.stride(3) != 1 or k_res.stride() != v_res.stride():
                k_res, v_res = k_res.contiguous(), v_res.contiguous()
            Hkv, R = k_res.shape[1], k_res.shape[2]
            a.k_res, a.v_res = k_res.data_ptr(), v_res.data_ptr()
            a.res_stride_b, a.res_stride_h, a.res_stride_r = k_res.stride(0), k_res.stride(1), k_res.stride(2)
            keep += [k_res, v_res]
        if Hkv is None:
            raise _lib.CalibQuantError("decode_attn needs packed tokens or residual rows")
        if mask is not None:
            _need_gpu(mask, "mask")
            mask = mask.reshape(B, -1).to(torch.float32).contiguous()
            if mask.shape[1] != T + R:
                raise _lib.CalibQuantError(f"mask length {mask.shape[1]} != T + R = {T + R}")
            a.mask, a.mask_stride_b = mask.data_ptr(), mask.stride(0)
            keep.append(mask)
        if out is None:
            out = torch.empty_like(q)
        elif out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
            raise _lib.CalibQuantError("out must be a contiguous tensor shaped and typed like q")
        a.q, a.out = q.data_ptr(), out.data_ptr()
        a.dtype, a.B, a.Hq, a.Hkv, a.D, a.T, a.R = dt, B, Hq, Hkv, D, T, R
        a.sprompt_len, a.bits = int(sprompt_len), int(bits)
        a.calibrate = int(bool(calibrate))
        a.calib_off_max, a.calib_off_min = float(calib_off_max), float(calib_off_min)
        a.force_splits = int(force_splits)
        if v_mode not in ("channel", "token"):
            raise _lib.CalibQuantError("v_mode must be 'channel' or 'token'")
        a.v_mode = 1 if v_mode == "token" else 0
        if r_dev is not None:
            # residual row count read on the device at run time; k_res / v_res are then the
            # whole window buffers (capacity rows) and R is that capacity
            _need_gpu(r_dev, "r_dev")
            if r_dev.dtype != torch.int32 or r_dev.numel() != 1:
                raise _lib.CalibQuantError("r_dev must be a single int32 on the GPU")
            if mask is not None:
                raise _lib.CalibQuantError("r_dev and mask cannot be combined")
            a.r_dev = r_dev.data_ptr()
            keep.append(r_dev)
        self._lib = _lib.load()
        # static_scratch: `cq_decode_attn_static`, whose scratch is a static device buffer inside the
        # library - no workspace tensor, nothing allocated per call; calls on one GPU must not overlap
        self._entry = self._lib.cq_decode_attn_static if static_scratch else self._lib.cq_decode_attn
        need = 0 if static_scratch else self._lib.cq_decode_attn_workspace(C.byref(a))
        ws = _decode_workspace(need, q.device)
        if ws is not None:
            a.workspace, a.workspace_bytes = ws.data_ptr(), need
            keep.append(ws)
        self.args, self._ref, self._keep, self.out, self.device = a, C.byref(a), keep, out, q.device
        self.workspace, self.workspace_bytes = (None if ws is None else ws[:need]), need

    def plan(self) -> dict:
        """What the launch will be for the prepared arguments (`cq_decode_attn_plan`): threads per
        workgroup, query heads per workgroup, token chunks, launches, LDS bytes, packed-fp16 logits."""
        p = _lib.DecodePlan()
        _lib.check(self._lib.cq_decode_attn_plan(self._ref, C.byref(p)), "cq_decode_attn_plan")
        return {name: int(getattr(p, name)) for name, _ in p._fields_}

    def step(self, q: torch.Tensor, k_res: torch.Tensor, v_res: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """Re-aim the prepared call at this decode step's query, output and (grown) residual
        window and launch.  Only pointers, R and the strides change; packed state, dtype, head
        counts and options stay as prepared.  No validation beyond what the C entry point does."""
        a = self.args
        a.q, a.out = q.data_ptr(), out.data_ptr()
        a.k_res, a.v_res, a.R = k_res.data_ptr(), v_res.data_ptr(), k_res.shape[2]
        a.res_stride_b, a.res_stride_h, a.res_stride_r = k_res.stride(0), k_res.stride(1), k_res.stride(2)
        self._step_keep = (q, k_res, v_res, out)
        self.out = out
        return self.run()

    def run(self) -> torch.Tensor:
        rc = self._entry(self._ref, torch.cuda.current_stream(self.device).cuda_stream)
        if rc:
            _lib.check(rc, "cq_decode_attn")
        return self.out


def decode_attn(q: torch.Tensor, codes_k: Optional[torch.Tensor], codes_v: Optional[torch.Tensor],
                k_scale: Optional[torch.Tensor], k_zero: Optional[torch.Tensor],
                v_scale: Optional[torch.Tensor], v_zero: Optional[torch.Tensor],
                k_res: Optional[torch.Tensor], v_res: Optional[torch.Tensor],
                sprompt_len: int = 0, bits: int = 1, calibrate: bool = True,
                calib_off_max: float = -3.0, calib_off_min: float = 0.0,
                mask: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                force_splits: int = 0, r_dev: Optional[torch.Tensor] = None,
                v_mode: str = "channel") -> torch.Tensor:
    """One decode-attention step over packed image K/V plus the fp residual window.

    q (B, Hq, D); codes_* uint8 (B, Hkv, T, D*bits/8); *_scale, *_zero (B, Hkv, D);
    k_res, v_res (B, Hkv, R, D) (any b/h/r strides); mask optional additive
    (B, S + T + R - S) over the [sys | image | text] order.  `r_dev` (int32 GPU scalar): the
    number of valid rows of k_res / v_res, read on the device when the launch runs.
    `v_mode='token'`: codes_v / v_scale / v_zero as returned by `quantize_pack_token`.
    Returns (B, Hq, D)."""
    call = DecodeCall(q, codes_k, codes_v, k_scale, k_zero, v_scale, v_zero, k_res, v_res,
                      sprompt_len, bits, calibrate, calib_off_max, calib_off_min, mask, out, force_splits, r_dev, v_mode)
    with torch.cuda.device(call.device):
        return call.run()


class RopeAppendCall:
    """A prepared `cq_rope_append` launch over fixed buffers: the token's fused projection output
    `qkv` (B, 1, (Hq + 2 Hkv) * D) or (B, Hkv, Hq/Hkv + 2, D), rotary tables (rows, D), device
    position ids `pos` (B,) or (B, 1) int64, output query `q_out` (B, Hq, D), the window buffers
    (B, Hkv, capacity, D) and the device int64 `row` that names the window row to fill."""

    def __init__(self, qkv, cos, sin, pos, q_out, k_win, v_win, row):
        for t, name in ((qkv, "qkv"), (cos, "cos"), (sin, "sin"), (pos, "pos"), (q_out, "q_out"),
                        (k_win, "k_win"), (v_win, "v_win"), (row, "row")):
            _need_gpu(t, name)
        dt = _storage_dtype(qkv, "qkv")
        B, Hq, D = q_out.shape
        Hkv, cap = k_win.shape[1], k_win.shape[2]
        for t in (cos, sin, q_out, k_win, v_win):
            if t.dtype != qkv.dtype:
                raise _lib.CalibQuantError("rope_append: all floating tensors must share the storage dtype")
        if not (qkv.is_contiguous() and cos.is_contiguous() and sin.is_contiguous() and q_out.is_contiguous()):
            raise _lib.CalibQuantError("rope_append: qkv, cos, sin and q_out must be contiguous")
        if qkv.numel() != B * (Hq + 2 * Hkv) * D or cos.shape != sin.shape or cos.shape[-1] != D:
            raise _lib.CalibQuantError("rope_append: shape mismatch")
        if k_win.stride() != v_win.stride() or k_win.stride(3) != 1 or k_win.shape != v_win.shape:
            raise _lib.CalibQuantError("rope_append: window buffers must share shape and strides")
        if pos.dtype != torch.int64 or row.dtype != torch.int64 or pos.numel() != B or row.numel() != 1:
            raise _lib.CalibQuantError("rope_append: pos (B int64) / row (1 int64) expected")
        self._lib = _lib.load()
        self.device = qkv.device
        self.geometry = (B, Hq, Hkv, D)          # what a prepared call can be re-aimed within
        self.tables = (cos, sin)
        self._fixed = (dt, B, Hq, Hkv, D, cos.data_ptr(), sin.data_ptr(), cos.shape[0])
        self._aim(qkv, pos, q_out, k_win, v_win, row)

    def _aim(self, qkv, pos, q_out, k_win, v_win, row) -> None:
        self._keep = (qkv, pos, q_out, k_win, v_win, row)
        self._args = (qkv.data_ptr(),) + self._fixed + (
            pos.data_ptr(), pos.reshape(-1).stride(0), q_out.data_ptr(), k_win.data_ptr(), v_win.data_ptr(),
            k_win.stride(0), k_win.stride(1), k_win.stride(2), k_win.shape[2], row.data_ptr())

    def step(self, qkv, pos, q_out, k_win, v_win, row) -> None:
        """Re-aim the prepared launch at this step's projection output, position ids, query
        output, window buffers (same geometry, possibly regrown) and row cell, and launch.
        Only pointers, strides and the capacity change; no validation beyond the C entry point's."""
        self._aim(qkv, pos, q_out, k_win, v_win, row)
        self.run()

    def run(self) -> None:
        rc = self._lib.cq_rope_append(*self._args, torch.cuda.current_stream(self.device).cuda_stream)
        if rc:
            _lib.check(rc, "cq_rope_append")
