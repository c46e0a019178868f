"""The reference's `patch_internvl.py` surface for the CalibQuant method, routed to
the MI355X kernels: `patch_model`, `ATTN_FORWARD_FUNCTIONS`, `custom_generate`,
`forward_internlm2_calibquant`, the RoPE / GQA helpers and the module constants.

What changes behind the same call contract (patch_internvl.py:141-150, 484):
  * prefill: the image slice of K and V is quantised and packed by one HIP entry
    point per tensor, reading the strided views of the fused wqkv output in place
    (reference: quant + unique/compare/argmax + encode, patch_internvl.py:288-341);
  * decode: one fused HIP call replaces repeat_kv copies, two Triton LUT vec-mats,
    the calibration, softmax and residual matmuls (patch_internvl.py:344-436);
  * the fp residual window is appended in place instead of `torch.cat` per step
    (patch_internvl.py:264-266); callers still get and pass plain (K, V) tensors.
The QJL method of the reference (`quant_method='qjl'`) is a different algorithm
and is not provided.
"""
from __future__ import annotations

import ctypes as C
import os
import warnings
from typing import Optional, Tuple

import torch

from . import _lib, ops
from ._lib import CalibQuantError
from .kvbuffer import GrowingKV

# global hyper-parameters, as in patch_internvl.py:19-31
BITS_KV = 1

if BITS_KV == 1:
    SCALE_V = 0.3
    SCALE_K = 0.5
else:
    SCALE_V = 1
    SCALE_K = 1

LOW_BITS = True
SPROMPT_LEN = 41
CHUNK_SIZE = 1024
CALIB_OFFSET_MAX = -3.0    # literals at patch_internvl.py:379-380
CALIB_OFFSET_MIN = 0.0


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Hkv, S, D) -> (B, Hkv * n_rep, S, D), each kv head repeated consecutively (patch_internvl.py:97-107)."""
    b, h, s, d = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    return hidden_states[:, :, None, :, :].expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


def rotate_half(x):
    """(-x2, x1) for x = (x1, x2) split along the last axis (patch_internvl.py:110-115; this version
    leaves its argument untouched)."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def _rope_one(x, cos, sin):
    # rnd(x * cos), then the fp32 sum with the exact fp32 product rotate_half(x) * sin, rounded once
    return torch.add((x * cos).float(), rotate_half(x).float() * sin.float()).to(x.dtype)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids, unsqueeze_dim=1):
    """Rotary position embedding of q and k with the rounding of the ops the reference runs
    (patch_internvl.py:125-128, 131-134): `copy_().mul_(cos)` rounds `x * cos` to the storage
    dtype, then `addcmul_(rotate_half(x), sin)` adds the product in fp32 and rounds the sum once.
    (The two-rounding form `(x * cos) + (rotate_half(x) * sin)` is the commented-out line :123 and
    differs from this by one unit in the last place in about a quarter of the elements.)

    The sum is written out as separate fp32 ops instead of calling `addcmul`: the device kernel the
    reference ran rounds the fp32 sum to fp32 and then to the storage dtype, and so do these ops
    and `cq_rope_append`; torch-ROCm's own `addcmul` on strided fp16 operands is compiled to a
    mixed-precision multiply-add that rounds the exact sum once, which differs in about 7 of a
    million fp16 elements (the fp32 sum lands exactly between two fp16 values).
    The inputs are left untouched; the reference's `rotate_half` negates the upper half of its
    argument in place."""
    cos = cos[position_ids].unsqueeze(unsqueeze_dim)
    sin = sin[position_ids].unsqueeze(unsqueeze_dim)
    return _rope_one(q, cos, sin), _rope_one(k, cos, sin)


@torch.no_grad()
def custom_generate(self, pixel_values=None, input_ids=None, attention_mask=None, visual_features=None,
                    generation_config=None, output_hidden_states=None, **generate_kwargs):
    """`InternVLChatModel.generate` replacement (patch_internvl.py:34-93): vision features in chunks
    of 10 tiles, splice them over the image-context tokens, publish the per-sample image token count,
    run the language model's generate."""
    assert self.img_context_token_id is not None
    lm = self.language_model
    if pixel_values is not None:
        if visual_features is not None:
            vit_embeds = visual_features
        else:
            chunks = [self.extract_feature(pixel_values[i:i + 10]) for i in range(0, pixel_values.size(0), 10)]
            vit_embeds = torch.cat(chunks, dim=0)
        input_embeds = lm.get_input_embeddings()(input_ids)
        B, N, C = input_embeds.shape
        input_embeds = input_embeds.reshape(B * N, C)
        selected = input_ids.reshape(B * N) == self.img_context_token_id
        assert selected.sum() != 0
        input_embeds[selected] = vit_embeds.reshape(-1, C).to(input_embeds.device, input_embeds.dtype)
        image_token_num = int(vit_embeds.shape[0] * vit_embeds.shape[1] / B)
        os.environ["IMAGE_TOKEN_NUM"] = str(image_token_num)
        for layer in lm.model.layers:      # the explicit per-module channel; wins over the env var
            layer.attention.cq_image_token_num = image_token_num
        input_embeds = input_embeds.reshape(B, N, C)
    else:
        input_embeds = lm.get_input_embeddings()(input_ids)
    return lm.generate(inputs_embeds=input_embeds, attention_mask=attention_mask,
                       generation_config=generation_config, output_hidden_states=output_hidden_states,
                       use_cache=True, **generate_kwargs)


def _image_token_num(self) -> int:
    """The image token count of this forward: the explicit override `cq_image_token_num` on the
    module if a caller set one (`custom_generate` does), else the `IMAGE_TOKEN_NUM` environment
    variable, re-read on every prefill and on every decode step that does not take the prepared
    steady-state step (the reference re-reads it per forward, patch_internvl.py:189,251) - a caller
    that updates the variable between prompts gets the new count with the next prefill."""
    n = getattr(self, "cq_image_token_num", None)
    if n is None:
        env = os.environ.get("IMAGE_TOKEN_NUM")
        if env is None:
            raise CalibQuantError("image token count unknown: set attention.cq_image_token_num or IMAGE_TOKEN_NUM")
        n = int(env)
    return int(n)


def forward_internlm2_calibquant(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                                 position_ids: Optional[torch.LongTensor] = None,
                                 past_key_value: Optional[Tuple[torch.Tensor]] = None,
                                 output_attentions: bool = False, use_cache: bool = False, **kwargs):
    """Attention forward with a 1-/2-bit image KV cache (patch_internvl.py:141-484).

    Returns `(attn_output, None, past_key_value)`; `past_key_value` is the fp pair
    (K, V) of shape (B, Hkv, R, D) holding the system prompt rows [0, S), the text rows and every
    generated token; the image rows live packed on the module
    (`encoded_features_k/v`, `scale_key/value`, `zero_point_key/value`, `unique_values_k/v`)."""
    # steady-state decode: the step object the first decode step prepared runs the whole step (rotary
    # embedding + window append launch, attention launch) in one call into the host shim; it declines
    # (returns None) when this is not the next token of the window it owns.  The hyper-parameters
    # (`cq_sprompt_len`, `cq_bits`, `cq_v_mode`, the image token count) are the ones of the first decode
    # step after a prefill: on this path they are not read again until the next prefill or a decline.
    fast = self.__dict__.get("_cq_step")
    if (fast is not None and attention_mask is None and past_key_value is not None and position_ids is not None
            and not kwargs and hidden_states.shape[1] == 1):
        got = fast[0].step(self.wqkv(hidden_states), position_ids, past_key_value[0])
        if got is not None:
            return self.wo(got[0]), None, ((got[1], got[2]) if use_cache else None)
        del self.__dict__["_cq_step"]
    # hyper-parameters published on the module, as patch_internvl.py:175-191 does
    self.sprompt_len = getattr(self, "cq_sprompt_len", SPROMPT_LEN)
    self.bits_k = self.bits_v = getattr(self, "cq_bits", BITS_KV)
    one_bit = self.bits_k == 1
    self.scale_k = getattr(self, "cq_scale_k", 0.5 if one_bit else 1)
    self.scale_v = getattr(self, "cq_scale_v", 0.3 if one_bit else 1)
    # values: per channel (CalibQuant) or per token in groups of 32 channels (the layout of
    # qjl/new_pack.py:53-82 that the reference's per-token branch reads, patch_internvl.py:560-577)
    self.v_mode = getattr(self, "cq_v_mode", "channel")
    self.per_channel_k = True
    self.per_channel_v = self.v_mode == "channel"
    self.image_token_num = _image_token_num(self)
    self.normalize = self.bits_k <= 2
    if "padding_mask" in kwargs:
        warnings.warn("Passing `padding_mask` is deprecated; use `attention_mask` instead.")
        attention_mask = kwargs.pop("padding_mask")

    bsz, q_len, _ = hidden_states.size()
    G, D, Hq = self.num_key_value_groups, self.head_dim, self.num_heads
    Hkv = Hq // G
    S, T = self.sprompt_len, self.image_token_num

    # (h gs d) de-interleave of the fused projection: views only (patch_internvl.py:214-234)
    qkv = self.wqkv(hidden_states).view(bsz, q_len, Hkv, 2 + G, D)
    if (q_len == 1 and past_key_value is not None and position_ids is not None and position_ids.is_cuda
            and position_ids.dtype == torch.int64 and position_ids.numel() == bsz and qkv.is_contiguous()
            and qkv.dtype in (torch.bfloat16, torch.float16)):
        return _decode_step_fused(self, qkv, position_ids, past_key_value, attention_mask, use_cache)
    value_states = qkv[..., -1, :].transpose(1, 2)                                 # (B, Hkv, q, D)
    kv_seq_len = q_len
    if past_key_value is not None:
        kv_seq_len += past_key_value[0].shape[-2] + T                               # patch_internvl.py:246-251
    cos, sin = self.rotary_emb(value_states, seq_len=kv_seq_len)
    # Prefill on the GPU: the rotary embedding runs in HIP kernels with the rounding of the reference's op
    # chain (`cq_rope_rows` for queries and keys), then the image block of the rotated keys is quantised.
    # The reference rotates the whole tensors with a chain of torch ops first (patch_internvl.py:258-260) and
    # quantises afterwards (:295-297).  With `cq_fused_rope` set on the module the image block of the keys is
    # rotated inside the quantise-and-pack pass instead (`cq_rope_quantize_pack`: un-rotated keys read once,
    # rotated rows written once, quantised from the registers) - same bits, one launch fewer, but slower at the
    # benchmark shape (348 against 309 us: a slice then reads two 32-byte pieces per row instead of one of 64,
    # which HBM serves as 64-byte fetches), so it is not the default.
    hip_rope = (q_len > 1 and qkv.is_cuda and qkv.dtype in (torch.bfloat16, torch.float16) and D == 128
                and position_ids is not None and position_ids.is_cuda and position_ids.dtype == torch.int64
                and tuple(position_ids.shape) == (bsz, q_len))
    k_rot = None
    if hip_rope:
        cos, sin = cos.contiguous(), sin.contiguous()
        q_rot = torch.empty((bsz, q_len, Hkv, G, D), dtype=qkv.dtype, device=qkv.device)
        ops.rope_rows_grouped(qkv[..., :G, :], cos, sin, position_ids, out=q_rot)   # all query heads: one launch
        query_states = q_rot.view(bsz, q_len, Hq, D).transpose(1, 2)               # (B, Hq, q, D)
        k_raw = qkv[..., -2, :]                                                    # (B, q, Hkv, D), un-rotated
        k_rot = ops.empty_token_rows(bsz, q_len, Hkv, D, qkv.dtype, qkv.device)    # (padded rows where that helps the quantiser)
        key_states = k_rot.transpose(1, 2)                                         # filled in the prefill branch
    else:
        query_states = qkv[..., :G, :].reshape(bsz, q_len, Hq, D).transpose(1, 2)  # (B, Hq, q, D)
        key_states = qkv[..., -2, :].transpose(1, 2)                               # (B, Hkv, q, D)
        query_states, key_states = apply_rotary_pos_emb(query_states, key_states, cos, sin, position_ids)

    if not hasattr(self, "_cq_window"):
        self._cq_window = GrowingKV()

    if q_len > 1:
        # ---- prefill (patch_internvl.py:268-341, 461-476) -------------------------------------
        if past_key_value is not None:
            raise CalibQuantError("prefill with an existing cache is not supported (the reference quantises "
                                  "the image block of a fresh prompt)")
        if S + T > q_len:
            raise CalibQuantError(f"prompt of {q_len} tokens is shorter than sprompt_len + image tokens = {S + T}")
        self._cq_call = None
        self.__dict__.pop("_cq_step", None)
        fused_rope = hip_rope and 0 < T <= ops.ROPE_FUSED_MAX_T and bool(getattr(self, "cq_fused_rope", False))
        if hip_rope:
            if fused_rope:      # image block: rotated inside the quantiser; the rows around it on their own
                ck, ks, kz = ops.rope_quantize_pack(k_raw[:, S:S + T], cos, sin, position_ids[:, S:S + T],
                                                    k_rot[:, S:S + T], self.bits_k, self.scale_k)
                if S > 0:
                    ops.rope_rows(k_raw[:, :S], cos, sin, position_ids[:, :S], out=k_rot[:, :S])
                if S + T < q_len:
                    ops.rope_rows(k_raw[:, S + T:], cos, sin, position_ids[:, S + T:], out=k_rot[:, S + T:])
            else:               # no image block, or one beyond the one-pass quantiser: rotate everything first
                ops.rope_rows(k_raw, cos, sin, position_ids, out=k_rot)
        if T > 0:
            k_img = key_states[:, :, S:S + T, :].transpose(1, 2)      # (B, T, Hkv, D) strided views
            v_img = value_states[:, :, S:S + T, :].transpose(1, 2)
            if not fused_rope:
                ck, ks, kz = ops.quantize_pack(k_img, self.bits_k, self.scale_k)
            if self.v_mode == "token":
                cv, vs, vz = ops.quantize_pack_token(v_img, self.bits_v)      # words, scale, minimum per (token, group)
            else:
                cv, vs, vz = ops.quantize_pack(v_img, self.bits_v, self.scale_v)
            self.encoded_features_k, self.encoded_features_v = ck, cv
            self._cq_stats = (ks, kz, vs, vz)                          # compact (B, Hkv, D)
            # reference-shaped views of the statistics: (B, Hq, 1, D) after repeat_kv (patch_internvl.py:300-309)
            self.scale_key = repeat_kv(ks.unsqueeze(2), G)
            self.zero_point_key = repeat_kv(kz.unsqueeze(2), G)
            if self.v_mode == "token":
                self.scale_value, self.zero_point_value = repeat_kv(vs, G), repeat_kv(vz, G)   # (B, Hq, T, D/32)
            else:
                self.scale_value = repeat_kv(vs.unsqueeze(2), G)
                self.zero_point_value = repeat_kv(vz.unsqueeze(2), G)
            lut = torch.arange(2 ** self.bits_k, device=hidden_states.device, dtype=hidden_states.dtype)
            self.unique_values_k, self.unique_values_v = lut, lut.half()
        else:
            self.encoded_features_k = self.encoded_features_v = None
            self._cq_stats = None
        if use_cache:
            k_st = torch.cat([key_states[:, :, :S], key_states[:, :, S + T:]], dim=2)
            v_st = torch.cat([value_states[:, :, :S], value_states[:, :, S + T:]], dim=2)
            self._cq_window = GrowingKV()
            past_key_value = self._cq_window.append(None, k_st, v_st)
        else:
            past_key_value = None
        # full-precision causal attention over the whole prompt, in query chunks
        # The reference hands `attention_mask` to `_flash_attention_forward` as it is
        # (patch_internvl.py:465-467), which takes a (B, kv) key-padding mask.  Any other layout
        # (the 4-D additive masks of the eager / SDPA attention classes) cannot be honoured by that
        # call: refuse it instead of attending to the padding.
        if attention_mask is not None and attention_mask.dim() != 2:
            raise CalibQuantError(f"prefill: attention_mask must be a (B, kv) key-padding mask or None, got a "
                                  f"{attention_mask.dim()}-D tensor of shape {tuple(attention_mask.shape)}")
        q_t, k_t, v_t = query_states.transpose(1, 2), key_states.transpose(1, 2), value_states.transpose(1, 2)
        outs = []
        for i in range(0, q_len, CHUNK_SIZE):
            outs.append(self._flash_attention_forward(q_t[:, i:i + CHUNK_SIZE], k_t[:, :i + CHUNK_SIZE],
                                                      v_t[:, :i + CHUNK_SIZE], attention_mask,
                                                      q_t[:, :i + CHUNK_SIZE].shape[1]))
        attn_output = torch.cat(outs, dim=1).reshape(bsz, q_len, self.hidden_size)
        return self.wo(attn_output), None, past_key_value

    # ---- decode (patch_internvl.py:344-457) -------------------------------------------------------
    k_res, v_res = self._cq_window.append(past_key_value, key_states, value_states)
    past_key_value = (k_res, v_res) if use_cache else None
    R = k_res.shape[2]
    if kv_seq_len != R + T:
        raise ValueError(f"Attention weights should be of size {(bsz, Hq, q_len, kv_seq_len)}, but is "
                         f"{(bsz, Hq, q_len, R + T)}")
    mask = None
    if attention_mask is not None:
        if attention_mask.size() != (bsz, 1, q_len, kv_seq_len):
            raise ValueError(f"Attention mask should be of size {(bsz, 1, q_len, kv_seq_len)}, "
                             f"but is {attention_mask.size()}")
        mask = attention_mask[:, 0, 0, :]
    out = _attend(self, query_states[:, :, 0, :], k_res, v_res, mask)
    attn_output = self.wo(out.reshape(bsz, 1, self.hidden_size))
    return attn_output, None, past_key_value


def _attend(self, q1, k_res, v_res, mask):
    """The fused decode attention of one step over the module's packed state and the full-precision
    window (k_res, v_res): q1 (B, Hq, D) -> (B, Hq, D).  In the steady state (no mask, same batch and
    dtype) the prepared call of the previous step is re-aimed at this step's tensors (a chunked call keeps
    its plan and its workspace: both depend on the packed tokens only, once the window has a row)."""
    bsz = q1.shape[0]
    S, T = self.sprompt_len, self.image_token_num
    R = k_res.shape[2]
    call = getattr(self, "_cq_call", None)
    if (mask is None and call is not None and call.args.B == bsz and call.args.R > 0
            and q1.is_contiguous() and call.args.dtype == (0 if q1.dtype == torch.bfloat16 else 1)):
        return call.step(q1, k_res, v_res, torch.empty_like(q1))
    stats = self._cq_stats if T > 0 else (None,) * 4
    call = ops.DecodeCall(q1, self.encoded_features_k if T > 0 else None,
                          self.encoded_features_v if T > 0 else None, stats[0], stats[1], stats[2], stats[3],
                          k_res, v_res, sprompt_len=min(S, R), bits=self.bits_k, calibrate=self.normalize,
                          calib_off_max=CALIB_OFFSET_MAX, calib_off_min=CALIB_OFFSET_MIN, mask=mask,
                          v_mode=self.v_mode)
    with torch.cuda.device(call.device):
        out = call.run()
    self._cq_call = call if mask is None else None
    return out


def _decode_step_fused(self, qkv, position_ids, past_key_value, attention_mask, use_cache):
    """One decode step with the split of the fused projection, the rotary embedding of q and k and
    the append of the new key / value row in one launch (`cq_rope_append`, bit-identical to the
    torch ops that run at patch_internvl.py:125-134, 219-266), then the fused attention launch."""
    bsz = qkv.shape[0]
    G, D, Hq = self.num_key_value_groups, self.head_dim, self.num_heads
    Hkv = Hq // G
    T = self.image_token_num
    R0 = past_key_value[0].shape[2]
    R = R0 + 1
    kv_seq_len = R + T
    # rotary tables in the storage dtype, kept on the module with room to spare
    tabs = getattr(self, "_cq_rope_tables", None)
    if tabs is None or tabs[0].shape[0] < kv_seq_len or tabs[0].dtype != qkv.dtype or tabs[0].device != qkv.device:
        cos, sin = self.rotary_emb(qkv, seq_len=kv_seq_len + 512)
        tabs = self._cq_rope_tables = (cos.contiguous(), sin.contiguous())
    if not hasattr(self, "_cq_window"):
        self._cq_window = GrowingKV()
    win = self._cq_window
    k_buf, v_buf = win.reserve(past_key_value, R, qkv, (bsz, Hkv), D)
    # a cell that holds the row index on the device: cell i of a ramp holds i
    rows = getattr(self, "_cq_row_ramp", None)
    if rows is None or rows.numel() <= R0 or rows.device != qkv.device:
        rows = self._cq_row_ramp = torch.arange(max(4096, 2 * R), dtype=torch.int64, device=qkv.device)
    row = rows[R0:R0 + 1]
    q1 = torch.empty((bsz, Hq, D), dtype=qkv.dtype, device=qkv.device)
    rope = getattr(self, "_cq_rope_call", None)
    with torch.cuda.device(qkv.device):
        if rope is None or rope.geometry != (bsz, Hq, Hkv, D) or rope.tables[0] is not tabs[0]:
            rope = self._cq_rope_call = ops.RopeAppendCall(qkv, tabs[0], tabs[1], position_ids, q1, k_buf, v_buf, row)
            rope.run()
        else:
            rope.step(qkv, position_ids, q1, k_buf, v_buf, row)
    k_res, v_res = win.extended(R)
    past_key_value = (k_res, v_res) if use_cache else None
    mask = None
    if attention_mask is not None:
        if attention_mask.size() != (bsz, 1, 1, kv_seq_len):
            raise ValueError(f"Attention mask should be of size {(bsz, 1, 1, kv_seq_len)}, "
                             f"but is {attention_mask.size()}")
        mask = attention_mask[:, 0, 0, :]
    out = _attend(self, q1, k_res, v_res, mask)
    call = getattr(self, "_cq_call", None)
    if (mask is None and use_cache and call is not None and call.args.B == bsz
            and not getattr(self, "cq_no_step_shim", False)):
        # from the next token on the host shim runs this whole function in one call; it takes over the
        # window buffers (this step's past_key_value are views of them) and keeps `call`'s tensors alive
        shim = _lib.load_step_shim()
        self.__dict__["_cq_step"] = (shim.LayerStep(C.addressof(call.args), C.sizeof(call.args), tabs[0], tabs[1],
                                                    win.k, win.v, win.len, rows), call)
    return self.wo(out.reshape(bsz, 1, self.hidden_size)), None, past_key_value


def _no_qjl(*args, **kwargs):
    raise CalibQuantError("quant_method='qjl' (the QJL sketch method) is not part of this build; use 'calibquant'")


ATTN_FORWARD_FUNCTIONS = {
    "calibquant": forward_internlm2_calibquant,
    "qjl": _no_qjl,
}


def patch_model(model, quant_method="calibquant", **kwargs):
    """Route a chat model's generate and its attention forward to the quantised-KV path
    (patch_internvl.py:645-660).  Works on any object exposing
    `language_model.model.layers[i].attention` and a class-level `generate`.
    Optional keyword overrides: bits, scale_k, scale_v, sprompt_len, v_mode ("channel" | "token")."""
    if quant_method not in ATTN_FORWARD_FUNCTIONS:
        raise KeyError(quant_method)
    if quant_method == "qjl":
        _no_qjl()
    print("Patching InternVLChatModel.generate function ...")
    model.__class__.generate = custom_generate
    print(f"Patching InternLM2FlashAttention2.forward function ... {quant_method}")
    layers = model.language_model.model.layers
    layers[0].attention.__class__.forward = ATTN_FORWARD_FUNCTIONS[quant_method]
    for name in ("bits", "scale_k", "scale_v", "sprompt_len", "v_mode"):
        if name in kwargs:
            for layer in layers:
                setattr(layer.attention, "cq_" + name, kwargs[name])
    return model
