"""Decode loop of an InternLM2-shaped language model recorded once as a HIP graph.

The reference decodes through `transformers`' eager `generate` loop: every
step re-reads tensor shapes on the host (patch_internvl.py:246-251), grows the
fp window with `torch.cat` (:265-266) and issues some hundreds of small
launches per token, so at batch 64 the step time is set by the host, not by
the GPU.  Here one decode step is expressed over buffers of fixed shape and
address - the window buffers have their final capacity, the number of valid
rows, the append position and the token position live in device scalars, and
the attention kernel reads the row count on the device
(`cq_decode_args.r_dev`) - so the step can be captured with
`torch.cuda.CUDAGraph` and replayed once per token.

Two variants share the step: attention modules patched by
`patch_internvl.patch_model` run the packed-KV kernel; unpatched modules keep
a full-precision cache and use either torch's scaled-dot-product attention over
the whole buffer with a length mask computed on the device, or (`fp_kernel=True`)
this library's attention kernel with every cached token as a row of its
full-precision window.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn.functional as F

from . import _lib, ops
from ._lib import CalibQuantError
from .patch_internvl import CALIB_OFFSET_MAX, CALIB_OFFSET_MIN


class _LayerState:
    """Fixed-address decode state of one attention module."""

    def __init__(self, att, past, capacity: int, r_len: torch.Tensor, quantized: bool, cos, sin, pos, row,
                 fp_kernel: bool = False):
        k_old, v_old = past
        B, Hkv, R0, D = k_old.shape
        self.quantized = quantized
        self.kbuf = torch.empty((B, Hkv, capacity, D), dtype=k_old.dtype, device=k_old.device)
        self.vbuf = torch.empty_like(self.kbuf)
        self.kbuf[:, :, :R0] = k_old
        self.vbuf[:, :, :R0] = v_old
        self.kbuf[:, :, R0:].zero_()
        self.vbuf[:, :, R0:].zero_()
        Hq = att.num_heads
        self.q = torch.empty((B, Hq, D), dtype=k_old.dtype, device=k_old.device)
        self.out = torch.empty_like(self.q)
        # fused projection output of the step's token, and the launch that splits it, applies
        # the rotary embedding and appends the key / value row to the window
        self.qkv = torch.empty((B, (Hq + 2 * Hkv) * D), dtype=k_old.dtype, device=k_old.device)
        self.rope = ops.RopeAppendCall(self.qkv, cos, sin, pos, self.q, self.kbuf, self.vbuf, row)
        self.call = None
        if quantized:
            T = att.image_token_num
            stats = att._cq_stats if T > 0 else (None,) * 4
            self.call = ops.DecodeCall(self.q, att.encoded_features_k if T > 0 else None,
                                       att.encoded_features_v if T > 0 else None, stats[0], stats[1], stats[2],
                                       stats[3], self.kbuf, self.vbuf, sprompt_len=min(att.sprompt_len, R0),
                                       bits=att.bits_k, calibrate=att.normalize, calib_off_max=CALIB_OFFSET_MAX,
                                       calib_off_min=CALIB_OFFSET_MIN, out=self.out, r_dev=r_len,
                                       v_mode=getattr(att, "v_mode", "channel"))
        elif fp_kernel:
            self.call = ops.DecodeCall(self.q, None, None, None, None, None, None, self.kbuf, self.vbuf,
                                       sprompt_len=0, bits=1, out=self.out, r_dev=r_len)


class StaticDecoder:
    """Greedy decoding after a prefill, one recorded step per token.

    lm: an `InternLM2ForCausalLM`-shaped module; past: the per-layer (K, V)
    pairs its prefill returned (fp window rows for patched attention modules,
    the whole cache otherwise); prompt_len: tokens in the prompt (the position
    of the first generated token); logits: the prefill's last-position logits."""

    def __init__(self, lm, past, prompt_len: int, max_new_tokens: int, fp_kernel: bool = False):
        layers = lm.model.layers
        att0 = layers[0].attention
        self.lm = lm
        self.quantized = hasattr(att0, "_cq_stats")
        k0 = past[0][0]
        self.B = k0.shape[0]
        dev = k0.device
        self.device = dev
        R0 = k0.shape[2]
        self.capacity = R0 + max_new_tokens
        # device scalars: rows in the window after this step's append, the append position,
        # and the position id of the token being processed
        self.r_len = torch.full((1,), R0 + 1, dtype=torch.int32, device=dev)
        self.r_idx = torch.full((1,), R0, dtype=torch.long, device=dev)
        self.pos = torch.full((self.B, 1), prompt_len, dtype=torch.long, device=dev)
        self.tok = torch.zeros((self.B,), dtype=torch.long, device=dev)
        cos, sin = att0.rotary_emb(k0, seq_len=prompt_len + max_new_tokens + 1)
        self.cos, self.sin = cos.contiguous(), sin.contiguous()
        self.state: List[_LayerState] = [
            _LayerState(l.attention, past[i], self.capacity, self.r_len, self.quantized, self.cos, self.sin,
                        self.pos, self.r_idx, fp_kernel) for i, l in enumerate(layers)]
        self.col = torch.arange(self.capacity, device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.steps_left = max_new_tokens

    # -- one decode step over the fixed buffers: consumes self.tok, leaves the next token there
    def _step(self):
        lm = self.lm
        x = lm.get_input_embeddings()(self.tok)[:, None]                      # (B, 1, hidden)
        for layer, st in zip(lm.model.layers, self.state):
            att = layer.attention
            B = self.B
            h = F.rms_norm(x, (x.shape[-1],), layer.attention_norm.weight, layer.attention_norm.eps)
            torch.matmul(h.view(B, -1), att.wqkv.weight.t(), out=st.qkv)
            st.rope.run()            # st.q <- rotated query heads; window row r_idx <- rotated key, value
            if st.call is not None:
                st.call.run()
                o = st.out
            else:
                keep = (self.col < self.r_len.to(torch.long))[None, None, None, :]
                o = F.scaled_dot_product_attention(st.q[:, :, None, :], st.kbuf, st.vbuf, attn_mask=keep,
                                                   enable_gqa=True)
            x = x + att.wo(o.reshape(B, 1, att.hidden_size))
            h = F.rms_norm(x, (x.shape[-1],), layer.ffn_norm.weight, layer.ffn_norm.eps)
            x = x + layer.feed_forward(h)
        x = F.rms_norm(x, (x.shape[-1],), lm.model.norm.weight, lm.model.norm.eps)
        logits = lm.output(x[:, -1, :])
        self.tok.copy_(logits.argmax(-1))
        self.r_len.add_(1)
        self.r_idx.add_(1)
        self.pos.add_(1)

    @torch.no_grad()
    def step(self) -> torch.Tensor:
        """Process the token in `self.tok`; afterwards `self.tok` holds the next one."""
        if self.steps_left <= 0:
            raise CalibQuantError("StaticDecoder: window capacity exhausted")
        self.steps_left -= 1
        if self.graph is not None:
            self.graph.replay()
        else:
            self._step()
        return self.tok

    @torch.no_grad()
    def capture(self, warmup: int = 2):
        """Run `warmup` steps eagerly (they are real steps: tokens are consumed and produced),
        then record the step.  Recording executes nothing."""
        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize(self.device)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._step()
        self.graph = g

    @torch.no_grad()
    def generate(self, first_token: torch.Tensor, max_new_tokens: int, use_graph: bool = True, on_step=None):
        """Greedy continuation: `first_token` (B,) is the token chosen from the prefill logits;
        returns (B, max_new_tokens) including it."""
        out = [first_token.clone()]
        self.tok.copy_(first_token)
        if on_step is not None:
            on_step(0)
        for i in range(1, max_new_tokens):
            # the first step runs eagerly (kernels set themselves up on their first launch);
            # the step is recorded before the second and replayed from there on
            if use_graph and self.graph is None and i == 2:
                self.capture(warmup=0)
            out.append(self.step().clone())
            if on_step is not None:
                on_step(i)
        tokens = torch.stack(out, dim=1)
        # A replayed launch does not pass through the library's own check of the single-launch chunked step's
        # bounded wait (long contexts only): ask once the replays are done.
        if self.graph is not None:
            torch.cuda.synchronize()
            if _lib.load().cq_decode_attn_gave_up():
                raise CalibQuantError("a recorded decode step did not complete (single-launch chunked step gave "
                                           "up waiting); rerun with cq_decode_attn_single_launch(0)")
        return tokens
