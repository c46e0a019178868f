"""The patched attention forward / model routing on the GPU: cache bookkeeping,
prefill quantisation of the strided wqkv views, decode through the fused kernel."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import to_np

pytestmark = pytest.mark.gpu


def _tiny_model(layers=2, seed=0, vit=None):
    from calibquant_amd.internlm2 import InternLM2Config, InternVLChatStandIn
    torch.manual_seed(seed)
    m = InternVLChatStandIn(InternLM2Config.tiny(layers), vit=vit).cuda().to(torch.bfloat16).eval()
    return m


def test_patched_forward_decode_matches_oracle_on_one_layer():
    """Prefill S + T + text tokens, then one decode step: the layer's attention output equals
    wo(oracle attention) built from the module's own packed state and fp window."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    torch.manual_seed(1)
    cfg = InternLM2Config.tiny()
    att = InternLM2Attention(cfg).cuda().to(torch.bfloat16)
    att.cq_sprompt_len, att.cq_image_token_num = 5, 200
    B, S, T, TXT = 2, 5, 200, 11
    N = S + T + TXT
    x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    pos = torch.arange(N, device="cuda")[None].expand(B, N)
    with torch.no_grad():
        out_p, _, past = pi.forward_internlm2_calibquant(att, x, None, pos, None, False, True)
        assert out_p.shape == (B, N, cfg.hidden_size)
        assert past[0].shape == (B, cfg.num_key_value_heads, S + TXT, 128)
        assert att.encoded_features_k.shape == (B, cfg.num_key_value_heads, T, 16)
        assert att.scale_key.shape == (B, cfg.num_attention_heads, 1, 128)
        # the packed state equals the oracle's quantisation of the post-RoPE image keys / raw values
        q, k, v = att.split_qkv(x)
        cos, sin = att.rotary_emb(v, seq_len=N)
        qr, kr = pi.apply_rotary_pos_emb(q.transpose(1, 2), k.transpose(1, 2), cos, sin, pos)
        ck, sk, zk = O.quantize_pack(to_np(kr[:, :, S:S + T].transpose(1, 2)), 1, 0.5, "bf16")
        cv, sv, zv = O.quantize_pack(to_np(v[:, S:S + T]), 1, 0.3, "bf16")
        assert np.array_equal(att.encoded_features_k.cpu().numpy(), ck)
        assert np.array_equal(att.encoded_features_v.cpu().numpy(), cv)
        # one decode step with an additive mask that hides two positions
        xd = torch.randn(B, 1, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
        posd = torch.full((B, 1), N, device="cuda", dtype=torch.long)
        mask = torch.zeros(B, 1, 1, N + 1, device="cuda", dtype=torch.bfloat16)
        mask[0, 0, 0, 2] = mask[1, 0, 0, S + 7] = torch.finfo(torch.bfloat16).min
        out_d, _, past2 = pi.forward_internlm2_calibquant(att, xd, mask, posd, past, False, True)
        assert past2[0].shape[2] == S + TXT + 1 and past2[0].data_ptr() == past[0].data_ptr()
        qd, kd, vd = att.split_qkv(xd)
        cos, sin = att.rotary_emb(vd, seq_len=N + 1)
        qd, kd = pi.apply_rotary_pos_emb(qd.transpose(1, 2), kd.transpose(1, 2), cos, sin, posd)
        want = O.decode_attention(to_np(qd[:, :, 0]), ck, cv, sk, zk, sv, zv, to_np(past2[0]), to_np(past2[1]),
                                  S, 1, mask=to_np(mask[:, 0, 0]))
        want = torch.from_numpy(want).cuda().to(torch.bfloat16).reshape(B, 1, -1)
        ref = att.wo(want)
        err = (out_d.float() - ref.float()).abs()
        assert err.max().item() < 2e-2 and err.mean().item() < 2e-3


def test_masked_steady_state_decode_of_a_left_padded_batch():
    """A batch whose second sample is left-padded by four positions: prefill with the (B, kv) padding mask,
    then eight decode steps that each pass the additive (B, 1, 1, kv) mask the reference adds per step
    (patch_internvl.py:404-410).  Every step's attention output equals wo(oracle attention with that mask) on
    the module's own packed state and window; the step times with and without the mask are printed (a masked
    step cannot take the prepared-call fast path: its call object is rebuilt every step)."""
    import time
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    torch.manual_seed(7)
    cfg = InternLM2Config.tiny()
    B, S, T, TXT, PAD, STEPS = 2, 5, 200, 11, 4, 8
    N = S + T + TXT
    lo = torch.finfo(torch.bfloat16).min

    def run(masked):
        torch.manual_seed(8)
        att = InternLM2Attention(cfg).cuda().to(torch.bfloat16)
        att.cq_sprompt_len, att.cq_image_token_num = S, T
        x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
        pos = torch.arange(N, device="cuda")[None].expand(B, N).clone()
        pad = None
        if masked:
            pad = torch.ones(B, N, device="cuda", dtype=torch.bool)
            pad[1, :PAD] = False
            pos[1] = (pos[1] - PAD).clamp_(min=0)
        outs, times = [], []
        with torch.no_grad():
            _, _, past = pi.forward_internlm2_calibquant(att, x, pad, pos, None, False, True)
            ck, cv = att.encoded_features_k.cpu().numpy(), att.encoded_features_v.cpu().numpy()
            sk, zk, sv, zv = (to_np(t) for t in att._cq_stats)
            for i in range(STEPS):
                xd = torch.randn(B, 1, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
                posd = pos[:, -1:] + 1 + i
                mask = None
                if masked:
                    mask = torch.zeros(B, 1, 1, N + 1 + i, device="cuda", dtype=torch.bfloat16)
                    mask[1, 0, 0, :PAD] = lo
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                out_d, _, past = pi.forward_internlm2_calibquant(att, xd, mask, posd, past, False, True)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                qd, kd, vd = att.split_qkv(xd)
                cos, sin = att.rotary_emb(vd, seq_len=N + 1 + i)
                qd, _ = pi.apply_rotary_pos_emb(qd.transpose(1, 2), kd.transpose(1, 2), cos, sin, posd)
                m = None if mask is None else to_np(mask[:, 0, 0])
                want = O.decode_attention(to_np(qd[:, :, 0]), ck, cv, sk, zk, sv, zv, to_np(past[0]), to_np(past[1]), S, 1, mask=m)
                ref = att.wo(torch.from_numpy(want).cuda().to(torch.bfloat16).reshape(B, 1, -1))
                err = (out_d.float() - ref.float()).abs()
                assert err.max().item() < 2e-2 and err.mean().item() < 2e-3, (masked, i, err.max().item())
                outs.append(out_d)
        return outs, sorted(times)[len(times) // 2]

    _, t_mask = run(True)
    _, t_plain = run(False)
    print(f"\nmasked decode step {t_mask * 1e6:.0f} us, unmasked {t_plain * 1e6:.0f} us per layer (host-inclusive, tiny layer)")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_decode_step_equals_the_unfused_op_chain(dtype):
    """Several decode steps through the one-launch split + rotary + append path - once driven by the host
    shim's `LayerStep` (the default), once by the Python call objects - and through the chain of torch ops
    (forced by int32 position ids): same outputs and same window, bit for bit."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    cfg = InternLM2Config.tiny()
    B, S, T, TXT = 3, 4, 130, 9
    N = S + T + TXT
    outs, wins = [], []
    for fused, shim in ((True, True), (True, False), (False, False)):
        torch.manual_seed(7)
        att = InternLM2Attention(cfg).cuda().to(dtype)
        att.cq_sprompt_len, att.cq_image_token_num = S, T
        att.cq_no_step_shim = not shim
        x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=dtype)
        pos = torch.arange(N, device="cuda")[None].expand(B, N)
        with torch.no_grad():
            _, _, past = pi.forward_internlm2_calibquant(att, x, None, pos, None, False, True)
            step_out = []
            for i in range(300):   # beyond the first window capacity: the buffers are regrown on the way
                xd = torch.randn(B, 1, cfg.hidden_size, device="cuda", dtype=dtype)
                posd = torch.full((B, 1), N + i, device="cuda", dtype=torch.long)
                o, _, past = pi.forward_internlm2_calibquant(att, xd, None, posd if fused else posd.int(), past,
                                                            False, True)
                if i % 37 == 0 or i == 299:
                    step_out.append(o.clone())
        assert hasattr(att, "_cq_rope_call") == fused
        if shim:    # every step after the first went through the shim, which regrew the window on the way
            step = att._cq_step[0]
            assert step.steps == 299 and step.length == S + TXT + 300 and step.capacity >= step.length
        else:
            assert "_cq_step" not in att.__dict__
        outs.append(torch.stack(step_out))
        wins.append((past[0].clone(), past[1].clone()))
    assert wins[0][0].shape == (B, cfg.num_key_value_heads, S + TXT + 300, 128)
    for other in (1, 2):
        assert torch.equal(wins[0][0], wins[other][0]) and torch.equal(wins[0][1], wins[other][1])
        assert torch.equal(outs[0], outs[other])


def test_fused_decode_step_on_a_chunked_context():
    """A context whose packed tokens take several chunks (a call with a workspace): the steady-state decode step
    goes through the host shim and the re-aimed call object all the same, and both give the bits of the path that
    prepares a new call on every step."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    cfg = InternLM2Config.tiny()
    dtype = torch.bfloat16
    B, S, T, TXT = 2, 4, 20000, 9
    N = S + T + TXT
    outs = []
    for mode in ("shim", "call", "fresh"):
        torch.manual_seed(11)
        att = InternLM2Attention(cfg).cuda().to(dtype)
        att.cq_sprompt_len, att.cq_image_token_num = S, T
        att.cq_no_step_shim = mode != "shim"
        x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=dtype)
        pos = torch.arange(N, device="cuda")[None].expand(B, N)
        with torch.no_grad():
            _, _, past = pi.forward_internlm2_calibquant(att, x, None, pos, None, False, True)
            step_out = []
            for i in range(12):
                xd = torch.randn(B, 1, cfg.hidden_size, device="cuda", dtype=dtype)
                posd = torch.full((B, 1), N + i, device="cuda", dtype=torch.long)
                if mode == "fresh":
                    att._cq_call = None     # a new prepared call (and plan) on every step
                o, _, past = pi.forward_internlm2_calibquant(att, xd, None, posd, past, False, True)
                step_out.append(o.clone())
                if i == 0:
                    plan = att._cq_call.plan()
                    assert plan["chunks"] > 1 and att._cq_call.workspace_bytes > 0
        if mode == "shim":
            assert att._cq_step[0].steps == 11
        else:
            assert "_cq_step" not in att.__dict__
        outs.append(torch.stack(step_out))
    assert torch.isfinite(outs[0].float()).all()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_patched_model_without_image_tokens_equals_the_fp_model():
    """With zero packed tokens the quantised path is plain attention over the fp window."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention
    from calibquant_amd.internlm2 import InternVLChatStandIn
    m = _tiny_model()
    lm = m.language_model
    fp_forward, fp_generate = InternLM2Attention.forward, InternVLChatStandIn.generate
    ids = torch.randint(0, 500, (2, 40), device="cuda")
    nxt = torch.randint(0, 500, (2, 1), device="cuda")
    pos = torch.arange(40, device="cuda")[None].expand(2, 40)
    pos1 = torch.full((2, 1), 40, device="cuda", dtype=torch.long)

    def two_steps():
        emb = lm.get_input_embeddings()
        l0, past = lm.forward_step(emb(ids), pos, None)
        l1, past = lm.forward_step(emb(nxt), pos1, past)
        return l0.float(), l1.float()

    try:
        with torch.no_grad():
            b0, b1 = two_steps()
            pi.patch_model(m, "calibquant", sprompt_len=0)
            for layer in lm.model.layers:
                layer.attention.cq_image_token_num = 0
            p0, p1 = two_steps()
        assert torch.allclose(b0, p0, atol=3e-2, rtol=3e-2)
        assert torch.allclose(b1, p1, atol=3e-2, rtol=3e-2)
    finally:
        InternLM2Attention.forward, InternVLChatStandIn.generate = fp_forward, fp_generate


@pytest.mark.parametrize("tower", ["stand-in", "internvit"])
def test_patch_model_and_custom_generate_end_to_end(tower):
    """Synthetic tiles -> 256 image tokens each, quantised at prefill, 8 greedy tokens.  With the
    InternViT-shaped tower the 12 tiles go through `extract_feature` in two chunks (10 + 2), as the
    reference's `custom_generate` runs them (patch_internvl.py:53-65)."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternVLChatStandIn
    from calibquant_amd.internvit import InternViTConfig
    fp_forward, fp_generate = InternLM2Attention.forward, InternVLChatStandIn.generate
    m = _tiny_model(seed=3, vit=InternViTConfig.tiny() if tower == "internvit" else None)
    B, S, tiles, txt = (2, 41, 6, 9) if tower == "internvit" else (2, 41, 2, 9)
    T = tiles * 256
    ids = torch.randint(0, 500, (B, S + T + txt), device="cuda")
    ids[:, S:S + T] = m.img_context_token_id
    pix = torch.rand(B * tiles, 3, 448, 448, device="cuda", dtype=torch.bfloat16)
    try:
        pi.patch_model(m, "calibquant")
        os.environ.pop("IMAGE_TOKEN_NUM", None)
        out = m.generate(pixel_values=pix, input_ids=ids, max_new_tokens=8)
        assert out.shape == (B, 8)
        assert os.environ["IMAGE_TOKEN_NUM"] == str(T)
        att = m.language_model.model.layers[0].attention
        assert att.encoded_features_k.shape == (B, 2, T, 16) and att.encoded_features_k.dtype == torch.uint8
        assert att._cq_step[0].length == S + txt + 7
        out2 = m.generate(pixel_values=pix, input_ids=ids, max_new_tokens=8)
        assert torch.equal(out, out2)
    finally:
        InternLM2Attention.forward, InternVLChatStandIn.generate = fp_forward, fp_generate


def _prefill(m, ids, pix=None):
    """Prompt embeddings (image features spliced in) -> last-position logits and the per-layer cache."""
    lm = m.language_model
    emb = lm.get_input_embeddings()(ids)
    if pix is not None:
        vit = m.extract_feature(pix)
        emb = emb.clone()
        emb[ids == m.img_context_token_id] = vit.reshape(-1, emb.shape[-1]).to(emb.dtype)
    B, N = ids.shape
    pos = torch.arange(N, device=ids.device)[None].expand(B, N)
    return lm.forward_step(emb, pos, None)


@pytest.mark.parametrize("quantized,fp_kernel,width", [(True, False, "tiny"), (False, False, "tiny"), (False, True, "tiny"),
                                                       (True, False, "26b")])
def test_static_decoder_graph_replays_equal_eager_steps(quantized, fp_kernel, width):
    """The recorded decode step, replayed per token, produces the tokens of the same step run
    eagerly, and its first step agrees with the model's own eager step.  `26b`: two layers of the
    InternLM2-20B width (hidden 6 144, 48 query / 8 kv heads: units of three heads) at batch 6."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.graph_decode import StaticDecoder
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config, InternVLChatStandIn
    fp_forward, fp_generate = InternLM2Attention.forward, InternVLChatStandIn.generate
    if width == "26b":
        torch.manual_seed(5)
        cfg = InternLM2Config(vocab_size=512, hidden_size=6144, intermediate_size=16384, num_hidden_layers=2,
                              num_attention_heads=48, num_key_value_heads=8, max_position_embeddings=8192)
        m = InternVLChatStandIn(cfg).cuda().to(torch.bfloat16).eval()
    else:
        m = _tiny_model(seed=5)
    lm = m.language_model
    B, S, tiles, txt, NEW = (6 if width == "26b" else 2), 41, 2, 9, 12
    T = tiles * 256
    ids = torch.randint(0, 500, (B, S + T + txt), device="cuda")
    ids[:, S:S + T] = m.img_context_token_id
    pix = torch.rand(B * tiles, 3, 448, 448, device="cuda", dtype=torch.bfloat16)
    N = ids.shape[1]
    try:
        with torch.no_grad():
            if quantized:
                pi.patch_model(m, "calibquant")
                for layer in lm.model.layers:
                    layer.attention.cq_image_token_num = T
            runs = []
            for use_graph in (False, True):
                logits, past = _prefill(m, ids, pix)
                first = logits[:, -1].argmax(-1)
                dec = StaticDecoder(lm, past, N, NEW, fp_kernel=fp_kernel)
                toks = dec.generate(first, NEW, use_graph=use_graph)
                torch.cuda.synchronize()
                assert (dec.graph is not None) == use_graph
                runs.append(toks)
            assert torch.equal(runs[0], runs[1])
            # first decode step against the model's eager forward_step (different norm kernel,
            # same arithmetic up to rounding)
            logits, past = _prefill(m, ids, pix)
            first = logits[:, -1].argmax(-1)
            dec = StaticDecoder(lm, past, N, 2, fp_kernel=fp_kernel)
            dec.tok.copy_(first)
            x = lm.get_input_embeddings()(first)[:, None]
            pos1 = torch.full((B, 1), N, device="cuda", dtype=torch.long)
            want, _ = lm.forward_step(x, pos1, past)
            lay = lm.model.layers
            got_tok = dec.step().clone()
            assert runs[0][:, 1].tolist() == got_tok.tolist()
            # the eager model's choice has (near-)maximal logit under the static step as well
            w = want[:, -1].float()
            assert ((w.max(-1).values - w.gather(1, got_tok[:, None])[:, 0]) < 0.15).all()
    finally:
        InternLM2Attention.forward, InternVLChatStandIn.generate = fp_forward, fp_generate


def test_patched_model_with_per_token_values():
    """`patch_model(..., v_mode="token")`: values quantised per token at prefill, decoded by the
    fused kernel; one layer's decode output against the oracle on the module's own state."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    torch.manual_seed(9)
    cfg = InternLM2Config.tiny()
    att = InternLM2Attention(cfg).cuda().to(torch.bfloat16)
    att.cq_sprompt_len, att.cq_image_token_num, att.cq_v_mode = 4, 300, "token"
    B, S, T, TXT = 2, 4, 300, 6
    N = S + T + TXT
    x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    pos = torch.arange(N, device="cuda")[None].expand(B, N)
    with torch.no_grad():
        _, _, past = pi.forward_internlm2_calibquant(att, x, None, pos, None, False, True)
        assert att.encoded_features_v.dtype == torch.int32 and att.encoded_features_v.shape == (B, 2, T, 4)
        assert att.scale_value.shape == (B, cfg.num_attention_heads, T, 4)
        _, _, v = att.split_qkv(x)
        w_ref, s_ref, m_ref = O.kivi_quantize_pack(to_np(v[:, S:S + T].transpose(1, 2)), 32, 1, "bf16")
        assert np.array_equal(att.encoded_features_v.cpu().numpy(), w_ref)
        xd = torch.randn(B, 1, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
        posd = torch.full((B, 1), N, device="cuda", dtype=torch.long)
        out_d, _, past2 = pi.forward_internlm2_calibquant(att, xd, None, posd, past, False, True)
        qd, kd, vd = att.split_qkv(xd)
        cos, sin = att.rotary_emb(vd, seq_len=N + 1)
        qd, kd = pi.apply_rotary_pos_emb(qd.transpose(1, 2), kd.transpose(1, 2), cos, sin, posd)
        ks, kz, _, _ = att._cq_stats
        want = O.decode_attention(to_np(qd[:, :, 0]), att.encoded_features_k.cpu().numpy(), w_ref, to_np(ks), to_np(kz),
                                  s_ref, m_ref, to_np(past2[0]), to_np(past2[1]), S, 1, v_token_group=32)
        ref = att.wo(torch.from_numpy(want).cuda().to(torch.bfloat16).reshape(B, 1, -1))
        err = (out_d.float() - ref.float()).abs()
        assert err.max().item() < 2e-2 and err.mean().item() < 2e-3


def test_two_prefills_follow_the_environment_variable(monkeypatch):
    """Two prompts through the patched forward with only IMAGE_TOKEN_NUM updated in between
    (no custom_generate, no attribute): each prefill quantises its own image slice, and a 4-D
    prefill mask is refused instead of being dropped."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd._lib import CalibQuantError
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config
    torch.manual_seed(3)
    cfg = InternLM2Config.tiny()
    att = InternLM2Attention(cfg).cuda().to(torch.bfloat16)
    att.cq_sprompt_len = 3
    B = 2
    with torch.no_grad():
        for T in (200, 72):
            monkeypatch.setenv("IMAGE_TOKEN_NUM", str(T))
            N = 3 + T + 5
            x = torch.randn(B, N, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
            pos = torch.arange(N, device="cuda")[None].expand(B, N)
            _, _, past = pi.forward_internlm2_calibquant(att, x, None, pos, None, False, True)
            assert att.image_token_num == T and att.encoded_features_k.shape[2] == T
            assert past[0].shape[2] == N - T
            q, k, v = att.split_qkv(x)
            cv, _, _ = O.quantize_pack(to_np(v[:, 3:3 + T]), 1, 0.3, "bf16")
            assert np.array_equal(att.encoded_features_v.cpu().numpy(), cv)
        with pytest.raises(CalibQuantError):
            pi.forward_internlm2_calibquant(att, x, torch.zeros(B, 1, N, N, device="cuda"), pos, None, False, True)
