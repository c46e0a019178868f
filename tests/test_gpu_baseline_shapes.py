"""The benchmark configurations at their full sizes, checked on the GPU.

Every batch row of the decode path is an independent problem, so a case of one or two
oracle rows repeated to the full batch pins every row: the repetitions must be
bit-identical to each other and the first rows within the tolerance of the oracle
(1e-2 max-abs / 1e-3 mean-abs against the fp32 dequant-attention).

  layer, 2 bits      batch 64, 32/8 heads, 3 328 packed + 128 window rows, bf16, Student-t outliers
  26B layer          batch 16, 48/8 heads, 9 984 packed + 64 window rows, 1 bit
  long context       batch 8, 32 768 packed tokens (chunked launch)
  wide batch         batch 256, 3 328 packed tokens
  8B-shaped model    32 layers, hidden 4 096, batch 64: first and last layer's decode output against
                     the oracle on the module's own state, recorded step == eager step
"""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import case_to_gpu, make_case, to_np

pytestmark = pytest.mark.gpu


def _check(got, want, what=""):
    err = np.abs(got - want)
    assert err.max() < 1e-2 and err.mean() < 1e-3, (what, float(err.max()), float(err.mean()))


def _repeated(ops, rows, reps, Hq, Hkv, T, R, S, bits, seed, expect_plan=None, **kw):
    c = make_case(rows, Hq, Hkv, 128, T, max(R, 1), bits, "bf16", seed=seed, outlier_kind="student")
    g = case_to_gpu(c, "bf16")
    rep = {k: torch.cat([v] * reps, 0) for k, v in g.items()}
    call = ops.DecodeCall(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"],
                          rep["kr"] if R else None, rep["vr"] if R else None, sprompt_len=S, bits=bits, **kw)
    plan = call.plan()
    for key, val in (expect_plan or {}).items():
        assert plan[key] == val, (key, plan)
    print("plan", plan, flush=True)
    out = call.run()
    torch.cuda.synchronize()
    assert out.shape[0] == rows * reps
    assert torch.equal(out, out[:rows].repeat(reps, 1, 1))
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                              c["kr"][:, :, :R], c["vr"][:, :, :R], S, bits)
    _check(to_np(out[:rows]), want, plan)
    return plan


@pytest.fixture(scope="module")
def ops():
    from calibquant_amd import ops as o
    return o


def test_layer_shape_two_bits_batch_64(ops):
    _repeated(ops, 2, 32, 32, 8, 3328, 128, 0, 2, seed=301, expect_plan={"launches": 1, "heads_per_unit": 4})


def test_layer_shape_one_bit_batch_64_with_system_rows(ops):
    """The headline shape with the reference's 41 system-prompt rows ahead of the image block."""
    _repeated(ops, 2, 32, 32, 8, 3328, 128, 41, 1, seed=302, expect_plan={"launches": 1, "heads_per_unit": 4})


def test_26b_layer_shape_batch_16(ops):
    """48 query / 8 kv heads, 9 984 packed tokens + 64 window rows: two exact units of three heads per kv
    head that hold the whole token axis in one launch with the logits in registers."""
    _repeated(ops, 2, 8, 48, 8, 9984, 64, 0, 1, seed=303,
              expect_plan={"launches": 1, "heads_per_unit": 3, "register_logits": 10})


def test_long_context_batch_8_kv_32768(ops):
    plan = _repeated(ops, 1, 8, 32, 8, 32768, 0, 0, 1, seed=304)
    assert plan["chunks"] > 1


def test_long_context_batch_8_kv_32768_with_window(ops):
    _repeated(ops, 1, 8, 32, 8, 32768, 77, 41, 1, seed=305)


def test_wide_batch_256_kv_3328(ops):
    _repeated(ops, 2, 128, 32, 8, 3328, 0, 0, 1, seed=306, expect_plan={"launches": 1, "threads": 512})


def test_wide_batch_256_kv_3328_two_bits(ops):
    _repeated(ops, 2, 128, 32, 8, 3328, 0, 0, 2, seed=307)


def test_full_8b_shaped_model_batch_64_first_and_last_layer_and_recorded_step():
    """InternLM2.5-7B-shaped language model (32 layers, hidden 4 096, 32/8 heads, vocab 92 553), random
    bf16 weights, batch 64, 41 + 3 328 + 23 prompt tokens.  Two prompt rows are repeated to the batch.
    After the prefill, one eager decode step: the attention outputs of layers 0 and 31 equal
    wo(oracle attention) on each module's own packed state and window, for the first two and the
    last two batch rows.  Then four tokens through the recorded step equal the same four through
    the eager step."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.graph_decode import StaticDecoder
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config, InternVLChatStandIn
    fp_forward, fp_generate = InternLM2Attention.forward, InternVLChatStandIn.generate
    dev = torch.device("cuda:0")
    torch.manual_seed(11)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            m = InternVLChatStandIn(InternLM2Config.internvl2_5_8b()).eval()
    finally:
        torch.set_default_dtype(prev)
    lm = m.language_model
    cfg = lm.config
    B, S, T, TXT, NEW = 64, 41, 3328, 23, 5
    N = S + T + TXT
    ids2 = torch.randint(0, 90000, (2, N), device=dev)
    emb2 = lm.get_input_embeddings()(ids2)
    # image rows: feature-like values with a few strong channels
    g = torch.Generator(device=dev).manual_seed(3)
    img = torch.randn((2, T, cfg.hidden_size), generator=g, device=dev, dtype=torch.float32) * 0.02
    emb2[:, S:S + T] = img.to(torch.bfloat16)
    try:
        import contextlib
        import io
        with contextlib.redirect_stdout(io.StringIO()):
            pi.patch_model(m, "calibquant")
        layers = lm.model.layers
        for layer in layers:
            layer.attention.cq_image_token_num = T
        pos = torch.arange(N, device=dev)[None].expand(B, N)

        def prefill():
            with torch.no_grad():
                return lm.forward_step(emb2.repeat(B // 2, 1, 1), pos, None)

        print("prefill", flush=True)
        logits, past = prefill()
        first = logits[:, -1].argmax(-1)
        # ---- one eager decode step with the first and the last layer's attention observed
        seen = {}

        def watch(i):
            def hook(mod, args, kwargs, output):
                seen[i] = (args[0].detach().clone(), output[0].detach().clone(), output[2])
            return hook

        handles = [layers[i].attention.register_forward_hook(watch(i), with_kwargs=True) for i in (0, len(layers) - 1)]
        x = lm.get_input_embeddings()(first)[:, None]
        pos1 = torch.full((B, 1), N, device=dev, dtype=torch.long)
        print("decode step", flush=True)
        with torch.no_grad():
            logits1, past1 = lm.forward_step(x, pos1, past)
        for h in handles:
            h.remove()
        rows = torch.tensor([0, 1, B - 2, B - 1], device=dev)
        for i, (hid, out_d, pkv) in seen.items():
            att = layers[i].attention
            assert att.encoded_features_k.shape == (B, 8, T, 16) and pkv[0].shape == (B, 8, S + TXT + 1, 128)
            with torch.no_grad():
                qd, kd, vd = att.split_qkv(hid)       # the same projection call as the step's own, then the rows
                qd, kd, vd = qd[rows], kd[rows], vd[rows]
                cos, sin = att.rotary_emb(vd, seq_len=N + 1)
                qd, kd = pi.apply_rotary_pos_emb(qd.transpose(1, 2), kd.transpose(1, 2), cos, sin, pos1[rows])
            ks, kz, vs, vz = (to_np(t[rows]) for t in att._cq_stats)
            want = O.decode_attention(to_np(qd[:, :, 0]), att.encoded_features_k[rows].cpu().numpy(),
                                      att.encoded_features_v[rows].cpu().numpy(), ks, kz, vs, vz,
                                      to_np(pkv[0][rows]), to_np(pkv[1][rows]), S, 1)
            # the new window row is the rotated key / the value of this step
            assert torch.equal(pkv[0][rows][:, :, -1], kd[:, :, 0]) and torch.equal(pkv[1][rows][:, :, -1], vd[:, 0])
            with torch.no_grad():
                ref = att.wo(torch.from_numpy(want).to(dev).to(torch.bfloat16).reshape(len(rows), 1, -1))
            err = (out_d[rows].float() - ref.float()).abs()
            scale = ref.float().abs().mean().item()
            print(f"layer {i}: max-abs {err.max().item():.3e} mean-abs {err.mean().item():.3e} (|ref| {scale:.3e})", flush=True)
            assert err.max().item() < 2e-2 and err.mean().item() < 2e-3
        del seen, past1, logits1
        # ---- recorded step == eager step over four more tokens
        runs = []
        for use_graph in (False, True):
            if use_graph:
                print("prefill again", flush=True)
                logits, past = prefill()
            dec = StaticDecoder(lm, past, N, NEW)
            del past
            toks = dec.generate(first, NEW, use_graph=use_graph)
            torch.cuda.synchronize()
            assert (dec.graph is not None) == use_graph
            runs.append(toks)
            del dec
        assert torch.equal(runs[0], runs[1])
    finally:
        InternLM2Attention.forward, InternVLChatStandIn.generate = fp_forward, fp_generate


@pytest.mark.parametrize("bits", [1, 2])
def test_long_context_chunked_step_is_deterministic_back_to_back(ops, bits):
    """Sixty chunked steps queued back to back on one stream (the unit counters are cleared by each step's first
    launch, the partials merged by whichever workgroup of a unit finishes last): every output equals the first,
    which is checked against the oracle."""
    c = make_case(1, 32, 8, 128, 32768, 16, bits, "bf16", seed=330 + bits, outlier_kind="student")
    g = {k: torch.cat([v] * 8, 0) for k, v in case_to_gpu(c, "bf16").items()}
    outs = [torch.empty((8, 32, 128), dtype=torch.bfloat16, device="cuda") for _ in range(60)]
    call = ops.DecodeCall(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"],
                          sprompt_len=3, bits=bits, out=outs[0])
    assert call.plan()["chunks"] > 1
    for o in outs:
        call.args.out = o.data_ptr()
        call.run()
    torch.cuda.synchronize()
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], 3, bits)
    _check(to_np(outs[0][:1]), want, "first of sixty")
    for i, o in enumerate(outs[1:]):
        assert torch.equal(o, outs[0]), i + 1
