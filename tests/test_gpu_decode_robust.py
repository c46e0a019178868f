"""Robustness of the fused decode kernel's other instantiations against the fp32 dequant-attention
oracle (1e-2 max-abs, 1e-3 mean-abs beyond the storage rounding of the result, see `_check`): logits of magnitude 50-300 (key outlier channels x100, queries
x3) through the 2-bit paired launch, the 1024-thread launch that keeps a long chunk's logits in
registers, the chunked step in one launch and in two (both hand-over modes) and per-token values; and softmax weights built so
that the packed-fp16 partial sums of the value loop sit next to 1.0."""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import CLIPS, case_to_gpu, to_np

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1e-2, 1e-3


@pytest.fixture(scope="module")
def ops():
    from calibquant_amd import ops
    return ops


def _check(got, want, dtype="bf16"):
    """The tolerance, on top of what storing the oracle's own result in the storage dtype costs: with a
    peaked softmax the outputs are of magnitude 1, where half a bf16 step is 2e-3 to 4e-3 - a kernel
    that is exact before its one rounding would already sit at 1e-3 mean-abs (measured: the rounding of
    the oracle's result alone is 1.02e-3 / 1.44e-3 mean-abs on two of the cases below)."""
    err = np.abs(got - want)
    rnd = np.abs(O.round_to(want, dtype) - want)
    assert np.isfinite(got).all()
    assert err.max() < MAX_ABS + rnd.max(), f"max-abs {err.max():.3e} (storage rounding alone {rnd.max():.3e})"
    assert err.mean() < MEAN_ABS + rnd.mean(), f"mean-abs {err.mean():.3e} (storage rounding alone {rnd.mean():.3e})"


def _large_logit_case(B, Hq, Hkv, T, R, bits, mult, qscale, seed, token_values=False):
    D = 128
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
    v = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
    for h in range(Hkv):
        k[:, :, h, rng.permutation(D)[:4]] *= mult
    k, v = O.round_to(k, "bf16"), O.round_to(v, "bf16")
    ck, sk, zk = O.quantize_pack(k, bits, CLIPS[bits][0], "bf16")
    if token_values:
        cv, sv, zv = O.kivi_quantize_pack(np.transpose(v, (0, 2, 1, 3)), 32, bits, "bf16")
    else:
        cv, sv, zv = O.quantize_pack(v, bits, CLIPS[bits][1], "bf16")
    return dict(q=O.round_to(qscale * rng.standard_normal((B, Hq, D), dtype=np.float32), "bf16"), ck=ck, cv=cv,
                sk=sk, zk=zk, sv=sv, zv=zv, kr=O.round_to(rng.standard_normal((B, Hkv, R, D), dtype=np.float32), "bf16"),
                vr=O.round_to(rng.standard_normal((B, Hkv, R, D), dtype=np.float32), "bf16"))


# name: (rows of the oracle case, repetitions, Hq, Hkv, T, R, bits, per-token values, what the plan must say)
LARGE = {
    "2bit-paired": (2, 20, 32, 8, 3328, 128, 2, False, dict(threads=512, chunks=1)),
    "26b-register-logits": (1, 16, 48, 8, 9984, 64, 1, False, dict(threads=1024, chunks=1, register_logits=10)),
    "chunked-one-launch": (1, 8, 32, 8, 20000, 70, 1, False, dict(launches=1)),
    "chunked-one-launch-2bit": (1, 8, 32, 8, 12000, 70, 2, False, dict(launches=1)),
    "chunked-recompute": (1, 12, 32, 8, 20000, 70, 1, False, dict(launches=2)),       # 96 units x 6 chunks: too many to wait
    "chunked-logits-buffer": (1, 12, 32, 8, 20000, 70, 2, False, dict(launches=2)),
    "token-values": (2, 20, 32, 8, 3328, 128, 1, True, dict(chunks=1)),
    "token-values-2bit": (1, 8, 32, 8, 2000, 40, 2, True, dict(chunks=1)),
}


@pytest.mark.parametrize("mult, qscale", [(100.0, 1.0), (30.0, 3.0)])
@pytest.mark.parametrize("name", sorted(LARGE))
def test_large_logits(ops, name, mult, qscale):
    rows, reps, Hq, Hkv, T, R, bits, tokv, plan_want = LARGE[name]
    c = _large_logit_case(rows, Hq, Hkv, T, R, bits, mult, qscale, seed=11, token_values=tokv)
    g = case_to_gpu(c, "bf16")
    rep = {n: torch.cat([t] * reps, 0) for n, t in g.items()}
    call = ops.DecodeCall(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"], rep["kr"], rep["vr"],
                          bits=bits, v_mode="token" if tokv else "channel")
    plan = call.plan()
    for key, val in plan_want.items():
        assert plan[key] == val, (key, plan)
    if name.startswith("chunked"):
        assert plan["chunks"] > 1
    out = call.run()
    torch.cuda.synchronize()
    assert torch.equal(out, out[:rows].repeat(reps, 1, 1))
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], 0, bits,
                              v_token_group=32 if tokv else 0)
    _check(to_np(out[:rows]), want)


@pytest.mark.parametrize("reps, T", [(20, 3328), (1, 3328), (1, 1000)])
def test_value_sums_next_to_one(ops, reps, T):
    """One token in every 32 carries weight 1 and the other 31 a weight just under half a unit in the last
    place of an fp16 1.0: the value loop adds the subset sums of 32 tokens as packed fp16 before it goes to
    fp32, so these sums sit where that format rounds hardest.  The logits take exactly two values (one key
    channel with a non-zero query weight), chosen so that the calibrated gap is ln(1 / 2.3e-4)."""
    B, Hq, Hkv, D, R = 2, 32, 8, 128, 0
    rng = np.random.default_rng(T)
    code = np.zeros((B, Hkv, T, D), np.uint8)
    hot = np.zeros((B, Hkv, T), bool)
    for w0 in range(0, T, 32):
        pick = rng.integers(0, min(32, T - w0), size=(B, Hkv))
        for b in range(B):
            for h in range(Hkv):
                hot[b, h, w0 + pick[b, h]] = True
    c0 = 5
    code[..., c0] = hot
    ck = O.encode(code, 1)
    cv = O.encode(rng.integers(0, 2, size=(B, Hkv, T, D)).astype(np.uint8), 1)
    gap = 3.0 + np.log(1.0 / 2.3e-4)          # calibration takes 3 off the top
    q = np.zeros((B, Hq, D), np.float32)
    q[:, :, c0] = 8.0 * (1.0 + 0.03 * (np.arange(Hq) % 4))
    sk = np.ones((B, Hkv, D), np.float32)
    sk[..., c0] = gap * np.sqrt(D) / 8.0
    zk = np.full((B, Hkv, D), 0.5, np.float32)
    c = dict(q=O.round_to(q, "bf16"), ck=ck, cv=cv, sk=O.round_to(sk, "bf16"), zk=O.round_to(zk, "bf16"),
             sv=O.round_to(0.5 + rng.random((B, Hkv, D), dtype=np.float32), "bf16"),
             sz=None, zv=O.round_to(rng.random((B, Hkv, D), dtype=np.float32), "bf16"))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16).cuda()  # noqa: E731
    rp = lambda x: torch.cat([x] * reps, 0)   # noqa: E731
    out = ops.decode_attn(rp(t(c["q"])), rp(torch.from_numpy(ck).cuda()), rp(torch.from_numpy(cv).cuda()),
                          rp(t(c["sk"])), rp(t(c["zk"])), rp(t(c["sv"])), rp(t(c["zv"])), None, None, bits=1)
    torch.cuda.synchronize()
    assert torch.equal(out, out[:B].repeat(reps, 1, 1))
    want = O.decode_attention(c["q"], ck, cv, c["sk"], c["zk"], c["sv"], c["zv"], None, None, 0, 1)
    # the weights are what the case was built for: 1 for the picked tokens, about 2.3e-4 (x the head's factor) elsewhere
    _check(to_np(out[:B]), want)


def test_single_launch_chunked_step_gives_up_and_the_host_reports_it(ops):
    """The wait inside the single-launch chunked step is bounded.  With the bound set to zero polls every
    workgroup gives up at once (each kernel still ends normally, nothing hangs, and the workspace's hand-over
    words are left empty as after a finished launch): the call that launched it returns success, the next chunked call on the device reports CQ_ERR_LAUNCH once, and from then on the
    process takes two launches - with results equal to the oracle - until the bound is set again."""
    from calibquant_amd import _lib
    from tests.util import make_case
    lib = _lib.load()
    B, Hq, Hkv, T, R = 2, 32, 8, 20000, 40
    c = make_case(B, Hq, Hkv, 128, T, R, 1, "bf16", seed=901, outlier_kind="student")
    g = case_to_gpu(c, "bf16")
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], c["kr"], c["vr"], 0, 1)
    call = ops.DecodeCall(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"], bits=1)
    assert call.plan()["chunks"] > 1 and call.plan()["launches"] == 1
    good = call.run().clone()
    torch.cuda.synchronize()
    _check(to_np(good), want)
    assert lib.cq_decode_attn_gave_up() == 0
    # the hand-over words (a counter per unit, then two records per head and chunk) are the tail of the workspace
    units, heads, chunks = B * Hkv, call.plan()["heads_per_unit"], call.plan()["chunks"]
    rec = units * heads * chunks * 16
    cnt = (units * 8 + 255) // 256 * 256 + rec

    def handover_words():
        return torch.cat([call.workspace[-cnt:][:units * 8], call.workspace[-rec:]])
    assert not handover_words().any(), "a finished launch leaves its hand-over words empty"
    before = lib.cq_decode_attn_wait_polls(0)
    try:
        call.run()                       # launched; its workgroups give up
        torch.cuda.synchronize()
        # ... and so does one whose workgroups gave up: a replay of that very launch (a recorded step comes
        # back with the same epoch) must not find this launch's records
        assert not handover_words().any()
        assert lib.cq_decode_attn_gave_up() == 1
        with pytest.raises(_lib.CalibQuantError):
            call.run()                   # the host finds the word set
        assert lib.cq_decode_attn_gave_up() == 0      # reported
        out = call.run().clone()         # two launches from here on
        torch.cuda.synchronize()
        _check(to_np(out), want)
    finally:
        lib.cq_decode_attn_wait_polls(before)      # also re-enables the single launch
    again = call.run().clone()
    torch.cuda.synchronize()
    assert torch.equal(again, good)
