"""GPU parity of the fused decode-attention kernel against the fp32
dequant-attention oracle computed from the same packed codes and statistics.
Tolerance (stated by the task): 1e-2 max-abs, 1e-3 mean-abs."""
import numpy as np
import pytest
import torch

from oracle import cq_oracle as O
from tests.util import case_to_gpu, make_case, to_np

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1e-2, 1e-3


@pytest.fixture(scope="module")
def ops():
    from calibquant_amd import ops
    return ops


def _run(ops, c, dtype, S, bits, mask=None, **kw):
    g = case_to_gpu(c, dtype)
    m = None if mask is None else torch.from_numpy(mask.astype(np.float32)).cuda()
    out = ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"],
                          sprompt_len=S, bits=bits, mask=m, **kw)
    torch.cuda.synchronize()
    return to_np(out)


def _oracle(c, S, bits, mask=None, **kw):
    kr = c["kr"] if c["kr"].shape[2] else None
    vr = c["vr"] if c["vr"].shape[2] else None
    return O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], kr, vr, S, bits,
                              mask=mask, **kw)


def _check(got, want):
    err = np.abs(got - want)
    assert np.isfinite(got).all()
    assert err.max() < MAX_ABS, f"max-abs {err.max():.3e}"
    assert err.mean() < MEAN_ABS, f"mean-abs {err.mean():.3e}"


CASES = [
    # B, Hq, Hkv, T, R, S
    (2, 32, 8, 3328, 128, 0),      # InternVL2.5-8B layer shape, small batch
    (1, 32, 8, 1024, 0, 0),        # CPU-reference configuration: no residual
    (2, 32, 8, 777, 60, 41),       # ragged T, system prompt of the reference (41 rows)
    (1, 8, 8, 130, 5, 2),          # MHA-like: one q head per kv head
    (1, 16, 8, 259, 70, 10),       # two q heads per kv head
    (1, 48, 8, 1000, 33, 0),       # InternLM2-20B grouping: six q heads per kv head
    (3, 32, 8, 7, 1, 1),           # a handful of packed tokens
]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("case", CASES)
def test_decode_attn_matches_oracle(ops, case, bits, dtype):
    B, Hq, Hkv, T, R, S = case
    print(f"case decode_attn {case} bits={bits} dtype={dtype}", flush=True)
    c = make_case(B, Hq, Hkv, 128, T, R, bits, dtype, seed=T + R)
    _check(_run(ops, c, dtype, S, bits), _oracle(c, S, bits))


def test_decode_attn_single_token_is_nan_like_the_reference(ops):
    """One packed token makes every channel constant: scale 0, zero-point
    inf, and the reference's bias term 0 * inf = NaN poisons the row
    (patch_internvl.py:369-370).  The kernel reproduces that, as the oracle does."""
    c = make_case(1, 32, 8, 128, 1, 4, 1, "bf16", seed=1)
    got, want = _run(ops, c, "bf16", 0, 1), _oracle(c, 0, 1)
    assert np.isnan(want).all() and np.isnan(got).all()


@pytest.mark.parametrize("bits", [1, 2])
def test_decode_attn_without_calibration_and_custom_offsets(ops, bits):
    c = make_case(2, 32, 8, 128, 500, 40, bits, "bf16", seed=9)
    _check(_run(ops, c, "bf16", 7, bits, calibrate=False), _oracle(c, 7, bits, calibrate_logits=False))
    _check(_run(ops, c, "bf16", 7, bits, calib_off_max=-1.5, calib_off_min=0.5),
           _oracle(c, 7, bits, off_max=-1.5, off_min=0.5))


@pytest.mark.parametrize("bits", [1, 2])
def test_decode_attn_with_additive_mask(ops, bits):
    B, Hq, Hkv, T, R, S = 2, 32, 8, 600, 50, 41
    c = make_case(B, Hq, Hkv, 128, T, R, bits, "bf16", seed=4)
    rng = np.random.default_rng(0)
    mask = np.zeros((B, T + R), np.float32)
    mask[0, :30] = -1e4                      # left padding inside the system prompt
    mask[1, rng.integers(0, T + R, 100)] = -1e4
    _check(_run(ops, c, "bf16", S, bits, mask=mask), _oracle(c, S, bits, mask=mask))


def test_decode_attn_residual_only_and_strided_cache(ops):
    """No packed tokens: plain attention over the fp window, read through a
    view of a larger pre-allocated cache."""
    B, Hq, Hkv, R = 2, 32, 8, 200
    c = make_case(B, Hq, Hkv, 128, 64, R, 1, "bf16", seed=2)
    g = case_to_gpu(c, "bf16")
    cap = 512
    kbuf = torch.zeros((B, Hkv, cap, 128), dtype=torch.bfloat16, device="cuda")
    vbuf = torch.zeros_like(kbuf)
    kbuf[:, :, :R] = g["kr"]
    vbuf[:, :, :R] = g["vr"]
    out = ops.decode_attn(g["q"], None, None, None, None, None, None, kbuf[:, :, :R], vbuf[:, :, :R])
    want = O.decode_attention(c["q"], c["ck"][:, :, :0], c["cv"][:, :, :0], c["sk"], c["zk"], c["sv"], c["zv"],
                              c["kr"], c["vr"], 0, 1)
    _check(to_np(out), want)
    out2 = ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"],
                           kbuf[:, :, :R], vbuf[:, :, :R], sprompt_len=41)
    _check(to_np(out2), _oracle(c, 41, 1))


@pytest.mark.parametrize("splits", [0, 3])
def test_decode_attn_row_count_read_on_device(ops, splits):
    """Window buffers of fixed capacity, the number of valid rows in a device
    scalar: the same prepared launch follows the window as it grows (what a
    recorded decode step needs).  Rows past the count hold garbage."""
    B, Hq, Hkv, T, R, S = 2, 32, 8, 1500, 150, 41
    c = make_case(B, Hq, Hkv, 128, T, R, 1, "bf16", seed=21)
    g = case_to_gpu(c, "bf16")
    cap = 192
    kbuf = torch.full((B, Hkv, cap, 128), 1e4, dtype=torch.bfloat16, device="cuda")
    vbuf = torch.full_like(kbuf, -1e4)
    kbuf[:, :, :R] = g["kr"]
    vbuf[:, :, :R] = g["vr"]
    r_dev = torch.zeros(1, dtype=torch.int32, device="cuda")
    call = ops.DecodeCall(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], kbuf, vbuf,
                          sprompt_len=S, bits=1, force_splits=splits, r_dev=r_dev)
    for rows in (60, 150, 129):          # grow, then shrink: only the scalar changes
        r_dev.fill_(rows)
        got = to_np(call.run())
        torch.cuda.synchronize()
        want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                                  c["kr"][:, :, :rows], c["vr"][:, :, :rows], S, 1)
        _check(got, want)


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("splits", [2, 5])
def test_decode_attn_split_path_matches_fused_path(ops, bits, splits):
    B, Hq, Hkv, T, R, S = 1, 32, 8, 2000, 70, 3
    c = make_case(B, Hq, Hkv, 128, T, R, bits, "bf16", seed=8)
    want = _oracle(c, S, bits)
    _check(_run(ops, c, "bf16", S, bits, force_splits=splits), want)
    rng = np.random.default_rng(1)
    mask = np.where(rng.random((B, T + R)) < 0.1, -1e4, 0.0).astype(np.float32)
    _check(_run(ops, c, "bf16", S, bits, mask=mask, force_splits=splits), _oracle(c, S, bits, mask=mask))


def test_decode_attn_long_context_auto_split(ops):
    """KV 32768 at batch 1: the chunked path (min/max launch, main launch, merge)."""
    B, Hq, Hkv, T, R = 1, 32, 8, 32768, 16
    c = make_case(B, Hq, Hkv, 128, T, R, 1, "bf16", seed=12)
    _check(_run(ops, c, "bf16", 0, 1), _oracle(c, 0, 1))


def _sweep_cases(n, seed):
    """Seeded draws over the options that select a code path: grouping (1 / 2 / 4 / 6 query heads per
    kv head), token counts either side of the chunking thresholds, window lengths either side of the
    128-row tile, dtype, bits, mask, calibration, forced chunk counts."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        Hkv = int(rng.choice([1, 2, 8]))
        G = int(rng.choice([1, 2, 4, 6]))
        T = int(rng.choice([5, 63, 64, 300, 1023, 2047, 2049, 4097, 6000]))
        B = 1 if Hkv * T > 20000 else int(rng.integers(1, 4))
        R = int(rng.choice([0, 1, 7, 128, 129, 200, 300]))
        S = int(rng.integers(0, min(R, 41) + 1))
        out.append((i, B, Hkv * G, Hkv, T, R, S, int(rng.integers(1, 3)), str(rng.choice(["bf16", "fp16"])),
                    bool(rng.random() < 0.3), bool(rng.random() < 0.8),
                    int(rng.choice([0, 0, 2, 3])) if T >= 300 else 0))
    return out


@pytest.mark.parametrize("case", _sweep_cases(24, seed=5), ids=lambda c: "-".join(str(x) for x in c[1:]))
def test_decode_attn_seeded_option_sweep(ops, case):
    i, B, Hq, Hkv, T, R, S, bits, dtype, use_mask, calibrate, splits = case
    c = make_case(B, Hq, Hkv, 128, T, R, bits, dtype, seed=500 + i, outlier_kind="student" if i % 2 else "x10")
    mask = None
    if use_mask:
        mask = np.where(np.random.default_rng(i).random((B, T + R)) < 0.15, -1e4, 0.0).astype(np.float32)
    got = _run(ops, c, dtype, S, bits, mask=mask, calibrate=calibrate, force_splits=splits)
    _check(got, _oracle(c, S, bits, mask=mask, calibrate_logits=calibrate))


def test_decode_attn_degenerate_range_and_peaked_softmax(ops):
    """All packed keys identical (logit range 0) and a residual row that takes
    nearly all the probability mass."""
    c = make_case(1, 32, 8, 128, 256, 8, 1, "bf16", seed=6)
    c["ck"][:] = c["ck"][:, :, :1]
    c["kr"][:, :, 3] = O.round_to(c["q"].reshape(1, 8, 4, 128)[:, :, 0] * 4.0, "bf16")
    _check(_run(ops, c, "bf16", 0, 1), _oracle(c, 0, 1))


def test_decode_attn_full_batch_properties(ops):
    """Batch 64, KV 3328 + 128 (the benchmark shape): every batch row is an
    independent problem, so (a) a batch built by repeating one row gives
    identical outputs per row, and (b) rows 0..1 equal the oracle."""
    B, Hq, Hkv, T, R = 64, 32, 8, 3328, 128
    c = make_case(2, Hq, Hkv, 128, T, R, 1, "bf16", seed=20, outlier_kind="student")
    g = case_to_gpu(c, "bf16")
    rep = {k: torch.cat([v] * (B // 2), 0) for k, v in g.items()}
    out = ops.decode_attn(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"],
                          rep["kr"], rep["vr"])
    torch.cuda.synchronize()
    assert torch.equal(out[0::2], out[0:1].expand(B // 2, -1, -1))
    assert torch.equal(out[1::2], out[1:2].expand(B // 2, -1, -1))
    _check(to_np(out[:2]), _oracle(c, 0, 1))


MID_BATCH = [
    # reps, Hq, Hkv, T, R, S, bits, dtype, mask, token values — 65..256 units of four heads: one 1024-thread workgroup
    # per unit, logits waiting in the token slots (smaller batches get fewer heads per unit)
    (6, 32, 8, 3328, 128, 0, 1, "bf16", False, False),
    (6, 32, 8, 777, 60, 41, 2, "fp16", True, False),     # 2 bits: K table in two passes, partial logits in the slots
    (6, 32, 8, 1500, 33, 0, 1, "bf16", False, True),     # per-token values
    (5, 48, 8, 1000, 70, 3, 2, "bf16", False, False),    # six q heads per kv head: exact units of three heads
    (6, 32, 8, 0, 150, 5, 1, "fp16", False, False),      # window only
    (6, 56, 8, 900, 40, 0, 1, "bf16", False, False),     # seven q heads per kv head: units of 4 + 3
    (8, 40, 8, 600, 70, 9, 2, "fp16", True, False),      # five: units of 4 + 1
    (10, 24, 8, 700, 20, 0, 1, "bf16", False, False),    # three: one exact unit of three heads
]


@pytest.mark.parametrize("case", MID_BATCH, ids=lambda c: "-".join(str(x) for x in c))
def test_decode_attn_mid_batch_four_heads_per_unit(ops, case):
    reps, Hq, Hkv, T, R, S, bits, dtype, use_mask, token = case
    c = make_case(2, Hq, Hkv, 128, max(T, 1), R, bits, dtype, seed=80 + T)
    kw, okw = {}, {}
    if token:
        words, scale, mins = O.kivi_quantize_pack(np.transpose(c["v"], (0, 2, 1, 3)), 32, bits, dtype)
        c["cv"], c["sv"], c["zv"] = words, scale, mins
        kw["v_mode"], okw["v_token_group"] = "token", 32
    if T == 0:
        c["ck"], c["cv"] = c["ck"][:, :, :0], c["cv"][:, :, :0]
    mask = None
    if use_mask:
        mask = np.where(np.random.default_rng(T).random((2, T + R)) < 0.15, -1e4, 0.0).astype(np.float32)
    g = case_to_gpu(c, dtype)
    rep = {k: torch.cat([v] * reps, 0) for k, v in g.items()}
    m = None if mask is None else torch.from_numpy(mask).cuda().repeat(reps, 1)
    args = [rep[k] if T else None for k in ("ck", "cv", "sk", "zk", "sv", "zv")]
    call = ops.DecodeCall(rep["q"], *args, rep["kr"] if R else None, rep["vr"] if R else None,
                          sprompt_len=S, bits=bits, mask=m, **kw)
    plan = call.plan()
    assert (plan["threads"], plan["heads_per_unit"], plan["launches"]) == (1024, 3 if (Hq // Hkv) % 3 == 0 and not token else 4, 1)
    out = call.run()
    torch.cuda.synchronize()
    assert torch.equal(out, out[:2].repeat(reps, 1, 1))
    _check(to_np(out[:2]), _oracle(c, S, bits, mask=mask, **okw))


PAIRED = [
    # reps, Hq, Hkv, T, R, S, dtype, mask, calibrate — more than 256 units of work, a unit's layout within half the LDS:
    # the launch uses 512-thread workgroups, two per compute unit (four heads per unit: logits kept in registers, K table in two passes)
    (20, 32, 8, 777, 60, 41, "bf16", False, True),
    (20, 32, 8, 3328, 128, 0, "fp16", False, True),
    (20, 32, 8, 2100, 70, 5, "bf16", True, True),       # two blocks of staged value rows, mask
    (20, 32, 8, 300, 0, 0, "fp16", False, False),
    (20, 16, 8, 1500, 130, 3, "bf16", True, True),      # two heads per unit: logits wait in the token slots
    (17, 48, 8, 1000, 33, 0, "fp16", False, True),      # six q heads per kv head: three units of two heads
    (20, 32, 8, 0, 200, 0, "bf16", False, True),        # window only
    (12, 56, 8, 1200, 64, 2, "fp16", False, True),      # seven q heads per kv head: padded four-head units, paired
    (12, 32, 8, 5000, 64, 0, "bf16", False, True),      # 192 units, T beyond the layout with logits in the slots: one launch, logits in registers
    (8, 48, 8, 5000, 64, 3, "fp16", False, True),       # six q heads per kv head: two units of four heads, the second half padding
    (4, 32, 8, 9000, 100, 7, "bf16", False, True),      # chunked: 64 units x 8 chunks, min/max launch + merge
    (4, 32, 8, 9000, 0, 0, "fp16", True, True),
]


PAIRED_2BIT = [
    # reps, Hq, Hkv, T, R, S, dtype, mask — 2 bits, more than 256 four-head units: 512-thread workgroups, K table in four passes
    (20, 32, 8, 3328, 128, 0, "bf16", False),
    (20, 32, 8, 777, 60, 41, "fp16", True),
    (17, 48, 8, 2100, 33, 0, "bf16", False),     # padded four-head units, two blocks of staged value rows
    (4, 32, 8, 9000, 100, 7, "bf16", False),     # chunked
]


@pytest.mark.parametrize("case", PAIRED_2BIT, ids=lambda c: "-".join(str(x) for x in c))
def test_decode_attn_paired_workgroups_two_bits(ops, case):
    reps, Hq, Hkv, T, R, S, dtype, use_mask = case
    c = make_case(2, Hq, Hkv, 128, T, R, 2, dtype, seed=90 + T, outlier_kind="x10" if T % 2 else "student")
    mask = None
    if use_mask:
        mask = np.where(np.random.default_rng(T).random((2, T + R)) < 0.15, -1e4, 0.0).astype(np.float32)
    g = case_to_gpu(c, dtype)
    rep = {k: torch.cat([v] * reps, 0) for k, v in g.items()}
    m = None if mask is None else torch.from_numpy(mask).cuda().repeat(reps, 1)
    call = ops.DecodeCall(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"], rep["kr"], rep["vr"],
                          sprompt_len=S, bits=2, mask=m)
    assert call.plan()["threads"] == 512
    out = call.run()
    torch.cuda.synchronize()
    assert torch.equal(out, out[:2].repeat(reps, 1, 1))
    _check(to_np(out[:2]), _oracle(c, S, 2, mask=mask))


@pytest.mark.parametrize("case", PAIRED, ids=lambda c: "-".join(str(x) for x in c))
def test_decode_attn_paired_workgroups(ops, case):
    """Batches with more units of work than compute units: every batch row is an independent problem, so
    a two-row case repeated `reps` times gives identical outputs per repetition, and the first two
    rows equal the oracle."""
    reps, Hq, Hkv, T, R, S, dtype, use_mask, calibrate = case
    c = make_case(2, Hq, Hkv, 128, max(T, 1), R, 1, dtype, seed=60 + T, outlier_kind="x10" if T % 2 else "student")
    if T == 0:
        c["ck"], c["cv"] = c["ck"][:, :, :0], c["cv"][:, :, :0]
    mask = None
    if use_mask:
        mask = np.where(np.random.default_rng(T).random((2, T + R)) < 0.15, -1e4, 0.0).astype(np.float32)
    g = case_to_gpu(c, dtype)
    rep = {k: torch.cat([v] * reps, 0) for k, v in g.items()}
    m = None if mask is None else torch.from_numpy(mask).cuda().repeat(reps, 1)
    args = [rep[k] if T else None for k in ("ck", "cv", "sk", "zk", "sv", "zv")]
    out = ops.decode_attn(rep["q"], *args, rep["kr"] if R else None, rep["vr"] if R else None,
                          sprompt_len=S, bits=1, mask=m, calibrate=calibrate)
    torch.cuda.synchronize()
    assert torch.equal(out, out[:2].repeat(reps, 1, 1))
    _check(to_np(out[:2]), _oracle(c, S, 1, mask=mask, calibrate_logits=calibrate))


@pytest.mark.parametrize("mult, qscale", [(100.0, 1.0), (30.0, 3.0)])
def test_decode_attn_paired_workgroups_large_logits(ops, mult, qscale):
    """Key outlier channels x100 / queries x3: logits of magnitude 50-300 and a peaked softmax.  The
    512-thread launch keeps its logits in fp32 (a 16-bit logit would be off by 2-4e-2 here)."""
    from tests.util import CLIPS
    reps, Hq, Hkv, T, R, D = 20, 32, 8, 3328, 128, 128
    rng = np.random.default_rng(5)
    k = rng.standard_normal((2, T, Hkv, D), dtype=np.float32)
    v = rng.standard_normal((2, T, Hkv, D), dtype=np.float32)
    for h in range(Hkv):
        k[:, :, h, rng.permutation(D)[:4]] *= mult
    k, v = O.round_to(k, "bf16"), O.round_to(v, "bf16")
    ck, sk, zk = O.quantize_pack(k, 1, CLIPS[1][0], "bf16")
    cv, sv, zv = O.quantize_pack(v, 1, CLIPS[1][1], "bf16")
    c = dict(q=O.round_to(qscale * rng.standard_normal((2, Hq, D), dtype=np.float32), "bf16"), ck=ck, cv=cv, sk=sk, zk=zk,
             sv=sv, zv=zv, kr=O.round_to(rng.standard_normal((2, Hkv, R, D), dtype=np.float32), "bf16"),
             vr=O.round_to(rng.standard_normal((2, Hkv, R, D), dtype=np.float32), "bf16"))
    g = case_to_gpu(c, "bf16")
    rep = {n: torch.cat([t] * reps, 0) for n, t in g.items()}
    out = ops.decode_attn(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"], rep["kr"], rep["vr"])
    torch.cuda.synchronize()
    assert torch.equal(out, out[:2].repeat(reps, 1, 1))
    _check(to_np(out[:2]), _oracle(c, 0, 1))


def test_decode_attn_paired_workgroups_row_count_on_device(ops):
    """The 512-thread launch with the window's row count in a device scalar (a recorded decode step at a
    large batch)."""
    reps, Hq, Hkv, T, R, S = 20, 32, 8, 1500, 150, 41
    c = make_case(2, Hq, Hkv, 128, T, R, 1, "bf16", seed=23)
    g = case_to_gpu(c, "bf16")
    rep = {k: torch.cat([v] * reps, 0) for k, v in g.items()}
    cap = 192
    kbuf = torch.full((2 * reps, Hkv, cap, 128), 1e4, dtype=torch.bfloat16, device="cuda")
    vbuf = torch.full_like(kbuf, -1e4)
    kbuf[:, :, :R] = rep["kr"]
    vbuf[:, :, :R] = rep["vr"]
    r_dev = torch.zeros(1, dtype=torch.int32, device="cuda")
    call = ops.DecodeCall(rep["q"], rep["ck"], rep["cv"], rep["sk"], rep["zk"], rep["sv"], rep["zv"], kbuf, vbuf,
                          sprompt_len=S, bits=1, r_dev=r_dev)
    for rows in (60, 150, 129):
        r_dev.fill_(rows)
        out = call.run()
        torch.cuda.synchronize()
        assert torch.equal(out, out[:2].repeat(reps, 1, 1))
        want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                                  c["kr"][:, :, :rows], c["vr"][:, :, :rows], S, 1)
        _check(to_np(out[:2]), want)


def test_decode_attn_rejects_bad_arguments(ops):
    from calibquant_amd._lib import CalibQuantError
    c = make_case(1, 32, 8, 128, 64, 8, 1, "bf16", seed=1)
    g = case_to_gpu(c, "bf16")
    with pytest.raises(CalibQuantError):
        ops.decode_attn(g["q"].float(), g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"])
    with pytest.raises(CalibQuantError):
        ops.decode_attn(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"],
                        sprompt_len=9)
    with pytest.raises(CalibQuantError):
        ops.decode_attn(g["q"].cpu(), g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"], g["vr"])
    with pytest.raises(CalibQuantError):
        ops.decode_attn(g["q"][:, :, :64].contiguous(), g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"],
                        g["kr"], g["vr"])


@pytest.fixture
def two_launches():
    """Chunked shapes take two launches for the test (the process-wide switch of the single-launch step)."""
    from calibquant_amd import _lib
    lib = _lib.load()
    before = lib.cq_decode_attn_single_launch(0)
    yield
    lib.cq_decode_attn_single_launch(before)


@pytest.mark.parametrize("case", [(2, 16, 8, 20000, 50, 3, 1), (2, 8, 8, 20000, 0, 0, 1), (1, 32, 8, 20000, 33, 5, 2),
                                  (1, 16, 8, 20000, 33, 0, 2)], ids=lambda c: "-".join(str(x) for x in c))
def test_decode_attn_chunked_with_the_logits_buffer(ops, case, two_launches):
    """Chunked launches whose first launch hands the logits to the second through the workspace (a packed K row
    of more bytes than the logits: 2 bits, or fewer than four heads per unit), against the oracle.  (Four-head
    units at 1 bit recompute their logits: `test_long_context_batch_8_kv_32768` and the chunked cases above.)"""
    B, Hq, Hkv, T, R, S, bits = case
    c = make_case(B, Hq, Hkv, 128, T, max(R, 1), bits, "bf16", seed=500 + Hq + bits, outlier_kind="student")
    g = case_to_gpu(c, "bf16")
    call = ops.DecodeCall(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"] if R else None,
                          g["vr"] if R else None, sprompt_len=S, bits=bits)
    plan = call.plan()
    assert plan["chunks"] > 1 and plan["launches"] == 2
    units = B * Hkv * ((Hq // Hkv + plan["heads_per_unit"] - 1) // plan["heads_per_unit"])
    assert call.workspace_bytes >= units * T * plan["heads_per_unit"] * 4      # the logits are part of it
    out = call.run()
    torch.cuda.synchronize()
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                              c["kr"][:, :, :R] if R else None, c["vr"][:, :, :R] if R else None, S, bits)
    _check(to_np(out), want)
    # twice in a row on the same workspace: the counters start from zero again
    out2 = call.run()
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("single", [True, False], ids=["one-launch", "two-launches"])
@pytest.mark.parametrize("case", [(1, 32, 8, 20000, 40, 3, 1), (8, 32, 8, 12000, 0, 0, 1), (2, 32, 8, 12000, 33, 0, 2)],
                         ids=lambda c: "-".join(str(x) for x in c))
def test_decode_attn_chunked_launches_replayed_from_a_graph(ops, case, single, request):
    """The chunked step - two launches (counters cleared by the first, partials merged by the last workgroup of a
    unit in the second; logits through the workspace or recomputed), or one launch whose chunks exchange their
    min / max inside it (the records and counters it leaves are emptied by the merging workgroup, so a replay
    with the same epoch starts clean) - recorded into a HIP graph: every replay, with eager work and
    synchronisations in between, gives the bits of the eager call."""
    if not single:
        request.getfixturevalue("two_launches")
    B, Hq, Hkv, T, R, S, bits = case
    c = make_case(1, Hq, Hkv, 128, T, max(R, 1), bits, "bf16", seed=700 + T + bits, outlier_kind="student")
    g = {k: torch.cat([v] * B, 0) for k, v in case_to_gpu(c, "bf16").items()}
    call = ops.DecodeCall(g["q"], g["ck"], g["cv"], g["sk"], g["zk"], g["sv"], g["zv"], g["kr"] if R else None,
                          g["vr"] if R else None, sprompt_len=S, bits=bits)
    assert call.plan()["chunks"] > 1 and call.plan()["launches"] == (1 if single else 2)
    eager = call.run().clone()
    torch.cuda.synchronize()
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"],
                              c["kr"][:, :, :R] if R else None, c["vr"][:, :, :R] if R else None, S, bits)
    _check(to_np(eager[:1]), want)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        call.run()                                   # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            call.run()
    for i in range(4):
        call.out.zero_()
        other = call.run().clone() if i == 2 else None       # an eager call between two replays
        call.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(call.out, eager), i
        if other is not None:
            assert torch.equal(other, eager)
