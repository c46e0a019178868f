"""The C restatement (timed CPU port) against the numpy oracle."""
import numpy as np
import pytest

from oracle import c_port
from oracle import cq_oracle as O
from tests.util import make_case, same_bits


@pytest.fixture(scope="module", autouse=True)
def _built():
    c_port.build()


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("S,R,masked", [(0, 0, False), (5, 17, False), (5, 17, True)])
def test_c_decode_attention_matches_numpy(bits, S, R, masked):
    c = make_case(2, 8, 2, 64, 130, R, bits, "bf16", seed=bits + R)
    mask = None
    if masked:
        mask = np.where(np.random.default_rng(0).random((2, 130 + R)) < 0.2, -1e4, 0.0).astype(np.float32)
    kr = c["kr"] if R else None
    vr = c["vr"] if R else None
    want = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], kr, vr, S, bits,
                              mask=mask, ftype=np.float64)
    got = c_port.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], kr, vr, S, bits,
                                  mask=mask)
    assert np.abs(got - want).max() < 2e-4


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("bits,clip", [(1, 0.5), (1, 0.3), (2, 1.0)])
def test_c_quantize_pack_matches_numpy(bits, clip, dtype):
    k, _ = O.synth_kv(2, 200, 3, 64, dtype, seed=2)
    codes, s, z = c_port.quantize_pack(k, bits, clip, dtype)
    oc, os_, oz = O.quantize_pack(k, bits, clip, dtype)
    assert same_bits(s, os_) and same_bits(z, oz) and np.array_equal(codes, oc)
