"""ctypes loader of the C restatement (oracle/cq_oracle.c).  Test
infrastructure only; see that file's header."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(_HERE, "libcq_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "libcq_oracle.so"], check=True, stdout=subprocess.DEVNULL)
    return LIB


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def decode_attention(q, ck, cv, ks, kz, vs, vz, kres, vres, S, bits, off_max=-3.0, off_min=0.0,
                     calibrate=True, mask=None):
    lib = load()
    q = _f(q)
    B, Hq, D = q.shape
    ck, cv = np.ascontiguousarray(ck), np.ascontiguousarray(cv)
    Hkv, T = ck.shape[1], ck.shape[2]
    kres, vres = _f(kres), _f(vres)
    R = 0 if kres is None else kres.shape[2]
    ks, kz, vs, vz, mask = _f(ks), _f(kz), _f(vs), _f(vz), _f(mask)
    out = np.empty((B, Hq, D), np.float32)
    lib.cqo_decode_attention(_p(q), _p(ck), _p(cv), _p(ks), _p(kz), _p(vs), _p(vz), _p(kres), _p(vres), _p(mask),
                             B, Hq, Hkv, D, T, R, int(S), int(bits), int(calibrate), C.c_float(off_max),
                             C.c_float(off_min), _p(out))
    return out


def quantize_pack(x, bits, clip, dtype):
    lib = load()
    x = _f(x)
    B, T, H, D = x.shape
    codes = np.empty((B, H, T, D * bits // 8), np.uint8)
    s = np.empty((B, H, D), np.float32)
    z = np.empty((B, H, D), np.float32)
    lib.cqo_quantize_pack(_p(x), B, T, H, D, int(bits), C.c_float(clip), {"bf16": 0, "fp16": 1, "fp32": 2}[dtype],
                          _p(codes), _p(s), _p(z))
    return codes, s, z
