"""Reader of the record format written by ck_tile_host_golden.cpp."""
import os
import struct

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
_NP = {0: np.float32, 3: np.uint16, 4: np.uint16, 6: np.int32}
_TORCH16 = {3: torch.float16, 4: torch.bfloat16}


def load(name="ck_tile_host_golden.bin"):
    out = {}
    with open(os.path.join(HERE, name), "rb") as f:
        data = f.read()
    at = 0
    while at < len(data):
        (nl,) = struct.unpack_from("<I", data, at)
        at += 4
        key = data[at:at + nl].decode()
        at += nl
        code, nd = struct.unpack_from("<II", data, at)
        at += 8
        dims = struct.unpack_from("<" + "I" * nd, data, at)
        at += 4 * nd
        n = int(np.prod(dims))
        arr = np.frombuffer(data, dtype=_NP[code], count=n, offset=at).reshape(dims).copy()
        at += arr.nbytes
        t = torch.from_numpy(arr.view(np.int16) if code in _TORCH16 else arr)
        out[key] = t.view(_TORCH16[code]) if code in _TORCH16 else t
    return out
