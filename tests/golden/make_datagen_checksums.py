#!/usr/bin/env python3
"""Writes tests/golden/datagen_checksums.json: CRC32 of the seeded tensors of the benchmark configurations
(as the in-repo generator makes them) and of the oracle's outputs for small cases.  The fixtures pin the
generator and the oracle against silent changes: inputs are regenerated from the seed, only checksums and
a few leading values are stored.   python tests/golden/make_datagen_checksums.py"""
import json
import os
import sys
import zlib

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from nnfusion_amd import datagen  # noqa: E402


def crc(a):
    return zlib.crc32(np.ascontiguousarray(a).view(np.uint8).tobytes()) & 0xFFFFFFFF


out = {"tensors": {}, "oracle": {}}
a, wq, s = datagen.w4a16_case(0, 1, 4096, 4096)
out["tensors"]["cfg0_A"] = {"crc32": crc(a), "head": [float(v) for v in a[0, :4]]}
out["tensors"]["cfg0_Wq"] = {"crc32": crc(wq), "head": [int(v) for v in wq[0, :4]]}
out["tensors"]["cfg0_S"] = {"crc32": crc(s), "head": [float(v) for v in s[0, :4]]}
y = oracle.w4a16_gemm(a, wq, s)
out["oracle"]["cfg0_Y_f16"] = {"crc32": crc(y), "head": [float(v) for v in y[0, :8]]}
a8, st, w8, sc = datagen.w8a8_case(0, 4, 256, 512)
out["tensors"]["w8a8_A"] = {"crc32": crc(a8)}
out["tensors"]["w8a8_W"] = {"crc32": crc(w8)}
out["tensors"]["w8a8_s_tok"] = {"crc32": crc(st), "head": [float(v) for v in st]}
out["oracle"]["w8a8_acc"] = {"crc32": crc(oracle.w8a8_acc(a8, w8)), "head": [int(v) for v in oracle.w8a8_acc(a8, w8)[0, :4]]}
out["oracle"]["w8a8_Y_f16"] = {"crc32": crc(oracle.w8a8_gemm(a8, st, w8, sc))}
x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, 4, 256, 384)
out["tensors"]["mlp_gamma"] = {"crc32": crc(gamma), "head": [float(v) for v in gamma[:4]]}
out["oracle"]["mlp_out_f16"] = {"crc32": crc(oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd))}
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "datagen_checksums.json")
json.dump(out, open(dst, "w"), indent=1)
print("wrote", dst)
