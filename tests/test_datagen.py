"""The seeded generator: golden checksums, determinism, independence of streams, distributions."""
import json
import os
import zlib

import numpy as np

import oracle
from nnfusion_amd import datagen

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "datagen_checksums.json")))


def crc(a):
    return zlib.crc32(np.ascontiguousarray(a).view(np.uint8).tobytes()) & 0xFFFFFFFF


def test_config0_tensors_and_oracle_output_match_the_golden_fixture():
    a, wq, s = datagen.w4a16_case(0, 1, 4096, 4096)
    t = GOLDEN["tensors"]
    assert crc(a) == t["cfg0_A"]["crc32"] and crc(wq) == t["cfg0_Wq"]["crc32"] and crc(s) == t["cfg0_S"]["crc32"]
    assert [float(v) for v in a[0, :4]] == t["cfg0_A"]["head"]
    y = oracle.w4a16_gemm(a, wq, s)
    assert crc(y) == GOLDEN["oracle"]["cfg0_Y_f16"]["crc32"]


def test_w8a8_and_mlp_golden_fixture():
    a8, st, w8, sc = datagen.w8a8_case(0, 4, 256, 512)
    assert crc(a8) == GOLDEN["tensors"]["w8a8_A"]["crc32"] and crc(w8) == GOLDEN["tensors"]["w8a8_W"]["crc32"]
    assert crc(oracle.w8a8_acc(a8, w8)) == GOLDEN["oracle"]["w8a8_acc"]["crc32"]
    assert crc(oracle.w8a8_gemm(a8, st, w8, sc)) == GOLDEN["oracle"]["w8a8_Y_f16"]["crc32"]
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, 4, 256, 384)
    assert crc(gamma) == GOLDEN["tensors"]["mlp_gamma"]["crc32"]
    assert crc(oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)) == GOLDEN["oracle"]["mlp_out_f16"]["crc32"]


def test_prefix_property_and_stream_independence():
    big = datagen.normal_f16(3, datagen.S_ACT, (4096,))
    small = datagen.normal_f16(3, datagen.S_ACT, (100,))
    np.testing.assert_array_equal(big[:100].view(np.uint16), small.view(np.uint16))
    other_seed = datagen.normal_f16(4, datagen.S_ACT, (100,))
    other_stream = datagen.normal_f16(3, datagen.S_GAMMA, (100,))
    assert not np.array_equal(small, other_seed) and not np.array_equal(small, other_stream)


def test_distributions():
    n = 1 << 20
    x = datagen.normal_f16(0, 1, (n,)).astype(np.float64)
    assert abs(x.mean()) < 5e-3 and abs(x.std() - 1.0) < 5e-3
    assert abs((np.abs(x) > 1.959964).mean() - 0.05) < 2e-3
    wq = datagen.uniform_u4_packed(0, 2, 1024, 2048)
    nibbles = np.concatenate([(wq & 0xF).ravel(), (wq >> 4).ravel()])
    counts = np.bincount(nibbles, minlength=16) / nibbles.size
    assert np.all(np.abs(counts - 1 / 16) < 2e-3)
    s = datagen.uniform_f16(0, 3, (n,), 0.005, 0.02).astype(np.float64)
    assert s.min() >= 0.005 - 1e-5 and s.max() <= 0.02 + 1e-5 and abs(s.mean() - 0.0125) < 1e-4
    i8 = datagen.uniform_i8(0, 4, (n,))
    assert i8.min() == -127 and i8.max() == 127 and abs(i8.astype(np.float64).mean()) < 0.5
    f = datagen.uniform_f32(0, 5, (n,), 0.001, 0.01)
    assert f.min() >= 0.001 and f.max() < 0.01
    g = datagen.normal_f16(0, 6, (n,), 1.0, 0.1).astype(np.float64)
    assert abs(g.mean() - 1.0) < 1e-3 and abs(g.std() - 0.1) < 1e-3
