"""Randomised parity against the CPU oracle over the entry points (HIP through the C ABI): random M, N, K, block
parameters and optional fused parts, the residual in place or not, with and without synchronisation words, workspaces
sized by the library's own queries (what a caller that follows the header allocates).

Bars: W8A8 bit for bit (accumulators and fp16 output); floating point within 1e-2 * RMS of the oracle's
fp32-accumulated result (2e-2 with bias / residual added on top, whose own rounding counts; the SiLU-gate product
against the bound derived from that tolerance on gate and up).  A shape an entry point declines (status -2) is skipped.
"""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu


def _rms(x):
    return float(np.sqrt(np.mean(np.asarray(x, np.float64) ** 2)))


@pytest.mark.parametrize("seed", list(range(8)))
def test_random_products_match_the_oracle(gpu, seed):
    import torch

    from nnfusion_amd import ops

    rng = np.random.default_rng(1000 + seed)
    sync = ops.sync_flags(gpu)

    def t(a):
        return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(gpu)

    def pick_m():
        c = int(rng.integers(0, 5))
        return [1, int(rng.integers(2, 17)), int(rng.integers(17, 41)), int(rng.integers(41, 200)), int(rng.integers(200, 700))][c]

    failures = []
    for c in range(60):
        kind = int(rng.integers(0, 5))
        m = pick_m()
        use_sync = rng.random() < 0.5
        words = sync if use_sync else None
        desc = ""
        try:
            if kind == 0:  # W8A8: fp16 output and accumulators
                n = int(rng.integers(1, 2500)) if rng.random() < 0.5 else int(rng.integers(1, 400)) * 16
                k = int(rng.integers(1, 80)) * 128 if rng.random() < 0.6 else int(rng.choice([128, 256, 8192, 9216, 11008, 16384]))
                if m * n * k > 400 * 2000 * 4096:
                    n = 256
                desc = f"w8a8 M={m} N={n} K={k} sync={use_sync}"
                a8, s_tok, w8, s_ch = datagen.w8a8_case(c, m, n, k)
                y = ops.w8a8_gemm(t(a8), t(s_tok), t(w8), t(s_ch), sync=words).cpu().numpy()
                acc = ops.w8a8_gemm_acc(t(a8), t(w8), sync=words).cpu().numpy()
                ref_acc = oracle.w8a8_acc(a8, w8)
                ref = oracle.w8a8_epilogue(ref_acc, s_tok, s_ch)
                ok = np.array_equal(acc, ref_acc) and np.array_equal(y.view(np.uint16), ref.view(np.uint16))
                err = 0.0 if ok else 1.0
            elif kind == 1:  # MLP block, fp16 x int4
                h = int(rng.integers(2, 24)) * 128
                i = int(rng.integers(2, 48)) * 128
                if rng.random() < 0.3:
                    h, i = int(rng.choice([1024, 2048, 4096])), int(rng.choice([2816, 5632, 8704, 11008]))
                if m > 300:
                    m = int(rng.integers(41, 300))
                in_place = rng.random() < 0.3
                desc = f"mlp M={m} H={h} I={i} sync={use_sync} in_place={in_place}"
                x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(c, m, h, i)
                tx = t(x)
                out = ops.fused_mlp_w4a16(tx, t(gamma), t(wgu), t(sgu), t(wd), t(sd), sync=words,
                                          out=tx if in_place else None).cpu().numpy()
                ref = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd)
                err = float(np.abs(out.astype(np.float32) - ref.astype(np.float32)).max()) / max(_rms(ref), 1e-6)
                ok = err <= 1e-2
            elif kind == 2:  # other block parameters
                bits = int(rng.choice([4, 8, 8]))
                group = int(rng.choice([32, 64, 128]))
                zpt = bool(rng.integers(0, 2))
                n = int(rng.integers(1, 3000)) if rng.random() < 0.5 else int(rng.integers(1, 300)) * 16
                k = int(rng.integers(1, 90)) * 128 if rng.random() < 0.5 else int(rng.choice([2048, 4096, 8192, 11008, 5120, 1024, 16384]))
                if rng.random() < 0.1:
                    k = int(rng.integers(1, 40)) * group
                if m * n * k > 400 * 2000 * 4096:
                    n = 256
                desc = f"wna16 M={m} N={n} K={k} bits={bits} group={group} zero-point tensor={zpt} sync={use_sync}"
                a, wq, s, z = datagen.wna16_case(c, m, n, k, bits, group, zpt)
                zp = int(rng.integers(0, 1 << bits))
                y = ops.wna16_gemm(t(a), t(wq), t(s), bits=bits, group=group, zp=zp, zero_points=t(z) if zpt else None,
                                   sync=words).cpu().numpy()
                ref = oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=z if zpt else None, f32_out=True)
                err = float(np.abs(y.astype(np.float32) - ref).max()) / max(_rms(ref), 1e-6)
                ok = err <= 1e-2
            elif kind == 3:  # fp16 x int4 with any of the optional parts
                n = int(rng.integers(1, 3000)) if rng.random() < 0.5 else int(rng.integers(1, 300)) * 16
                k = int(rng.integers(1, 96)) * 128 if rng.random() < 0.6 else int(rng.choice([1024, 2048, 4096, 8192, 11008]))
                if m * n * k > 400 * 2000 * 4096:
                    n = 256
                a, wq, s = datagen.w4a16_case(c, m, n, k)
                gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if rng.random() < 0.5 else None
                bias = rng.standard_normal(n).astype(np.float16) if rng.random() < 0.5 else None
                resid = rng.standard_normal((m, n)).astype(np.float16) if rng.random() < 0.5 else None
                in_place = resid is not None and rng.random() < 0.4
                desc = (f"fused M={m} N={n} K={k} gamma={gamma is not None} bias={bias is not None} "
                        f"residual={resid is not None} in_place={in_place} sync={use_sync}")
                tr = t(resid)
                y = ops.w4a16_gemm_fused(t(a), t(wq), t(s), rms_gamma=t(gamma), bias=t(bias), residual=tr,
                                         out=tr if in_place else None, sync=words).cpu().numpy()
                xin = oracle.rmsnorm_f16(a, gamma) if gamma is not None else a
                ref = oracle.w4a16_gemm(xin, wq, s, f32_out=True)
                scale = max(_rms(ref), 1e-6)
                if bias is not None:
                    ref = ref + bias.astype(np.float32)[None]
                if resid is not None:
                    ref = ref + resid.astype(np.float32)
                err = float(np.abs(y.astype(np.float32) - ref).max()) / scale
                ok = err <= 2e-2
            else:  # SiLU-gate product
                n = int(rng.integers(1, 120)) * 16 if rng.random() < 0.7 else int(rng.integers(1, 1500))
                k = int(rng.integers(1, 64)) * 128 if rng.random() < 0.6 else int(rng.choice([1024, 2048, 4096, 8192]))
                if m * n * k > 200 * 2000 * 4096:
                    n = 128
                a, wq, s = datagen.w4a16_case(c, m, 2 * n, k)
                gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16) if rng.random() < 0.5 else None
                desc = f"gate M={m} N={n} K={k} gamma={gamma is not None} sync={use_sync}"
                y = ops.w4a16_gemm_fused(t(a), t(wq), t(s), rms_gamma=t(gamma), act=1, sync=words).cpu().numpy()
                xin = oracle.rmsnorm_f16(a, gamma) if gamma is not None else a
                gu = oracle.w4a16_gemm(xin, wq, s)
                g, u = np.ascontiguousarray(gu[:, :n]), np.ascontiguousarray(gu[:, n:])
                ref = oracle.silu_mul_f16(g, u).astype(np.float32)
                delta = 1e-2 * _rms(gu)
                g32, u32 = g.astype(np.float32), u.astype(np.float32)
                silu = g32 / (1.0 + np.exp(-g32))
                bound = delta * (1.1 * np.abs(u32) + np.abs(silu)) + np.abs(ref) * 2.0 ** -10 + 1e-6
                e = np.abs(y.astype(np.float32) - ref)
                ok = bool(np.all(e <= bound))
                err = float((e - bound).max())
            torch.cuda.synchronize()
            if int(sync.count_nonzero()) != 0:
                ok, err = False, "synchronisation words left non-zero"
                sync.zero_()
        except ops.NnfError as e:
            if e.status == -2:  # a shape this entry point declines
                continue
            ok, err = False, str(e)
        if not ok:
            failures.append((desc, err))
    assert not failures, failures
