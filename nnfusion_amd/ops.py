"""Thin torch-tensor front over the C ABI (device pointers + the current HIP stream).

torch is used for device memory and streams only; every computation happens in
libnnf_hip_kernels.so.  A non-zero status from the library raises NnfError (the emitted host
wrappers of the codegen path throw std::runtime_error in the same situation).
"""
import ctypes

import torch

from . import _lib


class NnfPlan(ctypes.Structure):
    """struct nnf_plan of the C header: what a kernel-selection candidate fixes about the tile GEMM, and the
    synchronisation words that make the fp16 x int4 tile GEMM a single launch."""
    _fields_ = [("tile_rows", ctypes.c_int), ("k_parts", ctypes.c_int), ("tile_cols", ctypes.c_int),
                ("sync_flags", ctypes.c_void_p), ("sync_flags_bytes", ctypes.c_size_t), ("spin_limit", ctypes.c_int)]


SYNC_FLAGS_BYTES = 64 << 10  # NNF_SYNC_FLAGS_BYTES


def sync_flags(device):
    """A zeroed buffer for nnf_plan::sync_flags (cleared once here; every call leaves it zero again)."""
    return torch.zeros(SYNC_FLAGS_BYTES, dtype=torch.uint8, device=device)


def _plan_arg(plan, sync=None, spin_limit=0):
    """None, an NnfPlan or a (tile_rows, k_parts[, tile_cols]) tuple, plus an optional sync_flags tensor
    -> (object to keep alive, pointer argument)."""
    if plan is None and sync is None:
        return None, None
    if not isinstance(plan, NnfPlan):
        t = tuple(plan) if plan is not None else (0, 0, 0)
        plan = NnfPlan(int(t[0]), int(t[1]), int(t[2]) if len(t) > 2 else 0, None, 0, 0)
    if sync is not None:
        plan.sync_flags = sync.data_ptr()
        plan.sync_flags_bytes = sync.numel() * sync.element_size()
        plan.spin_limit = int(spin_limit)
    return plan, ctypes.cast(ctypes.pointer(plan), ctypes.c_void_p)


class NnfError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = _lib.kernels().nnf_status_string(status).decode()
        super().__init__(f"{where}: status {status} ({msg})")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check(status, where):
    if status != 0:
        raise NnfError(status, where)


def _ws(nbytes, device):
    # the library never allocates; the caller (here: the test/bench harness) owns the workspace
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def _p(t):
    return 0 if t is None else t.data_ptr()


def w4a16_gemm(a, wq, scales, group=128, zp=8, out=None, workspace=None):
    """Y[M,N] = A[M,K] . ((Wq - zp) * scales)^T ; a fp16 [M,K], wq u8 [N,K/2], scales fp16 [N,K/group]."""
    lib = _lib.kernels()
    m, k = a.shape
    n = wq.shape[0]
    assert a.dtype == torch.float16 and wq.dtype == torch.uint8 and scales.dtype == torch.float16
    assert a.is_contiguous() and wq.is_contiguous() and scales.is_contiguous()
    assert wq.shape[1] * 2 == k and tuple(scales.shape) == (n, k // group)
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    need = lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, group)
    if workspace is None:
        workspace = _ws(need, a.device)
    _check(lib.nnf_w4a16_gemm(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(),
                              m, n, k, group, zp, workspace.data_ptr(), workspace.numel()), "nnf_w4a16_gemm")
    return out


class NnfQuant(ctypes.Structure):
    """struct nnf_quant of the C header: the block parameters of the weights."""
    _fields_ = [("bits", ctypes.c_int), ("group", ctypes.c_int), ("zero_point", ctypes.c_int),
                ("zero_points", ctypes.c_void_p)]


def _quant_arg(bits, group, zp, zero_points):
    q = NnfQuant(int(bits), int(group), int(zp), _p(zero_points))
    return q, ctypes.cast(ctypes.pointer(q), ctypes.c_void_p)


def wna16_supported(m, n, k, bits, group, zp=8):
    _, qp = _quant_arg(bits, group, zp, None)
    return bool(_lib.kernels().nnf_wna16_supported(m, n, k, qp))


def wna16_workspace_bytes(m, n, k, bits, group, zero_points=None):
    """Bytes of workspace nnf_wna16_gemm wants for this product (0: none)."""
    _, qp = _quant_arg(bits, group, 0, zero_points)
    return int(_lib.kernels().nnf_wna16_gemm_workspace_bytes(m, n, k, qp))


def wna16_gemm(a, wq, scales, bits=4, group=128, zp=8, zero_points=None, out=None, workspace=None, sync=None, spin_limit=0):
    """Y[M,N] = A[M,K] . ((Wq - z) * scales)^T with 4- or 8-bit weights (wq u8 [N, K*bits/8]), groups of 32 / 64 / 128
    and either a scalar zero point or zero_points u8 [N, ceil(K/group*bits/8)] (4-bit: two per byte, even group low).
    sync: synchronisation words (sync_flags()) for the one-launch form of the tile GEMM: nnf_wna16_gemm_planned."""
    lib = _lib.kernels()
    m, k = a.shape
    n = wq.shape[0]
    assert a.dtype == torch.float16 and wq.dtype == torch.uint8 and scales.dtype == torch.float16
    assert a.is_contiguous() and wq.is_contiguous() and scales.is_contiguous()
    assert wq.shape[1] * 8 == k * bits and tuple(scales.shape) == (n, k // group)
    if zero_points is not None:
        assert zero_points.dtype == torch.uint8 and zero_points.is_contiguous()
        assert tuple(zero_points.shape) == (n, (k // group * bits + 7) // 8)
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    keep, qp = _quant_arg(bits, group, zp, zero_points)
    if workspace is None:
        workspace = _ws(lib.nnf_wna16_gemm_workspace_bytes(m, n, k, qp), a.device)
    if sync is not None:
        keep_plan, plan_ptr = _plan_arg(None, sync, spin_limit)
        _check(lib.nnf_wna16_gemm_planned(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(), m, n, k, qp,
                                          plan_ptr, workspace.data_ptr(), workspace.numel()), "nnf_wna16_gemm_planned")
        return out
    _check(lib.nnf_wna16_gemm(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(), m, n, k, qp,
                              workspace.data_ptr(), workspace.numel()), "nnf_wna16_gemm")
    return out


VARIANTS = {"auto": 0, "gemv_valu": 1, "gemv_mfma": 2, "gemm_mfma": 3, "gemv_rows": 4}


def w4a16_variant_supported(m, n, k, variant, group=128):
    return bool(_lib.kernels().nnf_w4a16_variant_supported(m, n, k, group, VARIANTS[variant]))


def w4a16_gemm_variant(a, wq, scales, variant, plan=None, group=128, zp=8, out=None, workspace=None, sync=None,
                       spin_limit=0):
    """As w4a16_gemm through one kernel variant (a key of VARIANTS) and, for the tile GEMM, a plan (tile_rows,
    k_parts); raises NnfError with status -2 when the variant cannot serve the shape."""
    lib = _lib.kernels()
    m, k = a.shape
    n = wq.shape[0]
    v = VARIANTS[variant]
    assert a.dtype == torch.float16 and wq.dtype == torch.uint8 and scales.dtype == torch.float16
    assert a.is_contiguous() and wq.is_contiguous() and scales.is_contiguous()
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    keep, plan_ptr = _plan_arg(plan, sync, spin_limit)
    if workspace is None:
        workspace = _ws(lib.nnf_w4a16_gemm_variant_workspace_bytes(m, n, k, group, v, plan_ptr), a.device)
    _check(lib.nnf_w4a16_gemm_variant(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(),
                                      m, n, k, group, zp, v, plan_ptr, workspace.data_ptr(), workspace.numel()),
           "nnf_w4a16_gemm_variant")
    return out


def w4a16_gemm_fused(a, wq, scales, group=128, zp=8, rms_gamma=None, rms_eps=1e-6, bias=None, residual=None,
                     act=0, out=None, workspace=None, variant="auto", plan=None, sync=None, spin_limit=0):
    """GEMM with the fused RMSNorm prologue / bias, residual, SiLU-gate epilogues (see the C header); variant
    "gemm_mfma" and a plan (tile_rows, k_parts) go through nnf_w4a16_gemm_fused_variant."""
    lib = _lib.kernels()
    m, k = a.shape
    n = wq.shape[0] // (2 if act == 1 else 1)
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    need = lib.nnf_w4a16_gemm_fused_workspace_bytes(m, n, k, group, act)
    if variant != "auto" or plan is not None or sync is not None:
        keep, plan_ptr = _plan_arg(plan, sync, spin_limit)
        v = VARIANTS[variant]
        if workspace is None:
            workspace = _ws(need + lib.nnf_w4a16_gemm_variant_workspace_bytes(m, wq.shape[0], k, group, v, plan_ptr),
                            a.device)
        _check(lib.nnf_w4a16_gemm_fused_variant(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(),
                                                out.data_ptr(), m, n, k, group, zp, _p(rms_gamma), float(rms_eps),
                                                _p(bias), _p(residual), int(act), v, plan_ptr, workspace.data_ptr(),
                                                workspace.numel()), "nnf_w4a16_gemm_fused_variant")
        return out
    if workspace is None:
        workspace = _ws(need, a.device)
    _check(lib.nnf_w4a16_gemm_fused(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(),
                                    m, n, k, group, zp, _p(rms_gamma), float(rms_eps), _p(bias), _p(residual),
                                    int(act), workspace.data_ptr(), workspace.numel()), "nnf_w4a16_gemm_fused")
    return out


W8A8_VARIANTS = {"auto": 0, "gemv_mfma": 1, "gemm_mfma": 2, "gemv_rows": 3}


def w8a8_variant_supported(m, n, k, variant):
    return bool(_lib.kernels().nnf_w8a8_variant_supported(m, n, k, W8A8_VARIANTS[variant]))


def _w8a8_variant(a, s_tok, w, s_ch, y, acc, variant, plan, workspace, sync=None):
    lib = _lib.kernels()
    m, k = a.shape
    n = w.shape[0]
    v = W8A8_VARIANTS[variant]
    keep, plan_ptr = _plan_arg(plan, sync)
    if workspace is None:
        workspace = _ws(lib.nnf_w8a8_gemm_variant_workspace_bytes(m, n, k, v, plan_ptr), a.device)
    _check(lib.nnf_w8a8_gemm_variant(_stream(), a.data_ptr(), _p(s_tok), w.data_ptr(), _p(s_ch), _p(y), _p(acc), m, n, k,
                                     v, plan_ptr, workspace.data_ptr(), workspace.numel()), "nnf_w8a8_gemm_variant")


def w8a8_gemm(a, s_tok, w, s_ch, out=None, workspace=None, variant="auto", plan=None, sync=None):
    """Y fp16 [M,N] = fp16((float)(A . W^T) * s_tok[m] * s_ch[n]) ; a i8 [M,K], w i8 [N,K].  A variant (a key of
    W8A8_VARIANTS), a plan (tile_rows, k_parts) or `sync` (see sync_flags: a few rows with a long K then run over
    two ranges of K in one launch) goes through nnf_w8a8_gemm_variant."""
    lib = _lib.kernels()
    m, k = a.shape
    n = w.shape[0]
    assert a.dtype == torch.int8 and w.dtype == torch.int8
    assert s_tok.dtype == torch.float32 and s_ch.dtype == torch.float32
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    if variant != "auto" or plan is not None or sync is not None:
        _w8a8_variant(a, s_tok, w, s_ch, out, None, variant, plan, workspace, sync)
        return out
    need = lib.nnf_w8a8_gemm_workspace_bytes(m, n, k)
    if workspace is None:
        workspace = _ws(need, a.device)
    _check(lib.nnf_w8a8_gemm(_stream(), a.data_ptr(), s_tok.data_ptr(), w.data_ptr(), s_ch.data_ptr(),
                             out.data_ptr(), m, n, k, workspace.data_ptr(), workspace.numel()), "nnf_w8a8_gemm")
    return out


def w8a8_gemm_acc(a, w, out=None, workspace=None, variant="auto", plan=None, sync=None):
    """acc i32 [M,N] = A . W^T, exact."""
    lib = _lib.kernels()
    m, k = a.shape
    n = w.shape[0]
    assert a.dtype == torch.int8 and w.dtype == torch.int8
    if out is None:
        out = torch.empty((m, n), dtype=torch.int32, device=a.device)
    if variant != "auto" or plan is not None or sync is not None:
        _w8a8_variant(a, None, w, None, None, out, variant, plan, workspace, sync)
        return out
    need = lib.nnf_w8a8_gemm_workspace_bytes(m, n, k)
    if workspace is None:
        workspace = _ws(need, a.device)
    _check(lib.nnf_w8a8_gemm_acc(_stream(), a.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k,
                                 workspace.data_ptr(), workspace.numel()), "nnf_w8a8_gemm_acc")
    return out


def fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd, eps=1e-6, group=128, zp=8, out=None, workspace=None, sync=None,
                    spin_limit=0, gate_up_plan=None, down_plan=None):
    """out = x + Wd . (SiLU(Wg . n) * (Wu . n)), n = RMSNorm(x, gamma, eps).  `sync` (see sync_flags) or a plan for
    either product goes through nnf_fused_mlp_w4a16_planned."""
    lib = _lib.kernels()
    m, h = x.shape
    i = wgu.shape[0] // 2
    if out is None:
        out = torch.empty((m, h), dtype=torch.float16, device=x.device)
    need = lib.nnf_fused_mlp_w4a16_workspace_bytes(m, h, i, group)
    if sync is not None or gate_up_plan is not None or down_plan is not None:
        keep_a, plan_a = _plan_arg(gate_up_plan, sync, spin_limit)
        keep_b, plan_b = _plan_arg(down_plan, sync, spin_limit)
        if workspace is None:
            v = VARIANTS["gemm_mfma"]
            extra = (lib.nnf_w4a16_gemm_variant_workspace_bytes(m, 2 * i, h, group, v, plan_a) if gate_up_plan is not None else 0) + \
                    (lib.nnf_w4a16_gemm_variant_workspace_bytes(m, h, i, group, v, plan_b) if down_plan is not None else 0)
            workspace = _ws(need + extra, x.device)
        _check(lib.nnf_fused_mlp_w4a16_planned(_stream(), x.data_ptr(), gamma.data_ptr(), float(eps), wgu.data_ptr(),
                                               sgu.data_ptr(), wd.data_ptr(), sd.data_ptr(), out.data_ptr(), m, h, i, group,
                                               zp, plan_a, plan_b, workspace.data_ptr(), workspace.numel()),
               "nnf_fused_mlp_w4a16_planned")
        return out
    if workspace is None:
        workspace = _ws(need, x.device)
    _check(lib.nnf_fused_mlp_w4a16(_stream(), x.data_ptr(), gamma.data_ptr(), float(eps), wgu.data_ptr(),
                                   sgu.data_ptr(), wd.data_ptr(), sd.data_ptr(), out.data_ptr(), m, h, i, group, zp,
                                   workspace.data_ptr(), workspace.numel()), "nnf_fused_mlp_w4a16")
    return out


EW_OPS = {"add": 0, "multiply": 1, "sigmoid": 2, "swish": 3}


def elementwise(op, a, b=None, out=None):
    """y = op(a, b) over fp16 tensors (b of a's shape, or a row [cols] broadcast over a's leading axes)."""
    lib = _lib.kernels()
    assert a.dtype == torch.float16 and a.is_contiguous()
    cols = a.shape[-1]
    rows = a.numel() // cols
    b_is_row = 0
    if b is not None:
        assert b.dtype == torch.float16 and b.is_contiguous()
        b_is_row = 1 if (b.dim() == 1 and a.dim() > 1) else 0
        assert b_is_row or b.shape == a.shape
    if out is None:
        out = torch.empty_like(a)
    _check(lib.nnf_elementwise_f16(_stream(), EW_OPS[op], a.data_ptr(), _p(b), out.data_ptr(), rows, cols, b_is_row),
           "nnf_elementwise_f16")
    return out


def rms_norm(x, gamma, eps=1e-6, out=None):
    lib = _lib.kernels()
    m, k = x.shape
    if out is None:
        out = torch.empty_like(x)
    _check(lib.nnf_rms_norm_f16(_stream(), x.data_ptr(), gamma.data_ptr(), out.data_ptr(), m, k, float(eps)), "nnf_rms_norm_f16")
    return out


def dequantize(wq, scales, bits=4, group=128, zp=8, zero_points=None, out=None):
    """W fp16 [N, K] = (q - z) * s per block of `group` weights."""
    lib = _lib.kernels()
    n = wq.shape[0]
    k = wq.shape[1] * 8 // bits
    if out is None:
        out = torch.empty((n, k), dtype=torch.float16, device=wq.device)
    keep, qp = _quant_arg(bits, group, zp, zero_points)
    _check(lib.nnf_dequantize_f16(_stream(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(), n, k, qp), "nnf_dequantize_f16")
    return out


def wna16_gemm_fused(a, wq, scales, bits=4, group=128, zp=8, zero_points=None, rms_gamma=None, rms_eps=1e-6, bias=None,
                     residual=None, act=0, out=None, workspace=None):
    """nnf_wna16_gemm_fused: the fused product for every block parameter."""
    lib = _lib.kernels()
    m, k = a.shape
    n = wq.shape[0] // (2 if act == 1 else 1)
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    keep, qp = _quant_arg(bits, group, zp, zero_points)
    if workspace is None:
        workspace = _ws(lib.nnf_wna16_gemm_fused_workspace_bytes(m, n, k, qp, int(act)), a.device)
    _check(lib.nnf_wna16_gemm_fused(_stream(), a.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(), m, n, k, qp,
                                    _p(rms_gamma), float(rms_eps), _p(bias), _p(residual), int(act), workspace.data_ptr(),
                                    workspace.numel()), "nnf_wna16_gemm_fused")
    return out


def fused_mlp_wna16(x, gamma, wgu, sgu, wd, sd, bits=4, group=128, zp=8, zgu=None, zd=None, eps=1e-6, out=None, workspace=None):
    """The MLP block for every block parameter (zgu / zd: zero-point tensors of the two weight matrices, or None)."""
    lib = _lib.kernels()
    m, h = x.shape
    i = wgu.shape[0] // 2
    if out is None:
        out = torch.empty((m, h), dtype=torch.float16, device=x.device)
    keep_a, qa = _quant_arg(bits, group, zp, zgu)
    keep_b, qb = _quant_arg(bits, group, zp, zd)
    if workspace is None:
        workspace = _ws(lib.nnf_fused_mlp_wna16_workspace_bytes(m, h, i, qa, qb), x.device)
    _check(lib.nnf_fused_mlp_wna16(_stream(), x.data_ptr(), gamma.data_ptr(), float(eps), wgu.data_ptr(), sgu.data_ptr(),
                                   wd.data_ptr(), sd.data_ptr(), out.data_ptr(), m, h, i, qa, qb, workspace.data_ptr(),
                                   workspace.numel()), "nnf_fused_mlp_wna16")
    return out
