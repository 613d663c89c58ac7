"""numpy-level access to the CPU oracle (oracle/libcf_oracle.so) and, when built,
to the reference's own E4M3 header (oracle/_ref/libcf_ref_e4m3.so).

Test infrastructure: the oracle is the checker, never the thing measured or shipped.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_DIR = ROOT / "oracle"
_SO = ORACLE_DIR / "libcf_oracle.so"
_REF_SO = ORACLE_DIR / "_ref" / "libcf_ref_e4m3.so"

E4M3_MAX = 448.0
E5M2_MAX = 57344.0
THREADS = min(16, os.cpu_count() or 1)


def _load():
    if not _SO.exists():
        subprocess.run(["make", "-C", str(ORACLE_DIR), "libcf_oracle.so"], check=True, capture_output=True)
    return ctypes.CDLL(str(_SO))


_o = _load()
_o.orc_expf.restype = ctypes.c_float
_o.orc_expf.argtypes = [ctypes.c_float]

c_f = ctypes.c_float
c_i = ctypes.c_int
c_sz = ctypes.c_size_t
c_d = ctypes.c_double
P = ctypes.c_void_p


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(P)


def _f32(v):
    return np.array([v], dtype=np.float32)


def _call(name, *args):
    fn = getattr(_o, name)
    conv = []
    for a in args:
        if isinstance(a, np.ndarray) or a is None:
            conv.append(_p(a))
        else:
            conv.append(a)
    fn.restype = None
    fn(*conv)


def ref_available() -> bool:
    return _REF_SO.exists()


def ref_lib():
    return ctypes.CDLL(str(_REF_SO))


# ---- scalar / vector conversions ---------------------------------------------
def bf16_from_f32(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    _call("orc_bf16_from_f32_n", x, out, c_sz(x.size))
    return out


def bf16_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, np.float32)
    _call("orc_bf16_to_f32_n", b, out, c_sz(b.size))
    return out


def e4m3_pack(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    fin = np.empty(x.shape, np.uint8)
    _call("orc_e4m3_pack_n", x, out, fin, c_sz(x.size))
    return out, fin.astype(bool)


def e4m3_satfinite(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    _call("orc_e4m3_satfinite_n", x, out, c_sz(x.size))
    return out


def e5m2_satfinite(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    _call("orc_e5m2_satfinite_n", x, out, c_sz(x.size))
    return out


def e4m3_unpack(b):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape, np.float32)
    _call("orc_e4m3_unpack_n", b, out, c_sz(b.size))
    return out


def e5m2_unpack(b):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape, np.float32)
    _call("orc_e5m2_unpack_n", b, out, c_sz(b.size))
    return out


def expf(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.float32)
    _call("orc_expf_n", x, out, c_sz(x.size))
    return out


# ---- per-tensor quantize family ------------------------------------------------
def amax_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    a = _f32(-1.0)
    _call("orc_amax_bf16", x, c_sz(x.size), a)
    return a[0]


def amax_f32(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = _f32(-1.0)
    _call("orc_amax_f32", x, c_sz(x.size), a)
    return a[0]


def scale_from_amax(amax, fp8_max):
    s, d = _f32(0), _f32(0)
    _call("orc_scale_from_amax", _f32(amax), c_f(fp8_max), s, d)
    return s[0], d[0]


def quantize_e4m3(x, scale):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, np.uint8)
    _call("orc_quantize_e4m3", x, out, _f32(scale), c_sz(x.size))
    return out


def quantize_e5m2(x, scale):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, np.uint8)
    _call("orc_quantize_e5m2", x, out, _f32(scale), c_sz(x.size))
    return out


def quantize_f32_e4m3(x, scale):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    _call("orc_quantize_f32_e4m3", x, out, _f32(scale), c_sz(x.size))
    return out


def quantize_record(x, scale, amax_in, e5m2=False):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, np.uint8)
    a = _f32(amax_in)
    _call("orc_quantize_e5m2_record" if e5m2 else "orc_quantize_e4m3_record", x, out, _f32(scale), a, c_sz(x.size))
    return out, a[0]


class DelayedState:
    """Host mirror of one delayed-scaling slot's device scalars."""

    def __init__(self, history_len, cursor=0, count=0):
        self.history = np.zeros(max(history_len, 1), np.float32)
        self.history_len = history_len
        self.cursor = np.array([cursor], np.int32)
        self.count = np.array([count], np.int32)
        self.scale = _f32(0)
        self.descale = _f32(0)

    def update(self, amax, fp8_max):
        _call("orc_update_delayed_scale", _f32(amax), c_f(fp8_max), self.scale, self.descale,
              self.history, c_i(self.history_len), self.cursor, self.count)


def quantize_transpose_e4m3(w, scale):
    w = np.ascontiguousarray(w, dtype=np.uint16)
    K, N = w.shape
    out = np.empty((N, K), np.uint8)
    _call("orc_quantize_transpose_e4m3", w, out, _f32(scale), c_i(K), c_i(N))
    return out


def quant_and_transpose_e4m3(x, scale):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    K, N = x.shape
    act8 = np.empty((K, N), np.uint8)
    snap = np.empty((N, K), np.uint8)
    _call("orc_quant_and_transpose_e4m3", x, act8, snap, _f32(scale), c_i(K), c_i(N))
    return act8, snap


def transpose_u8(x):
    x = np.ascontiguousarray(x, dtype=np.uint8)
    r, c = x.shape
    out = np.empty((c, r), np.uint8)
    _call("orc_transpose_u8", x, out, c_i(r), c_i(c))
    return out


def clip_probe(amax, scale, fp8_max, stats):
    stats = np.ascontiguousarray(stats, dtype=np.float32).copy()
    _call("orc_clip_probe", _f32(amax), _f32(scale), c_f(fp8_max), stats)
    return stats


def elem_clip_count(x, scale, fp8_max, out):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.ascontiguousarray(out, dtype=np.float32).copy()
    _call("orc_elem_clip_count", x, _f32(scale), c_f(fp8_max), c_sz(x.size), out)
    return out


def pack_raw(x, dequant=False):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, np.uint8)
    amax, scale, desc = _f32(0), _f32(0), _f32(0)
    bad = np.zeros(1, np.int32)
    if dequant:
        deq = np.empty(x.shape, np.uint16)
        _call("orc_pack_bf16_e4m3_raw_and_dequant", x, out, deq, amax, scale, desc, bad, c_sz(x.size))
        return out, deq, amax[0], scale[0], desc[0], int(bad[0])
    _call("orc_pack_bf16_e4m3_raw", x, out, amax, scale, desc, bad, c_sz(x.size))
    return out, amax[0], scale[0], desc[0], int(bad[0])


def unpack_raw(b, descale):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape, np.uint16)
    _call("orc_unpack_e4m3_raw_bf16", b, _f32(descale), out, c_sz(b.size))
    return out


def calib_minmax_update(amax, cmin, cmax):
    mn, mx = _f32(cmin), _f32(cmax)
    _call("orc_calib_minmax_update", _f32(amax), mn, mx)
    return mn[0], mx[0]


# ---- scale groups ---------------------------------------------------------------
def quantize_rows(x, e5m2=False):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    rows, K = x.shape
    out = np.empty((rows, K), np.uint8)
    s = np.empty(rows, np.float32)
    d = np.empty(rows, np.float32)
    _call("orc_quantize_rows", x, c_i(rows), c_i(K), c_i(int(e5m2)), out, s, d)
    return out, s, d


def quantize_block_1x128(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    rows, K = x.shape
    kb = (K + 127) // 128
    out = np.empty((rows, K), np.uint8)
    s = np.empty((rows, kb), np.float32)
    d = np.empty((rows, kb), np.float32)
    _call("orc_quantize_block_1x128", x, c_i(rows), c_i(K), out, s, d)
    return out, s, d


def quantize_block_128x128(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    rows, K = x.shape
    kb, rb = (K + 127) // 128, (rows + 127) // 128
    out = np.empty((rows, K), np.uint8)
    s = np.empty((rb, kb), np.float32)
    d = np.empty((rb, kb), np.float32)
    _call("orc_quantize_block_128x128", x, c_i(rows), c_i(K), out, s, d)
    return out, s, d


# ---- elementwise ------------------------------------------------------------------
def swiglu_forward(gate, up):
    gate = np.ascontiguousarray(gate, dtype=np.uint16)
    up = np.ascontiguousarray(up, dtype=np.uint16)
    out = np.empty(gate.shape, np.uint16)
    _call("orc_swiglu_forward", gate, up, out, c_i(gate.size))
    return out


def bias_add_strided(inout, bias, rows, cols, row_stride, base):
    inout = np.ascontiguousarray(inout, dtype=np.uint16).copy()
    _call("orc_bias_add_strided_bf16", inout, np.ascontiguousarray(bias, dtype=np.uint16),
          c_i(rows), c_i(cols), c_i(row_stride), c_i(base))
    return inout


def swiglu_backward(grad_out, gate, up):
    grad_out = np.ascontiguousarray(grad_out, dtype=np.uint16)
    gate = np.ascontiguousarray(gate, dtype=np.uint16)
    up = np.ascontiguousarray(up, dtype=np.uint16)
    dg = np.empty(gate.shape, np.uint16)
    du = np.empty(gate.shape, np.uint16)
    _call("orc_swiglu_backward", grad_out, gate, up, dg, du, c_i(gate.size))
    return dg, du


def col_sum_strided(x, out_accum, rows, cols, row_stride, base):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.ascontiguousarray(out_accum, dtype=np.float32).copy()
    _call("orc_col_sum_strided_bf16", x, out, c_i(rows), c_i(cols), c_i(row_stride), c_i(base))
    return out


# ---- producers of the quantizer's input ----------------------------------------------
def rmsnorm_forward(x, weight, eps=1e-6):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    weight = np.ascontiguousarray(weight, dtype=np.uint16)
    rows, H = x.shape
    out = np.empty((rows, H), np.uint16)
    rms = np.empty(rows, np.float32)
    _o.orc_rmsnorm_forward.restype = ctypes.c_int
    rc = _o.orc_rmsnorm_forward(_p(x), _p(weight), _p(out), _p(rms), c_i(rows), c_i(H), c_f(eps))
    if rc != 0:
        raise ValueError(f"orc_rmsnorm_forward: unsupported H={H}")
    return out, rms


def act_row_clip_abs(x, ceiling):
    x = np.ascontiguousarray(x, dtype=np.uint16).copy()
    rows, cols = x.shape
    normsq = np.zeros(rows, np.float32)
    _call("orc_act_row_clip_abs", x, c_i(rows), c_i(cols), c_f(ceiling), normsq)
    return x, normsq


# ---- chunked cross-entropy -----------------------------------------------------------
def cross_entropy_count_valid(labels):
    labels = np.ascontiguousarray(labels, dtype=np.int32)
    n = np.zeros(1, np.int32)
    _call("orc_cross_entropy_count_valid", labels, c_i(labels.size), n)
    return int(n[0])


def cross_entropy_fwd_bwd_chunk(logits, labels, n_valid, loss_in=0.0):
    logits = np.ascontiguousarray(logits, dtype=np.uint16)
    labels = np.ascontiguousarray(labels, dtype=np.int32)
    rows, V = logits.shape
    grad = np.empty((rows, V), np.uint16)
    loss = _f32(loss_in)
    _call("orc_cross_entropy_fwd_bwd_chunk", logits, labels, loss, grad, c_i(rows), c_i(V), np.array([n_valid], np.int32))
    return grad, loss[0]


# ---- GEMM ---------------------------------------------------------------------------
def gemm_nt_ref(A, B, a_descale, b_descale, a_e5m2=False, b_e5m2=False, scale_mode=0, lda=None, want_abs=True):
    """A[M,K] fp8 bytes (row stride lda), B[N,K] fp8 bytes -> (ref[M,N] f64, absdot[M,N] f64)."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    N, K = B.shape
    M = A.shape[0]
    lda = A.shape[1] if lda is None else lda
    ref = np.empty((M, N), np.float64)
    absdot = np.empty((M, N), np.float64) if want_abs else None
    _call("orc_gemm_nt_ref", c_i(M), c_i(N), c_i(K), A, c_i(lda), c_i(int(a_e5m2)),
          np.ascontiguousarray(a_descale, dtype=np.float32), B, c_i(B.shape[1]), c_i(int(b_e5m2)),
          np.ascontiguousarray(b_descale, dtype=np.float32), c_i(scale_mode), ref, absdot, c_i(THREADS))
    return ref, absdot


def gemm_bf16_nn_ref(A, B):
    """gemm_bf16 (src/trainer.cu:3069-3090) on bf16 bit patterns, carried in double: A[M,K] . B[K,N]."""
    return bf16_to_f32(np.asarray(A)).astype(np.float64) @ bf16_to_f32(np.asarray(B)).astype(np.float64)


def gemm_bf16_tn_ref(A, B):
    """gemm_bf16_tn_f32 (src/trainer.cu:3116-3160) without the beta term, in double: A[K,M]^T . B[K,N]."""
    return bf16_to_f32(np.asarray(A)).astype(np.float64).T @ bf16_to_f32(np.asarray(B)).astype(np.float64)


def bf16_ulp(x):
    """Spacing of bf16 at |x| (8 significand bits), floor at the smallest normal."""
    ax = np.maximum(np.abs(np.asarray(x, dtype=np.float64)), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(ax)) - 7)


def gemm_error(got, ref):
    got = np.asarray(got, np.float64)
    diff = got - ref
    rel_l2 = float(np.sqrt((diff ** 2).sum() / max((ref ** 2).sum(), 1e-300)))
    return rel_l2, diff


# Allowance for the accumulation itself, as a multiple of sum_k |a_k b_k|:
#  - an fp32 FMA chain (the naive kernel, the CPU path) differs from the exact sum by a few 2^-24;
#  - gfx950's v_mfma_f32_32x32x64_f8f6f4 aligns the 64 products of one instruction to a common
#    exponent and keeps fewer bits than fp32: measured max error 2.1e-5 * sum|a_k b_k| at K=128
#    and 1.8e-6 at K=4096 (rms 2e-6 / 3.6e-7); relative L2 error 1.5e-5.
ACC_FP32 = 8.0 * 2.0 ** -24
ACC_MFMA = 2.0 ** -15


def assert_gemm_close(got, ref, absdot, rel_l2_tol=1e-3, ulps=2.0, what="gemm", acc=ACC_MFMA, out_bf16=True):
    """The stated GEMM bar: relative L2 error <= 1e-3 and |got - ref| <= 2 bf16 ulps of |ref|, ref being
    the matmul of the dequantised operands carried in double.

    Two clarifications, both forced by arithmetic rather than chosen:
      * a bf16 output cannot be closer than 1.66e-3 relative L2 to an unrounded reference (half an ulp of
        an 8-bit significand, uniformly distributed), so for bf16 outputs the L2 bar is applied against
        the reference rounded to bf16, which is also what the reference's own GEMM returns;
      * where cancellation makes |ref| much smaller than sum|a_k b_k|, the error of the accumulation
        (`acc` * absdot, see above) is allowed on top of the 2 ulps of |ref|."""
    got = np.asarray(got, np.float64)
    l2_ref = ref
    if out_bf16:
        l2_ref = bf16_to_f32(bf16_from_f32(ref.astype(np.float32))).astype(np.float64)
    rel_l2, _ = gemm_error(got, l2_ref)
    assert rel_l2 <= rel_l2_tol, f"{what}: relative L2 error {rel_l2:.3e} > {rel_l2_tol}"
    diff = got - ref
    tol = ulps * bf16_ulp(ref) + acc * absdot
    bad = np.abs(diff) > tol
    if bad.any():
        i = np.unravel_index(np.argmax(np.abs(diff) / tol), diff.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} elements outside tolerance; worst at {i}: "
                             f"got {got[i]!r} ref {ref[i]!r} tol {tol[i]!r}")
    return rel_l2


def strict_ulp_fraction(got, ref, ulps=2.0):
    """Fraction of elements whose error exceeds `ulps` bf16 ulps of |ref| with no accumulation allowance."""
    return float((np.abs(np.asarray(got, np.float64) - ref) > ulps * bf16_ulp(ref)).mean())


def dequant(q, descale, e5m2=False):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    out = np.empty(q.shape, np.float32)
    _call("orc_dequant_n", q, c_i(int(e5m2)), c_f(descale), out, c_sz(q.size))
    return out


def linear_forward_f32(xq, wq, bias=None, threads=1):
    xq = np.ascontiguousarray(xq, dtype=np.float32)
    wq = np.ascontiguousarray(wq, dtype=np.float32)
    T, K = xq.shape
    N = wq.shape[0]
    y = np.empty((T, N), np.uint16)
    _call("orc_linear_forward_f32", xq, wq, None if bias is None else np.ascontiguousarray(bias, dtype=np.uint16),
          y, c_i(T), c_i(K), c_i(N), c_i(threads))
    return y


# ---- MoE ------------------------------------------------------------------------------
def softmax(x):
    x = np.ascontiguousarray(x, dtype=np.float32).copy()
    _call("orc_softmax_inplace_f32", x, c_i(x.shape[0]), c_i(x.shape[1]))
    return x


def moe_topk_route(scores, top_k, normalize=True, want_saves=False):
    s = np.ascontiguousarray(scores, dtype=np.float32).copy()
    rows, E = s.shape
    row_sum = np.empty(rows, np.float32) if want_saves else None
    save = np.empty((rows, E), np.float32) if want_saves else None
    _call("orc_moe_topk_route_f32", s, c_i(rows), c_i(E), c_i(top_k), row_sum, save, c_i(int(normalize)))
    return (s, row_sum, save) if want_saves else s


def moe_build_expert_row_lists(route_weights):
    rw = np.ascontiguousarray(route_weights, dtype=np.float32)
    rows, E = rw.shape
    counts = np.empty(E, np.int32)
    idx = np.full((E, rows), -1, np.int32)
    _call("orc_moe_build_expert_row_lists", rw, counts, idx, c_i(rows), c_i(E))
    return counts, idx


def moe_expert_offsets(counts):
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    off = np.empty(counts.shape, np.int32)
    _call("orc_moe_expert_offsets_from_counts", counts, off, c_i(counts.size))
    return off


def moe_gather_rows_u8(src, row_indices):
    src = np.ascontiguousarray(src, dtype=np.uint8)
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    dst = np.empty((ri.size, src.shape[1]), np.uint8)
    _call("orc_moe_gather_rows_u8", src, dst, ri, c_i(ri.size), c_i(src.shape[1]))
    return dst


def moe_gather_rows_bf16(src, row_indices):
    src = np.ascontiguousarray(src, dtype=np.uint16)
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    dst = np.empty((ri.size, src.shape[1]), np.uint16)
    _call("orc_moe_gather_rows_bf16", src, dst, ri, c_i(ri.size), c_i(src.shape[1]))
    return dst


def moe_scatter_accumulate(mixed, compact, route_weights, row_indices, expert_idx):
    mixed = np.ascontiguousarray(mixed, dtype=np.uint16).copy()
    compact = np.ascontiguousarray(compact, dtype=np.uint16)
    rw = np.ascontiguousarray(route_weights, dtype=np.float32)
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    _call("orc_moe_scatter_accumulate_rows_bf16", mixed, compact, rw, ri, c_i(ri.size), c_i(expert_idx),
          c_i(rw.shape[1]), c_i(mixed.shape[1]))
    return mixed


# ---- MoE expert-bank backward helpers -------------------------------------------------
def gelu_forward(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty_like(x)
    _call("orc_gelu_forward_bf16", x, out, c_sz(x.size))
    return out


def gelu_backward(pre, d_post):
    pre = np.ascontiguousarray(pre, dtype=np.uint16)
    d_post = np.ascontiguousarray(d_post, dtype=np.uint16)
    out = np.empty_like(pre)
    _call("orc_gelu_backward_bf16", pre, d_post, out, c_sz(pre.size))
    return out


def moe_row_dot_selected(a_full, b_compact, out, row_indices, out_col):
    """out is [rows, out_stride] float32; returns a copy with column out_col filled at the listed rows."""
    a_full = np.ascontiguousarray(a_full, dtype=np.uint16)
    b_compact = np.ascontiguousarray(b_compact, dtype=np.uint16)
    out = np.ascontiguousarray(out, dtype=np.float32).copy()
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    _call("orc_moe_row_dot_selected_bf16", a_full, b_compact, out, ri, c_i(ri.size), c_i(a_full.shape[1]),
          c_i(out.shape[1]), c_i(out_col))
    return out


def moe_gather_scale_rows(src, route_weights, row_indices, expert_idx):
    src = np.ascontiguousarray(src, dtype=np.uint16)
    rw = np.ascontiguousarray(route_weights, dtype=np.float32)
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    dst = np.empty((ri.size, src.shape[1]), np.uint16)
    _call("orc_moe_gather_scale_rows_bf16", src, dst, rw, ri, c_i(ri.size), c_i(expert_idx), c_i(rw.shape[1]),
          c_i(src.shape[1]))
    return dst


def moe_scatter_add_rows(dst_full, src_compact, row_indices):
    dst_full = np.ascontiguousarray(dst_full, dtype=np.uint16).copy()
    src_compact = np.ascontiguousarray(src_compact, dtype=np.uint16)
    ri = np.ascontiguousarray(row_indices, dtype=np.int32)
    _call("orc_moe_scatter_add_rows_bf16", dst_full, src_compact, ri, c_i(ri.size), c_i(dst_full.shape[1]))
    return dst_full


def moe_scale_accumulate(mixed, term, route_weights, expert_idx):
    mixed = np.ascontiguousarray(mixed, dtype=np.uint16).copy()
    term = np.ascontiguousarray(term, dtype=np.uint16)
    rw = np.ascontiguousarray(route_weights, dtype=np.float32)
    _call("orc_moe_scale_accumulate_bf16", mixed, term, rw, c_i(mixed.shape[0]), c_i(expert_idx),
          c_i(rw.shape[1]), c_i(mixed.shape[1]))
    return mixed


def moe_grouped_expert_forward_fp8_ref(hidden, fcin_descale, fcin_e5m2, route_weights, counts, row_indices,
                                       fc_in_w, fc_in_descale, fc_out_w, fc_out_descale, mixed0):
    hidden = np.ascontiguousarray(hidden, dtype=np.uint8)
    rows, H = hidden.shape
    rw = np.ascontiguousarray(route_weights, dtype=np.float32)
    E = rw.shape[1]
    fc_in_w = np.ascontiguousarray(fc_in_w, dtype=np.uint8)
    Ie = fc_in_w.shape[1]
    mixed = np.ascontiguousarray(mixed0, dtype=np.float64).copy()
    _call("orc_moe_grouped_expert_forward_fp8_ref", hidden, c_f(fcin_descale), c_i(int(fcin_e5m2)), rw,
          np.ascontiguousarray(counts, dtype=np.int32), np.ascontiguousarray(row_indices, dtype=np.int32),
          fc_in_w, c_f(fc_in_descale), np.ascontiguousarray(fc_out_w, dtype=np.uint8), c_f(fc_out_descale),
          mixed, c_i(rows), c_i(H), c_i(Ie), c_i(E), c_i(THREADS))
    return mixed


def moe_grouped_expert_forward_bf16_ref(hidden, route_weights, counts, row_indices, fc_in_w, fc_out_w, mixed0):
    """moe_grouped_expert_forward_bf16 (kernels/moe.cu, the bf16 sibling of the grouped FP8 expert forward) in
    float64 numpy: per expert, its listed rows through fc_in [Ie,H], exact-erf GELU rounded to bf16 as the kernel parks
    it in shared memory before fc_out (kernels/moe.cu:845), fc_out [H,Ie], times the route weight, summed into mixed.
    hidden / weights are bf16 bit patterns; returns float64 [rows,H]."""
    import math
    erf = np.vectorize(math.erf, otypes=[np.float64])
    x = bf16_to_f32(hidden).astype(np.float64)
    w_in = bf16_to_f32(fc_in_w).astype(np.float64)
    w_out = bf16_to_f32(fc_out_w).astype(np.float64)
    rw = np.asarray(route_weights, dtype=np.float64)
    out = np.array(mixed0, dtype=np.float64, copy=True)
    for e in range(rw.shape[1]):
        rows = np.asarray(row_indices)[e, : int(counts[e])]
        if rows.size == 0:
            continue
        pre = x[rows] @ w_in[e].T
        act = 0.5 * pre * (1.0 + erf(pre * 0.70710678118654752440))
        act = bf16_to_f32(bf16_from_f32(act.astype(np.float32))).astype(np.float64)
        out[rows] += rw[rows, e][:, None] * (act @ w_out[e].T)
    return out
