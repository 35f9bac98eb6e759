"""ctypes front-end of the CPU oracle (oracle/smlm_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The shipped package never imports it.

All matrices are numpy float32 arrays holding values representable in the I/O
dtype (call :func:`round_to` first).  dtype names: "fp32", "fp16", "bf16".
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libsmlm_oracle.so")
DTYPES = {"fp32": 0, "fp16": 1, "bf16": 2}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (no GPU toolchain involved)."""
    newest = max(os.path.getmtime(os.path.join(_HERE, f)) for f in ("smlm_oracle.c", "rms_norm_oracle.c", "dropout_oracle.c"))
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < newest:
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        for name in ("oracle_smlm_gemm", "oracle_add_lora_forward", "oracle_mixed_lora_linear",
                     "oracle_lora_fused", "oracle_add_lora_backward_rowmajor",
                     "oracle_add_lora_backward", "oracle_build_segments", "oracle_batch_len_info",
                     "oracle_prepare_weight", "oracle_rms_norm_fwd", "oracle_rms_norm_bwd",
                     "oracle_dropout_mask", "oracle_dropout_rows"):
            getattr(_lib, name).restype = C.c_int
        _lib.oracle_round.restype = None
        _lib.oracle_philox4x32_10.restype = None
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _fp(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _ptr_table(mats: Sequence[np.ndarray]):
    arr = (C.POINTER(C.c_float) * max(len(mats), 1))()
    for i, m in enumerate(mats):
        assert m.dtype == np.float32 and m.flags["C_CONTIGUOUS"]
        arr[i] = _fp(m)
    return arr


def _check(rc: int, what: str) -> None:
    if rc < 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def round_to(a, dtype: str) -> np.ndarray:
    """Round to the nearest fp16/bf16 value (ties to even), kept as float32."""
    out = _f32(a).copy()
    lib().oracle_round(_fp(out), C.c_size_t(out.size), C.c_int(DTYPES[dtype]))
    return out


def smlm_gemm(y: np.ndarray, x: np.ndarray, w: Sequence[np.ndarray], s, row_major: bool,
              dtype: str = "fp32", acc64: bool = True) -> np.ndarray:
    """Grouped GEMM Y_i = X_i W_i written into y in place (rows of empty or
    uncovered ranges untouched).  w[i] is stored [d_in, d_out] when row_major
    else [d_out, d_in]."""
    x = _f32(x)
    s = _i32(s)
    S = len(s) - 1
    assert y.dtype == np.float32 and y.flags["C_CONTIGUOUS"]
    d_in, d_out = x.shape[1], y.shape[1]
    w = [_f32(m) for m in w]
    for m in w:
        assert m.shape == ((d_in, d_out) if row_major else (d_out, d_in)), m.shape
    w_ld = d_out if row_major else d_in
    tab = _ptr_table(w)
    _check(lib().oracle_smlm_gemm(_fp(y), _fp(x), tab, _ip(s), S, d_in, d_out, w_ld,
                                  int(row_major), DTYPES[dtype], int(acc64)), "oracle_smlm_gemm")
    return y


def add_lora_forward(x, wa: Sequence[np.ndarray], wb: Sequence[np.ndarray], s, h_out: int,
                     dtype: str = "fp32", acc64: bool = True,
                     y_init: Optional[np.ndarray] = None) -> Tuple[np.ndarray, np.ndarray]:
    """Returns (y, v).  wa[i] is [r, h_in], wb[i] is [h_out, r] for segment i."""
    x = _f32(x)
    s = _i32(s)
    S = len(s) - 1
    T, h_in = x.shape
    wa = [_f32(m) for m in wa]
    wb = [_f32(m) for m in wb]
    r = wa[0].shape[0] if wa else 0
    y = np.zeros((T, h_out), np.float32) if y_init is None else _f32(y_init).copy()
    v = np.zeros((T, max(r, 1)), np.float32)[:, :r].copy()
    ta, tb = _ptr_table(wa), _ptr_table(wb)
    _check(lib().oracle_add_lora_forward(_fp(y), _fp(v), _fp(x), ta, tb, _ip(s), S, h_in, h_out, r,
                                         DTYPES[dtype], int(acc64)), "oracle_add_lora_forward")
    return y, v


def mixed_lora_linear(base, x, wa, wb, s, seg_scale=None, dtype="fp32", acc64=True) -> np.ndarray:
    """result = base + scale * add_lora(x), with the reference's roundings."""
    x = _f32(x)
    y = _f32(base).copy()
    s = _i32(s)
    S = len(s) - 1
    wa = [_f32(m) for m in wa]
    wb = [_f32(m) for m in wb]
    r = wa[0].shape[0]
    sc = None if seg_scale is None else _f32(seg_scale)
    _check(lib().oracle_mixed_lora_linear(_fp(y), _fp(x), _ptr_table(wa), _ptr_table(wb), _ip(s), S,
                                          _fp(sc) if sc is not None else None, x.shape[1],
                                          y.shape[1], r, DTYPES[dtype], int(acc64)),
           "oracle_mixed_lora_linear")
    return y


def lora_fused(y0, x, wa, wb, s, seg_scale=None, beta: float = 1.0, dtype="fp32",
               acc64=True) -> Tuple[np.ndarray, np.ndarray]:
    """y = beta*y0 + scale_seg * round(x A^T) B^T with a single final rounding."""
    x = _f32(x)
    y = _f32(y0).copy()
    s = _i32(s)
    S = len(s) - 1
    wa = [_f32(m) for m in wa]
    wb = [_f32(m) for m in wb]
    r = wa[0].shape[0]
    v = np.zeros((x.shape[0], r), np.float32)
    sc = None if seg_scale is None else _f32(seg_scale)
    _check(lib().oracle_lora_fused(_fp(y), _fp(v), _fp(x), _ptr_table(wa), _ptr_table(wb), _ip(s), S,
                                   _fp(sc) if sc is not None else None, C.c_float(beta), x.shape[1],
                                   y.shape[1], r, DTYPES[dtype], int(acc64)), "oracle_lora_fused")
    return y, v


def add_lora_backward_rowmajor(g, x, wa, wb, tp, dtype="fp32", acc64=True):
    """Literal reference backward; wa[p] is [h_in, r], wb[p] is [r, h_out].
    Returns (grad_x, [grad_wa_p], [grad_wb_p])."""
    g, x = _f32(g), _f32(x)
    tp = _i32(tp)
    P = len(tp) - 1
    T, h_out = g.shape
    h_in = x.shape[1]
    wa = [_f32(m) for m in wa]
    wb = [_f32(m) for m in wb]
    r = wa[0].shape[1]
    gx = np.zeros((T, h_in), np.float32)
    gwa = [np.zeros((h_in, r), np.float32) for _ in range(P)]
    gwb = [np.zeros((r, h_out), np.float32) for _ in range(P)]
    _check(lib().oracle_add_lora_backward_rowmajor(_fp(gx), _ptr_table(gwa), _ptr_table(gwb), _fp(g),
                                                   _fp(x), _ptr_table(wa), _ptr_table(wb), _ip(tp), P,
                                                   T, h_in, h_out, r, DTYPES[dtype], int(acc64)),
           "oracle_add_lora_backward_rowmajor")
    return gx, gwa, gwb


def add_lora_backward(g, x, a_w, b_w, tp, part_adapter, dtype="fp32", acc64=True):
    """Backward for A [r,h_in], B [h_out,r]; per-adapter summed gradients.
    Returns (grad_x [T,h_in], [dA_a], [dB_a]) over the adapters in a_w."""
    g, x = _f32(g), _f32(x)
    tp = _i32(tp)
    pa = _i32(part_adapter)
    P = len(tp) - 1
    T, h_out = g.shape
    h_in = x.shape[1]
    a_w = [_f32(m) for m in a_w]
    b_w = [_f32(m) for m in b_w]
    NA = len(a_w)
    r = a_w[0].shape[0]
    gx = np.zeros((T, h_in), np.float32)
    ga = [np.zeros((r, h_in), np.float32) for _ in range(NA)]
    gb = [np.zeros((h_out, r), np.float32) for _ in range(NA)]
    _check(lib().oracle_add_lora_backward(_fp(gx), _ptr_table(ga), _ptr_table(gb), _fp(g), _fp(x),
                                          _ptr_table(a_w), _ptr_table(b_w), _ip(tp), _ip(pa), P, NA, T,
                                          h_in, h_out, r, DTYPES[dtype], int(acc64)),
           "oracle_add_lora_backward")
    return gx, ga, gb


def build_segments(req_lora_id, req_len) -> Tuple[List[int], np.ndarray, np.ndarray]:
    """Returns (lora_ids list, lora_len int32 [S], segment int32 [S+1])."""
    ids, lens = _i32(req_lora_id), _i32(req_len)
    n = len(ids)
    o_ids = np.zeros(max(n, 1), np.int32)
    o_len = np.zeros(max(n, 1), np.int32)
    o_seg = np.zeros(max(n, 1) + 1, np.int32)
    S = lib().oracle_build_segments(_ip(ids), _ip(lens), n, _ip(o_ids), _ip(o_len), _ip(o_seg))
    _check(S, "oracle_build_segments")
    return o_ids[:S].tolist(), o_len[:S].copy(), o_seg[:S + 1].copy()


def batch_len_info(trains: Sequence[Tuple[int, int]], prefills: Sequence[int]):
    """Returns (train_partition int32 [n+1], tlen, doff)."""
    n = len(trains)
    bsz = _i32([t[0] for t in trains]) if n else np.zeros(1, np.int32)
    sl = _i32([t[1] for t in trains]) if n else np.zeros(1, np.int32)
    pf = _i32(list(prefills)) if len(prefills) else np.zeros(1, np.int32)
    tp = np.zeros(n + 1, np.int32)
    tlen, doff = C.c_int32(0), C.c_int32(0)
    _check(lib().oracle_batch_len_info(_ip(bsz), _ip(sl), n, _ip(pf), len(prefills), _ip(tp),
                                       C.byref(tlen), C.byref(doff)), "oracle_batch_len_info")
    return tp, tlen.value, doff.value


def prepare_weight(w, rank_dim: int, rank: int, scaling: Optional[float], dtype: str) -> np.ndarray:
    w = _f32(w)
    rows, cols = w.shape
    shape = (rank, cols) if rank_dim == 0 else (rows, rank)
    out = np.zeros(shape, np.float32)
    _check(lib().oracle_prepare_weight(_fp(out), _fp(w), rows, cols, rank_dim, rank,
                                       C.c_float(0.0 if scaling is None else scaling), DTYPES[dtype]),
           "oracle_prepare_weight")
    return out


def rms_norm_fwd(x, w, eps: float, dtype: str, acc64: bool = True) -> Tuple[np.ndarray, np.ndarray]:
    """Returns (out [rows, cols], rms [rows]); reference: rms_norm_cutlass.cu:81-159."""
    x, w = _f32(x), _f32(w)
    rows, cols = x.shape
    out = np.zeros((rows, cols), np.float32)
    rms = np.zeros(max(rows, 1), np.float32)
    _check(lib().oracle_rms_norm_fwd(_fp(out), _fp(rms), _fp(x), _fp(w), rows, cols, C.c_float(eps),
                                     DTYPES[dtype], int(acc64)), "oracle_rms_norm_fwd")
    return out, rms[:rows]


def rms_norm_bwd(g, x, w, rms, dtype: str, literal: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    """Returns (dx [rows, cols], dw [cols]); reference: kernel_utils.py:169-176."""
    g, x, w, rms = _f32(g), _f32(x), _f32(w), _f32(rms)
    rows, cols = x.shape
    dx = np.zeros((rows, cols), np.float32)
    dw = np.zeros(cols, np.float32)
    _check(lib().oracle_rms_norm_bwd(_fp(dx), _fp(dw), _fp(g), _fp(x), _fp(w), _fp(rms), rows, cols,
                                     DTYPES[dtype], int(literal)), "oracle_rms_norm_bwd")
    return dx, dw


def philox4x32_10(ctr: Sequence[int], key: Sequence[int]) -> List[int]:
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib().oracle_philox4x32_10(c, k, o)
    return list(o)


def dropout_mask(rows: int, cols: int, row_p, seed: int, offset: int, row0: int = 0) -> np.ndarray:
    """keep[t, j] of the counter-based dropout mask (1 = kept)."""
    rp = _f32(row_p)
    assert rp.shape == (rows,)
    keep = np.zeros((rows, cols), np.uint8)
    _check(lib().oracle_dropout_mask(keep.ctypes.data_as(C.c_void_p), rows, cols, row0, _fp(rp),
                                     C.c_uint64(seed), C.c_uint64(offset)), "oracle_dropout_mask")
    return keep


def dropout_rows(x, row_p, seed: int, offset: int, dtype: str, row0: int = 0) -> np.ndarray:
    """nn.Dropout on the rows of x (row t with probability row_p[t]), mask from the
    counter-based generator; see dropout_oracle.c."""
    x = _f32(x)
    rp = _f32(row_p)
    assert rp.shape == (x.shape[0],)
    out = np.empty_like(x)
    _check(lib().oracle_dropout_rows(_fp(out), _fp(x), x.shape[0], x.shape[1], row0, _fp(rp),
                                     C.c_uint64(seed), C.c_uint64(offset), DTYPES[dtype]),
           "oracle_dropout_rows")
    return out
