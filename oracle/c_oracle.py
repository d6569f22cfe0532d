"""TEST INFRASTRUCTURE -- NOT PRODUCT CODE.

ctypes binding of ``bf_oracle.c`` (the C restatement of the reference's int8-simulated
forward with explicit fp32 operation order).  Imported only by ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Dict, Optional

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbf_oracle.so")


def build(force: bool = False) -> str:
    """Compile the checker with gcc (``make -C oracle``)."""
    if force:
        subprocess.run(["make", "-C", HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)
    return LIB_PATH


class _Config(C.Structure):
    _fields_ = [("d_model", C.c_int), ("n_layers", C.c_int), ("n_heads", C.c_int),
                ("d_ff", C.c_int), ("n_value", C.c_int), ("eps", C.c_float), ("value_mode", C.c_int)]


_PARAM_FIELDS = ["emb_square", "emb_type_special", "emb_color_turn", "emb_clock", "emb_rep",
                 "in_proj_w", "in_proj_b", "out_proj_w", "out_proj_b", "linear1_w", "linear1_b",
                 "linear2_w", "linear2_b", "norm1_w", "norm1_b", "norm2_w", "norm2_b",
                 "norm_f_w", "norm_f_b", "policy_w", "promo_w", "value_w"]


class _Params(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in _PARAM_FIELDS]


_TAP_FIELDS = ["embed", "qa_qkv", "acc_qkv", "qa_out", "acc_out", "qa_ff1", "acc_ff1",
               "qa_ff2", "acc_ff2", "resid", "normed"]


class _Taps(C.Structure):
    _fields_ = ([("x_in", C.c_void_p), ("layer_begin", C.c_int), ("layer_end", C.c_int)]
                + [(n, C.c_void_p) for n in _TAP_FIELDS])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.bfo_model_create.restype = C.c_void_p
        L.bfo_model_create.argtypes = [C.POINTER(_Config), C.POINTER(_Params)]
        L.bfo_model_destroy.argtypes = [C.c_void_p]
        L.bfo_forward.restype = C.c_int
        L.bfo_forward.argtypes = [C.c_void_p] + [C.c_void_p] * 4 + [C.c_int] + [C.c_void_p] * 4 + [C.POINTER(_Taps)]
        L.bfo_exp_neg.restype = C.c_float
        L.bfo_exp_neg.argtypes = [C.c_float]
        L.bfo_check_div_const.restype = C.c_long
        L.bfo_check_div_const.argtypes = [C.c_float, C.c_uint]
        L.bfo_tanh.restype = C.c_float
        L.bfo_tanh.argtypes = [C.c_float]
        L.bfo_quantise_weights_int8.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.bfo_quantise_activations_int8.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.bfo_int8_linear.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        L.bfo_int8_linear_q.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                                        C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.bfo_model_qweight.restype = C.c_void_p
        L.bfo_model_qweight.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_void_p)]
        _lib = L
    return _lib


def _f32(t) -> np.ndarray:
    return np.ascontiguousarray(t.detach().cpu().float().numpy() if isinstance(t, torch.Tensor) else t,
                                dtype=np.float32)


def quantise_weights_int8(w: np.ndarray):
    w = _f32(w)
    n, k = w.shape
    q = np.empty((n, k), np.int8)
    s = np.empty(n // 128, np.float32)
    lib().bfo_quantise_weights_int8(w.ctypes.data, n, k, q.ctypes.data, s.ctypes.data)
    return q, s


def quantise_activations_int8(x: np.ndarray, unsigned: bool = False):
    x = _f32(x)
    m, k = x.shape
    q = np.empty((m, k), np.int16)
    s = np.empty(m, np.float32)
    lib().bfo_quantise_activations_int8(x.ctypes.data, m, k, int(unsigned), q.ctypes.data, s.ctypes.data)
    return q, s


def int8_linear(x, w, bias=None, unsigned: bool = False) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    m, k = x.shape
    n = w.shape[0]
    b = _f32(bias) if bias is not None else None
    out = np.empty((m, n), np.float32)
    lib().bfo_int8_linear(x.ctypes.data, m, k, w.ctypes.data, n, b.ctypes.data if b is not None else None,
                          int(unsigned), out.ctypes.data)
    return out


def int8_linear_q(x, wq, ws, bias=None, unsigned: bool = False):
    """Pre-quantised weights; returns (out, qa int16 [m,k], sa [m,k/256], acc int32 [k/256,m,n])."""
    x = _f32(x)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    ws = _f32(ws)
    m, k = x.shape
    n = wq.shape[0]
    b = _f32(bias) if bias is not None else None
    out = np.empty((m, n), np.float32)
    qa = np.empty((m, k), np.int16)
    sa = np.empty((m, k // 256), np.float32)
    acc = np.empty((k // 256, m, n), np.int32)
    lib().bfo_int8_linear_q(x.ctypes.data, m, k, wq.ctypes.data, ws.ctypes.data, n,
                            b.ctypes.data if b is not None else None, int(unsigned), out.ctypes.data,
                            qa.ctypes.data, sa.ctypes.data, acc.ctypes.data)
    return out, qa, sa, acc


class COracle:
    """The C checker bound to one set of weights (a reference-style ``state_dict``)."""

    def __init__(self, sd: Dict[str, torch.Tensor], n_heads: Optional[int] = None, eps: float = 1e-5):
        L = 0
        while f"encoder.layers.{L}.linear1.weight" in sd:
            L += 1
        d = sd["norm_f.weight"].shape[0]
        f = sd["encoder.layers.0.linear1.weight"].shape[0]
        self.d, self.L, self.f = d, L, f
        self.n_heads = n_heads if n_heads is not None else d // 32
        self.n_value = int(sd["value.weight"].shape[0])

        def stack(fmt):
            return _f32(torch.stack([sd[fmt.format(i)].detach().float() for i in range(L)]))

        arrs = {
            "emb_square": _f32(sd["emb_square.weight"]),
            "emb_type_special": _f32(sd["emb_type_special.weight"]),
            "emb_color_turn": _f32(sd["emb_color_turn.weight"]),
            "emb_clock": _f32(sd["emb_clock.weight"]),
            "emb_rep": _f32(sd["emb_rep.weight"]),
            "in_proj_w": stack("encoder.layers.{}.self_attn.in_proj_weight"),
            "in_proj_b": stack("encoder.layers.{}.self_attn.in_proj_bias"),
            "out_proj_w": stack("encoder.layers.{}.self_attn.out_proj.weight"),
            "out_proj_b": stack("encoder.layers.{}.self_attn.out_proj.bias"),
            "linear1_w": stack("encoder.layers.{}.linear1.weight"),
            "linear1_b": stack("encoder.layers.{}.linear1.bias"),
            "linear2_w": stack("encoder.layers.{}.linear2.weight"),
            "linear2_b": stack("encoder.layers.{}.linear2.bias"),
            "norm1_w": stack("encoder.layers.{}.norm1.weight"),
            "norm1_b": stack("encoder.layers.{}.norm1.bias"),
            "norm2_w": stack("encoder.layers.{}.norm2.weight"),
            "norm2_b": stack("encoder.layers.{}.norm2.bias"),
            "norm_f_w": _f32(sd["norm_f.weight"]), "norm_f_b": _f32(sd["norm_f.bias"]),
            "policy_w": _f32(sd["policy.weight"]), "promo_w": _f32(sd["promo.weight"]),
            "value_w": _f32(sd["value.weight"]),
        }
        self._keep = arrs
        # the marker buffer of the pooled heads (brokefish/nn/model.py:318-331); absent: king row
        self.value_mode = int(sd["value_mode"]) if "value_mode" in sd else 0
        cfg = _Config(d, L, self.n_heads, f, self.n_value, eps, self.value_mode)
        prm = _Params(**{k: v.ctypes.data for k, v in arrs.items()})
        self._h = lib().bfo_model_create(C.byref(cfg), C.byref(prm))
        if not self._h:
            raise ValueError("unsupported dimensions for the C checker")

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.bfo_model_destroy(self._h)
            self._h = None

    def qweight(self, which: str, layer: int):
        """(int8 [n,k], scale [n/128]) of matmul ``which`` in {"qkv","out","ff1","ff2"}."""
        idx = {"qkv": 0, "out": 1, "ff1": 2, "ff2": 3}[which]
        d, f = self.d, self.f
        n, k = {"qkv": (3 * d, d), "out": (d, d), "ff1": (f, d), "ff2": (d, f)}[which]
        sp = C.c_void_p()
        qp = lib().bfo_model_qweight(self._h, idx, layer, C.byref(sp))
        q = np.ctypeslib.as_array(C.cast(qp, C.POINTER(C.c_int8)), shape=(n, k)).copy()
        s = np.ctypeslib.as_array(C.cast(sp, C.POINTER(C.c_float)), shape=(n // 128,)).copy()
        return q, s

    def forward(self, boards, control, rep, mask=None, taps: bool = False, x_in=None,
                layer_begin: int = 0, layer_end: Optional[int] = None):
        """numpy in, dict of numpy out: policy, promo, value, [best], [taps...].

        ``x_in`` ([n,32,d] fp32) replaces the embedding as the residual stream entering
        ``layer_begin``; layers ``[layer_begin, layer_end)`` run, then the heads."""
        b = np.ascontiguousarray(np.asarray(boards).astype(np.int16).view(np.uint16))
        c = np.ascontiguousarray(np.asarray(control), dtype=np.int16)
        r = np.ascontiguousarray(np.asarray(rep), dtype=np.uint8)
        n = b.shape[0]
        d, f = self.d, self.f
        layer_end = self.L if layer_end is None else layer_end
        L = layer_end - layer_begin
        out = {"policy": np.empty((n, 32, 64), np.float32), "promo": np.empty((n, 32, 4), np.float32),
               "value": np.empty(n, np.float32)}
        mk = None
        best = None
        if mask is not None:
            mk = np.ascontiguousarray(np.asarray(mask).astype(np.int64).view(np.uint64))
            best = np.empty(n, np.int32)
            out["best"] = best
        tp = None
        xin = None
        if x_in is not None:
            xin = _f32(x_in)
            assert xin.shape == (n, 32, d)
        if taps or xin is not None:
            kd, kf = d // 256, f // 256
            t = {"embed": np.empty((n, 32, d), np.float32),
                 "qa_qkv": np.empty((n, L, 32, d), np.int8), "acc_qkv": np.empty((n, L, kd, 32, 3 * d), np.int32),
                 "qa_out": np.empty((n, L, 32, d), np.int8), "acc_out": np.empty((n, L, kd, 32, d), np.int32),
                 "qa_ff1": np.empty((n, L, 32, d), np.int8), "acc_ff1": np.empty((n, L, kd, 32, f), np.int32),
                 "qa_ff2": np.empty((n, L, 32, f), np.int8), "acc_ff2": np.empty((n, L, kf, 32, d), np.int32),
                 "resid": np.empty((n, L, 32, d), np.float32), "normed": np.empty((n, 32, d), np.float32)}
            if taps:
                out.update(t)
            tp = _Taps(**({k: v.ctypes.data for k, v in t.items()} if taps else {}))
            tp.x_in = xin.ctypes.data if xin is not None else None
            tp.layer_begin, tp.layer_end = layer_begin, layer_end
        rc = lib().bfo_forward(self._h, b.ctypes.data, c.ctypes.data, r.ctypes.data,
                               mk.ctypes.data if mk is not None else None, n,
                               out["policy"].ctypes.data, out["promo"].ctypes.data, out["value"].ctypes.data,
                               best.ctypes.data if best is not None else None,
                               C.byref(tp) if tp is not None else None)
        if rc:
            raise RuntimeError(f"bfo_forward returned {rc}")
        return out
