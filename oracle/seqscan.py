"""ORACLE (test infrastructure, not part of the product).

numpy-facing loader of oracle/seqscan.c: the sequential fp64 recurrences that
define the operator.  Inputs are fp32 (or complex64) arrays of shape
(..., T); results are float64 (complex128).
"""

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libseqscan.so"
_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(_HERE), "all"], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        p = ctypes.c_void_p
        i64 = ctypes.c_int64
        lib.seq_forward_f32.argtypes = [p, p, p, i64, i64, ctypes.c_int]
        lib.seq_forward_c64.argtypes = [p, p, p, i64, i64, ctypes.c_int]
        lib.seq_backward_f32.argtypes = [p, p, p, p, p, i64, i64]
        lib.seq_backward_c64.argtypes = [p, p, p, p, p, i64, i64]
        lib.seq_forward_from_f32.argtypes = [p, p, p, p, i64, i64, ctypes.c_int]
        lib.seq_forward_from_c64.argtypes = [p, p, p, p, i64, i64, ctypes.c_int]
        lib.seq_backward_from_f32.argtypes = [p, p, p, p, p, p, p, i64, i64]
        lib.seq_backward_from_c64.argtypes = [p, p, p, p, p, p, p, i64, i64]
        lib.seq_forward_sigmoid_f32.argtypes = [p, p, p, p, i64, i64]
        lib.seq_forward_exp_f32.argtypes = [p, p, p, p, i64, i64]
        lib.seq_backward_exp_f32.argtypes = [p, p, p, p, p, p, p, i64, i64]
        lib.seq_backward_sigmoid_f32.argtypes = [p, p, p, p, p, p, p, i64, i64]
        lib.seq_forward_lerp_f32.argtypes = [p, p, p, p, i64, i64]
        lib.seq_backward_lerp_f32.argtypes = [p, p, p, p, p, p, p, p, i64, i64]
        lib.seq_forward_expnorm_f32.argtypes = [p, p, p, p, i64, i64]
        lib.seq_backward_expnorm_f32.argtypes = [p, p, p, p, p, p, p, p, i64, i64]
        for f in (lib.seq_forward_f32, lib.seq_forward_c64, lib.seq_backward_f32, lib.seq_backward_c64,
                  lib.seq_forward_from_f32, lib.seq_forward_from_c64, lib.seq_backward_from_f32,
                  lib.seq_backward_from_c64, lib.seq_forward_sigmoid_f32, lib.seq_backward_sigmoid_f32,
                  lib.seq_forward_lerp_f32, lib.seq_backward_lerp_f32, lib.seq_forward_exp_f32,
                  lib.seq_backward_exp_f32, lib.seq_forward_expnorm_f32, lib.seq_backward_expnorm_f32):
            f.restype = None
        _lib = lib
    return _lib


def _prep(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a, a.ctypes.data_as(ctypes.c_void_p)


def forward(gates, tokens, reverse=False):
    """Sequential scan in fp64.  Real (float32) or complex (complex64) inputs."""
    lib = _load()
    cplx = np.iscomplexobj(gates) or np.iscomplexobj(tokens)
    dt = np.complex64 if cplx else np.float32
    g, gp = _prep(gates, dt)
    x, xp = _prep(tokens, dt)
    assert g.shape == x.shape
    T = g.shape[-1]
    rows = g.size // T if T else 0
    out = np.empty(g.shape, dtype=np.complex128 if cplx else np.float64)
    fn = lib.seq_forward_c64 if cplx else lib.seq_forward_f32
    fn(gp, xp, out.ctypes.data_as(ctypes.c_void_p), rows, T, int(bool(reverse)))
    return out


def backward(gates, states, grad_out):
    """(d_gates, d_tokens) of the scan for an incoming gradient, in fp64."""
    lib = _load()
    cplx = np.iscomplexobj(gates) or np.iscomplexobj(states) or np.iscomplexobj(grad_out)
    dt = np.complex64 if cplx else np.float32
    g, gp = _prep(gates, dt)
    s, sp = _prep(states, dt)
    d, dp = _prep(grad_out, dt)
    assert g.shape == s.shape == d.shape
    T = g.shape[-1]
    rows = g.size // T if T else 0
    odt = np.complex128 if cplx else np.float64
    dg = np.empty(g.shape, dtype=odt)
    dx = np.empty(g.shape, dtype=odt)
    fn = lib.seq_backward_c64 if cplx else lib.seq_backward_f32
    fn(gp, sp, dp, dg.ctypes.data_as(ctypes.c_void_p), dx.ctypes.data_as(ctypes.c_void_p), rows, T)
    return dg, dx


def forward_from(gates, tokens, initial, reverse=False):
    """Sequential scan in fp64 started from ``initial`` (shape = gates.shape[:-1])."""
    lib = _load()
    cplx = np.iscomplexobj(gates) or np.iscomplexobj(tokens) or np.iscomplexobj(initial)
    dt = np.complex64 if cplx else np.float32
    g, gp = _prep(gates, dt)
    x, xp = _prep(tokens, dt)
    i, ip = _prep(initial, dt)
    assert g.shape == x.shape and i.shape == g.shape[:-1]
    T = g.shape[-1]
    rows = g.size // T if T else 0
    out = np.empty(g.shape, dtype=np.complex128 if cplx else np.float64)
    fn = lib.seq_forward_from_c64 if cplx else lib.seq_forward_from_f32
    fn(gp, xp, ip, out.ctypes.data_as(ctypes.c_void_p), rows, T, int(bool(reverse)))
    return out


def backward_from(gates, states, initial, grad_out, reverse=False):
    """(d_gates, d_tokens, d_initial) of the scan started from ``initial``, in fp64.
    ``reverse``: of the reverse scan ``forward_from(..., reverse=True)``, which is the forward scan of the
    sequences flipped in time, flipped: its gradients are those of that scan, flipped."""
    if reverse:
        flip = lambda a: np.ascontiguousarray(np.flip(np.asarray(a), -1))
        dg, dx, di = backward_from(flip(gates), flip(states), initial, flip(grad_out))
        return flip(dg), flip(dx), di
    lib = _load()
    cplx = any(np.iscomplexobj(a) for a in (gates, states, initial, grad_out))
    dt = np.complex64 if cplx else np.float32
    g, gp = _prep(gates, dt)
    s, sp = _prep(states, dt)
    i, ip = _prep(initial, dt)
    d, dp = _prep(grad_out, dt)
    assert g.shape == s.shape == d.shape and i.shape == g.shape[:-1]
    T = g.shape[-1]
    rows = g.size // T if T else 0
    odt = np.complex128 if cplx else np.float64
    dg = np.empty(g.shape, dtype=odt)
    dx = np.empty(g.shape, dtype=odt)
    di = np.zeros(i.shape, dtype=odt)
    if rows:
        fn = lib.seq_backward_from_c64 if cplx else lib.seq_backward_from_f32
        fn(gp, sp, ip, dp, dg.ctypes.data_as(ctypes.c_void_p), dx.ctypes.data_as(ctypes.c_void_p),
           di.ctypes.data_as(ctypes.c_void_p), rows, T)
    return dg, dx, di


def _forward_gated(name, gate_inputs, tokens, initial):
    lib = _load()
    z, zp = _prep(gate_inputs, np.float32)
    x, xp = _prep(tokens, np.float32)
    assert z.shape == x.shape
    ip = None
    if initial is not None:
        i, ip = _prep(initial, np.float32)
        assert i.shape == z.shape[:-1]
    T = z.shape[-1]
    rows = z.size // T if T else 0
    out = np.empty(z.shape, dtype=np.float64)
    getattr(lib, name)(zp, xp, ip, out.ctypes.data_as(ctypes.c_void_p), rows, T)
    return out


def _backward_gated(name, gate_inputs, states, grad_out, initial):
    lib = _load()
    z, zp = _prep(gate_inputs, np.float32)
    s, sp = _prep(states, np.float32)
    d, dp = _prep(grad_out, np.float32)
    assert z.shape == s.shape == d.shape
    ip = None
    if initial is not None:
        i, ip = _prep(initial, np.float32)
        assert i.shape == z.shape[:-1]
    T = z.shape[-1]
    rows = z.size // T if T else 0
    dz = np.empty(z.shape, dtype=np.float64)
    dx = np.empty(z.shape, dtype=np.float64)
    di = np.zeros(z.shape[:-1], dtype=np.float64)
    if rows:
        getattr(lib, name)(zp, sp, ip, dp, dz.ctypes.data_as(ctypes.c_void_p), dx.ctypes.data_as(ctypes.c_void_p),
                           di.ctypes.data_as(ctypes.c_void_p), rows, T)
    return dz, dx, di


def forward_sigmoid(gate_logits, tokens, initial=None):
    """Sequential scan in fp64 with gates = sigmoid(gate_logits) (real inputs)."""
    return _forward_gated("seq_forward_sigmoid_f32", gate_logits, tokens, initial)


def backward_sigmoid(gate_logits, states, grad_out, initial=None):
    """(d_gate_logits, d_tokens, d_initial) of the sigmoid-gated scan, in fp64."""
    return _backward_gated("seq_backward_sigmoid_f32", gate_logits, states, grad_out, initial)


def forward_exp(log_gates, tokens, initial=None):
    """Sequential scan in fp64 with gates = exp(log_gates) (real inputs)."""
    return _forward_gated("seq_forward_exp_f32", log_gates, tokens, initial)


def backward_exp(log_gates, states, grad_out, initial=None):
    """(d_log_gates, d_tokens, d_initial) of the exponentially gated scan, in fp64."""
    return _backward_gated("seq_backward_exp_f32", log_gates, states, grad_out, initial)


def _forward_values(name, gate_inputs, values, initial):
    lib = _load()
    z, zp = _prep(gate_inputs, np.float32)
    v, vp = _prep(values, np.float32)
    assert z.shape == v.shape
    ip = None
    if initial is not None:
        i, ip = _prep(initial, np.float32)
        assert i.shape == z.shape[:-1]
    T = z.shape[-1]
    rows = z.size // T if T else 0
    out = np.empty(z.shape, dtype=np.float64)
    getattr(lib, name)(zp, vp, ip, out.ctypes.data_as(ctypes.c_void_p), rows, T)
    return out


def _backward_values(name, gate_inputs, values, states, grad_out, initial):
    lib = _load()
    z, zp = _prep(gate_inputs, np.float32)
    v, vp = _prep(values, np.float32)
    s, sp = _prep(states, np.float32)
    d, dp = _prep(grad_out, np.float32)
    assert z.shape == v.shape == s.shape == d.shape
    ip = None
    if initial is not None:
        i, ip = _prep(initial, np.float32)
        assert i.shape == z.shape[:-1]
    T = z.shape[-1]
    rows = z.size // T if T else 0
    dz = np.empty(z.shape, dtype=np.float64)
    dv = np.empty(z.shape, dtype=np.float64)
    di = np.zeros(z.shape[:-1], dtype=np.float64)
    if rows:
        getattr(lib, name)(zp, vp, sp, ip, dp, dz.ctypes.data_as(ctypes.c_void_p), dv.ctypes.data_as(ctypes.c_void_p),
                           di.ctypes.data_as(ctypes.c_void_p), rows, T)
    return dz, dv, di


def forward_lerp(gate_logits, values, initial=None):
    """Sequential gated interpolation in fp64:
    x[t] = a[t] * x[t-1] + (1 - a[t]) * values[t], a = sigmoid(gate_logits) (real inputs)."""
    return _forward_values("seq_forward_lerp_f32", gate_logits, values, initial)


def backward_lerp(gate_logits, values, states, grad_out, initial=None):
    """(d_gate_logits, d_values, d_initial) of the gated interpolation, in fp64."""
    return _backward_values("seq_backward_lerp_f32", gate_logits, values, states, grad_out, initial)


def forward_expnorm(log_gates, values, initial=None):
    """Sequential scan in fp64 with an exponential gate and the input scale that goes with it:
    x[t] = a[t] * x[t-1] + sqrt(1 - a[t]^2) * values[t], a = exp(log_gates) (real inputs, log_gates <= 0)."""
    return _forward_values("seq_forward_expnorm_f32", log_gates, values, initial)


def backward_expnorm(log_gates, values, states, grad_out, initial=None):
    """(d_log_gates, d_values, d_initial) of that scan, in fp64."""
    return _backward_values("seq_backward_expnorm_f32", log_gates, values, states, grad_out, initial)
