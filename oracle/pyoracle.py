"""ctypes/numpy front end of the CPU oracle (liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg, as the checker.  Product code never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32 = 0
BF16 = 1


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    # make compares time stamps itself: a stale library is rebuilt, a current
    # one costs a few milliseconds
    subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


class AttentionParams(ctypes.Structure):
    _fields_ = [
        ("query_heads", ctypes.c_int),
        ("key_value_heads", ctypes.c_int),
        ("head_dim", ctypes.c_int),
        ("rotary_dim", ctypes.c_int),
        ("capacity", ctypes.c_int),
        ("rms_norm_epsilon", ctypes.c_float),
        ("rope_theta", ctypes.c_float),
        ("round_to_bfloat16", ctypes.c_int),
    ]


class DeltaParams(ctypes.Structure):
    _fields_ = [
        ("key_heads", ctypes.c_int),
        ("value_heads", ctypes.c_int),
        ("key_head_dim", ctypes.c_int),
        ("value_head_dim", ctypes.c_int),
        ("conv_kernel_dim", ctypes.c_int),
        ("rms_norm_epsilon", ctypes.c_float),
        ("round_to_bfloat16", ctypes.c_int),
    ]


def attention_params(query_heads=24, key_value_heads=4, head_dim=256,
                     rotary_dim=64, capacity=4096, rms_norm_epsilon=1e-6,
                     rope_theta=10000000.0, round_to_bfloat16=True):
    return AttentionParams(query_heads, key_value_heads, head_dim, rotary_dim,
                           capacity, rms_norm_epsilon, rope_theta,
                           int(bool(round_to_bfloat16)))


def delta_params(key_heads=16, value_heads=48, key_head_dim=128,
                 value_head_dim=128, conv_kernel_dim=4, rms_norm_epsilon=1e-6,
                 round_to_bfloat16=True):
    return DeltaParams(key_heads, value_heads, key_head_dim, value_head_dim,
                       conv_kernel_dim, rms_norm_epsilon,
                       int(bool(round_to_bfloat16)))


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.pluto_oracle_bf16_round.restype = ctypes.c_float
        _lib.pluto_oracle_bf16_round.argtypes = [ctypes.c_float]
        _lib.pluto_oracle_gqa_attend.argtypes = [
            ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t] + [ctypes.c_void_p] * 5
        _lib.pluto_oracle_gdn_scan.argtypes = [
            ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5 + [
            ctypes.c_int, ctypes.c_double, ctypes.c_void_p, ctypes.c_void_p,
            ctypes.c_int, ctypes.c_int]
    return _lib


def _ptr(array):
    if array is None:
        return None
    assert array.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(array.ctypes.data)


def _f32(array):
    return np.ascontiguousarray(array, dtype=np.float32)


# ---- bf16 helpers (numpy, vectorised; same RNE rule as the C code) --------

def f32_to_bf16_bits(x):
    bits = _f32(x).view(np.uint32).astype(np.uint64)
    bits = bits + 0x7FFF + ((bits >> 16) & 1)
    return ((bits >> 16) & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32)
            << 16).view(np.float32)


def bf16_round(x):
    return bf16_bits_to_f32(f32_to_bf16_bits(x)).reshape(np.shape(x))


# ---- GPT-2 causal MHA ------------------------------------------------------

def mha_fwd(qkv, context_length, num_heads, dtype=F32, seqs=None, heads=None):
    """qkv: [rows, 3E] float32, or uint16 bf16 bits when dtype == BF16.
    Returns (out, maxima, normalizers); out has qkv's storage type."""
    rows, packed = qkv.shape
    E = packed // 3
    qkv = np.ascontiguousarray(qkv)
    out = np.zeros((rows, E), dtype=qkv.dtype)
    stats_shape = (rows // context_length * num_heads, context_length)
    maxima = np.zeros(stats_shape, np.float32)
    normalizers = np.zeros(stats_shape, np.float32)
    s0, s1 = seqs if seqs else (0, rows // context_length)
    h0, h1 = heads if heads else (0, num_heads)
    rc = lib().pluto_oracle_mha_fwd(dtype, _ptr(qkv), rows, context_length,
                                    num_heads, E, _ptr(out), _ptr(maxima),
                                    _ptr(normalizers), s0, s1, h0, h1)
    if rc != 0:
        raise ValueError("oracle rejected the attention shape")
    return out, maxima, normalizers


def mha_bwd(qkv, out, d_out, context_length, num_heads, dtype=F32, seqs=None,
            heads=None):
    rows, packed = qkv.shape
    E = packed // 3
    qkv = np.ascontiguousarray(qkv)
    out = np.ascontiguousarray(out)
    d_out = _f32(d_out)
    d_qkv = np.zeros((rows, 3 * E), np.float32)
    s0, s1 = seqs if seqs else (0, rows // context_length)
    h0, h1 = heads if heads else (0, num_heads)
    rc = lib().pluto_oracle_mha_bwd(dtype, _ptr(qkv), _ptr(out), _ptr(d_out),
                                    rows, context_length, num_heads, E,
                                    _ptr(d_qkv), s0, s1, h0, h1)
    if rc != 0:
        raise ValueError("oracle rejected the attention shape")
    return d_qkv


# ---- Qwen GQA --------------------------------------------------------------

def gqa_normalize_rotate(p, position, x, weight):
    x = _f32(x)
    weight = _f32(weight)
    out = np.zeros(p.head_dim, np.float32)
    lib().pluto_oracle_gqa_normalize_rotate(ctypes.byref(p), position, _ptr(x),
                                            _ptr(weight), _ptr(out))
    return out


class CachedAttention:
    """Stateful mirror of the reference test's AttentionReference: a token-major
    FP32 cache [capacity, kv_heads, head_dim] and a position."""

    def __init__(self, p):
        self.p = p
        shape = (p.capacity, p.key_value_heads, p.head_dim)
        self.keys = np.full(shape, np.nan, np.float32)
        self.values = np.full(shape, np.nan, np.float32)
        self.position = 0

    def reset(self):
        self.position = 0

    def step(self, q_gate, k, v, q_norm, k_norm, want_probabilities=False):
        p = self.p
        q_gate, k, v = _f32(q_gate), _f32(k), _f32(v)
        q_norm, k_norm = _f32(q_norm), _f32(k_norm)
        out = np.zeros((p.query_heads, p.head_dim), np.float32)
        probs = (np.zeros((p.query_heads, self.position + 1), np.float32)
                 if want_probabilities else None)
        rc = lib().pluto_oracle_gqa_cached_step(
            ctypes.byref(p), _ptr(self.keys), _ptr(self.values), self.position,
            _ptr(q_gate), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm),
            _ptr(out), _ptr(probs))
        if rc == -2:
            raise OverflowError("full-attention cache capacity reached")
        if rc != 0:
            raise ValueError("invalid full-attention dimensions or parameters")
        self.position += 1
        return (out, probs) if want_probabilities else out


def gqa_sequence(p, qg, k, v, q_norm, k_norm, rows=None, heads=None):
    """qg [T, qh, 2, d], k/v [T, kh, d] float32 (bf16 representable values).
    Returns dict(out [T, qh, d], keys [T, kh, d], values [T, kh, d], lse [T, qh]);
    only the requested rows/heads of out and lse are filled."""
    qg, k, v = _f32(qg), _f32(k), _f32(v)
    T = qg.shape[0]
    r0, r1 = rows if rows else (0, T)
    h0, h1 = heads if heads else (0, p.query_heads)
    out = np.zeros((T, p.query_heads, p.head_dim), np.float32)
    keys = np.zeros((T, p.key_value_heads, p.head_dim), np.float32)
    values = np.zeros_like(keys)
    lse = np.zeros((T, p.query_heads), np.float32)
    q_norm, k_norm = _f32(q_norm), _f32(k_norm)
    rc = lib().pluto_oracle_gqa_sequence(
        ctypes.byref(p), T, _ptr(qg), _ptr(k), _ptr(v), _ptr(q_norm),
        _ptr(k_norm), _ptr(out), _ptr(keys), _ptr(values), _ptr(lse), r0, r1,
        h0, h1)
    if rc != 0:
        raise ValueError("oracle rejected the GQA sequence")
    return dict(out=out, keys=keys, values=values, lse=lse)


def gqa_sequence_backward(p, qg, k, v, q_norm, k_norm, dy, weight_grads=True):
    """Gradients of gqa_sequence for the upstream gradient dy [T, qh, d].
    Returns dict(dqg [T, qh, 2, d], dk, dv [T, kh, d], dq_norm, dk_norm [d])."""
    qg, k, v, dy = _f32(qg), _f32(k), _f32(v), _f32(dy)
    q_norm, k_norm = _f32(q_norm), _f32(k_norm)
    T = qg.shape[0]
    dqg = np.zeros((T, p.query_heads, 2, p.head_dim), np.float32)
    dk = np.zeros((T, p.key_value_heads, p.head_dim), np.float32)
    dv = np.zeros_like(dk)
    dq_norm = np.zeros(p.head_dim, np.float32)
    dk_norm = np.zeros(p.head_dim, np.float32)
    fn = lib().pluto_oracle_gqa_sequence_backward
    fn.restype = ctypes.c_int
    rc = fn(ctypes.byref(p), T, _ptr(qg), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm),
            _ptr(dy), _ptr(dqg), _ptr(dk), _ptr(dv),
            _ptr(dq_norm) if weight_grads else None, _ptr(dk_norm) if weight_grads else None)
    if rc != 0:
        raise ValueError("oracle rejected the GQA sequence backward")
    return dict(dqg=dqg, dk=dk, dv=dv, dq_norm=dq_norm, dk_norm=dk_norm)


def gqa_attend(p, q, gate, keys, values):
    """q, gate [qh, d]; keys/values [kh, L, d] head-major float32."""
    q, gate = _f32(q), _f32(gate)
    keys, values = _f32(keys), _f32(values)
    L = keys.shape[1]
    out = np.zeros((p.query_heads, p.head_dim), np.float32)
    rc = lib().pluto_oracle_gqa_attend(ctypes.byref(p), L, L * p.head_dim,
                                       _ptr(q), _ptr(gate), _ptr(keys),
                                       _ptr(values), _ptr(out))
    if rc != 0:
        raise ValueError("oracle rejected the attend call")
    return out


# ---- gated delta-net -------------------------------------------------------

def gdn_scan(p, q, k, v, log_decay, beta, normalize_qk, q_scale, state=None,
             heads=None):
    """q,k [T, kh, kd]; v [T, vh, vd]; log_decay, beta [T, vh].
    Returns (core [T, vh, vd] float32, final_state [vh, kd, vd] float64)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    log_decay, beta = _f32(log_decay), _f32(beta)
    T = q.shape[0]
    if state is None:
        state = np.zeros((p.value_heads, p.key_head_dim, p.value_head_dim),
                         np.float64)
    else:
        state = np.array(state, dtype=np.float64, order="C", copy=True)
    core = np.zeros((T, p.value_heads, p.value_head_dim), np.float32)
    h0, h1 = heads if heads else (0, p.value_heads)
    rc = lib().pluto_oracle_gdn_scan(ctypes.byref(p), T, _ptr(q), _ptr(k),
                                     _ptr(v), _ptr(log_decay), _ptr(beta),
                                     int(bool(normalize_qk)), float(q_scale),
                                     _ptr(state), _ptr(core), h0, h1)
    if rc != 0:
        raise ValueError("oracle rejected the delta-net scan")
    return core, state


def gdn_sequence(p, qkv, z, a, b, conv_weight, a_log, dt_bias, norm):
    qkv, z, a, b = _f32(qkv), _f32(z), _f32(a), _f32(b)
    conv_weight, a_log = _f32(conv_weight), _f32(a_log)
    dt_bias, norm = _f32(dt_bias), _f32(norm)
    T = qkv.shape[0]
    width = p.value_heads * p.value_head_dim
    out = np.zeros((T, width), np.float32)
    core = np.zeros((T, p.value_heads, p.value_head_dim), np.float32)
    state = np.zeros((p.value_heads, p.key_head_dim, p.value_head_dim),
                     np.float64)
    rc = lib().pluto_oracle_gdn_sequence(
        ctypes.byref(p), T, _ptr(qkv), _ptr(z), _ptr(a), _ptr(b),
        _ptr(conv_weight), _ptr(a_log), _ptr(dt_bias), _ptr(norm), _ptr(out),
        _ptr(core), _ptr(state))
    if rc != 0:
        raise ValueError("oracle rejected the delta-net sequence")
    return dict(out=out, core=core, state=state)


def gdn_sequence_backward(p, qkv, z, a, b, conv_weight, a_log, dt_bias, norm, dy,
                          parameter_grads=True):
    """Gradients of gdn_sequence for the upstream gradient dy [T, vh*vd].
    Returns dict(dqkv, dz, da, db, d_conv_weight, d_a_log, d_dt_bias, d_norm)."""
    qkv, z, a, b, dy = _f32(qkv), _f32(z), _f32(a), _f32(b), _f32(dy)
    conv_weight, a_log = _f32(conv_weight), _f32(a_log)
    dt_bias, norm = _f32(dt_bias), _f32(norm)
    T = qkv.shape[0]
    out = dict(dqkv=np.zeros_like(qkv), dz=np.zeros_like(z), da=np.zeros_like(a),
               db=np.zeros_like(b), d_conv_weight=np.zeros_like(conv_weight),
               d_a_log=np.zeros_like(a_log), d_dt_bias=np.zeros_like(dt_bias),
               d_norm=np.zeros_like(norm))
    fn = lib().pluto_oracle_gdn_sequence_backward
    fn.restype = ctypes.c_int
    grads = [_ptr(out[n]) if parameter_grads else None
             for n in ("d_conv_weight", "d_a_log", "d_dt_bias", "d_norm")]
    rc = fn(ctypes.byref(p), T, _ptr(qkv), _ptr(z), _ptr(a), _ptr(b), _ptr(conv_weight),
            _ptr(a_log), _ptr(dt_bias), _ptr(norm), _ptr(dy), _ptr(out["dqkv"]), _ptr(out["dz"]),
            _ptr(out["da"]), _ptr(out["db"]), *grads)
    if rc != 0:
        raise ValueError("oracle rejected the delta-net backward")
    return out


class DeltaNetStep:
    """Stateful mirror of the reference test's DeltaReference."""

    def __init__(self, p):
        self.p = p
        channels = (2 * p.key_heads * p.key_head_dim +
                    p.value_heads * p.value_head_dim)
        self.conv = np.zeros((channels, p.conv_kernel_dim), np.float32)
        self.state = np.zeros(
            (p.value_heads, p.key_head_dim, p.value_head_dim), np.float64)

    def reset(self):
        self.conv[:] = 0
        self.state[:] = 0

    def step(self, qkv, z, a, b, conv_weight, a_log, dt_bias, norm):
        p = self.p
        args = [_f32(x) for x in (qkv, z, a, b, conv_weight, a_log, dt_bias,
                                  norm)]
        out = np.zeros(p.value_heads * p.value_head_dim, np.float32)
        rc = lib().pluto_oracle_gdn_step(
            ctypes.byref(p), _ptr(self.conv), _ptr(self.state),
            *[_ptr(x) for x in args], _ptr(out))
        if rc != 0:
            raise ValueError("oracle rejected the delta-net step")
        return out


def half_round(x):
    """float32 -> IEEE half -> float32 (round to nearest even), elementwise."""
    x = _f32(x)
    out = np.empty_like(x)
    fn = lib().pluto_oracle_half_round
    fn.restype = ctypes.c_float
    fn.argtypes = [ctypes.c_float]
    flat_in, flat_out = x.ravel(), out.ravel()
    for i in range(flat_in.size):
        flat_out[i] = fn(float(flat_in[i]))
    return out


def dense_forward(dtype, x, matrix, bias):
    """FullyConnectedLayer forward: x [rows, in] (float values), matrix [in, out],
    bias [out] -> y [rows, out] in the activation type's value set."""
    x, matrix, bias = _f32(x), _f32(matrix), _f32(bias)
    rows, input_dim = x.shape
    output_dim = matrix.shape[1]
    y = np.zeros((rows, output_dim), np.float32)
    fn = lib().pluto_oracle_dense_forward
    fn.restype = ctypes.c_int
    if fn(dtype, rows, input_dim, output_dim, _ptr(x), _ptr(matrix), _ptr(bias), _ptr(y)) != 0:
        raise ValueError("oracle rejected the dense forward")
    return y


def dense_backward(dtype, x, matrix, dy):
    """Gradients (dx [rows, in], d_matrix [in, out], d_bias [out]) of dense_forward."""
    x, matrix, dy = _f32(x), _f32(matrix), _f32(dy)
    rows, input_dim = x.shape
    output_dim = matrix.shape[1]
    dx = np.zeros((rows, input_dim), np.float32)
    dw = np.zeros((input_dim, output_dim), np.float32)
    db = np.zeros(output_dim, np.float32)
    fn = lib().pluto_oracle_dense_backward
    fn.restype = ctypes.c_int
    if fn(dtype, rows, input_dim, output_dim, _ptr(x), _ptr(matrix), _ptr(dy), _ptr(dx), _ptr(dw),
          _ptr(db)) != 0:
        raise ValueError("oracle rejected the dense backward")
    return dx, dw, db


MATRIX_BF16, MATRIX_F32, MATRIX_FP8_E4M3 = 0, 1, 2


def fp8_e4m3_to_f32(bits):
    """Values of OCP FP8 E4M3 codes (uint8 array)."""
    bits = np.ascontiguousarray(bits, np.uint8)
    fn = lib().pluto_oracle_fp8_e4m3_to_f32
    fn.restype = ctypes.c_float
    fn.argtypes = [ctypes.c_uint8]
    return np.array([fn(int(b)) for b in bits.ravel()], np.float32).reshape(bits.shape)


def f32_to_fp8_e4m3(values):
    """FP8 E4M3 codes of floats: nearest even, saturating to +-448."""
    values = _f32(values)
    fn = lib().pluto_oracle_f32_to_fp8_e4m3
    fn.restype = ctypes.c_uint8
    fn.argtypes = [ctypes.c_float]
    return np.array([fn(float(v)) for v in values.ravel()], np.uint8).reshape(values.shape)


def imported_quantize(x):
    """Dynamic FP8 quantization of a token in groups of 128 (fully_connected.cc:70-88)."""
    x = _f32(x)
    out = np.zeros_like(x)
    fn = lib().pluto_oracle_imported_quantize
    fn.restype = None
    fn(_ptr(x), ctypes.c_int(x.size), _ptr(out))
    return out


def imported_matvec(storage, weights, scales, x):
    """Frozen output-major projection of one bf16 token: weights [out, in] as
    uint16 bf16 bits, float32 or uint8 FP8 codes (+ float32 block scales)."""
    weights = np.ascontiguousarray(weights)
    output_dim, input_dim = weights.shape
    x = _f32(x)
    y = np.zeros(output_dim, np.float32)
    fn = lib().pluto_oracle_imported_matvec
    fn.restype = ctypes.c_int
    s = None if scales is None else _f32(scales)
    if fn(ctypes.c_int(storage), weights.ctypes.data_as(ctypes.c_void_p),
          None if s is None else _ptr(s), _ptr(x), ctypes.c_int(input_dim),
          ctypes.c_int(output_dim), _ptr(y)) != 0:
        raise ValueError("oracle rejected the imported projection")
    return y
