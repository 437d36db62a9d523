"""ctypes binding of libpluto_hip.so (the C ABI declared in include/pluto_hip.h).

torch is used for plumbing only: device memory (tensors) and the current HIP
stream.  It is imported before the library is loaded so that both share one
HIP runtime.  There is no fallback: if the library is missing or a call
fails, an exception is raised.
"""
import ctypes
import os

import torch  # noqa: F401  (must precede loading the library, see above)

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpluto_hip.so")

F32 = 0
BF16 = 1

EINVAL, ERANGE, EUNSUPPORTED, EWORKSPACE, ELIMIT = -1, -2, -3, -4, -5


class PlutoHipError(RuntimeError):
    def __init__(self, code, name, text):
        super().__init__("%s (%d): %s" % (name, code, text))
        self.code = code


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


class KvCacheView(ctypes.Structure):
    _fields_ = [
        ("keys", ctypes.c_void_p),
        ("values", ctypes.c_void_p),
        ("dtype", ctypes.c_int),
        ("token_stride", ctypes.c_longlong),
        ("head_stride", ctypes.c_longlong),
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


_VP = ctypes.c_void_p
_I = ctypes.c_int
_SZ = ctypes.c_size_t

# name -> (restype, argtypes); every symbol declared in include/pluto_hip.h
SIGNATURES = {
    "pluto_hip_error_name": (ctypes.c_char_p, [_I]),
    "pluto_hip_error_string": (ctypes.c_char_p, [_I]),
    "pluto_hip_test_force_generic": (_I, [_I]),
    "pluto_hip_test_kernel_classes": (ctypes.c_uint, [ctypes.c_uint]),
    "pluto_hip_test_last_path": (_I, []),
    "pluto_hip_test_forward_schedule": (_I, [_I] * 8 + [ctypes.POINTER(ctypes.c_uint16), _I,
                                                        ctypes.POINTER(_I), ctypes.POINTER(_I)]),
    "pluto_hip_abi_version": (_I, []),
    "pluto_hip_target_arch": (ctypes.c_char_p, []),
    "pluto_hip_executor_create": (_I, [ctypes.POINTER(_VP)]),
    "pluto_hip_executor_destroy": (_I, [_VP]),
    "pluto_hip_executor_synchronize": (_I, [_VP]),
    "pluto_hip_executor_stream": (_VP, [_VP]),
    "pluto_hip_executor_immediate_stream": (_VP, [_VP]),
    "pluto_hip_malloc_async": (_I, [_VP, _SZ, ctypes.POINTER(_VP)]),
    "pluto_hip_free_async": (_I, [_VP, _VP]),
    "pluto_hip_host_alloc": (_I, [_VP, _SZ, ctypes.POINTER(_VP)]),
    "pluto_hip_host_free_async": (_I, [_VP, _VP]),
    "pluto_hip_memcpy_async": (_I, [_VP, _VP, _VP, _SZ, _I]),
    "pluto_hip_memset_async": (_I, [_VP, _VP, _I, _SZ]),
    "pluto_hip_stream_synchronize": (_I, [_VP]),
    "pluto_hip_cast_bf16_to_f32": (_I, [_VP, _VP, _VP, _SZ]),
    "pluto_hip_cast_f32_to_bf16": (_I, [_VP, _VP, _VP, _SZ]),
    "pluto_hip_mha_forward": (_I, [_VP, _I, _VP, _I, _I, _I, _I, _VP, _VP, _VP]),
    "pluto_hip_mha_probabilities": (_I, [_VP, _I, _VP, _VP, _VP, _I, _I, _I, _I, _VP]),
    "pluto_hip_mha_backward_workspace_bytes": (_SZ, [_I, _I, _I, _I, _I]),
    "pluto_hip_mha_backward": (_I, [_VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I,
                                    _VP, _VP, _SZ]),
    "pluto_hip_attention_params_validate": (_I, [ctypes.POINTER(AttentionParams)]),
    "pluto_hip_gqa_prefill_workspace_bytes": (_SZ, [ctypes.POINTER(AttentionParams), _I]),
    "pluto_hip_gqa_prefill_saved_bytes": (_SZ, [ctypes.POINTER(AttentionParams), _I, _I]),
    "pluto_hip_gqa_prefill": (_I, [_VP, ctypes.POINTER(AttentionParams), _I, _I, _VP,
                                   _VP, _VP, _VP, _VP, ctypes.POINTER(KvCacheView),
                                   _VP, _VP, _VP, _VP, _SZ]),
    "pluto_hip_gqa_prefill_probabilities": (_I, [_VP, ctypes.POINTER(AttentionParams), _I, _I,
                                                 ctypes.POINTER(KvCacheView), _VP, _SZ, _VP]),
    "pluto_hip_gqa_prefill_backward_workspace_bytes": (_SZ, [ctypes.POINTER(AttentionParams), _I,
                                                             _I, _I]),
    "pluto_hip_gqa_prefill_backward": (_I, [_VP, ctypes.POINTER(AttentionParams), _I] +
                                       [_VP] * 12 + [_VP, _SZ]),
    "pluto_hip_gqa_decode_workspace_bytes": (_SZ, [ctypes.POINTER(AttentionParams), _I,
                                                   ctypes.POINTER(_I), _I]),
    "pluto_hip_gqa_decode": (_I, [_VP, ctypes.POINTER(AttentionParams), _I, _I, _VP,
                                  _VP, _VP, _VP, _VP, ctypes.POINTER(_I),
                                  ctypes.POINTER(KvCacheView), _VP,
                                  ctypes.POINTER(_VP), _I, _VP, _SZ]),
    "pluto_hip_gqa_decode_static_bytes": (_SZ, []),
    "pluto_hip_gqa_decode_static_prepare": (_I, []),
    "pluto_hip_gqa_decode_static_reset": (_I, [_VP]),
    "pluto_hip_gqa_decode_static": (_I, [_VP, ctypes.POINTER(AttentionParams), _I, _I, _VP,
                                         _VP, _VP, _VP, _VP, ctypes.POINTER(_I),
                                         ctypes.POINTER(KvCacheView), _VP,
                                         ctypes.POINTER(_VP), _I]),
    "pluto_hip_gdn_scan_workspace_bytes": (_SZ, [ctypes.POINTER(DeltaParams), _I, _I, _I]),
    "pluto_hip_gdn_scan": (_I, [_VP, ctypes.POINTER(DeltaParams), _I, _I, _I, _VP, _VP,
                                _VP, _VP, _VP, _I, ctypes.c_float, _VP, _VP, _VP, _SZ]),
    "pluto_hip_gdn_layer_workspace_bytes": (_SZ, [ctypes.POINTER(DeltaParams), _I, _I]),
    "pluto_hip_gdn_layer_forward": (_I, [_VP, ctypes.POINTER(DeltaParams), _I, _I] + [_VP] * 10 +
                                    [_VP, _SZ]),
    "pluto_hip_gdn_layer_backward_workspace_bytes": (_SZ, [ctypes.POINTER(DeltaParams), _I, _I]),
    "pluto_hip_gdn_layer_backward": (_I, [_VP, ctypes.POINTER(DeltaParams), _I, _I] + [_VP] * 17 +
                                     [_VP, _SZ]),
    "pluto_hip_gdn_step_workspace_bytes": (_SZ, [ctypes.POINTER(DeltaParams)]),
    "pluto_hip_gdn_step": (_I, [_VP, ctypes.POINTER(DeltaParams)] + [_VP] * 11 + [_VP, _SZ]),
    "pluto_hip_gdn_step_batch_workspace_bytes": (_SZ, [ctypes.POINTER(DeltaParams), _I]),
    "pluto_hip_gdn_step_batch": (_I, [_VP, ctypes.POINTER(DeltaParams), _I, _I] + [_VP] * 11 +
                                 [_VP, _SZ]),
    "pluto_hip_dense_workspace_bytes": (_SZ, [_I, _I, _I, _I]),
    "pluto_hip_dense_forward": (_I, [_VP, _I, _VP, _VP, _VP, _I, _I, _I, _VP, _VP, _SZ]),
    "pluto_hip_dense_backward": (_I, [_VP, _I, _VP, _VP, _VP, _I, _I, _I, _VP, _VP, _VP, _VP,
                                      _SZ]),
    "pluto_hip_dense_imported_workspace_bytes": (_SZ, [_I]),
    "pluto_hip_dense_imported_forward": (_I, [_VP, _I, _VP, _VP, _VP, _I, _I, _VP, _VP, _SZ]),
    "pluto_hip_dense_imported_batch_workspace_bytes": (_SZ, [_I, _I]),
    "pluto_hip_dense_imported_forward_batch": (_I, [_VP, _I, _VP, _VP, _VP, _I, _I, _I, _VP, _VP,
                                                    _SZ]),
    "pluto_hip_dense_imported_forward_many": (_I, [_VP, _I, _I, ctypes.POINTER(_VP),
                                                   ctypes.POINTER(_VP), ctypes.POINTER(_I), _VP,
                                                   _I, _I, ctypes.POINTER(_VP), _VP, _SZ]),
    "pluto_hip_gdn_recurrence": (_I, [_VP, ctypes.POINTER(DeltaParams), _I, _I, _VP, _VP,
                                      _VP, _VP, _VP, _I, ctypes.c_float, _VP, _VP, _I]),
}

_lib = None


def lib():
    """Loads libpluto_hip.so (built in-tree by pluto_amd.build) or raises."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: run `python -m pluto_amd.build`" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError: the build is stale
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


class force_generic:
    """Context manager around the library's test switch: inside it every call
    runs the any-shape FP32-arithmetic kernels."""

    def __enter__(self):
        self.previous = lib().pluto_hip_test_force_generic(1)

    def __exit__(self, *exc):
        lib().pluto_hip_test_force_generic(self.previous)
        return False


MAIN_KERNEL, QUERY_KERNEL, AUXILIARY_KERNELS = 1, 2, 4
EIGHT_WAVE = 16  # permission bit, not a kernel: see pluto_hip_test_kernel_classes
FROM_LENGTH = 32  # cleared: hand-scheduled kernels at every length (same header comment)
(PATH_NONE, PATH_GENERIC, PATH_MATRIX_F32, PATH_FLASH, PATH_SPLIT_K, PATH_CHUNKED,
 PATH_RECURRENCE) = range(7)


def last_path():
    """Kernel family the calling thread's most recent compute call chose."""
    return lib().pluto_hip_test_last_path()


class only_kernels:
    """Context manager around the library's measurement hook: inside it the
    multi-launch entry points queue only the kernel classes in `mask`."""

    def __init__(self, mask):
        self.mask = mask

    def __enter__(self):
        self.previous = lib().pluto_hip_test_kernel_classes(self.mask)

    def __exit__(self, *exc):
        lib().pluto_hip_test_kernel_classes(self.previous)
        return False


def check(code):
    if code != 0:
        l = lib()
        raise PlutoHipError(code, l.pluto_hip_error_name(code).decode(),
                            l.pluto_hip_error_string(code).decode())


def current_stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(tensor):
    return None if tensor is None else ctypes.c_void_p(tensor.data_ptr())


def dtype_code(tensor):
    if tensor.dtype == torch.bfloat16:
        return BF16
    if tensor.dtype == torch.float32:
        return F32
    raise TypeError("activations must be float32 or bfloat16")


# ---- GPT-2 causal MHA ------------------------------------------------------

def mha_forward(qkv, context_length, num_heads, stream=None, into=None):
    """qkv [rows, 3E] (float32 or bfloat16, contiguous, on the GPU).
    Returns (out [rows, E], maxima [rows/T*H, T], normalizers); `into` is an
    earlier result whose three tensors are written again instead of new ones."""
    assert qkv.is_contiguous()
    rows, packed = qkv.shape
    E = packed // 3
    if into is not None:
        out, maxima, normalizers = into
    else:
        out = torch.empty((rows, E), dtype=qkv.dtype, device=qkv.device)
        stats = (max(rows // max(context_length, 1), 0) * num_heads, context_length)
        maxima = torch.empty(stats, dtype=torch.float32, device=qkv.device)
        normalizers = torch.empty(stats, dtype=torch.float32, device=qkv.device)
    check(lib().pluto_hip_mha_forward(stream or current_stream(), dtype_code(qkv),
                                      ptr(qkv), rows, context_length, num_heads, E,
                                      ptr(out), ptr(maxima), ptr(normalizers)))
    return out, maxima, normalizers


def mha_probabilities(qkv, maxima, normalizers, context_length, num_heads, stream=None):
    rows, packed = qkv.shape
    E = packed // 3
    probs = torch.empty((rows // context_length, num_heads, context_length, context_length),
                        dtype=torch.float32, device=qkv.device)
    check(lib().pluto_hip_mha_probabilities(stream or current_stream(), dtype_code(qkv),
                                            ptr(qkv), ptr(maxima), ptr(normalizers), rows,
                                            context_length, num_heads, E, ptr(probs)))
    return probs


def mha_backward_workspace(qkv, context_length, num_heads):
    rows, packed = qkv.shape
    size = lib().pluto_hip_mha_backward_workspace_bytes(
        dtype_code(qkv), rows, context_length, num_heads, packed // 3)
    return torch.empty(size, dtype=torch.uint8, device=qkv.device)


def mha_backward(qkv, out, d_out, maxima, normalizers, context_length, num_heads,
                 workspace=None, d_qkv=None, stream=None):
    rows, packed = qkv.shape
    E = packed // 3
    if workspace is None:
        workspace = mha_backward_workspace(qkv, context_length, num_heads)
    if d_qkv is None:
        d_qkv = torch.empty((rows, packed), dtype=torch.float32, device=qkv.device)
    check(lib().pluto_hip_mha_backward(stream or current_stream(), dtype_code(qkv), ptr(qkv),
                                       ptr(out), ptr(d_out), ptr(maxima), ptr(normalizers),
                                       rows, context_length, num_heads, E, ptr(d_qkv),
                                       ptr(workspace), workspace.numel()))
    return d_qkv


# ---- Qwen grouped-query attention -------------------------------------------

def attention_params(query_heads=24, key_value_heads=4, head_dim=256, rotary_dim=64,
                     capacity=4096, rms_norm_epsilon=1e-6, rope_theta=10000000.0,
                     round_to_bfloat16=True):
    return AttentionParams(query_heads, key_value_heads, head_dim, rotary_dim, capacity,
                           rms_norm_epsilon, rope_theta, int(bool(round_to_bfloat16)))


class KvCache:
    """One sequence's K and V storage plus the view handed to the C ABI.

    layout "head_major": [kv_heads, capacity, head_dim] (native, bf16 by default);
    layout "token_major": [capacity, kv_heads, head_dim] (the reference's layout)."""

    def __init__(self, capacity, kv_heads, head_dim, dtype=torch.bfloat16,
                 layout="head_major", device="cuda", fill=None):
        shape = ((kv_heads, capacity, head_dim) if layout == "head_major"
                 else (capacity, kv_heads, head_dim))
        self.keys = torch.empty(shape, dtype=dtype, device=device)
        self.values = torch.empty(shape, dtype=dtype, device=device)
        if fill is not None:
            self.keys.fill_(fill)
            self.values.fill_(fill)
        self.layout = layout
        self.capacity, self.kv_heads, self.head_dim = capacity, kv_heads, head_dim
        self.position = 0

    def view(self):
        if self.layout == "head_major":
            token_stride, head_stride = self.head_dim, self.capacity * self.head_dim
        else:
            token_stride, head_stride = self.kv_heads * self.head_dim, self.head_dim
        return KvCacheView(self.keys.data_ptr(), self.values.data_ptr(),
                           dtype_code(self.keys), token_stride, head_stride)

    def token_major(self, tensor):
        """[capacity, kv_heads, head_dim] float32 copy on the host."""
        t = tensor.float().cpu()
        return (t.permute(1, 0, 2) if self.layout == "head_major" else t).contiguous().numpy()


def gqa_prefill_saved(p, length, cache, device="cuda"):
    """Buffer for the state gqa_prefill can leave for gqa_prefill_backward, or
    None where the library keeps none (it then recomputes)."""
    size = lib().pluto_hip_gqa_prefill_saved_bytes(ctypes.byref(p), length, cache.view().dtype)
    return torch.empty(size, dtype=torch.uint8, device=device) if size else None


def gqa_prefill(p, qg, k, v, q_norm, k_norm, cache, start_position=0, want_lse=False,
                stream=None, want_probabilities=False, saved=None, out=None, workspace=None):
    """qg bf16 [T, qh, 2, d]; k, v bf16 [T, kh, d]; norms fp32 [d].

    want_probabilities appends fp32 [qh, T, start_position + T] to the result.
    saved: a gqa_prefill_saved(...) buffer to fill for the backward pass."""
    T = qg.shape[0]
    if out is None:
        out = torch.empty((T, p.query_heads, p.head_dim), dtype=torch.bfloat16, device=qg.device)
    lse = (torch.empty((T, p.query_heads), dtype=torch.float32, device=qg.device)
           if want_lse else None)
    size = lib().pluto_hip_gqa_prefill_workspace_bytes(ctypes.byref(p), T)
    if workspace is None:
        workspace = torch.empty(max(size, 1), dtype=torch.uint8, device=qg.device)
    view = cache.view()
    check(lib().pluto_hip_gqa_prefill(stream or current_stream(), ctypes.byref(p), T,
                                      start_position, ptr(qg), ptr(k), ptr(v), ptr(q_norm),
                                      ptr(k_norm), ctypes.byref(view), ptr(out), ptr(lse),
                                      ptr(saved), ptr(workspace), size))
    cache.position = start_position + T
    result = (out, lse) if want_lse else out
    if want_probabilities:
        probabilities = torch.empty((p.query_heads, T, start_position + T), dtype=torch.float32,
                                    device=qg.device)
        check(lib().pluto_hip_gqa_prefill_probabilities(
            stream or current_stream(), ctypes.byref(p), T, start_position, ctypes.byref(view),
            ptr(workspace), size, ptr(probabilities)))
        result = (result + (probabilities,)) if want_lse else (result, probabilities)
    return result


def gqa_prefill_backward(p, qg, k, v, q_norm, k_norm, dy, dq_norm=None, dk_norm=None,
                         stream=None, saved=None):
    """Gradients of the whole-sequence layer: (dqg fp32 [T, qh, 2, d], dk, dv fp32 [T, kh, d]).

    dq_norm / dk_norm: optional fp32 [d] accumulators the norm-weight gradients are added to.
    saved: the buffer gqa_prefill filled for the same inputs (skips the forward recomputation)."""
    T = qg.shape[0]
    dqg = torch.empty((T, p.query_heads, 2, p.head_dim), dtype=torch.float32, device=qg.device)
    dk = torch.empty((T, p.key_value_heads, p.head_dim), dtype=torch.float32, device=qg.device)
    dv = torch.empty_like(dk)
    size = lib().pluto_hip_gqa_prefill_backward_workspace_bytes(
        ctypes.byref(p), T, int(dq_norm is not None), int(dk_norm is not None))
    workspace = torch.empty(max(size, 1), dtype=torch.uint8, device=qg.device)
    check(lib().pluto_hip_gqa_prefill_backward(
        stream or current_stream(), ctypes.byref(p), T, ptr(qg), ptr(k), ptr(v), ptr(q_norm),
        ptr(k_norm), ptr(dy), ptr(saved), ptr(dqg), ptr(dk), ptr(dv), ptr(dq_norm),
        ptr(dk_norm), ptr(workspace), size))
    return dqg, dk, dv


def gqa_decode_workspace(p, positions, split_tokens=0, device="cuda"):
    batch = len(positions)
    pos = (ctypes.c_int * batch)(*positions)
    size = lib().pluto_hip_gqa_decode_workspace_bytes(ctypes.byref(p), batch, pos, split_tokens)
    return torch.empty(max(size, 1), dtype=torch.uint8, device=device)


def gqa_decode(p, q_gate, k, v, q_norm, k_norm, caches, positions=None, split_tokens=0,
               probabilities=None, workspace=None, out=None, advance=True, stream=None):
    """q_gate [batch, qh, 2, d]; k, v [batch, kh, d] (float32 or bfloat16);
    caches: list of KvCache.  positions default to the caches' own counters,
    which are advanced after a successful call."""
    batch = q_gate.shape[0]
    if positions is None:
        positions = [c.position for c in caches]
    pos = (ctypes.c_int * batch)(*positions)
    views = (KvCacheView * batch)(*[c.view() for c in caches])
    if workspace is None:
        workspace = gqa_decode_workspace(p, positions, split_tokens, q_gate.device)
    if out is None:
        out = torch.empty((batch, p.query_heads, p.head_dim), dtype=q_gate.dtype,
                          device=q_gate.device)
    probs = None
    if probabilities is not None:
        probs = (ctypes.c_void_p * batch)(*[None if t is None else t.data_ptr()
                                             for t in probabilities])
    check(lib().pluto_hip_gqa_decode(stream or current_stream(), ctypes.byref(p), batch,
                                     dtype_code(q_gate), ptr(q_gate), ptr(k), ptr(v),
                                     ptr(q_norm), ptr(k_norm), pos, views, ptr(out), probs,
                                     split_tokens, ptr(workspace), workspace.numel()))
    if advance:
        for c in caches:
            c.position += 1
    return out


def gqa_decode_static(p, q_gate, k, v, q_norm, k_norm, caches, positions, out, split_tokens=0,
                      stream=None):
    """pluto_hip_gqa_decode_static: the decode step on the library's fixed
    scratch.  Nothing is allocated here either: the caller passes `out`."""
    batch = q_gate.shape[0]
    pos = (ctypes.c_int * batch)(*positions)
    views = (KvCacheView * batch)(*[c.view() for c in caches])
    check(lib().pluto_hip_gqa_decode_static(stream or current_stream(), ctypes.byref(p), batch,
                                            dtype_code(q_gate), ptr(q_gate), ptr(k), ptr(v),
                                            ptr(q_norm), ptr(k_norm), pos, views, ptr(out), None,
                                            split_tokens))
    return out


# ---- gated delta-net -----------------------------------------------------------

def delta_params(key_heads=16, value_heads=48, key_head_dim=128, value_head_dim=128,
                 conv_kernel_dim=4, rms_norm_epsilon=1e-6, round_to_bfloat16=True):
    return DeltaParams(key_heads, value_heads, key_head_dim, value_head_dim, conv_kernel_dim,
                       rms_norm_epsilon, int(bool(round_to_bfloat16)))


def gdn_scan_workspace(p, batch, length, chunk=0, device="cuda"):
    size = lib().pluto_hip_gdn_scan_workspace_bytes(ctypes.byref(p), batch, length, chunk)
    return torch.empty(max(size, 16), dtype=torch.uint8, device=device)


def gdn_scan(p, q, k, v, log_decay, beta, state, normalize_qk=False, q_scale=1.0, chunk=0,
             workspace=None, out=None, stream=None):
    """q, k bf16 [B, T, kh, kd]; v bf16 [B, T, vh, vd]; log_decay, beta fp32 [B, T, vh];
    state fp32 [B, vh, kd, vd] (updated in place).  Returns out bf16 [B, T, vh, vd]."""
    batch, length = q.shape[0], q.shape[1]
    if workspace is None:
        workspace = gdn_scan_workspace(p, batch, length, chunk, q.device)
    if out is None:
        out = torch.empty(v.shape, dtype=torch.bfloat16, device=q.device)
    check(lib().pluto_hip_gdn_scan(stream or current_stream(), ctypes.byref(p), batch, length,
                                   chunk, ptr(q), ptr(k), ptr(v), ptr(log_decay), ptr(beta),
                                   int(bool(normalize_qk)), float(q_scale), ptr(state), ptr(out),
                                   ptr(workspace), workspace.numel()))
    return out


def gdn_recurrence(p, q, k, v, log_decay, beta, state, normalize_qk=False, q_scale=1.0,
                   out_dtype=None, stream=None):
    batch, length = q.shape[0], q.shape[1]
    out = torch.empty(v.shape, dtype=out_dtype or torch.bfloat16, device=q.device)
    check(lib().pluto_hip_gdn_recurrence(stream or current_stream(), ctypes.byref(p), batch,
                                         length, ptr(q), ptr(k), ptr(v), ptr(log_decay),
                                         ptr(beta), int(bool(normalize_qk)), float(q_scale),
                                         ptr(state), ptr(out), dtype_code(out)))
    return out


def gdn_layer_forward(p, qkv, z, a, b, conv_weight, a_log, dt_bias, norm, state, stream=None):
    """Whole delta-net layer: qkv bf16 [B, T, channels], z bf16 [B, T, vh*vd], a/b bf16
    [B, T, vh]; state fp32 [B, vh, kd, vd] updated in place.  Returns out bf16 [B, T, vh*vd]."""
    batch, length = qkv.shape[0], qkv.shape[1]
    size = lib().pluto_hip_gdn_layer_workspace_bytes(ctypes.byref(p), batch, length)
    workspace = torch.empty(max(size, 16), dtype=torch.uint8, device=qkv.device)
    out = torch.empty(z.shape, dtype=torch.bfloat16, device=qkv.device)
    check(lib().pluto_hip_gdn_layer_forward(stream or current_stream(), ctypes.byref(p), batch,
                                            length, ptr(qkv), ptr(z), ptr(a), ptr(b),
                                            ptr(conv_weight), ptr(a_log), ptr(dt_bias), ptr(norm),
                                            ptr(state), ptr(out), ptr(workspace), workspace.numel()))
    return out


def gdn_layer_backward(p, qkv, z, a, b, conv_weight, a_log, dt_bias, norm, dy,
                       parameter_grads=None, stream=None):
    """Gradients of gdn_layer_forward (zero initial state) for dy fp32 [B, T, vh*vd].

    Returns (dqkv, dz, da, db), all fp32 with the inputs' shapes.  parameter_grads: optional
    dict with fp32 accumulators "conv_weight", "a_log", "dt_bias", "norm" (any subset)."""
    batch, length = qkv.shape[0], qkv.shape[1]
    grads = parameter_grads or {}
    f32 = dict(dtype=torch.float32, device=qkv.device)
    dqkv, dz = torch.empty(qkv.shape, **f32), torch.empty(z.shape, **f32)
    da, db = torch.empty(a.shape, **f32), torch.empty(b.shape, **f32)
    size = lib().pluto_hip_gdn_layer_backward_workspace_bytes(ctypes.byref(p), length,
                                                              int("norm" in grads))
    workspace = torch.empty(max(size, 16), dtype=torch.uint8, device=qkv.device)
    check(lib().pluto_hip_gdn_layer_backward(
        stream or current_stream(), ctypes.byref(p), batch, length, ptr(qkv), ptr(z), ptr(a),
        ptr(b), ptr(conv_weight), ptr(a_log), ptr(dt_bias), ptr(norm), ptr(dy), ptr(dqkv), ptr(dz),
        ptr(da), ptr(db), ptr(grads.get("conv_weight")), ptr(grads.get("a_log")),
        ptr(grads.get("dt_bias")), ptr(grads.get("norm")), ptr(workspace), size))
    return dqkv, dz, da, db


class DeltaNetStep:
    """Single-token delta-net state (DeltaNetState of the reference): fp32 arrays.
    With batch > 1 it holds that many independent sequences (leading axis of
    every state and activation) advanced by one set of launches."""

    def __init__(self, p, device="cuda", batch=None):
        self.p = p
        self.batch = batch
        lead = () if batch is None else (batch,)
        channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim
        self.conv = torch.zeros(lead + (channels, p.conv_kernel_dim), device=device)
        self.state = torch.zeros(lead + (p.value_heads, p.key_head_dim, p.value_head_dim),
                                 device=device)
        size = lib().pluto_hip_gdn_step_batch_workspace_bytes(ctypes.byref(p), batch or 1)
        self.workspace = torch.empty(max(size, 16), dtype=torch.uint8, device=device)

    def reset(self):
        self.conv.zero_()
        self.state.zero_()

    def step(self, qkv, z, a, b, conv_weight, a_log, dt_bias, norm, stream=None):
        p = self.p
        width = p.value_heads * p.value_head_dim
        if self.batch is None:
            out = torch.empty(width, device=qkv.device)
            check(lib().pluto_hip_gdn_step(
                stream or current_stream(), ctypes.byref(p), ptr(self.conv), ptr(self.state),
                ptr(qkv), ptr(z), ptr(a), ptr(b), ptr(conv_weight), ptr(a_log), ptr(dt_bias),
                ptr(norm), ptr(out), ptr(self.workspace), self.workspace.numel()))
            return out
        # activations and result are FP32 or bf16, all of one type
        out = torch.empty((self.batch, width), device=qkv.device, dtype=qkv.dtype)
        check(lib().pluto_hip_gdn_step_batch(
            stream or current_stream(), ctypes.byref(p), self.batch, dtype_code(qkv), ptr(self.conv),
            ptr(self.state), ptr(qkv), ptr(z), ptr(a), ptr(b), ptr(conv_weight), ptr(a_log),
            ptr(dt_bias), ptr(norm), ptr(out), ptr(self.workspace), self.workspace.numel()))
        return out


def dense_workspace(x, output_dim):
    rows, input_dim = x.shape
    size = lib().pluto_hip_dense_workspace_bytes(dtype_code(x), rows, input_dim, output_dim)
    return torch.empty(max(size, 16), dtype=torch.uint8, device=x.device)


def dense_forward(x, matrix, bias, workspace=None, out=None, stream=None):
    """FullyConnectedLayer forward: x [rows, in] (float32 or bfloat16), matrix
    fp32 [in, out], bias fp32 [out] -> [rows, out] in x's type."""
    rows, input_dim = x.shape
    output_dim = matrix.shape[1]
    if workspace is None:
        workspace = dense_workspace(x, output_dim)
    if out is None:
        out = torch.empty((rows, output_dim), dtype=x.dtype, device=x.device)
    check(lib().pluto_hip_dense_forward(stream or current_stream(), dtype_code(x), ptr(x),
                                        ptr(matrix), ptr(bias), rows, input_dim, output_dim,
                                        ptr(out), ptr(workspace), workspace.numel()))
    return out


def dense_backward(x, matrix, d_out, workspace=None, stream=None):
    """(d_input [rows, in], d_matrix [in, out], d_bias [out]), all fp32."""
    rows, input_dim = x.shape
    output_dim = matrix.shape[1]
    if workspace is None:
        workspace = dense_workspace(x, output_dim)
    dx = torch.empty((rows, input_dim), dtype=torch.float32, device=x.device)
    dw = torch.empty((input_dim, output_dim), dtype=torch.float32, device=x.device)
    db = torch.empty(output_dim, dtype=torch.float32, device=x.device)
    check(lib().pluto_hip_dense_backward(stream or current_stream(), dtype_code(x), ptr(x),
                                         ptr(matrix), ptr(d_out), rows, input_dim, output_dim,
                                         ptr(dx), ptr(dw), ptr(db), ptr(workspace),
                                         workspace.numel()))
    return dx, dw, db


MATRIX_BF16, MATRIX_F32, MATRIX_FP8_E4M3 = 0, 1, 2


def dense_imported_workspace(input_dim, device):
    bytes_needed = lib().pluto_hip_dense_imported_workspace_bytes(input_dim)
    return torch.empty(max(bytes_needed, 1), dtype=torch.uint8, device=device)


def dense_imported_forward(storage, weights, scales, x, workspace=None, out=None, stream=None):
    """Imported FullyConnectedLayer projection of one bf16 token: weights
    [out, in] (bfloat16, float32, or uint8 FP8 E4M3 codes with float32 block
    scales) times x bf16 [in] -> bf16 [out]."""
    output_dim, input_dim = weights.shape
    if workspace is None:
        workspace = dense_imported_workspace(input_dim, x.device)
    if out is None:
        out = torch.empty(output_dim, dtype=torch.bfloat16, device=x.device)
    check(lib().pluto_hip_dense_imported_forward(
        stream or current_stream(), storage, ptr(weights), None if scales is None else ptr(scales),
        ptr(x), input_dim, output_dim, ptr(out), ptr(workspace), workspace.numel()))
    return out


def dense_imported_forward_batch(storage, weights, scales, x, workspace=None, out=None,
                                 stream=None):
    """The imported projection for x bf16 [tokens, in] -> bf16 [tokens, out]."""
    output_dim, input_dim = weights.shape
    tokens = x.shape[0]
    if workspace is None:
        bytes_needed = lib().pluto_hip_dense_imported_batch_workspace_bytes(tokens, input_dim)
        workspace = torch.empty(max(bytes_needed, 1), dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((tokens, output_dim), dtype=torch.bfloat16, device=x.device)
    check(lib().pluto_hip_dense_imported_forward_batch(
        stream or current_stream(), storage, ptr(weights), None if scales is None else ptr(scales),
        ptr(x), tokens, input_dim, output_dim, ptr(out), ptr(workspace), workspace.numel()))
    return out


def dense_imported_forward_many(storage, weights, scales, x, workspace=None, outs=None,
                                stream=None):
    """Several imported projections of the same tokens in one call: weights a list
    of [out_i, in] matrices, scales a list of the same length (entries None unless
    FP8); returns the list of bf16 [tokens, out_i] results."""
    count = len(weights)
    input_dim = weights[0].shape[1]
    tokens = x.shape[0]
    if workspace is None:
        bytes_needed = lib().pluto_hip_dense_imported_batch_workspace_bytes(tokens, input_dim)
        workspace = torch.empty(max(bytes_needed, 1), dtype=torch.uint8, device=x.device)
    if outs is None:
        outs = [torch.empty((tokens, w.shape[0]), dtype=torch.bfloat16, device=x.device)
                for w in weights]
    pointers = ctypes.c_void_p * count
    scale_list = scales if scales is not None else [None] * count
    check(lib().pluto_hip_dense_imported_forward_many(
        stream or current_stream(), storage, count,
        pointers(*[w.data_ptr() for w in weights]),
        pointers(*[None if s is None else s.data_ptr() for s in scale_list]),
        (ctypes.c_int * count)(*[w.shape[0] for w in weights]), ptr(x), tokens, input_dim,
        pointers(*[o.data_ptr() for o in outs]), ptr(workspace), workspace.numel()))
    return outs
