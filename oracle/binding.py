"""ctypes access to the CPU oracle (oracle/psi_oracle.c).  TEST INFRASTRUCTURE ONLY: imported by
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg -- never by the shipped package.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int, c_uint16, c_uint32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libpsi_oracle.so")

F32, BF16, F16 = 0, 1, 2
_lib = None


def build():
    subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = ctypes.CDLL(LIB_PATH)
    lib.psi_oracle_f32_to_bf16.restype = c_uint16
    lib.psi_oracle_f32_to_bf16.argtypes = [c_float]
    lib.psi_oracle_bf16_to_f32.restype = c_float
    lib.psi_oracle_bf16_to_f32.argtypes = [c_uint16]
    lib.psi_oracle_f32_to_f16.restype = c_uint16
    lib.psi_oracle_f32_to_f16.argtypes = [c_float]
    lib.psi_oracle_f16_to_f32.restype = c_float
    lib.psi_oracle_f16_to_f32.argtypes = [c_uint16]
    lib.psi_oracle_convert_from_f32.restype = None
    lib.psi_oracle_convert_from_f32.argtypes = [c_void_p, c_void_p, c_uint64, c_uint32]
    lib.psi_oracle_convert_to_f32.restype = None
    lib.psi_oracle_convert_to_f32.argtypes = [c_void_p, c_void_p, c_uint64, c_uint32]
    lib.psi_oracle_softmax.restype = c_int
    lib.psi_oracle_softmax.argtypes = [c_void_p, c_uint64, c_void_p]
    lib.psi_oracle_projected_gqa.restype = c_int
    lib.psi_oracle_projected_gqa.argtypes = [c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_void_p, c_void_p,
                                             c_void_p, POINTER(c_void_p), POINTER(c_void_p), c_void_p, c_int]
    lib.psi_oracle_tokens_per_page.restype = c_int
    lib.psi_oracle_tokens_per_page.argtypes = [c_uint32, c_uint32, c_uint32, c_uint32, POINTER(c_uint32)]
    lib.psi_oracle_kv_page_write.restype = c_int
    lib.psi_oracle_kv_page_write.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + \
        [c_uint32] * 9
    lib.psi_oracle_gather_context.restype = c_int
    lib.psi_oracle_gather_context.argtypes = [c_void_p, c_void_p] + [c_uint32] * 10 + [c_void_p, c_void_p]
    lib.psi_oracle_paged_gqa.restype = c_int
    lib.psi_oracle_paged_gqa.argtypes = [c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_uint32, c_uint32,
                                         c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int]
    lib.psi_oracle_qgkv_split.restype = c_int
    lib.psi_oracle_qgkv_split.argtypes = [c_void_p] * 5 + [c_uint32] * 5
    lib.psi_oracle_rope_parameters.restype = c_int
    lib.psi_oracle_rope_parameters.argtypes = [c_uint32, c_float, c_int, c_float, c_float, c_float, c_float, c_uint32,
                                               c_int, c_void_p, POINTER(c_float), c_void_p]
    lib.psi_oracle_rms_norm_rope.restype = c_int
    lib.psi_oracle_rms_norm_rope.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32,
                                             c_uint32, c_float, c_void_p, c_float, c_uint32]
    lib.psi_oracle_activation_gate.restype = c_int
    lib.psi_oracle_activation_gate.argtypes = [c_void_p, c_void_p, c_void_p, c_uint64, c_uint32]
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data_as(c_void_p)


def _u32(values):
    return np.ascontiguousarray(np.asarray(values, dtype=np.uint32))


def from_f32(values, dtype):
    """f32 array -> storage array of `dtype` (float32 or uint16 bit patterns)."""
    src = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == F32:
        return src.copy()
    dst = np.empty(src.shape, dtype=np.uint16)
    load().psi_oracle_convert_from_f32(_p(src), _p(dst), src.size, dtype)
    return dst


def to_f32(storage, dtype):
    src = np.ascontiguousarray(storage)
    if dtype == F32:
        return src.astype(np.float32)
    dst = np.empty(src.shape, dtype=np.float32)
    load().psi_oracle_convert_to_f32(_p(src), _p(dst), src.size, dtype)
    return dst


def softmax(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    out = np.empty_like(logits)
    if load().psi_oracle_softmax(_p(logits), logits.size, _p(out)) != 0:
        raise ValueError("softmax reference requires finite positive total")
    return out


def projected_gqa_reference(num_q_heads, num_kv_heads, head_dim, scale, cu_tokens, token_indices, q,
                            context_k_by_req, context_v_by_req, num_threads=1):
    cu, ti = _u32(cu_tokens), _u32(token_indices)
    q = np.ascontiguousarray(q, dtype=np.float32)
    ks = [np.ascontiguousarray(k, dtype=np.float32) for k in context_k_by_req]
    vs = [np.ascontiguousarray(v, dtype=np.float32) for v in context_v_by_req]
    assert len(cu) == len(ti) + 1 and len(ks) == len(ti) and len(vs) == len(ti)
    total = int(cu[-1])
    assert q.size == total * num_q_heads * head_dim
    for r in range(len(ti)):
        ctx = int(ti[r]) + int(cu[r + 1] - cu[r])
        assert ks[r].size == ctx * num_kv_heads * head_dim and vs[r].size == ks[r].size
    out = np.zeros(total * num_q_heads * head_dim, dtype=np.float32)
    kp = (c_void_p * max(len(ks), 1))(*[k.ctypes.data for k in ks])
    vp = (c_void_p * max(len(vs), 1))(*[v.ctypes.data for v in vs])
    rc = load().psi_oracle_projected_gqa(num_q_heads, num_kv_heads, head_dim, scale, len(ti), _p(cu), _p(ti), _p(q),
                                         kp, vp, _p(out), num_threads)
    if rc != 0:
        raise ValueError("projected_gqa_reference rejected its input")
    return out


def tokens_per_page(num_kv_heads, head_dim, page_bytes, dtype):
    out = c_uint32()
    if load().psi_oracle_tokens_per_page(num_kv_heads, head_dim, page_bytes, dtype, ctypes.byref(out)) != 0:
        raise ValueError("GQA page_bytes must be divisible by the K/V bytes per token")
    return out.value


def kv_page_write(pages, flat_k, flat_v, req_slots, flat_token_indices, page_ids, num_active, layer, layout,
                  num_kv_heads, head_dim, page_bytes, dtype):
    """In-place on `pages` (numpy storage array).  layout = (slots, layers, blocks, ids_per_block)."""
    rs, ft, pid = _u32(req_slots), _u32(flat_token_indices), _u32(page_ids)
    rc = load().psi_oracle_kv_page_write(_p(pages), _p(flat_k), _p(flat_v), _p(rs), _p(ft), _p(pid), num_active,
                                         layer, layout[1], layout[2], layout[3], num_kv_heads, head_dim, page_bytes,
                                         dtype)
    if rc != 0:
        raise ValueError("kv_page_write oracle rejected its input")


def gather_context(pages, page_ids, req_slot, layer, context_len, layout, num_kv_heads, head_dim, page_bytes, dtype):
    pid = _u32(page_ids)
    k = np.empty(context_len * num_kv_heads * head_dim, dtype=np.float32)
    v = np.empty_like(k)
    rc = load().psi_oracle_gather_context(_p(pages), _p(pid), req_slot, layer, context_len, layout[1], layout[2],
                                          layout[3], num_kv_heads, head_dim, page_bytes, dtype, _p(k), _p(v))
    if rc != 0:
        raise ValueError("gather_context oracle rejected its input")
    return k, v


def paged_gqa(num_q_heads, num_kv_heads, head_dim, scale, page_bytes, dtype, layout, layer, req_slots_by_req,
              token_indices, cu_tokens, q, pages, page_ids, num_threads=1):
    rs, ti, cu, pid = _u32(req_slots_by_req), _u32(token_indices), _u32(cu_tokens), _u32(page_ids)
    q = np.ascontiguousarray(q)
    out = np.zeros(int(cu[-1]) * num_q_heads * head_dim, dtype=np.float32)
    rc = load().psi_oracle_paged_gqa(num_q_heads, num_kv_heads, head_dim, scale, page_bytes, dtype, layout[0],
                                     layout[1], layout[2], layout[3], layer, len(ti), _p(rs), _p(ti), _p(cu), _p(q),
                                     _p(pages), _p(pid), _p(out), num_threads)
    if rc != 0:
        raise ValueError("paged_gqa oracle rejected its input")
    return out


def _storage(dtype):
    return np.float32 if dtype == F32 else np.uint16


def qgkv_split(qgkv, num_tokens, num_q_heads, num_kv_heads, head_dim, dtype):
    """Storage array [tokens][2*Hq*D + 2*Hkv*D] -> (q, g, k, v) storage arrays."""
    qgkv = np.ascontiguousarray(qgkv, dtype=_storage(dtype))
    q = np.zeros(num_tokens * num_q_heads * head_dim, _storage(dtype))
    g = np.zeros_like(q)
    k = np.zeros(num_tokens * num_kv_heads * head_dim, _storage(dtype))
    v = np.zeros_like(k)
    load().psi_oracle_qgkv_split(_p(qgkv), _p(q), _p(g), _p(k), _p(v), num_tokens, num_q_heads, num_kv_heads, head_dim,
                                 dtype)
    return q, g, k, v


def rope_parameters(rope_dim, rope_theta, yarn=None):
    """yarn: None or dict(factor, attention_factor, beta_fast, beta_slow, original_max_position_embeddings,
    truncate).  Returns (inverse_frequencies f32[rope_dim / 2], attention_factor, (low, high) or None)."""
    inv = np.zeros(rope_dim // 2, np.float32)
    corr = np.zeros(2, np.float32)
    factor = c_float()
    y = yarn or {}
    rc = load().psi_oracle_rope_parameters(
        rope_dim, rope_theta, 1 if yarn else 0, y.get("factor", 1.0), y.get("attention_factor", 1.0),
        y.get("beta_fast", 1.0), y.get("beta_slow", 1.0), y.get("original_max_position_embeddings", 1),
        1 if y.get("truncate", False) else 0, _p(inv), ctypes.byref(factor), _p(corr))
    if rc != 0:
        raise ValueError("rope parameters rejected")
    return inv, factor.value, (tuple(float(x) for x in corr) if yarn else None)


def rms_norm_rope(x, norm_weight_bf16, positions, num_heads, head_dim, rope_dim, eps, inverse_frequencies,
                  attention_factor, dtype):
    """x: storage array [tokens][heads][head_dim]; norm_weight_bf16: uint16[head_dim]; returns a storage array."""
    x = np.ascontiguousarray(x, dtype=_storage(dtype))
    w = np.ascontiguousarray(norm_weight_bf16, dtype=np.uint16)
    pos = _u32(positions)
    inv = np.ascontiguousarray(inverse_frequencies, dtype=np.float32)
    out = x.copy()
    rc = load().psi_oracle_rms_norm_rope(_p(x), _p(w), _p(pos), _p(out), len(pos), num_heads, head_dim, rope_dim, eps,
                                         _p(inv), attention_factor, dtype)
    if rc != 0:
        raise ValueError("rms_norm_rope oracle rejected its input")
    return out


def activation_gate(attention_output, gates, dtype):
    a = np.ascontiguousarray(attention_output, dtype=_storage(dtype)).ravel()
    g = np.ascontiguousarray(gates, dtype=_storage(dtype)).ravel()
    out = np.zeros_like(a)
    load().psi_oracle_activation_gate(_p(a), _p(g), _p(out), a.size, dtype)
    return out
