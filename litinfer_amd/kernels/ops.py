"""Python side of the HIP kernels: argument checks and the ctypes calls.

Every function checks on the host that devices, dtypes, shapes and strides are
what its kernel and launch assume, because a kernel that reads out of bounds
can take the GPU down.  There is no fallback: on a tensor that is not on the
GPU, or without the built library, a call raises.
"""
from __future__ import annotations

import ctypes
import math
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Dict, Optional

import numpy as np
import torch

from . import build
from ..utils.profiler import profiler

float32 = torch.float32
bfloat16 = torch.bfloat16

_DT = {torch.float32: 0, torch.bfloat16: 1}
MAX_HEAD_DIM = 256

P, I, F, L = c_void_p, c_int, c_float, c_long
_SIGNATURES = {
    "elementwise": {
        "li_embedding": [P, P, P, P, I, P, I, I, I],
        "li_rmsnorm": [P, I, P, F, P, I, I, I],
        "li_gather_rows": [P, P, P, I, I],
        "li_cast": [P, I, P, I, L],
        "li_swiglu": [P, P, I, I, I],
        "li_rope_table": [P, F, I, P, P, I],
        "li_rope_apply": [P, I, I, I, I, I, P, P, I],
        "li_kv_store": [P, I, I, I, I, I, P, P, P, I, I, I],
        "li_rope_kv_store": [P, I, I, I, I, I, I, P, P, P, P, P, I, I, I],
        "li_embedding_add": [P, P, P, P, I, P, P, I, I, I],
        "li_rmsnorm_add": [P, P, F, F, P, F, P, P, F, P, I, I, I, I],
        "li_gated_act": [P, I, P, I, I, I, I],
        "li_relu_squared": [P, I, P, I, L],
        "li_gelu_gate_rows": [P, P, P, P, P, I, I, I, I, P, I, I, I],
        "li_rope_freq_table": [P, P, I, F, P, P, I],
        "li_rope_pairs_apply": [P, I, I, I, I, I, P, P, I],
        "li_qk_norm_pairs_store": [P, I, I, I, I, I, I, P, P, F, P, P, P, P, P, I, I, I, I, I],
        "li_latent_norm_pairs_store": [P, L, I, I, I, P, L, I, P, F, P, P, P, P, I, P, I, I, P, L, I, P, P, I, I],
        "li_pair_embedding": [P, P, P, P, P, P, P, P, P, P, P, I, P, I, I, I, I, L, L],
        "li_layernorm": [P, P, P, F, P, I, I, I],
        "li_gelu_tanh": [P, I, P, I, L],
        "li_concat_rows": [P, P, P, I, I, I],
        "li_sinusoid_add": [P, P, P, I, I],
        "li_scale_softcap": [P, L, F, F],
        "li_paged_store": [P, L, I, I, I, P, I, I, I, P, I, I, I, P, I, P, I, I],
        "li_diff_combine": [P, P, I, F, F, F, P, I, L, I],
    },
    "recurrent": {
        "li_causal_conv_silu": [P, L, I, I, P, P, P, P, P, P, P, P, L, I, I, I],
        "li_ssm_scan": [P, L, P, L, P, P, P, P, P, P, P, P, L, I, I, I, I, I, I, I, I, P, L, P, F],
        "li_delta_scan": [P, L, P, L, P, P, P, P, P, P, P, L, I, I, I, I, F, I, I, I, I, P, L],
        "li_gated_group_norm": [P, L, P, L, P, F, P, I, L, I, I, I, I],
    },
    "moe": {
        "li_moe_route": [P, I, L, P, I, P, P, P, P, P, I, I, I, I, I, P, I, I],
        "li_moe_plan": [P, I, I, I, P, I, P, P, I],
        "li_moe_linear": [P, I, L, P, P, I, P, I, P, I, L, I, I, I, F, I, I],
        "li_moe_combine": [P, L, P, L, P, P, P, P, L, I, I, I, P, I, P, I, L],
    },
    "attention_masked": {
        "li_masked_attention": [P, I, I, P, I, P, P, I, I, I, P, I, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, P, L, I],
        "li_masked_attention_single": [P, I, I, P, P, P, I, I, P, I, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, P, L, I, P, L],
        "li_masked_attention_heads": [P, I, I, P, P, P, I, I, P, I, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, P, L, I, P, L],
        "li_masked_attention_tiles": [P, I, I, P, P, P, I, I, P, I, P, I, P, P, P, I, I, I, I, I, I, I, I, F, F, P, P, L, I, P, L, P, I, I],
        "li_headwise_linear": [P, I, L, I, P, I, P, I, L, I, I, I, I, I, P, L, I, I, P, P],
    },
    "gemm": {
        "li_linear": [P, P, P, P, I, I, I, I, I, I, P, L],
        "li_linear_skinny": [P, P, P, P, I, I, I, I, I, I],
        "li_linear_swiglu": [P, P, P, I, I, I, P, I, F],
        "li_linear_swiglu_f32": [P, P, P, I, I, I],
        "li_linear_residual_norm": [P, P, P, P, I, I, I, P, P, P],
        "li_linear_then_norm": [P, P, P, P, I, I, I, P, L, P, F, P, I],
        "li_linear_rope_store": [P, P, P, P, I, I, P, P, P, P, P, I, I, I, I, I, P, I, F],
        "li_linear_rope_store_parts": [P, P, P, P, I, I, P, P, P, P, P, I, I, I, I, I, P, L],
    },
    "attention": {
        "li_paged_attention": [P, I, P, P, P, I, P, I, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, F],
        "li_paged_attention_prefill": [P, I, P, P, P, P, I, P, I, P, P, P, I, I, I, I, I, I, F, I, P, P, P, I],
        "li_paged_attention_prefill_f32": [P, I, P, P, P, P, I, P, I, P, P, P, I, I, I, I, I, I, F],
        "li_paged_attention_decode": [P, I, P, P, P, I, P, I, P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, I, I, P, P],
        "li_decode_run_keys": [P, I, P, P, P, P, I, I, I, I, I, I, I, P],
    },
    "sampling": {
        "li_argmax_rows": [P, P, P, P, I, I],
        "li_sample_rows": [P, P, P, P, P, P, I, I, P, L],
        "li_sample_prepare": [P, I, P, I, P, P, P, P],
    },
}
_fn_cache = {}


def _fn(module: str, name: str):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = build.load(module)
        f = getattr(lib, name)
        f.argtypes = _SIGNATURES[module][name] + [c_void_p]      # + stream
        f.restype = c_int
        _fn_cache[key] = f
    return f


def _work_bytes(m: int, n: int, k: int, dtype: int) -> int:
    f = _fn_cache.get(("gemm", "li_linear_work_bytes"))
    if f is None:
        f = build.load("gemm").li_linear_work_bytes
        f.argtypes, f.restype = [c_int, c_int, c_int, c_int], c_long
        _fn_cache[("gemm", "li_linear_work_bytes")] = f
    return int(f(m, n, k, dtype))


def _sample_scratch_floats(n: int, v: int) -> int:
    f = _fn_cache.get(("sampling", "li_sample_rows_scratch_floats"))
    if f is None:
        f = build.load("sampling").li_sample_rows_scratch_floats
        f.argtypes, f.restype = [c_int, c_int], c_long
        _fn_cache[("sampling", "li_sample_rows_scratch_floats")] = f
    return int(f(n, v))


PREFILL_RUNS_MAX_BYTES = 1 << 30       # room that the runs of a prompt portion's keys may take in the workspace


def _prefill_runs(host_q_len, host_ctx_len, nh: int, nkv: int, dh: int, max_blocks: int, window: int, tokens: int) -> int:
    """How many runs the library cuts the keys of a prompt portion's tiles into (the batch's segments as
    int32 arrays in host memory)."""
    f = _fn_cache.get(("attention", "li_paged_attention_prefill_runs"))
    if f is None:
        f = build.load("attention").li_paged_attention_prefill_runs
        f.argtypes, f.restype = [c_int, c_void_p, c_void_p] + [c_int] * 6 + [c_long], c_int
        _fn_cache[("attention", "li_paged_attention_prefill_runs")] = f
    if host_q_len is None or host_ctx_len is None or host_q_len.dtype != "int32" or host_ctx_len.dtype != "int32":
        return 1
    return int(f(len(host_q_len), host_q_len.ctypes.data, host_ctx_len.ctypes.data, nh, nkv, dh, max_blocks,
                 int(window), tokens, PREFILL_RUNS_MAX_BYTES))


# the current stream's handle without the stream object around it (an op is called some hundred times a
# step, and the object's way through torch's Python layers took a quarter of a step's host time)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _get_device is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _run(module: str, name: str, *args) -> None:
    if profiler.enabled:
        rc = []
        profiler.timed(name[3:], lambda: rc.append(_fn(module, name)(*args, _stream())), torch.cuda.synchronize)
        rc = rc[0]
    else:
        rc = _fn(module, name)(*args, _stream())
    if rc != 0:
        raise RuntimeError(f"{name}: the kernel library refused the call (code {rc}): "
                           f"{_ERRORS.get(rc, 'unknown')}")


_ERRORS = {1: "unsupported dtype combination", 2: "unsupported size", 3: "launch failed"}


def require_gpu(device) -> None:
    if not torch.cuda.is_available():
        raise RuntimeError("litinfer_amd runs on an AMD GPU through its HIP kernels; "
                           "no GPU is visible and there is no CPU path")


def _gpu(*ts) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("kernel call on a tensor that is not on the GPU "
                               "(there is no CPU path)")


def _chk(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _rows_ok(t: torch.Tensor) -> bool:
    return t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1]


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Sizes the attention and position kernels take; anything else is refused
    here, when the model is built."""
    # (the texts are made only when they are needed: these checks run with every call of an op)
    if not (num_heads > 0 and num_kv_heads > 0 and num_heads % num_kv_heads == 0):
        _chk(False, f"attention: {num_heads} heads and {num_kv_heads} kv heads: the first must be a "
                    f"multiple of the second")
    if not (head_dim % 2 == 0 and 2 <= head_dim <= MAX_HEAD_DIM):
        _chk(False, f"attention: head size {head_dim} is not supported (even, at most {MAX_HEAD_DIM})")


# ---------------------------------------------------------------- elementwise
def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor,
              id_src: Optional[torch.Tensor] = None, feedback: Optional[torch.Tensor] = None) -> None:
    """out[t, :] = table[id(t), :] as float32 with id(t) = ids[t], or
    feedback[id_src[t]] where id_src is given and id_src[t] >= 0 (a token chosen
    on the device that the host has not seen yet).  Ids given by the host must
    already be inside the table (the step checks them); an id outside it (one
    that the device chose) gives a row of zeros, never a read outside the table."""
    _gpu(ids, table, out, id_src, feedback)
    t, h = out.shape
    _chk(ids.dtype is torch.int32 and ids.numel() == t and ids.is_contiguous(), "embedding: ids")
    _chk(table.dim() == 2 and table.shape[1] == h and table.is_contiguous() and table.dtype in _DT,
         "embedding: table")
    _chk(out.dtype is torch.float32 and out.is_contiguous(), "embedding: out must be float32")
    _chk(id_src is None or (feedback is not None and id_src.dtype is torch.int32 and id_src.numel() == t
                            and id_src.is_contiguous() and feedback.dtype is torch.int32
                            and feedback.is_contiguous()), "embedding: id_src / feedback")
    if t:
        _run("elementwise", "li_embedding", ids.data_ptr(), 0 if id_src is None else id_src.data_ptr(),
             0 if id_src is None else feedback.data_ptr(), table.data_ptr(), _DT[table.dtype],
             out.data_ptr(), t, h, table.shape[0])


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    _gpu(x, weight, out)
    _chk(x.dim() == 2 and x.shape == out.shape and x.is_contiguous() and out.is_contiguous(),
         "rmsnorm: x and out must be contiguous [T, H] of one shape")
    _chk(x.dtype in _DT and out.dtype in _DT, "rmsnorm: dtype")
    _chk(weight.dtype is torch.float32 and weight.numel() == x.shape[1] and weight.is_contiguous(),
         "rmsnorm: weight must be float32 [H]")
    if x.shape[0]:
        _run("elementwise", "li_rmsnorm", x.data_ptr(), _DT[x.dtype], weight.data_ptr(), float(eps),
             out.data_ptr(), _DT[out.dtype], x.shape[0], x.shape[1])


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """out[i, :] = x[rows[i], :]; rows must be valid row numbers of x."""
    _gpu(x, rows, out)
    _chk(x.dtype is torch.float32 and out.dtype is torch.float32 and x.is_contiguous()
         and out.is_contiguous() and x.dim() == 2 and out.dim() == 2 and x.shape[1] == out.shape[1],
         "gather_rows: x, out")
    _chk(rows.dtype is torch.int32 and rows.numel() == out.shape[0] and rows.is_contiguous(),
         "gather_rows: rows")
    if out.shape[0]:
        _run("elementwise", "li_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(),
             out.shape[0], x.shape[1])


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _gpu(src, dst)
    _chk(src.numel() == dst.numel() and src.is_contiguous() and dst.is_contiguous()
         and src.dtype in _DT and dst.dtype in _DT, "cast: src, dst")
    if src.numel():
        _run("elementwise", "li_cast", src.data_ptr(), _DT[src.dtype], dst.data_ptr(), _DT[dst.dtype],
             src.numel())


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = up * gate / (1 + exp(-gate)) with gate = gate_up[t, i],
    up = gate_up[t, I + i]."""
    _gpu(gate_up, out)
    t, inter = out.shape
    _chk(gate_up.shape == (t, 2 * inter) and gate_up.is_contiguous() and out.is_contiguous()
         and gate_up.dtype is out.dtype and out.dtype in _DT, "swiglu: gate_up [T, 2I], out [T, I]")
    if t:
        _run("elementwise", "li_swiglu", gate_up.data_ptr(), out.data_ptr(), _DT[out.dtype], t, inter)


def rope_table(positions: torch.Tensor, theta: float, rotary_dim: int, cos: torch.Tensor,
               sin: torch.Tensor) -> None:
    """cos/sin [T, rotary_dim/2] of angle = float(pos) / theta^(2j/rotary_dim), in float32."""
    _gpu(positions, cos, sin)
    t = positions.numel()
    _chk(positions.dtype is torch.int32 and positions.is_contiguous(), "rope_table: positions")
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and cos.is_contiguous()
         and sin.is_contiguous() and cos.dtype is torch.float32 and sin.dtype is torch.float32,
         "rope_table: cos, sin")
    if t:
        _run("elementwise", "li_rope_table", positions.data_ptr(), float(theta), rotary_dim,
             cos.data_ptr(), sin.data_ptr(), t)


def _check_qkv(qkv, heads_total, head_dim):
    _chk(_rows_ok(qkv) and qkv.dtype in _DT and qkv.shape[1] >= heads_total * head_dim,
         "qkv: needs rows of at least heads*head_dim elements")


def rope_apply(qkv: torch.Tensor, n_heads: int, head_dim: int, rotary_dim: int, cos: torch.Tensor,
               sin: torch.Tensor) -> None:
    """Rotate heads 0..n_heads-1 of every row of qkv in place (half-split pairs)."""
    _gpu(qkv, cos, sin)
    _check_qkv(qkv, n_heads, head_dim)
    t = qkv.shape[0]
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and rotary_dim <= head_dim,
         "rope_apply: tables")
    if t:
        _run("elementwise", "li_rope_apply", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), n_heads,
             head_dim, rotary_dim, cos.data_ptr(), sin.data_ptr(), t)


def _check_cache(k, v, nkv, dh, page_size, dtype):
    _chk(k.shape == v.shape and k.dim() == 4 and k.shape[1:] == (nkv, page_size, dh)
         and k.is_contiguous() and v.is_contiguous() and k.dtype is dtype and v.dtype is dtype,
         "kv cache: expected contiguous [pages, kv_heads, page_size, head_dim] of the activation dtype")


def kv_store(qkv: torch.Tensor, nh: int, nkv: int, dh: int, slot_map: torch.Tensor, k: torch.Tensor,
             v: torch.Tensor, page_size: int) -> None:
    """Write the key and value heads of every row of qkv (columns nh*dh.. and
    (nh+nkv)*dh..) to the page slot slot_map[t] = page*page_size + offset."""
    _gpu(qkv, slot_map, k, v)
    _check_qkv(qkv, nh + 2 * nkv, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == t and slot_map.is_contiguous(),
         "kv_store: slot_map")
    if t:
        _run("elementwise", "li_kv_store", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), nh, nkv, dh,
             slot_map.data_ptr(), k.data_ptr(), v.data_ptr(), page_size, k.shape[0], t)


def rope_kv_store(qkv: torch.Tensor, nh: int, nkv: int, dh: int, rotary_dim: int, cos: torch.Tensor,
                  sin: torch.Tensor, slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  page_size: int) -> None:
    """Fused: rotate the query heads in place, rotate the key heads and write
    them, and copy the value heads, to the pages."""
    _gpu(qkv, cos, sin, slot_map, k, v)
    _check_qkv(qkv, nh + 2 * nkv, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and rotary_dim <= dh
         and cos.dtype is torch.float32, "rope_kv_store: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == t and slot_map.is_contiguous(),
         "rope_kv_store: slot_map")
    if t:
        _run("elementwise", "li_rope_kv_store", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), nh, nkv,
             dh, rotary_dim, cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(),
             v.data_ptr(), page_size, k.shape[0], t)


def _ids_ok(ids, id_src, feedback, t) -> bool:
    return (ids.dtype is torch.int32 and ids.numel() == t and ids.is_contiguous()
            and (id_src is None or (feedback is not None and id_src.dtype is torch.int32 and id_src.numel() == t
                                    and id_src.is_contiguous() and feedback.dtype is torch.int32
                                    and feedback.is_contiguous())))


def embedding_add(out: torch.Tensor, ids: Optional[torch.Tensor] = None, table: Optional[torch.Tensor] = None,
                  vec: Optional[torch.Tensor] = None, id_src: Optional[torch.Tensor] = None,
                  feedback: Optional[torch.Tensor] = None) -> None:
    """out[t, :] += table[id(t), :] (if a table is given) + vec[:] (if given), in float32; ids as in
    `embedding` (an id outside the table adds nothing)."""
    _gpu(out, ids, table, vec, id_src, feedback)
    t, h = out.shape
    _chk(out.dtype is torch.float32 and out.is_contiguous(), "embedding_add: out must be float32")
    _chk(table is None or (ids is not None and table.dim() == 2 and table.shape[1] == h and table.is_contiguous()
                           and table.dtype in _DT and _ids_ok(ids, id_src, feedback, t)), "embedding_add: table, ids")
    _chk(vec is None or (vec.dtype is torch.float32 and vec.numel() == h and vec.is_contiguous()), "embedding_add: vec")
    if t and (table is not None or vec is not None):
        if table is None:
            ids = id_src = feedback = None
        _run("elementwise", "li_embedding_add", 0 if ids is None else ids.data_ptr(), 0 if id_src is None else id_src.data_ptr(),
             0 if id_src is None else feedback.data_ptr(), 0 if table is None else table.data_ptr(),
             _DT[table.dtype] if table is not None else 0, 0 if vec is None else vec.data_ptr(), out.data_ptr(), t, h,
             table.shape[0] if table is not None else 0)


def rmsnorm_add(y: torch.Tensor, weight: torch.Tensor, eps: float, x: torch.Tensor,
                next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0,
                next_out: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
                factors=(1.0, 1.0)) -> None:
    """x += b / sqrt(mean(b^2) + eps) * weight, row by row, in float32, for the branch b = y or, with `y2`,
    b = factors[0] * y + factors[1] * y2; with `next_weight` also next_out = the RMS norm of the new x with those
    weights and `next_eps`; with `next_out` alone, next_out = the new x in next_out's type."""
    _gpu(y, weight, x, next_weight, next_out, y2)
    _chk(y.dim() == 2 and y.shape == x.shape and y.is_contiguous() and x.is_contiguous()
         and y.dtype is torch.float32 and x.dtype is torch.float32, "rmsnorm_add: y and x must be contiguous float32 [T, H]")
    _chk(y2 is None or (y2.shape == x.shape and y2.is_contiguous() and y2.dtype is torch.float32), "rmsnorm_add: the second branch")
    h = x.shape[1]
    _chk(weight.dtype is torch.float32 and weight.numel() == h and weight.is_contiguous(), "rmsnorm_add: weight")
    if next_weight is not None:
        _chk(next_out is not None and next_weight.dtype is torch.float32 and next_weight.numel() == h and next_weight.is_contiguous(),
             "rmsnorm_add: the next norm's weight and out")
    if next_out is not None:
        _chk(next_out.shape == x.shape and next_out.is_contiguous() and next_out.dtype in _DT, "rmsnorm_add: out of the next reader")
    nxt = 0 if next_out is None else 1 if next_weight is not None else 2
    if x.shape[0]:
        _run("elementwise", "li_rmsnorm_add", y.data_ptr(), 0 if y2 is None else y2.data_ptr(), float(factors[0]), float(factors[1]),
             weight.data_ptr(), float(eps), x.data_ptr(), 0 if next_weight is None else next_weight.data_ptr(), float(next_eps),
             0 if next_out is None else next_out.data_ptr(), _DT[next_out.dtype] if next_out is not None else 0, nxt, x.shape[0], h)


def gated_act(gate_up: torch.Tensor, out: torch.Tensor, act: str) -> None:
    """out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]; act "silu" or "gelu_tanh"; float32 arithmetic; gate_up in
    float32 or the engine's dtype, out in the engine's."""
    _gpu(gate_up, out)
    t, i = out.shape
    _chk(act in ("silu", "gelu_tanh"), "gated_act: act")
    _chk(gate_up.shape == (t, 2 * i) and gate_up.is_contiguous() and out.is_contiguous() and gate_up.dtype in _DT and out.dtype in _DT
         and (gate_up.dtype is torch.float32 or out.dtype is torch.bfloat16), "gated_act: gate_up [T, 2 I], out [T, I]")
    if t:
        _run("elementwise", "li_gated_act", gate_up.data_ptr(), _DT[gate_up.dtype], out.data_ptr(), _DT[out.dtype], t, i,
             1 if act == "gelu_tanh" else 0)


def relu_squared(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = max(x, 0)^2."""
    _gpu(x, out)
    _chk(x.shape == out.shape and x.is_contiguous() and out.is_contiguous() and x.dtype in _DT and out.dtype in _DT
         and (x.dtype is torch.float32 or out.dtype is x.dtype), "relu_squared: x, out")
    if x.numel():
        _run("elementwise", "li_relu_squared", x.data_ptr(), _DT[x.dtype], out.data_ptr(), _DT[out.dtype], x.numel())


def gelu_gate_rows(a: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, offset: int, out: torch.Tensor,
                   id_src: Optional[torch.Tensor] = None, feedback: Optional[torch.Tensor] = None) -> None:
    """out[t, j] = gelu_tanh(a[t, j]) * table[id(t), offset + j]."""
    _gpu(a, ids, table, out, id_src, feedback)
    t, n = a.shape
    _chk(a.dtype is torch.float32 and a.is_contiguous() and out.shape == a.shape and out.is_contiguous()
         and out.dtype in _DT, "gelu_gate_rows: a float32 [T, n], out [T, n]")
    _chk(table.dim() == 2 and table.is_contiguous() and table.dtype in _DT and 0 <= offset
         and offset + n <= table.shape[1] and _ids_ok(ids, id_src, feedback, t), "gelu_gate_rows: table, ids")
    if t:
        _run("elementwise", "li_gelu_gate_rows", a.data_ptr(), ids.data_ptr(), 0 if id_src is None else id_src.data_ptr(),
             0 if id_src is None else feedback.data_ptr(), table.data_ptr(), _DT[table.dtype], table.shape[1], int(offset),
             table.shape[0], out.data_ptr(), _DT[out.dtype], t, n)


def rope_freq_table(positions: torch.Tensor, freq: torch.Tensor, amplitude: float, cos: torch.Tensor,
                    sin: torch.Tensor) -> None:
    """cos/sin [T, n] of angle = float(pos) * freq[i], times `amplitude`, in float32."""
    _gpu(positions, freq, cos, sin)
    t, n = positions.numel(), freq.numel()
    _chk(positions.dtype is torch.int32 and positions.is_contiguous() and freq.dtype is torch.float32
         and freq.is_contiguous(), "rope_freq_table: positions, freq")
    _chk(cos.shape == (t, n) and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous()
         and cos.dtype is torch.float32 and sin.dtype is torch.float32, "rope_freq_table: cos, sin")
    if t:
        _run("elementwise", "li_rope_freq_table", positions.data_ptr(), freq.data_ptr(), n, float(amplitude),
             cos.data_ptr(), sin.data_ptr(), t)


def rope_pairs_apply(qkv: torch.Tensor, n_heads: int, head_dim: int, rotary_dim: int, cos: torch.Tensor,
                     sin: torch.Tensor) -> None:
    """Rotate heads 0..n_heads-1 of every row in place, neighbouring columns (2i, 2i+1) forming a pair."""
    _gpu(qkv, cos, sin)
    _check_qkv(qkv, n_heads, head_dim)
    t = qkv.shape[0]
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and rotary_dim <= head_dim
         and cos.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), "rope_pairs_apply: tables")
    if t:
        _run("elementwise", "li_rope_pairs_apply", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), n_heads, head_dim,
             rotary_dim, cos.data_ptr(), sin.data_ptr(), t)


def _check_tables(what, t, rotary_dim, cos, sin, slot_map):
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and cos.dtype is torch.float32
         and sin.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), f"{what}: tables")
    _chk(slot_map is None or (slot_map.dtype is torch.int32 and slot_map.numel() == t and slot_map.is_contiguous()),
         f"{what}: slot_map")


def qk_norm_pairs_store(qkv: torch.Tensor, nh: int, nkv: int, dk: int, dv: int, rotary_dim: int,
                        wq: Optional[torch.Tensor], wk: Optional[torch.Tensor], eps: float, cos: torch.Tensor,
                        sin: torch.Tensor, slot_map: Optional[torch.Tensor], k: Optional[torch.Tensor],
                        v: Optional[torch.Tensor], page_size: int, half_split: bool = False) -> None:
    """qkv float32 rows [q (nh*dk) | k (nkv*dk) | v (nkv*dv)].  q and k are RMS-normed over their WHOLE
    width (weights wq, wk; None: no norm), their heads' first `rotary_dim` columns rotated in neighbouring
    pairs (`half_split`: column i with column i + rotary_dim / 2); q stays in place, k and v go to their page slots (k None: only q is prepared)."""
    _gpu(qkv, wq, wk, cos, sin, slot_map, k, v)
    t = qkv.shape[0]
    _chk(_rows_ok(qkv) and qkv.dtype is torch.float32 and qkv.shape[1] >= nh * dk + nkv * (dk + dv),
         "qk_norm_pairs_store: qkv must be float32 rows of q, k and v")
    _chk(rotary_dim % 2 == 0 and 0 <= rotary_dim <= dk, "qk_norm_pairs_store: rotary_dim")
    _check_tables("qk_norm_pairs_store", t, rotary_dim, cos, sin, slot_map if k is not None else None)
    for w_, n_ in ((wq, nh * dk), (wk, nkv * dk)):
        _chk(w_ is None or (w_.dtype is torch.float32 and w_.numel() == n_ and w_.is_contiguous()),
             "qk_norm_pairs_store: norm weights")
    if k is not None:
        _chk(k.dim() == 4 and v.dim() == 4 and k.shape[1:] == (nkv, page_size, dk) and v.shape[1:] == (nkv, page_size, dv)
             and k.shape[0] == v.shape[0] and k.is_contiguous() and v.is_contiguous() and k.dtype is v.dtype
             and k.dtype in _DT and slot_map is not None, "qk_norm_pairs_store: cache")
    if t:
        _run("elementwise", "li_qk_norm_pairs_store", qkv.data_ptr(), qkv.stride(0), nh, nkv, dk, dv, rotary_dim,
             0 if wq is None else wq.data_ptr(), 0 if wk is None else wk.data_ptr(), float(eps), cos.data_ptr(),
             sin.data_ptr(), 0 if k is None else slot_map.data_ptr(), 0 if k is None else k.data_ptr(),
             0 if k is None else v.data_ptr(), _DT[k.dtype] if k is not None else 0, page_size, int(k is not None),
             int(bool(half_split)), t)


def latent_norm_pairs_store(qd: Optional[torch.Tensor], nh: int, dn: int, dr: int, rank: int, wc: torch.Tensor, eps: float,
                            cos: torch.Tensor, sin: torch.Tensor, slot_map: Optional[torch.Tensor],
                            cache: Optional[torch.Tensor], qfull: Optional[torch.Tensor], down: Optional[torch.Tensor] = None,
                            half_split: bool = False, q_latent: Optional[torch.Tensor] = None,
                            wq: Optional[torch.Tensor] = None, cq: Optional[torch.Tensor] = None) -> None:
    """qd float32 rows [q (nh x (dn + dr)) | latent (rank) | shared rotated key part (dr)]; with `down` (float32 rows
    [latent | shared part], which may be a view of columns inside a wider buffer) qd holds the queries alone, and may
    be None: then no query is touched.  The latent is RMS-normed and written with the rotated shared part to the
    token's page row [rank + dr]; every query head's rotated part goes to columns rank.. of its row in qfull
    [T, nh, rank + dr] (float32).  Pairs are neighbouring columns, or column i with column i + dr/2 (`half_split`).
    With `q_latent` (float32 rows, a view is fine) also cq = the RMS norm of those rows with weights wq."""
    _gpu(qd, wc, cos, sin, slot_map, cache, qfull, down, q_latent, wq, cq)
    t = cos.shape[0]
    if qd is None:
        nh = 0
    if nh:
        need = nh * (dn + dr) + (0 if down is not None else rank + dr)
        _chk(_rows_ok(qd) and qd.dtype is torch.float32 and qd.shape[0] == t and qd.shape[1] >= need, "latent_norm_pairs_store: qd")
        _chk(qfull is not None and qfull.shape == (t, nh, rank + dr) and qfull.is_contiguous() and qfull.dtype is torch.float32,
             "latent_norm_pairs_store: qfull")
    if down is None and nh:
        down = qd[:, nh * (dn + dr):]
    _chk(dr % 2 == 0 and dr > 0, "latent_norm_pairs_store: the rotated size must be even")
    _check_tables("latent_norm_pairs_store", t, dr, cos, sin, slot_map if cache is not None else None)
    _chk(wc.dtype is torch.float32 and wc.numel() == rank and wc.is_contiguous(), "latent_norm_pairs_store: norm weight")
    if cache is not None:
        _chk(down is not None and _rows_ok(down) and down.dtype is torch.float32 and down.shape == (t, rank + dr),
             "latent_norm_pairs_store: the rows of latent and shared key part")
        _chk(cache.dim() == 4 and cache.shape[1] == 1 and cache.shape[3] == rank + dr and cache.is_contiguous()
             and cache.dtype in _DT and slot_map is not None, "latent_norm_pairs_store: cache [pages, 1, page, rank + dr]")
    q_rank = 0
    if q_latent is not None:
        q_rank = q_latent.shape[1]
        _chk(_rows_ok(q_latent) and q_latent.dtype is torch.float32 and q_latent.shape[0] == t and q_rank > 0
             and wq is not None and wq.dtype is torch.float32 and wq.numel() == q_rank and wq.is_contiguous()
             and cq is not None and cq.shape == (t, q_rank) and cq.is_contiguous() and cq.dtype in _DT,
             "latent_norm_pairs_store: the queries' latent, its norm weight and its output")
    if t and (nh or cache is not None or q_rank):
        _run("elementwise", "li_latent_norm_pairs_store", qd.data_ptr() if nh else 0, qd.stride(0) if nh else 0, nh, dn, dr,
             down.data_ptr() if cache is not None else 0, down.stride(0) if cache is not None else 0, rank, wc.data_ptr(),
             float(eps), cos.data_ptr(), sin.data_ptr(), 0 if cache is None else slot_map.data_ptr(),
             0 if cache is None else cache.data_ptr(), _DT[cache.dtype] if cache is not None else 0,
             qfull.data_ptr() if nh else 0, int(cache is not None), int(bool(half_split)),
             q_latent.data_ptr() if q_rank else 0, q_latent.stride(0) if q_rank else 0, q_rank,
             wq.data_ptr() if q_rank else 0, cq.data_ptr() if q_rank else 0, _DT[cq.dtype] if q_rank else 0, t)


def pair_embedding(ids: torch.Tensor, table: torch.Tensor, pair: torch.Tensor, out: torch.Tensor, positions: torch.Tensor,
                   seg_of_token: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
                   last: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int,
                   id_src: Optional[torch.Tensor] = None, feedback: Optional[torch.Tensor] = None) -> None:
    """out[t, :] = table[id(t), :] + pair[row(t), :] as float32, row(t) = (prev * mul_prev + id * mul_cur) mod buckets
    with prev the id of the token before t in its request, and the last row (number `buckets`) for a request's first
    token.  `last` [slots] int32 holds every live request's last token between steps and is brought up to date;
    the other arrays are the step's (segment of a token, a segment's first token, its length, its slot)."""
    _gpu(ids, table, pair, out, positions, seg_of_token, q_start, q_len, slots, last, id_src, feedback)
    t, h = out.shape
    nseg = q_start.numel()
    _chk(out.dtype is torch.float32 and out.is_contiguous() and _ids_ok(ids, id_src, feedback, t), "pair_embedding: out, ids")
    _chk(table.dim() == 2 and table.shape[1] == h and table.is_contiguous() and table.dtype in _DT
         and pair.shape == (buckets + 1, h) and pair.is_contiguous() and pair.dtype is table.dtype and buckets > 0
         and mul_prev >= 0 and mul_cur >= 0, "pair_embedding: the tables")
    for a_, n_ in ((positions, t), (seg_of_token, t), (q_start, nseg), (q_len, nseg), (slots, nseg)):
        _chk(a_.dtype is torch.int32 and a_.numel() == n_ and a_.is_contiguous(), "pair_embedding: the step's index arrays")
    _chk(last.dtype is torch.int32 and last.is_contiguous() and last.dim() == 1, "pair_embedding: the last tokens")
    if t:
        _run("elementwise", "li_pair_embedding", ids.data_ptr(), 0 if id_src is None else id_src.data_ptr(),
             0 if id_src is None else feedback.data_ptr(), positions.data_ptr(), seg_of_token.data_ptr(), q_start.data_ptr(),
             q_len.data_ptr(), slots.data_ptr(), last.data_ptr(), table.data_ptr(), pair.data_ptr(), _DT[table.dtype],
             out.data_ptr(), t, h, table.shape[0], int(buckets), int(mul_prev), int(mul_cur))


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float, out: torch.Tensor) -> None:
    """out = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias, row by row, in float32."""
    _gpu(x, weight, bias, out)
    _chk(x.dim() == 2 and x.shape == out.shape and x.is_contiguous() and out.is_contiguous() and x.dtype is torch.float32
         and out.dtype in _DT, "layernorm: x float32 and out must be contiguous [T, H] of one shape")
    for w_ in (weight, bias):
        _chk(w_ is None or (w_.dtype is torch.float32 and w_.numel() == x.shape[1] and w_.is_contiguous()),
             "layernorm: weight and bias must be float32 [H]")
    if x.shape[0]:
        _run("elementwise", "li_layernorm", x.data_ptr(), weight.data_ptr(), 0 if bias is None else bias.data_ptr(), float(eps),
             out.data_ptr(), _DT[out.dtype], x.shape[0], x.shape[1])


def gelu_tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))."""
    _gpu(x, out)
    _chk(x.shape == out.shape and x.is_contiguous() and out.is_contiguous() and x.dtype in _DT and out.dtype in _DT
         and (x.dtype is torch.float32 or out.dtype is x.dtype), "gelu_tanh: x, out")
    if x.numel():
        _run("elementwise", "li_gelu_tanh", x.data_ptr(), _DT[x.dtype], out.data_ptr(), _DT[out.dtype], x.numel())


def concat_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, :] = [a[t, :] | b[t, :]] for float32 a and b [T, H], in the dtype of out [T, 2H]."""
    _gpu(a, b, out)
    t, h = a.shape
    _chk(a.dtype is torch.float32 and b.dtype is torch.float32 and b.shape == a.shape and a.is_contiguous() and b.is_contiguous()
         and out.shape == (t, 2 * h) and out.is_contiguous() and out.dtype in _DT, "concat_rows: a, b [T, H] float32, out [T, 2H]")
    if t:
        _run("elementwise", "li_concat_rows", a.data_ptr(), b.data_ptr(), out.data_ptr(), _DT[out.dtype], t, h)


_CUS: Dict[int, int] = {}


def _compute_units(device: torch.device) -> int:
    idx = device.index or 0
    if idx not in _CUS:
        _CUS[idx] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _CUS[idx]



def _single_blocks(n: int, nh: int, nkv: int, dk: int, dv: int) -> int:
    f = _fn_cache.get(("attention_masked", "li_masked_attention_single_blocks"))
    if f is None:
        f = build.load("attention_masked").li_masked_attention_single_blocks
        f.argtypes, f.restype = [c_int] * 5, c_int
        _fn_cache[("attention_masked", "li_masked_attention_single_blocks")] = f
    return max(1, int(f(n, nh, nkv, dk, dv)))


def masked_attention(q: torch.Tensor, q_token_stride: int, q_head_stride: int, out: torch.Tensor, k: torch.Tensor,
                     v: torch.Tensor, meta, nh: int, nkv: int, dk: int, dv: int, page_size: int, window: int,
                     keep_first: int, softcap: float, scale: float, ws=None, sink: Optional[torch.Tensor] = None,
                     head_gate: Optional[torch.Tensor] = None) -> None:
    """Attention of every token of the step over its request's cached keys: position p sees j <= p with
    p - j < window (0: all) or j < keep_first; scores (q . k) * scale, then softcap * tanh(score / softcap)
    where softcap > 0; softmax and sums in float32.  q: a float32 tensor in which head h of token t starts at
    t * q_token_stride + h * q_head_stride; k [pages, nkv, page, >= dk] and v [pages, nkv, page, >= dv] (the two
    may be one tensor: then the value is the first dv columns of the key's row); out [T, nh * dv].
    `sink` (float32 [nh]): the softmax's denominator also holds exp(sink[head]), a term without key or value.
    `head_gate` (float32 rows [T, nh], a view of columns is fine): head h's output of token t is multiplied by
    sigmoid(head_gate[t, h])."""
    _gpu(q, out, k, v, meta.block_table, sink, head_gate)
    t = out.shape[0]
    _chk(q.dtype is torch.float32 and q.is_contiguous() and q.numel() >= (t - 1) * q_token_stride + (nh - 1) * q_head_stride + dk,
         "masked_attention: q")
    _chk(out.shape == (t, nh * dv) and out.is_contiguous() and out.dtype in _DT, "masked_attention: out")
    _chk(k.dim() == 4 and v.dim() == 4 and k.shape[:3] == (k.shape[0], nkv, page_size) and v.shape[:3] == k.shape[:3]
         and k.shape[3] >= dk and v.shape[3] >= dv and k.is_contiguous() and v.is_contiguous() and k.dtype is v.dtype
         and k.dtype in _DT and (out.dtype is k.dtype or out.dtype is torch.float32), "masked_attention: cache")
    _chk(nh % nkv == 0 and meta.num_tokens == t and meta.block_table.shape == (meta.num_segments, meta.max_blocks),
         "masked_attention: batch")
    _chk(sink is None or (sink.dtype is torch.float32 and sink.numel() == nh and sink.is_contiguous()), "masked_attention: sink")
    _chk(head_gate is None or (head_gate.dtype is torch.float32 and _rows_ok(head_gate) and head_gate.shape == (t, nh)),
         "masked_attention: head_gate")
    fin = (0 if sink is None else sink.data_ptr(), 0 if head_gate is None else head_gate.data_ptr(),
           0 if head_gate is None else head_gate.stride(0))
    if not t:
        return
    # keys that one query may see, as far as the host knows without looking at the contexts (a recorded step
    # must not depend on them): decides how many waves share a (token, head)'s keys in the general kernel
    bound = window + keep_first if window else meta.max_blocks * page_size
    waves = 8 if bound >= 512 else 4 if bound >= 128 else 1

    def general(token_list, n):
        _run("attention_masked", "li_masked_attention", q.data_ptr(), int(q_token_stride), int(q_head_stride),
             out.data_ptr(), _DT[out.dtype], k.data_ptr(), v.data_ptr(), _DT[k.dtype], k.shape[3], v.shape[3],
             meta.block_table.data_ptr(), meta.max_blocks, 0 if token_list is None else token_list.data_ptr(), n,
             meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dk, dv, page_size, k.shape[0], int(window), int(keep_first), float(softcap or 0.0), float(scale), *fin, waves)

    fast = (k.dtype is torch.bfloat16 and out.dtype is torch.bfloat16 and k.shape[3] % 8 == 0 and v.shape[3] % 8 == 0
            and q_token_stride % 4 == 0 and q_head_stride % 4 == 0 and q.data_ptr() % 16 == 0)

    def singles(token_list, n):
        # single tokens in bfloat16, at the sizes it has: rows spread over lanes, a row read once for a group's heads
        if fast and ws is not None and masked_tiles_take(dk, dv) and _heads_kernel_pays(n, nh // nkv, dk, dv):
            # many query heads on one kv head (a compressed cache: all of them): the heads are the columns of
            # matrix-core tiles, one wave a (token, kv head, 32 heads, split of the keys)
            blocks = n * nkv * -(-(nh // nkv) // 32)
            nsplit = max(1, min(3 * _compute_units(q.device) // blocks, bound // 64, 32))
            parts, parts_n = 0, 0
            if nsplit > 1:
                buf = ws.buffer("masked_attention.parts", (n * nh * nsplit * (dv + 2),), torch.float32)
                parts, parts_n = buf.data_ptr(), buf.numel()
            return _run("attention_masked", "li_masked_attention_heads", q.data_ptr(), int(q_token_stride),
                        int(q_head_stride), out.data_ptr(), k.data_ptr(), v.data_ptr(), k.shape[3], v.shape[3],
                        meta.block_table.data_ptr(), meta.max_blocks, 0 if token_list is None else token_list.data_ptr(), n,
                        meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
                        nh, nkv, dk, dv, page_size, k.shape[0], int(window), int(keep_first), float(softcap or 0.0),
                        float(scale), *fin, nsplit, parts, parts_n)
        if not (fast and masked_single_takes(dk, dv)):
            return general(token_list, n)
        # few blocks against many keys: the keys are cut into splits, each a block of its own, and joined by a second
        # kernel (the number follows the table's width or the window, not the contexts: a recorded step keeps it)
        blocks = _single_blocks(n, nh, nkv, dk, dv)
        # (whole rounds of blocks over the compute units: a block of this kernel is a chain of dependent trips to memory,
        # and a second round of a few blocks costs as much as the first)
        nsplit = max(1, min(_compute_units(q.device) * (1 if -(-dk // 64) + -(-dv // 64) > 6 else 2) // blocks,
                             bound // 128, 32)) if ws is not None else 1
        parts, parts_n = 0, 0
        if nsplit > 1:
            buf = ws.buffer("masked_attention.parts", (n * nh * nsplit * (dv + 2),), torch.float32)
            parts, parts_n = buf.data_ptr(), buf.numel()
        _run("attention_masked", "li_masked_attention_single", q.data_ptr(), int(q_token_stride), int(q_head_stride),
             out.data_ptr(), k.data_ptr(), v.data_ptr(), k.shape[3], v.shape[3], meta.block_table.data_ptr(), meta.max_blocks,
             0 if token_list is None else token_list.data_ptr(), n, meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(),
             meta.q_len.data_ptr(), meta.ctx_len.data_ptr(), nh, nkv, dk, dv, page_size, k.shape[0], int(window),
             int(keep_first), float(softcap or 0.0), float(scale), *fin, nsplit, parts, parts_n)

    if meta.num_single == t and not meta.num_multi:
        return singles(None, t)                                 # a decoding step
    # portions of prompts in bfloat16, at the sizes it has: tiles of queries on the matrix cores
    if (fast and meta.tiles is not None and meta.num_tiles and meta.tile_rows == MASKED_TILE_ROWS and masked_tiles_take(dk, dv)
            and meta.num_single + meta.num_multi == t):
        # few tiles (one prompt of a model with few kv heads): a wave's own chain of matrix products and softmax sets
        # the time of a block of keys, so the waves must fill the chip: a tile's blocks of keys are cut into splits,
        # each a block of its own, and joined by the kernel that joins single tokens' splits
        rep = nh // nkv
        nw = 8 if rep > 4 and (rep <= 8 or rep % 8 == 0 or rep % 8 > 4) else 4
        waves = meta.num_tiles * nkv * -(-rep // nw) * nw
        slots = (8 if dk + dv <= 384 else 4) * _compute_units(q.device)      # waves the chip holds of this kernel (its registers)
        nsplit = max(1, min(slots // waves, bound // 128, 4)) if ws is not None else 1
        n_multi = meta.num_multi or t
        parts, parts_n = 0, 0
        if nsplit > 1:
            buf = ws.buffer("masked_attention.parts", (t * nh * nsplit * (dv + 2),), torch.float32)
            parts, parts_n = buf.data_ptr(), buf.numel()
        _run("attention_masked", "li_masked_attention_tiles", q.data_ptr(), int(q_token_stride), int(q_head_stride),
             out.data_ptr(), k.data_ptr(), v.data_ptr(), k.shape[3], v.shape[3], meta.block_table.data_ptr(), meta.max_blocks,
             meta.tiles.data_ptr(), meta.num_tiles, meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dk, dv, page_size, k.shape[0], int(window), int(keep_first), float(softcap or 0.0), float(scale),
             *fin, nsplit, parts, parts_n, 0 if meta.multi_tokens is None else meta.multi_tokens.data_ptr(), n_multi, t)
        if meta.num_single:
            singles(meta.single_tokens, meta.num_single)       # (a list is there: the batch has tokens of both kinds)
        return
    general(None, t)


# Single tokens on the matrix cores (the heads of a kv head as a tile's columns) or on the vector ALU.  Measured on
# 8 / 64 / 256 requests of 1,028 visible keys (us a call, vector against matrix cores): rows of 128 + 128 columns,
# 28 heads on 4 kv heads 46/20, 84/49, 324/127; 12 on 2: 19/19, 36/33, 152/107; rows of 320 columns shared by keys and
# values (a compressed cache), 28 heads: 28/38, 144/112, 494/396; 12 heads: 21/36, 74/107, 225/381 (there one wave
# stages 36 KB a block of keys by itself, which sets its time whatever the heads).
# One and two requests: 28 on 4: 25/24, 24/24; 12 on 2: 19/23, 18/23; the long rows 20/40.
MASKED_HEADS_MIN = 4          # query heads a kv head from which rows of up to 384 columns (keys + values) take the matrix cores,
MASKED_HEADS_MIN_PAIRS = 48   # for at least so many (token, head) pairs a kv head
MASKED_HEADS_MIN_LONG = 24    # ... and from which longer rows do, for at least MASKED_HEADS_MIN_WORK (token, head) pairs a kv head
MASKED_HEADS_MIN_WORK = 1024


def _heads_kernel_pays(n: int, rep: int, dk: int, dv: int) -> bool:
    if dk + dv <= 384:
        return rep >= MASKED_HEADS_MIN and n * rep >= MASKED_HEADS_MIN_PAIRS
    return rep >= MASKED_HEADS_MIN_LONG and n * rep >= MASKED_HEADS_MIN_WORK


MASKED_TILE_ROWS = 32         # queries of one request that a block of the matrix-core kernel takes


def masked_single_takes(dk: int, dv: int) -> bool:
    """Whether the kernel for single tokens has these key and value sizes (bfloat16)."""
    f = _fn_cache.get(("attention_masked", "li_masked_attention_single_takes"))
    if f is None:
        f = build.load("attention_masked").li_masked_attention_single_takes
        f.argtypes, f.restype = [c_int, c_int], c_int
        _fn_cache[("attention_masked", "li_masked_attention_single_takes")] = f
    return bool(f(int(dk), int(dv)))


def masked_tiles_take(dk: int, dv: int) -> bool:
    """Whether the matrix-core kernel for portions has these key and value sizes (bfloat16)."""
    f = _fn_cache.get(("attention_masked", "li_masked_attention_tiles_takes"))
    if f is None:
        f = build.load("attention_masked").li_masked_attention_tiles_takes
        f.argtypes, f.restype = [c_int, c_int], c_int
        _fn_cache[("attention_masked", "li_masked_attention_tiles_takes")] = f
    return bool(f(int(dk), int(dv)))


def headwise_linear(x: torch.Tensor, x_token_stride: int, x_head_stride: int, m: torch.Tensor, out: torch.Tensor,
                    o_token_stride: int, o_head_stride: int, tokens: int, gate: Optional[torch.Tensor] = None,
                    rotate_tail=None) -> None:
    """out[t, h, j] = sum_k m[h, j, k] * x[t, h, k] for m [heads, n_out, n_in]; head h of token t starts at
    t * token_stride + h * head_stride in x (n_in values) and in out (n_out values).  With `gate` (float32 rows
    [tokens, heads], a view of columns is fine) head h's outputs of token t are multiplied by sigmoid(gate[t, h]).
    With `rotate_tail` = (n, cos, sin, half_split) the n columns behind a head's inputs are rotated by the token's
    angles (cos, sin [tokens, n / 2]) and written behind the head's outputs."""
    _gpu(x, m, out, gate)
    nh, n_out, n_in = m.shape
    tn, tcos, tsin, tsplit = rotate_tail if rotate_tail is not None else (0, None, None, False)
    if tn:
        _gpu(tcos, tsin)
        _check_tables("headwise_linear", tokens, tn, tcos, tsin, None)
        _chk(tn % 2 == 0 and x_head_stride >= n_in + tn and o_head_stride >= n_out + tn
             and x.numel() >= (tokens - 1) * x_token_stride + (nh - 1) * x_head_stride + n_in + tn
             and out.numel() >= (tokens - 1) * o_token_stride + (nh - 1) * o_head_stride + n_out + tn, "headwise_linear: the rotated tail")
    _chk(gate is None or (_rows_ok(gate) and gate.dtype is torch.float32 and gate.shape == (tokens, nh)), "headwise_linear: gate")
    _chk(m.is_contiguous() and m.dtype in _DT and x.dtype in _DT and out.dtype in _DT and x.is_contiguous()
         and out.is_contiguous(), "headwise_linear: operands")
    _chk(x.numel() >= (tokens - 1) * x_token_stride + (nh - 1) * x_head_stride + n_in
         and out.numel() >= (tokens - 1) * o_token_stride + (nh - 1) * o_head_stride + n_out
         and x_head_stride >= 0 and o_head_stride >= n_out, "headwise_linear: strides")
    _chk(m.dtype is torch.bfloat16 or (x.dtype is torch.float32 and out.dtype is torch.float32), "headwise_linear: dtypes")
    _chk(n_in <= 2048, "headwise_linear: at most 2048 inputs a head")
    if tokens:
        _run("attention_masked", "li_headwise_linear", x.data_ptr(), _DT[x.dtype], int(x_token_stride), int(x_head_stride),
             m.data_ptr(), _DT[m.dtype], out.data_ptr(), _DT[out.dtype], int(o_token_stride), int(o_head_stride),
             tokens, nh, n_out, n_in, 0 if gate is None else gate.data_ptr(), 0 if gate is None else gate.stride(0),
             int(tn), int(bool(tsplit)), tcos.data_ptr() if tn else 0, tsin.data_ptr() if tn else 0)


# ---------------------------------------------------------------------- gemm
SKINNY_MAX_ROWS = 64
SPLITK_MAX_PARTS = 8


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False, ws=None) -> None:
    """out = x w^T + bias, or out += x w^T + bias when `accumulate`.
    x [M, K] and w [N, K] of one dtype (float32 or bfloat16); out [M, N] of that
    dtype or float32; accumulation of the product is float32.  `ws` lends the
    memory for partial sums where the kernel cuts K into parts (17 rows and more
    against a matrix of few columns); without it
    such a product takes a slower kernel."""
    _gpu(x, w, bias, out)
    _chk(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear: needs matrices")
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape[1] == k and out.shape == (m, n)):
        _chk(False, f"linear: shapes x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear: contiguous operands")
    if not (x.dtype is w.dtype and x.dtype in _DT):
        _chk(False, f"linear: x is {x.dtype}, w is {w.dtype}")
    _chk(out.dtype is x.dtype or out.dtype is torch.float32, "linear: out dtype")
    _chk(not accumulate or out.dtype is torch.float32, "linear: accumulation needs a float32 out")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear: bias must be float32 [N]")
    if m:
        work, work_bytes = 0, 0
        if ws is not None and x.dtype is torch.bfloat16 and not few_rows_preferred(m, n, k):
            # few rows over a long k and few columns: the library cuts k into parts if it is lent room for their sums
            need = _work_bytes(m, n, k, _DT[x.dtype])
            if need:
                if m <= SKINNY_MAX_ROWS:            # one size for all row counts of a decode batch: the buffer does not move
                    need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
                buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
                work, work_bytes = buf.data_ptr(), buf.numel() * 4
        _run("gemm", "li_linear", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
             out.data_ptr(), m, n, k, _DT[x.dtype], _DT[out.dtype], int(bool(accumulate)), work, work_bytes)



def linear_row_tile(dtype: torch.dtype) -> int:
    """Rows of the smallest tile that `linear` cuts a product of many rows of this dtype into (the
    kernel library says): a few rows more than a multiple of it cost a whole tile more."""
    f = _fn_cache.get(("gemm", "li_linear_row_tile"))
    if f is None:
        f = build.load("gemm").li_linear_row_tile
        f.argtypes, f.restype = [c_int], c_int
        _fn_cache[("gemm", "li_linear_row_tile")] = f
    return int(f(_DT[dtype]))


def skinny_takes(m: int, k: int, w_dtype: torch.dtype) -> bool:
    """Whether `linear_skinny` takes a product of m rows over k with such a matrix."""
    return w_dtype is torch.bfloat16 and k % 8 == 0 and 0 < m <= SKINNY_MAX_ROWS


def linear_skinny(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, swiglu: bool = False) -> None:
    """The product for few rows (decoding).  swiglu: w is [gate; up] (2N rows)
    and out[m, n] = up * gate / (1 + exp(-gate)), the activation fused into the
    product's epilogue."""
    _gpu(x, w, bias, out)
    m, k = x.shape
    n = out.shape[1]
    _chk(skinny_takes(m, k, w.dtype), "linear_skinny: sizes or dtype not taken")
    _chk(w.shape == ((2 * n if swiglu else n), k) and out.shape[0] == m, "linear_skinny: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_skinny: contiguous operands")
    _chk(x.dtype is torch.bfloat16, "linear_skinny: x must be bfloat16")
    _chk(out.dtype in _DT and (not accumulate or out.dtype is torch.float32), "linear_skinny: out dtype")
    _chk(not swiglu or (bias is None and not accumulate and out.dtype is torch.bfloat16),
         "linear_skinny: swiglu takes no bias and no accumulation and writes bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_skinny: bias must be float32 [N]")
    _run("gemm", "li_linear_skinny", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, n, k, _DT[out.dtype], int(bool(accumulate)), int(bool(swiglu)))


def swiglu_takes(m: int, k: int, w_dtype: torch.dtype) -> bool:
    """Whether `linear_swiglu` takes a product of m rows over k with such a matrix (float32: the few rows of
    a decoding step)."""
    if w_dtype is torch.float32:
        # (more rows: a block's share of x grows with them while its gate and up columns stay 16 each; the
        # product without the activation takes wider blocks there)
        return 0 < m <= 16 and k % 4 == 0
    return w_dtype is torch.bfloat16 and m > 0 and (k % 8 == 0 if m <= SKINNY_MAX_ROWS else k % 64 == 0)


# An RMS norm between two products of few rows (a decoding step), without a pass of its own: the
# product before it, which adds to the float32 sum, also writes the sum times the norm's weights in
# bfloat16 and each block's share of the rows' sums of squares (`linear_residual_norm`); the product
# after it multiplies those rows and scales each row's result by the norm's factor (`row_scale` of
# `linear_swiglu` and `linear_rope_store`).
RESIDUAL_NORM_MAX_ROWS = 32
RESIDUAL_NORM_MAX_PARTS = 512
# The few-row kernels with their fused epilogues take up to 32 rows (two tiles of 16 a block); from 13 rows on
# the 64-row tiles with K in parts (and the kernels that add the parts up doing the norm, the rotation and the
# page write) are faster where the matrix is large, from 17 on also where it is of middling size.  Parts ask `few_rows_preferred` beside the `*_takes` of the few-row
# kernels; the kernel library holds the rule (its own entry points decide by it too).


def few_rows_preferred(m: int, n: int, k: int) -> bool:
    """Whether m rows against a matrix [n, k] should take the few-row kernels."""
    f = _fn_cache.get(("gemm", "li_few_rows_preferred"))
    if f is None:
        f = build.load("gemm").li_few_rows_preferred
        f.argtypes, f.restype = [c_int, c_long, c_long], c_int
        _fn_cache[("gemm", "li_few_rows_preferred")] = f
    return bool(f(int(m), int(n), int(k)))


class RowScale:
    """What the product after a fused RMS norm needs beside its rows: the shares of the rows' sums
    of squares [nparts * R] float32 (R = 16 for up to 16 rows, 32 above) and the norm's eps."""
    def __init__(self, sq_parts: torch.Tensor, nparts: int, eps: float):
        self.sq_parts, self.nparts, self.eps = sq_parts, int(nparts), float(eps)


def residual_norm_parts(n: int) -> int:
    """Blocks of `linear_residual_norm` over n columns, i.e. shares of a row's sum of squares (the
    library spreads a matrix of few columns evenly over the current device's compute units)."""
    f = _fn_cache.get(("gemm", "li_residual_norm_parts"))
    if f is None:
        f = build.load("gemm").li_residual_norm_parts
        f.argtypes, f.restype = [c_int], c_int
        _fn_cache[("gemm", "li_residual_norm_parts")] = f
    return int(f(int(n)))


def residual_norm_takes(m: int, n: int, k: int, w_dtype: torch.dtype) -> bool:
    return (w_dtype is torch.bfloat16 and 0 < m <= RESIDUAL_NORM_MAX_ROWS and k % 8 == 0
            and residual_norm_parts(n) <= RESIDUAL_NORM_MAX_PARTS)


def row_scale_rows(m: int) -> int:
    """Places a block's shares of the rows' sums of squares take: 16 for up to 16 rows, 32 above."""
    return 16 if m <= 16 else 32


def linear_residual_norm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                         gamma: torch.Tensor, xg: torch.Tensor, sq_parts: torch.Tensor) -> int:
    """out += x w^T + bias (float32); xg = bfloat16(gamma * out); sq_parts[p * R + m] = block p's
    share of sum_n out[m, n]^2 (R = `row_scale_rows(m)`).  Returns the number of blocks p."""
    _gpu(x, w, bias, out, gamma, xg, sq_parts)
    m, k = x.shape
    n = w.shape[0]
    _chk(residual_norm_takes(m, n, k, w.dtype), "linear_residual_norm: sizes or dtype not taken")
    _chk(x.dtype is torch.bfloat16 and w.shape == (n, k) and x.is_contiguous() and w.is_contiguous(),
         "linear_residual_norm: x and w must be contiguous bfloat16 [M, K] and [N, K]")
    _chk(out.dtype is torch.float32 and out.shape == (m, n) and out.is_contiguous(), "linear_residual_norm: out must be float32 [M, N]")
    _chk(xg.dtype is torch.bfloat16 and xg.shape == (m, n) and xg.is_contiguous(), "linear_residual_norm: xg must be bfloat16 [M, N]")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_residual_norm: bias must be float32 [N]")
    _chk(gamma.dtype is torch.float32 and gamma.shape == (n,) and gamma.is_contiguous(), "linear_residual_norm: gamma must be float32 [N]")
    parts = residual_norm_parts(n)
    _chk(sq_parts.dtype is torch.float32 and sq_parts.is_contiguous() and sq_parts.numel() >= parts * row_scale_rows(m),
         "linear_residual_norm: sq_parts must be float32 with 16 places a block (32 above 16 rows)")
    _run("gemm", "li_linear_residual_norm", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, n, k, gamma.data_ptr(), xg.data_ptr(), sq_parts.data_ptr())
    return parts


def linear_then_norm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                     gamma: torch.Tensor, eps: float, xn: torch.Tensor, ws) -> bool:
    """out += x w^T + bias (float32) and xn = gamma * out / sqrt(mean(out^2) + eps), in the kernel
    that adds up the parts of a product cut along K.  Returns False, having done nothing, where
    `linear` would not cut this product (then multiply and norm in two calls)."""
    _gpu(x, w, bias, out, gamma, xn)
    if ws is None or x.dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16:
        return False
    _chk(x.dim() == 2 and w.dim() == 2, "linear_then_norm: needs matrices")
    m, k = x.shape
    n = w.shape[0]
    need = _work_bytes(m, n, k, _DT[x.dtype])
    if not need:
        return False
    _chk(w.shape == (n, k) and x.is_contiguous() and w.is_contiguous(), "linear_then_norm: contiguous [M, K] and [N, K]")
    _chk(out.dtype is torch.float32 and out.shape == (m, n) and out.is_contiguous(), "linear_then_norm: out must be float32 [M, N]")
    _chk(xn.dtype in _DT and xn.shape == (m, n) and xn.is_contiguous(), "linear_then_norm: xn must be [M, N]")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_then_norm: bias must be float32 [N]")
    _chk(gamma.dtype is torch.float32 and gamma.shape == (n,) and gamma.is_contiguous() and eps >= 0,
         "linear_then_norm: gamma must be float32 [N], eps not negative")
    if m <= SKINNY_MAX_ROWS:                # one size for all row counts of a decode batch: the buffer does not move
        need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
    buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
    rc = _fn("gemm", "li_linear_then_norm")(x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
                                             out.data_ptr(), m, n, k, buf.data_ptr(), buf.numel() * 4, gamma.data_ptr(),
                                             float(eps), xn.data_ptr(), _DT[xn.dtype], _stream())
    if rc == -1:
        return False
    if rc != 0:
        raise RuntimeError(f"li_linear_then_norm: the kernel library refused the call (code {rc}): {_ERRORS.get(rc, 'unknown')}")
    return True


def _check_row_scale(what: str, m: int, row_scale: Optional[RowScale]):
    if row_scale is None:
        return 0, 0, 0.0
    _gpu(row_scale.sq_parts)
    _chk(0 < m <= RESIDUAL_NORM_MAX_ROWS, f"{what}: a row scale goes with up to {RESIDUAL_NORM_MAX_ROWS} rows")
    _chk(0 < row_scale.nparts <= RESIDUAL_NORM_MAX_PARTS and row_scale.eps >= 0, f"{what}: row scale out of range")
    _chk(row_scale.sq_parts.dtype is torch.float32 and row_scale.sq_parts.is_contiguous()
         and row_scale.sq_parts.numel() >= row_scale.nparts * row_scale_rows(m),
         f"{what}: the row scale's parts must be float32 [nparts * {row_scale_rows(m)}]")
    return row_scale.sq_parts.data_ptr(), row_scale.nparts, row_scale.eps


def linear_swiglu(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, row_scale: Optional[RowScale] = None) -> None:
    """out[m, n] = up * gate / (1 + exp(-gate)) with [gate, up] = x w^T, w = [gate; up]
    (2 N rows): the activation in the product's epilogue, from the product's float32 sums.
    With `row_scale`, x is the xg of `linear_residual_norm` and the result is that of the norm."""
    _gpu(x, w, out)
    _chk(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear_swiglu: needs matrices")
    m, k = x.shape
    n = out.shape[1]
    _chk(swiglu_takes(m, k, w.dtype) or (w.dtype is torch.float32 and 0 < m <= SKINNY_MAX_ROWS and k % 4 == 0),
         "linear_swiglu: sizes or dtype not taken")
    _chk(w.shape == (2 * n, k) and out.shape[0] == m, "linear_swiglu: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_swiglu: contiguous operands")
    if w.dtype is torch.float32:
        _chk(x.dtype is torch.float32 and out.dtype is torch.float32 and row_scale is None,
             "linear_swiglu: float32 w goes with float32 x and out, and no row scale")
        _chk(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "linear_swiglu: operands must start on 16 bytes")
        _run("gemm", "li_linear_swiglu_f32", x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k)
        return
    _chk(x.dtype is torch.bfloat16 and out.dtype is torch.bfloat16, "linear_swiglu: x and out must be bfloat16")
    _run("gemm", "li_linear_swiglu", x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k,
         *_check_row_scale("linear_swiglu", m, row_scale))


ROPE_STORE_MAX_ROWS = 32


def rope_store_takes(m: int, k: int, w_dtype: torch.dtype, dh: int, rotary_dim: int) -> bool:
    """Whether `linear_rope_store` takes the packed projection of m rows over k."""
    return (w_dtype is torch.bfloat16 and 0 < m <= ROPE_STORE_MAX_ROWS and k % 8 == 0
            and dh % 16 == 0 and rotary_dim == dh)


def linear_rope_store(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                      nh: int, nkv: int, dh: int, cos: torch.Tensor, sin: torch.Tensor,
                      slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor, page_size: int,
                      row_scale: Optional[RowScale] = None) -> None:
    """Fused for a decoding step: out = x w^T + bias with w the packed [q; k; v]
    projection, query and key heads rotated (half-split pairs, the whole head) by
    the rows' angles, keys and values written into their page slots.  out holds
    the rotated queries and keys and the values, as after the separate kernels.
    With `row_scale`, x is the xg of `linear_residual_norm` and the result is that of the norm."""
    _gpu(x, w, bias, out, cos, sin, slot_map, k, v)
    m, kk = x.shape
    n = (nh + 2 * nkv) * dh
    _chk(rope_store_takes(m, kk, w.dtype, dh, 2 * cos.shape[1]), "linear_rope_store: sizes or dtype not taken")
    _chk(w.shape == (n, kk) and out.shape == (m, n), "linear_rope_store: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_rope_store: contiguous operands")
    _chk(x.dtype is torch.bfloat16 and out.dtype is torch.bfloat16, "linear_rope_store: x and out must be bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_rope_store: bias must be float32 [N]")
    _check_cache(k, v, nkv, dh, page_size, out.dtype)
    _chk(cos.shape == (m, dh // 2) and sin.shape == cos.shape and cos.dtype is torch.float32
         and sin.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), "linear_rope_store: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == m and slot_map.is_contiguous(),
         "linear_rope_store: slot_map")
    _run("gemm", "li_linear_rope_store", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, kk, cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(), v.data_ptr(),
         nh, nkv, dh, page_size, k.shape[0], *_check_row_scale("linear_rope_store", m, row_scale))


def linear_rope_store_parts(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                            nh: int, nkv: int, dh: int, cos: torch.Tensor, sin: torch.Tensor,
                            slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor, page_size: int, ws) -> bool:
    """The same result as `linear_rope_store` for the rows of a large decoding batch, where the
    packed projection is cut along K anyway: the kernel that adds the parts up rotates and writes
    the pages.  Returns False, having done nothing, where `linear` would not cut this product."""
    _gpu(x, w, bias, out, cos, sin, slot_map, k, v)
    if ws is None or x.dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16 or 2 * cos.shape[1] != dh:
        return False
    m, kk = x.shape
    n = (nh + 2 * nkv) * dh
    need = _work_bytes(m, n, kk, _DT[x.dtype])
    if not need:
        return False
    _chk(w.shape == (n, kk) and out.shape == (m, n), "linear_rope_store_parts: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_rope_store_parts: contiguous operands")
    _chk(out.dtype is torch.bfloat16, "linear_rope_store_parts: out must be bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_rope_store_parts: bias must be float32 [N]")
    _check_cache(k, v, nkv, dh, page_size, out.dtype)
    _chk(cos.shape == (m, dh // 2) and sin.shape == cos.shape and cos.dtype is torch.float32
         and sin.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), "linear_rope_store_parts: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == m and slot_map.is_contiguous(),
         "linear_rope_store_parts: slot_map")
    if m <= SKINNY_MAX_ROWS:                # one size for all row counts of a decode batch: the buffer does not move
        need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
    buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
    rc = _fn("gemm", "li_linear_rope_store_parts")(
        x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(), out.data_ptr(), m, kk,
        cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(), v.data_ptr(), nh, nkv, dh, page_size,
        k.shape[0], buf.data_ptr(), buf.numel() * 4, _stream())
    if rc == -1:
        return False
    if rc != 0:
        raise RuntimeError(f"li_linear_rope_store_parts: the kernel library refused the call (code {rc}): {_ERRORS.get(rc, 'unknown')}")
    return True


# ----------------------------------------------------------------- attention
# waves that the split-key decode kernel on the matrix cores is cut into at least (where the keys allow):
# four a compute unit; more splits cost more in the merge than they gain (measured at 8 and 64 requests)
_DEC_WAVES = 1024
PREFILL_TILE_ROWS = 32       # queries of one segment that a block of the matrix-core kernel for portions takes
DECODE_MAX_SPLITS = 64       # the merge kernel keeps a weight per split
DECODE_TABLE_CAP = 1024      # pages of one split that the matrix-core decode kernel copies into LDS
DECODE_LIST_MAX_TOKENS = 4096    # single tokens whose runs the device lists (`decode_run_keys`)


_simds: Dict[int, int] = {}


def _simd_count(device: torch.device) -> int:
    """Waves of the decode kernel that run at one time: one on each SIMD, four SIMDs a compute unit."""
    i = device.index if device.index is not None else torch.cuda.current_device()
    if i not in _simds:
        _simds[i] = 4 * torch.cuda.get_device_properties(i).multi_processor_count
    return _simds[i]


DECODE_QUAD = 4              # runs of a token's keys that one block of the matrix-core decode kernel takes, one a wave
# measurements only: single-wave blocks and a merge kernel behind them, as before the blocks joined their runs
_decode_single_waves = False
# Share of the SIMDs that a step's waves must fill for the blocks of four waves (below).  Most batch sizes give a
# number of runs whose waves fill the SIMDs nearly, not wholly (17 requests x 2 kv heads x 28 runs = 952 of
# 1,024); asked for all of them, those took single-wave blocks and the merge kernel: 17 / 24 / 28 requests of
# 4,096 keys at the 1.5B head layout 23.5 / 29.4 / 31.5 us a layer against 21.8 / 26.9 / 29.9 with the blocks of
# four (7B layout, 28 requests: 53.6 against 50.0); from a half on the short contexts lose (17.0 against 16.0 us).
_DECODE_FILLS = 0.7


def decode_splits(pairs: int, keys: int, simds: int = _DEC_WAVES, quad: int = DECODE_QUAD) -> int:
    """Into how many runs the keys of a decoding token are cut.  Every (token, kv head) pair and
    run is one wave, and a SIMD holds one wave of this kernel: the waves go over the SIMDs in
    rounds, each as long as a run (plus a wave's start and end, about 24 keys' time), so the
    number of runs with the least rounds x run length is taken, a run being a multiple of 32
    keys and at least 128 where the keys allow; every run costs the join a little (4 keys' time).
    The runs come in blocks of `quad` waves (a block joins its runs itself), so their number is 1
    or a multiple of `quad`.  Few pairs: as many runs as fill the SIMDs once."""
    most = max(1, min(-(-keys // 128), DECODE_MAX_SPLITS))
    best, best_cost = 1, None
    for ns in [1] + list(range(quad, most + 1, quad)):
        run = (-(-keys // ns) + 31) & ~31
        cost = -(-pairs * ns // simds) * (run + 24) + 4 * ns
        if best_cost is None or cost < best_cost:
            best, best_cost = ns, cost
    return best


def _ragged_splits(nsplit: int, meta, window: int, quad: int = DECODE_QUAD) -> int:
    """More runs for the grid of a batch whose contexts differ: `nsplit` fits contexts that are all as
    long as the longest; with one run length for the batch (chosen on the device) the short ones fill
    few runs, and the same number of working waves needs the longest cut into more."""
    ql, cl = getattr(meta, "host_q_len", None), getattr(meta, "host_ctx_len", None)
    if ql is None or cl is None or nsplit >= DECODE_MAX_SPLITS:
        return nsplit
    keys = cl[ql == 1]
    if keys.size < 2:
        return nsplit
    if window > 0:
        keys = np.minimum(keys, window)
    ragged = float(keys.max()) * keys.size / max(float(keys.sum()), 1.0)
    if ragged < 1.15:
        return nsplit
    more = min(DECODE_MAX_SPLITS, int(math.ceil(nsplit * ragged * 1.25)))
    return min(DECODE_MAX_SPLITS, -(-more // quad) * quad)


def decode_run_keys(meta, token_list: Optional[torch.Tensor], n_tokens: int, page_size: int, window: int,
                    nkv: int, nsplit: int, simds: int, out: torch.Tensor, group: int = 1) -> None:
    """out[0] = the run length, in keys, for the split-key decode kernel over these single tokens
    (`token_list`, or the batch's first n_tokens tokens): the multiple of 32 with the least rounds of
    working waves over `simds` x (length + 24), between what the longest context needs to fit
    `nsplit` runs and what the block table's width would need.  out[1] = the number of runs with
    keys at that length, out[2 : 2 + n_tokens] = the runs of each token, then the runs themselves as
    token | run << 16.  With `group` > 1 the runs are taken `group` at a time (one block of the decode
    kernel): the list then holds the first run of every group, out[1] counts the groups, and a length's
    cost counts `group` waves a group.  At most 4,096 tokens."""
    _gpu(out, meta.ctx_len, token_list)
    _chk(0 < n_tokens <= DECODE_LIST_MAX_TOKENS, "decode_run_keys: too many tokens")
    _chk(out.dtype is torch.int32 and out.is_contiguous() and out.numel() >= 2 + n_tokens + n_tokens * nsplit,
         "decode_run_keys: out must be int32 [2 + tokens + tokens * nsplit]")
    _run("attention", "li_decode_run_keys", 0 if token_list is None else token_list.data_ptr(), n_tokens,
         meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
         meta.max_blocks, page_size, int(window), nkv, nsplit, simds, int(group), out.data_ptr())


def decode_split_blocks(max_blocks: int, page_size: int, window: int, nsplit: int) -> int:
    """The most pages one of `nsplit` splits of the keys can touch, for block tables of
    `max_blocks` pages: the keys (at most the table's, or the window's) are cut into runs
    of a multiple of 32, and a run that begins anywhere in a page touches one page more
    than its length fills.  The kernel library computes the same bound and refuses a call
    beyond its table."""
    keys = max_blocks * page_size
    if 0 < window < keys:
        keys = window
    per = (-(-keys // nsplit) + 31) & ~31
    return (per + page_size - 2) // page_size + 1

def _decode_kernel_takes(dtype: torch.dtype, dh: int) -> bool:
    """The single-query kernel spreads a key's row over dh / (16 bytes) lanes, a power of two."""
    per = 8 if dtype is torch.bfloat16 else 4
    return dh % per == 0 and (dh // per) & (dh // per - 1) == 0 and dh // per <= 64


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, k: torch.Tensor, v: torch.Tensor, meta,
                    nh: int, nkv: int, dh: int, page_size: int, window: int, scale: float,
                    ws=None) -> None:
    """Causal grouped-query attention of the batch's queries (heads 0..nh-1 of
    qkv's rows) over the paged keys and values; out [T, nh*dh].  Query i of a
    segment stands at position ctx_len - q_len + i and sees the keys at
    positions <= its own and, with window > 0, closer than `window`.  Tokens of
    segments that bring one token go to the split-key decode kernel, the others
    to the kernel for portions.  `ws` lends the buffers for the splits' partial
    results."""
    _gpu(qkv, out, k, v, meta.block_table)
    check_attention_sizes(nh, nkv, dh)
    _check_qkv(qkv, nh, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(out.shape == (t, nh * dh) and out.is_contiguous() and out.dtype is qkv.dtype, "attention: out")
    _chk(t == meta.num_tokens, "attention: batch metadata is of another batch")
    bt = meta.block_table
    _chk(bt.dtype is torch.int32 and bt.shape == (meta.num_segments, meta.max_blocks)
         and bt.is_contiguous(), "attention: block table")
    _chk(meta.max_blocks * page_size >= meta.max_ctx_len, "attention: block table too short")
    _chk(meta.num_single + meta.num_multi == t, "attention: token lists do not cover the batch")
    _chk(meta.num_single in (0, t) or (meta.single_tokens is not None and meta.multi_tokens is not None),
         "attention: a batch of single-token and longer segments needs their token lists (BatchNeeds.token_kinds)")
    if not t:
        return
    n_single, n_multi = meta.num_single, meta.num_multi
    if n_single and not _decode_kernel_takes(qkv.dtype, dh):
        n_single, n_multi = 0, t                      # every token through the general kernel
    if n_single:
        keys = min(meta.max_single_ctx, window) if window > 0 else meta.max_single_ctx
        # a head size of 64 or 128 (bfloat16, or float32 on the float32 matrix cores): one wave per split
        # on the matrix cores; else one block of four waves per split on the vector ALU
        mfma = dh in (64, 128)
        planned = 0
        if mfma:
            # (the kernel finds a key's page by a float32 product that is exact below 2^22)
            _chk(meta.max_blocks * page_size <= 1 << 21 and page_size <= 1 << 16,
                 f"attention: block tables of {meta.max_blocks} pages of {page_size} keys are beyond the decode "
                 f"kernel's {1 << 21} keys")
            # Blocks of four waves that join their runs themselves, or single-wave blocks and a merge kernel
            # behind them.  Four waves sit on ONE compute unit and the join is three trips to memory at the
            # kernel's end: it pays where one block holds all runs of a (token, kv head) (no join, no second
            # kernel: 64 requests at the 7B head layout 105 -> 96 us a layer), and where the waves fill the
            # chip anyway and the runs are not many or long (8 requests, 4,096 keys: 22.3 -> 21.6 us; 8
            # requests of the 1.5B layout with 64 short runs each: 17.3 -> 18.9 us, so not there).  Not for
            # contexts that differ (one run length for the batch and a list of the runs that have keys): a
            # token's runs then fill its last block of four only partly, and a block's waves end at different
            # times (64 requests with 16 to 4,600 keys, 7B head layout: 73.8 us against 82.7; 1.5B: 41.3 / 52.5).
            simds = _simd_count(qkv.device)
            quad = DECODE_QUAD
            planned = decode_splits(n_single * nkv, keys, simds, quad)
            nsplit = _ragged_splits(planned, meta, window)
            fills = n_single * nkv * nsplit >= _DECODE_FILLS * simds
            if (_decode_single_waves or nsplit > planned
                    or not (nsplit == DECODE_QUAD or (fills and (nsplit <= 32 or keys >= 8192)))):
                quad = 1
                planned = decode_splits(n_single * nkv, keys, simds, quad)
                nsplit = _ragged_splits(planned, meta, window, quad)
            # a split's pages must fit the kernel's copy of the block table
            while nsplit <= DECODE_MAX_SPLITS and decode_split_blocks(meta.max_blocks, page_size, window, nsplit) > DECODE_TABLE_CAP:
                nsplit += 1 if nsplit < quad else quad
            if 1 < nsplit < quad:
                nsplit = quad
            _chk(nsplit <= DECODE_MAX_SPLITS, f"attention: block tables of {meta.max_blocks} pages of {page_size} "
                                              f"are too long for the decode kernel")
        else:
            nsplit = max(1, min(-(-512 // (n_single * nkv)), -(-keys // 256), DECODE_MAX_SPLITS))
        acc = ml = None
        if nsplit > 1:
            shape_a, shape_m = (n_single, nh, nsplit, dh), (n_single, nh, nsplit, 2)
            if ws is not None:
                acc = ws.buffer("attn.part_acc", shape_a, torch.float32)
                ml = ws.buffer("attn.part_ml", shape_m, torch.float32)
            else:
                acc = torch.empty(shape_a, dtype=torch.float32, device=qkv.device)
                ml = torch.empty(shape_m, dtype=torch.float32, device=qkv.device)
        lst = meta.single_tokens if n_single < t else None
        run_keys = done = None
        if mfma and nsplit > DECODE_QUAD and quad > 1:
            # the blocks of a (token, kv head) count themselves here, and the last one joins their results
            # (zero before the first call; every call leaves it zero)
            done = (ws.buffer("attn.done", (n_single * nkv,), torch.int32, zero=True) if ws is not None
                    else torch.zeros(n_single * nkv, dtype=torch.int32, device=qkv.device))
        if mfma and nsplit > planned and n_single <= DECODE_LIST_MAX_TOKENS:
            # contexts that differ: one run length for the batch and the list of the runs that have keys, made
            # on the device from the context lengths, once a step for all layers with these numbers (a
            # recorded step makes them again at every replay)
            key = ("decode_run_keys", nkv, int(window), nsplit, meta.max_blocks, n_single)
            run_keys = meta.extra.get(key)
            if run_keys is None:
                # one buffer for every number of runs and (growing only with the batch) of tokens: a
                # name per combination would pile up over a serving run
                name = "attn.run_keys.%d.%d.%d" % (getattr(meta, "group", 0), nkv, int(window))
                size = 2 + n_single + n_single * DECODE_MAX_SPLITS
                run_keys = (ws.buffer(name, (size,), torch.int32) if ws is not None
                            else torch.empty(size, dtype=torch.int32, device=qkv.device))
                decode_run_keys(meta, lst, n_single, page_size, window, nkv, nsplit, _simd_count(qkv.device), run_keys,
                                group=quad)
                meta.extra[key] = run_keys
        _run("attention", "li_paged_attention_decode", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), _DT[qkv.dtype], bt.data_ptr(), meta.max_blocks,
             0 if lst is None else lst.data_ptr(), n_single, meta.seg_of_token.data_ptr(),
             meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             0 if acc is None else acc.data_ptr(), 0 if ml is None else ml.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale), nsplit,
             (2 if quad == 1 and nsplit > 1 else 1) if mfma else 0,
             0 if run_keys is None else run_keys.data_ptr(), 0 if done is None else done.data_ptr())
    # the matrix-core kernel for portions keeps a tile's pages in LDS (8192 entries) and divides
    # positions by the page size in float, exact below 2^21 keys; longer tables take the general kernel
    if (n_multi and qkv.dtype is torch.bfloat16 and dh in (64, 128) and meta.num_tiles
            and meta.tile_rows == PREFILL_TILE_ROWS and n_multi == meta.num_multi and meta.max_blocks <= 8192 and meta.max_blocks * page_size <= 1 << 21):
        # few tiles against long contexts: the tiles' keys in runs, joined by the kernel that joins the
        # decode attention's (the library says how many; their results take room in the workspace)
        runs = 1
        if ws is not None:
            runs = _prefill_runs(getattr(meta, "host_q_len", None), getattr(meta, "host_ctx_len", None), nh, nkv, dh,
                                 meta.max_blocks, window, t)
        acc = ml = lst = None
        if runs > 1:
            acc = ws.buffer("attn.runs_acc", (t, nh, runs, dh), torch.float32)
            ml = ws.buffer("attn.runs_ml", (t, nh, runs, 2), torch.float32)
            lst = meta.multi_tokens if n_multi < t else None
        _run("attention", "li_paged_attention_prefill", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), bt.data_ptr(), meta.max_blocks, meta.tiles.data_ptr(),
             meta.num_tiles, meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale), runs,
             0 if acc is None else acc.data_ptr(), 0 if ml is None else ml.data_ptr(),
             0 if lst is None else lst.data_ptr(), n_multi)
    elif (n_multi and qkv.dtype is torch.float32 and dh in (64, 128) and meta.num_tiles
            and meta.tile_rows == PREFILL_TILE_ROWS and n_multi == meta.num_multi):
        # the 32-bit path's tiled kernel for portions (other head sizes: the general kernel below)
        _run("attention", "li_paged_attention_prefill_f32", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), bt.data_ptr(), meta.max_blocks, meta.tiles.data_ptr(),
             meta.num_tiles, meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale))
    elif n_multi:
        lst = meta.multi_tokens if n_multi < t else None
        _run("attention", "li_paged_attention", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), _DT[qkv.dtype], bt.data_ptr(), meta.max_blocks,
             0 if lst is None else lst.data_ptr(), meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(),
             meta.q_len.data_ptr(), meta.ctx_len.data_ptr(), meta.num_segments, n_multi, meta.max_q_len,
             meta.max_ctx_len, nh, nkv, dh, page_size, k.shape[0], int(window), float(scale))


# ------------------------------------------------------------------ sampling
_argmax_scratch = {}
_sample_scratch = {}


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = index of the maximum of row i, the lowest index on ties."""
    _gpu(logits, out)
    _chk(logits.dim() == 2 and logits.dtype is torch.float32 and logits.is_contiguous(), "argmax: logits")
    _chk(out.dtype is torch.int32 and out.numel() == logits.shape[0] and out.is_contiguous(), "argmax: out")
    n = logits.shape[0]
    if n:
        key = (logits.device, n)
        if key not in _argmax_scratch:
            _argmax_scratch[key] = (torch.empty(n * 32, dtype=torch.float32, device=logits.device),
                                    torch.empty(n * 32, dtype=torch.int32, device=logits.device))
        sv, si = _argmax_scratch[key]
        _run("sampling", "li_argmax_rows", logits.data_ptr(), out.data_ptr(), sv.data_ptr(), si.data_ptr(),
             n, logits.shape[1])


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
                top_p: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor) -> None:
    """One token per row.  temperature <= 0: the argmax (lowest index on ties).
    Otherwise the candidates, ordered by (logit descending, index ascending),
    are cut to the first top_k (when 0 < top_k < V) and then to the shortest
    prefix whose softmax mass among them reaches top_p (when 0 < top_p < 1);
    the softmax of logits/temperature over the survivors is sampled by inverse
    CDF over ascending ids with the row's uniform number in [0, 1)."""
    _gpu(logits, temperature, top_k, top_p, uniform, out)
    _chk(logits.dim() == 2 and logits.dtype is torch.float32 and logits.is_contiguous(), "sample: logits")
    n = logits.shape[0]
    for t_, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p, torch.float32),
                   (uniform, torch.float32), (out, torch.int32)):
        _chk(t_.dtype is dt and t_.numel() == n and t_.is_contiguous(), "sample: per-row arrays")
    if n:
        v = logits.shape[1]
        key = (logits.device, n, v)
        if key not in _sample_scratch:               # what the first of the two kernels leaves for the second
            _sample_scratch[key] = torch.empty(_sample_scratch_floats(n, v), dtype=torch.float32, device=logits.device)
        tiles = _sample_scratch[key]
        _run("sampling", "li_sample_rows", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(),
             top_p.data_ptr(), uniform.data_ptr(), out.data_ptr(), n, v, tiles.data_ptr(), tiles.numel())


SAMPLE_SLOT_WORDS = 8          # 32-bit words of a slot's row in the sampling table (csrc/sampling.hip)
SAMPLE_ROW_GREEDY = 1 << 24    # flag of a step's row: greedy whatever its slot's row says


def sample_prepare(rows: torch.Tensor, table: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
                   top_p: torch.Tensor, uniform: torch.Tensor) -> None:
    """From the sampling table of the state slots (int32 [slots, 8]: temperature and top_p as float bits,
    top_k, the seed's two halves, the draws so far) and a step's rows (int32: slot | flags << 24), the
    per-row arrays that `sample_rows` takes; the uniform number of every sampling row is drawn on the
    device from its slot's seed and count, and the count goes up."""
    _gpu(rows, table, temperature, top_k, top_p, uniform)
    n = rows.numel()
    _chk(rows.dtype is torch.int32 and rows.is_contiguous(), "sample_prepare: rows must be int32")
    _chk(table.dtype is torch.int32 and table.dim() == 2 and table.shape[1] == SAMPLE_SLOT_WORDS and table.is_contiguous(),
         "sample_prepare: the table must be int32 [slots, 8]")
    for t_, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p, torch.float32), (uniform, torch.float32)):
        _chk(t_.dtype is dt and t_.numel() == n and t_.is_contiguous(), "sample_prepare: per-row arrays")
    if n:
        _run("sampling", "li_sample_prepare", rows.data_ptr(), n, table.data_ptr(), table.shape[0],
             temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), uniform.data_ptr())


# ------------------------------------------------------------- position vector, logits, pages, map difference
def sinusoid_add(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> None:
    """x[t, 2i] += sin(p f_i), x[t, 2i + 1] += cos(p f_i) for p = positions[t]; freq float32 [ceil(H / 2)]."""
    _gpu(x, positions, freq)
    t, h = x.shape
    _chk(x.dtype is torch.float32 and x.is_contiguous() and positions.dtype is torch.int32 and positions.numel() == t
         and positions.is_contiguous() and freq.dtype is torch.float32 and freq.is_contiguous()
         and freq.numel() == (h + 1) // 2, "sinusoid_add: x [T, H] float32, positions [T] int32, freq [ceil(H / 2)] float32")
    if t:
        _run("elementwise", "li_sinusoid_add", x.data_ptr(), positions.data_ptr(), freq.data_ptr(), t, h)


def scale_softcap(x: torch.Tensor, scale: float, cap: float) -> None:
    """x <- x * scale, then cap * tanh(x / cap) where cap > 0; in place, float32."""
    _gpu(x)
    _chk(x.dtype is torch.float32 and x.is_contiguous() and cap >= 0, "scale_softcap: a contiguous float32 tensor, cap >= 0")
    if x.numel():
        _run("elementwise", "li_scale_softcap", x.data_ptr(), x.numel(), float(scale), float(cap))


def paged_store(src: torch.Tensor, runs, slot_map: torch.Tensor, page_size: int) -> None:
    """Up to three runs (first column, heads, columns a head, paged tensor [pages, heads, page_size, columns]) of the
    float32 rows `src` [T, stride] go to every token's slot."""
    t = src.shape[0]
    _gpu(src, slot_map, *(r[3] for r in runs))
    _chk(src.dtype is torch.float32 and _rows_ok(src) and slot_map.dtype is torch.int32 and slot_map.numel() == t
         and slot_map.is_contiguous() and 1 <= len(runs) <= 3, "paged_store: src [T, stride] float32, slot_map [T] int32, 1 to 3 runs")
    dt = runs[0][3].dtype
    flat = []
    for col, heads, dim, dst in runs:
        _chk(dst.dtype is dt and dt in _DT and dst.dim() == 4 and dst.is_contiguous() and dst.shape[1:] == (heads, page_size, dim)
             and 0 <= col and col + heads * dim <= src.shape[1], "paged_store: a run does not fit its rows or its pages")
        flat += [int(col), int(heads), int(dim), dst.data_ptr()]
    flat += [0, 0, 0, 0] * (3 - len(runs))
    if t:
        _run("elementwise", "li_paged_store", src.data_ptr(), src.stride(0), *flat, _DT[dt], slot_map.data_ptr(), int(page_size), t)


def diff_combine(a1: torch.Tensor, a2: torch.Tensor, lam: float, eps: float, mult: float, out: torch.Tensor, dv: int) -> None:
    """out = mult * o / sqrt(mean(o^2) + eps) over every head's dv columns, o = a1 - lam * a2; all [T, heads * dv]."""
    _gpu(a1, a2, out)
    _chk(a1.shape == a2.shape == out.shape and a1.dtype is a2.dtype and a1.dtype in _DT and out.dtype in _DT
         and a1.is_contiguous() and a2.is_contiguous() and out.is_contiguous() and dv > 0 and a1.shape[1] % dv == 0,
         "diff_combine: a1, a2, out [T, heads * dv]")
    if a1.numel():
        _run("elementwise", "li_diff_combine", a1.data_ptr(), a2.data_ptr(), _DT[a1.dtype], float(lam), float(eps), float(mult),
             out.data_ptr(), _DT[out.dtype], a1.numel() // dv, int(dv))


# ------------------------------------------------------------------------------------------ recurrent mixers
SSM_CHUNK = 64          # tokens of a portion that one block of the recurrence takes; longer portions run as chunks side by side


def _lib_fn(module: str, name: str, argtypes, restype):
    f = _fn_cache.get((module, name))
    if f is None:
        f = getattr(build.load(module), name)
        f.argtypes, f.restype = argtypes, restype
        _fn_cache[(module, name)] = f
    return f


def ssm_scan_takes(state: int, vdim: int) -> bool:
    """Whether the recurrence kernel has a layout for states of `state` values a column."""
    return bool(_lib_fn("recurrent", "li_ssm_scan_layout", [c_int, c_int, c_void_p, c_void_p], c_int)(int(state), int(vdim), None, None))


def causal_conv_silu(u: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], tail: torch.Tensor, ctx, out: torch.Tensor) -> None:
    """out[t, c] = silu(b[c] + sum_j w[c, j] u[t - (taps - 1 - j), c]) over each request's own tokens; what lies before
    the step's portion comes from `tail` [slots, taps - 1, C] (zeros for a new request), which then takes the
    request's last taps - 1 inputs.  u: float32 rows (a view with a row stride), the first C columns are read."""
    _gpu(u, w, b, tail, out)
    t, (c, taps) = out.shape[0], w.shape
    _chk(u.dtype is torch.float32 and _rows_ok(u) and u.shape[0] == t and u.shape[1] >= c and out.dtype is torch.float32
         and _rows_ok(out) and out.shape[1] == c, "causal_conv_silu: u, out")
    _chk(w.dtype is torch.float32 and w.is_contiguous() and taps >= 1
         and (b is None or (b.dtype is torch.float32 and b.numel() == c and b.is_contiguous())), "causal_conv_silu: w [C, taps], b [C] float32")
    _chk(tail.dtype is torch.float32 and tail.is_contiguous() and tail.dim() == 3 and (taps == 1 or tail.shape[1:] == (taps - 1, c)),
         "causal_conv_silu: tail [slots, taps - 1, C] float32")
    _chk(ctx.num_tokens == t and int(ctx.host_state_slots.max(initial=0)) < tail.shape[0], "causal_conv_silu: batch")
    if t:
        _run("recurrent", "li_causal_conv_silu", u.data_ptr(), u.stride(0), c, taps, w.data_ptr(), 0 if b is None else b.data_ptr(),
             tail.data_ptr(), ctx.seg_of_token.data_ptr(), ctx.q_start.data_ptr(), ctx.q_len.data_ptr(), ctx.state_slots.data_ptr(),
             out.data_ptr(), out.stride(0), t, ctx.num_segments, int(ctx.max_q_len))


def ssm_scan(xbc: torch.Tensor, dt: Optional[torch.Tensor], dt_bias: Optional[torch.Tensor], a_log: Optional[torch.Tensor],
             d: Optional[torch.Tensor], state: torch.Tensor, ctx, y: torch.Tensor, heads: int, vdim: int, n_state: int,
             groups: int, ws, fixed_decay: Optional[torch.Tensor] = None, fixed_step: float = 1.0) -> None:
    """The state-space recurrence over each request's tokens of the step, from and into `state`
    [slots, heads, n_state, vdim] (float32):  S <- a S + dt B x^T,  y = S^T C + d_h x,  with a = exp(-exp(a_log_h) dt) and
    dt = softplus(dt_raw + dt_bias_h), or, with `fixed_decay` (float32 [heads]), a = fixed_decay[h] and dt = fixed_step
    for every token (dt, dt_bias and a_log are then not read; d None: no x term).
    xbc: float32 rows [x: heads * vdim | B: groups * n_state | C: groups * n_state];
    dt: float32 rows [heads] (raw); y: float32 rows [heads * vdim].  All float32."""
    fixed = fixed_decay is not None
    _gpu(xbc, dt, dt_bias, a_log, d, state, y, fixed_decay)
    t = y.shape[0]
    inner = heads * vdim
    _chk(all(x is None or x.dtype is torch.float32 for x in (xbc, dt, dt_bias, a_log, d, state, y, fixed_decay)), "ssm_scan: everything is float32")
    _chk(_rows_ok(xbc) and xbc.shape == (t, inner + 2 * groups * n_state) and _rows_ok(y) and y.shape == (t, inner), "ssm_scan: rows")
    _chk(fixed or (dt is not None and _rows_ok(dt) and dt.shape == (t, heads)
                   and all(v is not None and v.numel() == heads and v.is_contiguous() for v in (dt_bias, a_log))), "ssm_scan: dt")
    _chk(not fixed or (fixed_decay.numel() == heads and fixed_decay.is_contiguous()), "ssm_scan: fixed_decay [heads]")
    _chk(state.is_contiguous() and state.shape[1:] == (heads, n_state, vdim) and heads % groups == 0
         and (d is None or (d.numel() == heads and d.is_contiguous())), "ssm_scan: state [slots, heads, N, vdim]")
    _chk(ctx.num_tokens == t and int(ctx.host_state_slots.max(initial=0)) < state.shape[0], "ssm_scan: batch")
    _chk(ssm_scan_takes(n_state, vdim), f"ssm_scan: no kernel for a state of {n_state} values a column (at most 256)")
    if not t:
        return
    work, work_bytes = 0, 0
    if ctx.max_q_len > SSM_CHUNK:
        need = _lib_fn("recurrent", "li_ssm_scan_work_bytes", [c_int] * 6 + [c_void_p], c_long)(
            t, ctx.num_segments, heads, vdim, n_state, SSM_CHUNK, None)
        buf = ws.buffer("ssm_scan.work", ((int(need) + 3) // 4,), torch.float32)
        work, work_bytes = buf.data_ptr(), buf.numel() * 4

    def ptr(v):
        return 0 if v is None else v.data_ptr()
    _run("recurrent", "li_ssm_scan", xbc.data_ptr(), xbc.stride(0), ptr(dt), 0 if dt is None else dt.stride(0), ptr(dt_bias), ptr(a_log),
         ptr(d), state.data_ptr(), ctx.state_slots.data_ptr(), ctx.q_start.data_ptr(), ctx.q_len.data_ptr(), y.data_ptr(),
         y.stride(0), heads, vdim, n_state, groups, SSM_CHUNK, t, ctx.num_segments, int(ctx.max_q_len), work, work_bytes,
         ptr(fixed_decay), float(fixed_step))


# Portions of more than SSM_CHUNK tokens run through the delta rule as chunks side by side (their own states and transition
# matrices, the carry, the outputs); False: token after token, whatever the portion.
DELTA_CHUNKED = True


def delta_scan_takes(n_state: int, vdim: int) -> bool:
    """Whether the delta-rule kernel has a layout for states of `n_state` values a column."""
    return bool(_lib_fn("recurrent", "li_delta_scan_takes", [c_int, c_int], c_int)(int(n_state), int(vdim)))


def delta_scan(xkq: torch.Tensor, ba: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, state: torch.Tensor, ctx,
               y: torch.Tensor, heads: int, vdim: int, n_state: int, groups: int, q_scale: float, ws=None) -> None:
    """The gated delta rule over each request's tokens of the step, from and into `state` [slots, heads, n_state, vdim]
    (float32):  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  y = S^T q,  with k and q made unit vectors
    (x / sqrt(sum x^2 + 1e-6); q times q_scale), beta = sigmoid(b), g = exp(-exp(a_log_h) softplus(a + dt_bias_h)).
    xkq: float32 rows [v: heads * vdim | k: groups * n_state | q: groups * n_state]; ba: float32 rows [b: heads | a: heads]
    (raw); y: float32 rows [heads * vdim].  All float32.  With a workspace `ws`, portions longer than SSM_CHUNK tokens run
    as chunks side by side (every chunk's own state and its transition matrix, then the chunks' starting states one after
    the other, then the outputs); without one, token after token."""
    _gpu(xkq, ba, dt_bias, a_log, state, y)
    t = y.shape[0]
    inner = heads * vdim
    _chk(all(x.dtype is torch.float32 for x in (xkq, ba, dt_bias, a_log, state, y)), "delta_scan: everything is float32")
    _chk(_rows_ok(xkq) and xkq.shape == (t, inner + 2 * groups * n_state) and _rows_ok(ba) and ba.shape == (t, 2 * heads)
         and _rows_ok(y) and y.shape == (t, inner), "delta_scan: rows")
    _chk(state.is_contiguous() and state.shape[1:] == (heads, n_state, vdim) and heads % groups == 0
         and all(v.numel() == heads and v.is_contiguous() for v in (dt_bias, a_log)), "delta_scan: state [slots, heads, N, vdim]")
    _chk(ctx.num_tokens == t and int(ctx.host_state_slots.max(initial=0)) < state.shape[0], "delta_scan: batch")
    _chk(delta_scan_takes(n_state, vdim), f"delta_scan: no kernel for a state of {n_state} values a column (at most 256)")
    if not t:
        return
    work, work_bytes, q = 0, 0, SSM_CHUNK
    if not DELTA_CHUNKED:
        ws = None
    if ctx.max_q_len > SSM_CHUNK and ws is not None:
        need = _lib_fn("recurrent", "li_delta_scan_work_bytes", [c_int] * 6 + [c_void_p], c_long)(
            t, ctx.num_segments, heads, vdim, n_state, SSM_CHUNK, None)
        buf = ws.buffer("delta_scan.work", ((int(need) + 3) // 4,), torch.float32)
        work, work_bytes = buf.data_ptr(), buf.numel() * 4
    elif ctx.max_q_len > SSM_CHUNK:
        q = int(ctx.max_q_len)                       # one chunk a request: the recurrence token after token
    _run("recurrent", "li_delta_scan", xkq.data_ptr(), xkq.stride(0), ba.data_ptr(), ba.stride(0), dt_bias.data_ptr(),
         a_log.data_ptr(), state.data_ptr(), ctx.state_slots.data_ptr(), ctx.q_start.data_ptr(), ctx.q_len.data_ptr(),
         y.data_ptr(), y.stride(0), heads, vdim, n_state, groups, float(q_scale), q, t, ctx.num_segments, int(ctx.max_q_len),
         work, work_bytes)


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: Optional[torch.Tensor], eps: float, groups: int, out: torch.Tensor,
                     gate_after: bool = False) -> None:
    """out = weight * v / sqrt(mean over the group of v^2 + eps), v = y * silu(z), every one of `groups` equal runs of
    columns by its own mean; with `gate_after` the norm sees y alone and its result is multiplied by silu(z).
    weight None: ones.  y, z float32 rows; out in either dtype."""
    _gpu(y, z, weight, out)
    t, n = out.shape
    _chk(y.dtype is torch.float32 and z.dtype is torch.float32 and _rows_ok(y) and _rows_ok(z) and y.shape == (t, n) and z.shape == (t, n)
         and _rows_ok(out) and out.dtype in _DT and (weight is None or (weight.dtype is torch.float32 and weight.numel() == n and weight.is_contiguous()))
         and groups > 0 and n % groups == 0, "gated_group_norm: y, z [T, n] float32, weight [n], out [T, n]")
    if t:
        _run("recurrent", "li_gated_group_norm", y.data_ptr(), y.stride(0), z.data_ptr(), z.stride(0),
             0 if weight is None else weight.data_ptr(), float(eps), out.data_ptr(), _DT[out.dtype], out.stride(0), t, n, int(groups),
             int(bool(gate_after)))


# --------------------------------------------------------------------------------------- routed feed-forward
MOE_TILE_ROWS = 32       # rows of one expert that a block of the products takes


MOE_BIG_TILE_ROWS = 64   # ... where the experts get hundreds of rows each (a prompt's portion),
MOE_HUGE_TILE_ROWS = 128  # and where they get still more


def moe_tile_rows(tokens: int, top: int, experts: int, a_dtype, w_dtype, sizes) -> int:
    """Rows a tile for a step of this many tokens: the large tiles where every expert gets twice their rows on average
    and the kernel that takes them has these operands (`sizes`: (n_out, K) of every product)."""
    takes = _lib_fn("moe", "li_moe_linear_big_takes", [c_int] * 4, c_int)
    if tokens * top >= 2 * MOE_BIG_TILE_ROWS * experts and a_dtype in _DT and w_dtype in _DT and all(
            takes(_DT[a_dtype], _DT[w_dtype], int(n), int(k)) for n, k in sizes):
        return MOE_HUGE_TILE_ROWS if tokens * top >= 2 * MOE_HUGE_TILE_ROWS * experts else MOE_BIG_TILE_ROWS
    return MOE_TILE_ROWS


def moe_max_tiles(tokens: int, top: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    """The most tiles a step can have: every expert's rows end in a tile that may not be full."""
    pairs = tokens * top
    return min(pairs, pairs // tile_rows + experts)


def moe_route(x: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], gate_row: Optional[torch.Tensor],
              idx: torch.Tensor, wt: torch.Tensor, gate: Optional[torch.Tensor], scores: str = "softmax_chosen",
              correction: Optional[torch.Tensor] = None, groups: int = 1, keep_groups: int = 1,
              group_score: str = "top2_sum", normalize: bool = True) -> None:
    """idx [T, top] int32: the experts with the largest logits x router^T + bias (float32 sums; the lower index wins a
    tie); wt [T, top] float32: softmax over the chosen logits; gate [T] = sigmoid(x . gate_row) where a row is given.
    With scores = "sigmoid" an expert's score is sigmoid(logit); the choice goes by score + correction[e], and only
    among the experts of the `keep_groups` groups (of experts / groups neighbours each) whose two largest choice
    values have the largest sum (`group_score` = "max": whose largest choice value is largest); wt = the chosen scores
    over their sum (+ 1e-20), or, with `normalize` False, the chosen scores themselves.  scores = "softmax": the same
    with an expert's score = the softmax over ALL logits."""
    _gpu(x, router, bias, gate_row, idx, wt, gate, correction)
    t, k = x.shape
    e, top = router.shape[0], idx.shape[1]
    _chk(scores in ("softmax_chosen", "sigmoid", "softmax") and group_score in ("top2_sum", "max"), "moe_route: scores")
    mode = {"softmax_chosen": 0, "sigmoid": 1, "softmax": 2}[scores]
    _chk(correction is None or (mode != 0 and correction.dtype is torch.float32 and correction.numel() == e
                                and correction.is_contiguous()), "moe_route: correction")
    _chk(1 <= keep_groups <= groups and e % groups == 0 and (mode != 0 or groups == 1)
         and (mode == 0 or top <= keep_groups * (e // groups)), "moe_route: groups")
    _chk(x.dtype in _DT and _rows_ok(x) and router.dtype in _DT and router.is_contiguous() and router.shape == (e, k)
         and (bias is None or (bias.dtype is torch.float32 and bias.numel() == e and bias.is_contiguous())), "moe_route: x, router, bias")
    _chk(idx.dtype is torch.int32 and idx.is_contiguous() and idx.shape == (t, top) and wt.dtype is torch.float32 and wt.is_contiguous()
         and wt.shape == (t, top) and 1 <= top <= min(e, 64), "moe_route: idx, wt [T, top], top at most 64")
    _chk((gate_row is None) == (gate is None) and (gate_row is None or (gate_row.dtype is router.dtype and gate_row.numel() == k
         and gate_row.is_contiguous() and gate.dtype is torch.float32 and gate.numel() == t and gate.is_contiguous())), "moe_route: gate")
    _chk((k + 2 * e + groups + 4) * 4 <= 60000, "moe_route: the row and the logits must fit 60 KB of LDS")
    if t:
        _run("moe", "li_moe_route", x.data_ptr(), _DT[x.dtype], x.stride(0), router.data_ptr(), _DT[router.dtype],
             0 if bias is None else bias.data_ptr(), 0 if gate_row is None else gate_row.data_ptr(), idx.data_ptr(), wt.data_ptr(),
             0 if gate is None else gate.data_ptr(), t, k, e, top,
             mode | (4 if group_score == "max" else 0) | (0 if normalize or mode == 0 else 8), 0 if correction is None else correction.data_ptr(),
             int(groups), int(keep_groups))


def moe_plan(idx: torch.Tensor, experts: int, plan: torch.Tensor, row_token: torch.Tensor, pair_row: torch.Tensor,
             tile_rows: int = MOE_TILE_ROWS) -> int:
    """Sorts the (token, choice) pairs by expert.  plan int32 [4 + 4 * max_tiles]: the number of tiles, then (expert,
    first row, rows, 0) a tile; row_token [pairs]: the token of a sorted row; pair_row [pairs]: the row of a pair.
    Returns max_tiles."""
    _gpu(idx, plan, row_token, pair_row)
    t, top = idx.shape
    max_tiles = moe_max_tiles(t, top, experts, tile_rows)
    _chk(tile_rows in (MOE_TILE_ROWS, MOE_BIG_TILE_ROWS, MOE_HUGE_TILE_ROWS), "moe_plan: tiles of 32, 64 or 128 rows")
    _chk(all(x.dtype is torch.int32 and x.is_contiguous() for x in (idx, plan, row_token, pair_row))
         and plan.numel() >= 4 + 4 * max_tiles and row_token.numel() >= t * top and pair_row.numel() >= t * top and experts <= 8000,
         "moe_plan: int32 arrays of the step's sizes")
    if t:
        _run("moe", "li_moe_plan", idx.data_ptr(), t, top, experts, plan.data_ptr(), max_tiles, row_token.data_ptr(), pair_row.data_ptr(),
             int(tile_rows))
    return max_tiles


def moe_linear(a: torch.Tensor, row_token: Optional[torch.Tensor], w: torch.Tensor, plan: torch.Tensor, max_tiles: int,
               out: torch.Tensor, rows: int, act: int = 0, tile_rows: int = MOE_TILE_ROWS, limit: float = 0.0) -> None:
    """out[row] = act(W[expert of the row's tile] a[src(row)]) for the sorted rows of the plan; src(row) = row_token[row]
    where given (rows gathered from tokens), else the row.  w [experts, n_out, K]; act 1: max(., 0)^2; act 2: the
    matrix rows are (gate, up) pairs, out[row, j] = silu(W[2j] a) * (W[2j + 1] a) and out has n_out / 2 columns; act 3:
    the same pairs with g = min(gate, limit), u = clamp(up, -limit, limit) and out = g sigmoid(1.702 g) (u + 1)."""
    _gpu(a, row_token, w, plan, out)
    e, n_out, k = w.shape
    _chk(act in (0, 1, 2, 3) and (act < 2 or n_out % 2 == 0) and (act != 3 or limit > 0), "moe_linear: act")
    _chk(a.dtype in _DT and _rows_ok(a) and a.shape[1] == k and w.dtype in _DT and w.is_contiguous() and out.dtype in _DT and _rows_ok(out)
         and out.shape == (rows, n_out // 2 if act >= 2 else n_out)
         and (w.dtype is torch.bfloat16 or (a.dtype is torch.float32 and out.dtype is torch.float32)),
         "moe_linear: a [*, K], w [E, n_out, K], out [rows, n_out]")
    _chk(plan.dtype is torch.int32 and plan.numel() >= 4 + 4 * max_tiles and (row_token is not None or a.shape[0] >= rows)
         and (row_token is None or (row_token.dtype is torch.int32 and row_token.numel() >= rows)), "moe_linear: plan, rows")
    if rows:
        _run("moe", "li_moe_linear", a.data_ptr(), _DT[a.dtype], a.stride(0), 0 if row_token is None else row_token.data_ptr(),
             w.data_ptr(), _DT[w.dtype], plan.data_ptr(), int(max_tiles), out.data_ptr(), _DT[out.dtype], out.stride(0), n_out, k, int(act),
             float(limit), int(tile_rows), int(rows))


def moe_combine(x: torch.Tensor, yrows: torch.Tensor, pair_row: torch.Tensor, wt: torch.Tensor, gate: Optional[torch.Tensor],
                shared_out: Optional[torch.Tensor], idx: Optional[torch.Tensor] = None, experts: int = 0,
                identity_rows: Optional[torch.Tensor] = None) -> None:
    """x[t] += sum_c wt[t, c] * yrows[pair_row[t * top + c]] (in the order of c) + gate[t] * shared_out[t]; float32.
    With `identity_rows` [T, H] (the feed-forward's input), a choice idx[t, c] >= experts is an identity expert whose
    output is identity_rows[t]."""
    _gpu(x, yrows, pair_row, wt, gate, shared_out, idx, identity_rows)
    t, h = x.shape
    top = wt.shape[1]
    _chk(x.dtype is torch.float32 and _rows_ok(x) and yrows.dtype is torch.float32 and _rows_ok(yrows) and yrows.shape == (t * top, h)
         and pair_row.dtype is torch.int32 and pair_row.numel() >= t * top and wt.dtype is torch.float32 and wt.is_contiguous()
         and wt.shape[0] == t, "moe_combine: x [T, H], yrows [T * top, H], pair_row, wt")
    _chk(shared_out is None or (shared_out.dtype is torch.float32 and _rows_ok(shared_out) and shared_out.shape == (t, h)
                                and (gate is None or (gate.dtype is torch.float32 and gate.numel() == t))), "moe_combine: shared")
    _chk(identity_rows is None or (idx is not None and idx.dtype is torch.int32 and idx.is_contiguous() and idx.shape == (t, top)
                                   and identity_rows.dtype in _DT and _rows_ok(identity_rows) and identity_rows.shape == (t, h)
                                   and experts >= 0), "moe_combine: identity experts")
    if t:
        _run("moe", "li_moe_combine", x.data_ptr(), x.stride(0), yrows.data_ptr(), yrows.stride(0), pair_row.data_ptr(), wt.data_ptr(),
             0 if gate is None else gate.data_ptr(), 0 if shared_out is None else shared_out.data_ptr(),
             0 if shared_out is None else shared_out.stride(0), t, h, top,
             0 if identity_rows is None else idx.data_ptr(), int(experts), 0 if identity_rows is None else identity_rows.data_ptr(),
             _DT[identity_rows.dtype] if identity_rows is not None else 0, 0 if identity_rows is None else identity_rows.stride(0))
