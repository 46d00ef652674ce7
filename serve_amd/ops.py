"""Python face of the HIP kernels: argument checks on the host, then one C call.

Every function checks on the host that shapes, dtypes, contiguity and device match what the
kernel and its grid assume, so that a wrong call is an exception and never a wild access on
the GPU.  There is no CPU path: tensors that are not on a GPU are refused, and a missing
library that cannot be compiled is an error (`serve_amd.csrc.build.BuildError`).
"""
from __future__ import annotations

import ctypes
import functools
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from .csrc.build import load_library

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

c_int = ctypes.c_int
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("serve_amd kernels run on the GPU only; got a tensor on " + str(t.device))
        if not t.is_contiguous():
            raise KernelError("kernel arguments must be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel arguments lie on different devices")


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _stream() -> c_void_p:
    # the current stream of the current device as a raw handle (what torch.cuda.current_stream()
    # wraps into an object, at thirty times the cost: this runs once per kernel launch)
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _ret(code: int, what: str) -> None:
    if code != 0:
        reason = {-1: "bad argument", -2: "unsupported combination of dtypes"}.get(code, f"HIP error {code}")
        raise KernelError(f"{what}: {reason}")


_CU_COUNT = {}


def compute_units(device=None) -> int:
    """Compute units of the device (asked once): the launch policies below fill these."""
    if not torch.cuda.is_available():
        return 256                      # planning on a host without a GPU (tests of the policies)
    dev = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    n = _CU_COUNT.get(dev)
    if n is None:
        n = _CU_COUNT[dev] = int(torch.cuda.get_device_properties(dev).multi_processor_count)
    return n


def _i32(t: torch.Tensor, n: int, name: str) -> None:
    _check(t.dtype == torch.int32 and t.numel() >= n, f"{name} must be int32 with at least {n} entries")


# ---------------------------------------------------------------------------------------------

def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor,
          src_row: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None,
          scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[tokens[t]] * scale as fp32 (the product is taken in fp32).  Where src_row[t] >= 0 the id is prev[src_row[t]] instead:
    a token sampled on the device by an earlier step.  Host-given ids have been checked against
    the table by the batch builder; the kernel clamps as a last resort."""
    _dev(table, tokens, out, src_row, prev)
    T = tokens.numel()
    _check(table.dim() == 2, "embedding table must be [V, d]")
    V, d = table.shape
    _i32(tokens, T, "tokens")
    _check(out.dtype == torch.float32 and out.shape == (T, d), "embed output must be fp32 [T, d]")
    if src_row is not None:
        _i32(src_row, T, "src_row")
        _check(prev is not None and prev.dtype == torch.int32, "prev must be int32")
    lib = load_library("elementwise")
    _ret(lib.sa_embed(_ptr(table), c_int(_code(table)), _ptr(tokens), _ptr(src_row), _ptr(prev), _ptr(out),
                      c_int(T), c_int(d), c_int(V), c_float(scale), _stream()), "embed")
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += delta (fp32 residual stream, in place), out = rmsnorm(x) * weight.

    `delta` is [T, d] in the activation dtype or fp32, or fp32 [parts, T, d]: partial sums of a
    product whose inner dimension was cut across workgroups; the parts are added in order.
    With `rows`, only the listed rows are produced (out[r] from source row rows[r]) and x is
    left as it was."""
    _dev(x, delta, weight, out, rows)
    _check(x.dtype == torch.float32 and x.dim() == 2, "residual stream must be fp32 [T, d]")
    T, d = x.shape
    _check(weight.shape == (d,), f"norm weight must be [{d}]")
    R = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, R, "rows")
    _check(out.shape == (R, d), f"norm output must be [{R}, {d}]")
    parts, delta_code = 1, _code(out)
    if delta is not None:
        if delta.dim() == 3:
            parts = delta.shape[0]
            _check(delta.dtype == torch.float32 and delta.shape[1:] == (T, d), "partial deltas must be fp32 [parts, T, d]")
        else:
            _check(delta.shape == (T, d) and delta.dtype in (out.dtype, torch.float32),
                   "delta must be [T, d] in the activation dtype or fp32")
        delta_code = _code(delta)
    lib = load_library("elementwise")
    _ret(lib.sa_add_rmsnorm(_ptr(x), _ptr(delta), c_int(delta_code), c_int(parts), _ptr(weight),
                            c_int(_code(weight)), _ptr(out), c_int(_code(out)), _ptr(rows), c_float(eps),
                            c_int(R), c_int(T), c_int(d), _stream()), "add_rmsnorm")
    return out


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with fp32 multiply and accumulate (vector ALU)."""
    _dev(a, w, out)
    _check(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm operands must be matrices")
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape[1] == K, f"gemm: inner sizes differ ({K} vs {w.shape[1]})")
    _check(out.shape == (M, N), f"gemm: output must be [{M}, {N}]")
    lib = load_library("gemm")
    _ret(lib.sa_gemm_nt(_ptr(a), c_int(_code(a)), _ptr(w), c_int(_code(w)), _ptr(out), c_int(_code(out)),
                        c_int(M), c_int(N), c_int(K), _stream()), "gemm_nt")
    return out


# rows of float32 activations that take the matrix-core kernel with the weights streamed once per 64 rows
F32_MID_MIN_ROWS = 9
F32_MID_MAX_ROWS = 128


def f32_mid_parts(M: int, N: int, K: int) -> int:
    """Into how many slices the inner dimension of a float32 product of F32_MID_MIN_ROWS..F32_MID_MAX_ROWS
    rows is cut across workgroups when its consumer adds the parts: a workgroup takes 32 rows of the
    weights, one per compute unit and pass of 64 rows is wanted, slices of at least 512."""
    groups = -(-N // 32) * -(-M // 64)
    cus = compute_units()
    parts = 1
    while parts < 8 and groups * parts < cus and K // (parts * 2) >= 512:
        parts *= 2
    return parts


def gemm_f32_mid_available(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.is_cuda and a.dtype == torch.float32 and w.dtype == torch.float32 and a.dim() == 2 and w.dim() == 2
            and F32_MID_MIN_ROWS <= a.shape[0] <= F32_MID_MAX_ROWS and a.shape[1] % 4 == 0
            and a.is_contiguous() and w.is_contiguous() and _aligned16(a, w))


def gemm_f32_mid_parts(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[p] = a[:, slice p of K] @ w[:, slice p of K]^T in float32 on the matrix cores, for
    F32_MID_MIN_ROWS..F32_MID_MAX_ROWS rows: out is fp32 [parts, M, N] (1 to 8 parts), whose sum over the
    parts is the product; the consumer adds them in order."""
    _dev(a, w, out)
    _check(gemm_f32_mid_available(a, w), "gemm_f32_mid_parts takes 9 to 128 rows of contiguous, 16-byte aligned "
           "float32 with an inner size that is a multiple of 4")
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape[1] == K, f"gemm: inner sizes differ ({K} vs {w.shape[1]})")
    _check(out.dim() == 3 and out.shape[1:] == (M, N) and 1 <= out.shape[0] <= 8 and out.dtype == torch.float32
           and out.is_contiguous(), f"gemm_f32_mid_parts: output must be fp32 [1..8, {M}, {N}]")
    lib = load_library("gemm")
    _ret(lib.sa_gemm_f32_mid_parts(_ptr(a), _ptr(w), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(out.shape[0]),
                                   _stream()), "gemm_f32_mid_parts")
    return out


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                  slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                  rot_dim: int, adjacent_pairs: bool, page_size: int) -> None:
    """Rotate q (in place) and k; store rotated k and v of every token at its cache slot.

    qkv [T, (Hq + 2 Hk) D]; k_pages [P, Hk, page_size, D]; v_pages [P, Hk, D, page_size];
    slots[t] = page * page_size + offset.  With `slots=None` only q is rotated (a mixer that
    reads another layer's cache) and the row holds q alone: qkv is [T, Hq D], Hk = 0."""
    write = slots is not None
    _dev(qkv, positions, inv_freq, slots, k_pages, v_pages)
    T = qkv.shape[0]
    Hk = num_kv_heads if write else 0
    _check(qkv.dim() == 2 and qkv.shape[1] == (num_heads + 2 * Hk) * head_dim,
           f"qkv must be [T, {(num_heads + 2 * Hk) * head_dim}]")
    _i32(positions, T, "positions")
    _check(inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dim // 2,
           f"inv_freq must be fp32 [{rot_dim // 2}]")
    _check(rot_dim % 2 == 0 and 0 <= rot_dim <= head_dim, "rot_dim must be even and at most head_dim")
    if write:
        _i32(slots, T, "slots")
        P = k_pages.shape[0]
        _check(k_pages.shape == (P, Hk, page_size, head_dim), "k_pages must be [P, Hk, page_size, D]")
        _check(v_pages.shape == (P, Hk, head_dim, page_size), "v_pages must be [P, Hk, D, page_size]")
        _check(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype must match activations")
    lib = load_library("elementwise")
    _ret(lib.sa_rope_kv_write(_ptr(qkv), c_int(_code(qkv)), _ptr(positions), _ptr(inv_freq), _ptr(slots),
                              _ptr(k_pages), _ptr(v_pages), c_int(_code(qkv)), c_int(T), c_int(num_heads),
                              c_int(Hk), c_int(head_dim), c_int(rot_dim), c_int(1 if adjacent_pairs else 0),
                              c_int(page_size), c_int(1 if write else 0), _stream()), "rope_kv_write")


SIMPLE_ATTENTION_MAX_HEAD_DIM = 640     # (SA_MAX_D of csrc/attention_simple.hip)


def _check_sinks(sinks: Optional[torch.Tensor], num_heads: int) -> None:
    """`sinks`: per query head one more term exp(sinks[h]) in the softmax's denominator, which takes weight
    away from the keys and adds nothing to the output (fp32 [Hq] on the device); None: a plain softmax."""
    if sinks is not None:
        _check(sinks.is_cuda and sinks.is_contiguous() and sinks.dtype == torch.float32
               and sinks.numel() == num_heads, f"sinks must be contiguous fp32 [{num_heads}] on the GPU")


def paged_attention_simple(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                           v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                           ctx_len: torch.Tensor, seg_of_token: torch.Tensor, num_tokens: int,
                           num_heads: int, scale: float, window: Optional[int],
                           sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of every token of the step over its request's cached keys (fp32 arithmetic), a wave
    per (token, head): the general form, for sizes that the other kernels do not take.

    q is the start of the q block of the fused qkv rows (row stride `q_row_stride` elements)."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len, seg_of_token)
    _check_sinks(sinks, num_heads)
    P, Hk, page_size, D = k_pages.shape
    _check(v_pages.shape == (P, Hk, D, page_size), "v_pages must be [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    _check(D <= SIMPLE_ATTENTION_MAX_HEAD_DIM, f"head_dim {D} is above this kernel's limit of {SIMPLE_ATTENTION_MAX_HEAD_DIM}")
    T = num_tokens
    _check(out.shape == (T, num_heads * D) and out.dtype == q.dtype, "attention output must be [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "cache dtype must match activations")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _i32(seg_of_token, T, "seg_of_token")
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_simple(
        _ptr(q), c_int(q_row_stride), _ptr(out), c_int(_code(q)), _ptr(k_pages), _ptr(v_pages),
        c_int(_code(k_pages)), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len),
        _ptr(seg_of_token), c_int(T), c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size),
        c_float(scale), c_int(window or 0), _ptr(sinks), _stream()), "paged_attention_simple")
    return out


def tiled_attention_available(q: torch.Tensor, k_pages: torch.Tensor, q_row_stride: int) -> bool:
    """float32 throughout, head sizes 16..128 in steps of 16, page sizes that are multiples of 4."""
    P, Hk, page_size, D = k_pages.shape
    return (q.dtype == torch.float32 and k_pages.dtype == torch.float32 and D % 16 == 0 and D <= 128
            and page_size % 4 == 0 and q_row_stride % 4 == 0 and q.data_ptr() % 16 == 0)


def paged_attention_tiled_f32(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                              v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                              ctx_len: torch.Tensor, num_tokens: int, max_q_len: int, num_heads: int,
                              scale: float, window: Optional[int], num_splits: int = 1,
                              sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 attention: 64 rows (tokens x the query heads of a KV head) a workgroup share the keys
    and values of their KV head through LDS (fp32 arithmetic on the vector ALU).  `num_splits` > 1
    cuts the key range of every tile into that many parts across workgroups, merged by a second kernel
    (for few rows over long contexts, where there are few tiles; the segments then begin at token 0).
    The tables may describe a run of the step's segments only: `num_tokens` then counts the tokens up
    to the end of the last of them, and only their rows of `out` are written."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    _check_sinks(sinks, num_heads)
    P, Hk, page_size, D = k_pages.shape
    _check(tiled_attention_available(q, k_pages, q_row_stride),
           f"paged_attention_tiled_f32 takes float32, head sizes 16..128 in steps of 16 and page sizes that are "
           f"multiples of 4; got head size {D}, page size {page_size}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.float32,
           "v_pages must be fp32 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    T = num_tokens
    _check(out.dim() == 2 and out.shape[0] >= T and out.shape[1] == num_heads * D and out.dtype == torch.float32,
           "attention output must be fp32 [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _check(1 <= max_q_len <= max(T, 1) and 1 <= num_splits <= 64, "max_q_len / num_splits out of range")
    part_o = part_ml = None
    if num_splits > 1:
        part_o = torch.empty((T * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_tiled_f32(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(T), c_int(max_q_len),
        c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0),
        c_int(num_splits), _ptr(part_o), _ptr(part_ml), _ptr(sinks), _stream()), "paged_attention_tiled_f32")
    return out


def paged_attention_decode_f32(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                               v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                               ctx_len: torch.Tensor, num_heads: int, scale: float, window: Optional[int],
                               num_splits: int = 1, first_token: int = 0,
                               sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 attention of B segments of one token each, a run of the step's tokens that begins at
    token `first_token` (the tables may be a slice of a longer step's; cu_q[i] must be first_token + i,
    which the caller knows on the host and the kernels do not check): a wave takes up to four query
    heads of a KV head, so that the keys and values are read once for them.  `num_splits` > 1 cuts
    every key range into that many parts across workgroups, merged by a second kernel."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    _check_sinks(sinks, num_heads)
    P, Hk, page_size, D = k_pages.shape
    _check(tiled_attention_available(q, k_pages, q_row_stride),
           f"paged_attention_decode_f32 takes float32, head sizes 16..128 in steps of 16 and page sizes that are "
           f"multiples of 4; got head size {D}, page size {page_size}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.float32,
           "v_pages must be fp32 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B = block_table.shape[0]
    _check(B <= 65535, "paged_attention_decode_f32 takes at most 65,535 segments")
    rows = first_token + B
    _check(first_token >= 0, "first_token must not be negative")
    _check(out.dim() == 2 and out.shape[0] >= rows and out.shape[1] == num_heads * D and out.dtype == torch.float32,
           "attention output must be fp32 [T, Hq D] with a row for every segment's token")
    _check(q.numel() >= (rows - 1) * q_row_stride + num_heads * D if B else True, "q is too short")
    _i32(cu_q, B + 1, "cu_q")
    _i32(ctx_len, B, "ctx_len")
    _check(1 <= num_splits <= 64, "num_splits out of range")
    part_o = part_ml = None
    if num_splits > 1:
        # the parts are indexed by token, like q and out
        part_o = torch.empty((rows * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((rows * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_simple")
    _ret(lib.sa_paged_attention_decode_f32(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(first_token), c_int(num_heads),
        c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0), c_int(num_splits), _ptr(part_o),
        _ptr(part_ml), _ptr(sinks), _stream()), "paged_attention_decode_f32")
    return out


# The float32 path's attention: steps of single tokens take the kernel with a wave per (segment, up to four
# heads of a KV head), cut into about FP32_DECODE_WAVES waves along the keys (at the 1B shape, batch 8 and
# context 4,096: 3.07 ms a step against 4.54 with the tiled kernel, whose workgroups do the arithmetic of 64 rows).
# Other steps take the tiled kernel when their longest segment has more than TILED_MIN_ROWS rows (tokens x
# query heads of a KV head) or the context reaches TILED_MIN_CONTEXT (few rows over many keys: the keys cut
# across workgroups), and the kernel with a wave per (token, head) otherwise.
TILED_MIN_ROWS = 16
TILED_MIN_CONTEXT = 256
FP32_DECODE_WAVES = 2048


# gated activations (csrc/common.h, gate_mul): silu(g) u; gelu_tanh(g) u; and, with g' = min(g, limit) and
# u' = clamp(u, -limit, limit), g' sigmoid(1.702 g') (u' + 1)
GATES = {"silu": 0, "gelu_tanh": 1, "clamped_swish": 2}


def gate_mul(gate_up: torch.Tensor, out: torch.Tensor, kind: str = "silu", limit: float = 0.0) -> torch.Tensor:
    """out[t, i] = gate(gate_up[t, i], gate_up[t, I + i]) for one of GATES; fp32 arithmetic."""
    _dev(gate_up, out)
    T, two_i = gate_up.shape
    _check(kind in GATES, f"unknown gate {kind!r}; known: {sorted(GATES)}")
    _check(kind != "clamped_swish" or limit > 0.0, "the clamped gate needs a positive limit")
    _check(two_i % 2 == 0 and out.shape == (T, two_i // 2) and out.dtype == gate_up.dtype,
           "gate_mul: out must be [T, I] for gate_up [T, 2 I]")
    lib = load_library("elementwise")
    _ret(lib.sa_gate_mul(_ptr(gate_up), _ptr(out), c_int(_code(out)), c_int(T), c_int(two_i // 2),
                         c_int(GATES[kind]), c_float(limit), _stream()), "gate_mul")
    return out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    return gate_mul(gate_up, out, "silu")


# ---------------------------------------------------------------------------------------------
# layers whose norm sits on the sublayer's output; plain activations
# ---------------------------------------------------------------------------------------------

def _f32vec(t: torch.Tensor, n: int, name: str) -> None:
    _check(t.dtype == torch.float32 and t.numel() == n, f"{name} must be fp32 with {n} entries")


def output_norm_add(x: torch.Tensor, y: Optional[torch.Tensor], weight: Optional[torch.Tensor],
                    scale: Optional[torch.Tensor], eps: float, h: Optional[torch.Tensor],
                    next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0) -> Optional[torch.Tensor]:
    """x += (y / sqrt(mean(y^2) + eps) * weight) * scale on the fp32 residual stream x [T, d], in place;
    `h` (activation dtype [T, d]) receives a copy of the new x.  y is [T, d] in h's dtype or fp32, or
    fp32 [parts, T, d] partial sums that are added in order.  y None: only the copy is made.
    With `next_weight` (fp32 [d]; needs y and h): h = x / sqrt(mean(x^2) + next_eps) * next_weight of the new
    x instead of its copy: the norm in front of the sublayer that reads the stream next."""
    _dev(x, y, weight, scale, h, next_weight)
    _check(x.dtype == torch.float32 and x.dim() == 2, "residual stream must be fp32 [T, d]")
    T, d = x.shape
    act = h.dtype if h is not None else (y.dtype if y is not None and y.dim() == 2 else torch.float32)
    parts, ycode = 1, F32
    if y is not None:
        _f32vec(weight, d, "norm weight")
        _f32vec(scale, d, "layer scale")
        if y.dim() == 3:
            parts = y.shape[0]
            _check(y.dtype == torch.float32 and y.shape[1:] == (T, d), "partial sums must be fp32 [parts, T, d]")
        else:
            _check(y.shape == (T, d) and y.dtype in (act, torch.float32), "y must be [T, d] in the activation dtype or fp32")
        ycode = _code(y)
    if h is not None:
        _check(h.shape == (T, d), "the stream's copy must be [T, d]")
    if next_weight is not None:
        _check(y is not None and h is not None, "the norm of the new stream needs a sublayer's output and a place to go")
        _f32vec(next_weight, d, "the next norm's weight")
    lib = load_library("sublayer")
    _ret(lib.sa_output_norm_add(_ptr(x), _ptr(y), c_int(ycode), c_int(parts), _ptr(weight), _ptr(scale), _ptr(h),
                                c_int(_DT[act]), c_float(eps), c_int(T), c_int(d), _ptr(next_weight), c_float(next_eps),
                                _stream()), "output_norm_add")
    return h


ACTIVATIONS = {"gelu_tanh": 0, "silu": 1, "relu_squared": 2}


def activation(a: torch.Tensor, kind: str) -> torch.Tensor:
    """a = act(a) in place: 'gelu_tanh' (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))), 'silu' or
    'relu_squared' (max(z, 0)^2)."""
    _dev(a)
    _check(kind in ACTIVATIONS, f"unknown activation {kind!r}; known: {sorted(ACTIVATIONS)}")
    lib = load_library("sublayer")
    _ret(lib.sa_activation(_ptr(a), c_int(_code(a)), ctypes.c_longlong(a.numel()), c_int(ACTIVATIONS[kind]),
                           _stream()), "activation")
    return a


def sigmoid_mul(a: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """a *= sigmoid(g) in place, element by element (an output gate); a and g contiguous, of one shape and dtype."""
    _dev(a, g)
    _check(a.shape == g.shape and a.dtype == g.dtype and a.is_contiguous() and g.is_contiguous(),
           "the gate's logits must have the shape and dtype of what they gate, both contiguous")
    lib = load_library("sublayer")
    _ret(lib.sa_sigmoid_mul(_ptr(a), _ptr(g), c_int(_code(a)), ctypes.c_longlong(a.numel()), _stream()), "sigmoid_mul")
    return a


# ---------------------------------------------------------------------------------------------
# gated delta rule
# ---------------------------------------------------------------------------------------------
DELTA_MAX_DIM = 256
DELTA_MAX_TAPS = 16


def delta_rule(z: torch.Tensor, conv_w: torch.Tensor, ba: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor,
               norm_w: torch.Tensor, state: torch.Tensor, ctx, y: torch.Tensor, eps: float, heads: int,
               kv_heads: int, dk: int, dv: int, taps: int) -> torch.Tensor:
    """The gated delta rule over the step's tokens.  z [T, >= C + H dv]: the projections
    [q: Hk dk | k: Hk dk | v: H dv | gate: H dv] (C = the first three: the convolution's channels);
    conv_w fp32 [C, taps]; ba fp32 [T, 2 H] (beta's logits, then the decay's); state fp32
    [slots, H dk dv + (taps - 1) C], a request's row (ctx.state_slots, -1: none) read and written;
    y [T, H dv] in z's dtype: the normed, gated read-out."""
    _dev(z, conv_w, ba, A_log, dt_bias, norm_w, state, y, ctx.seg_of_token, ctx.cu_q, ctx.state_slots)
    T, B = ctx.num_tokens, ctx.num_segments
    H, Hk = heads, kv_heads
    C = 2 * Hk * dk + H * dv
    _check(z.dim() == 2 and z.shape[0] == T and z.shape[1] >= C + H * dv, f"z must be [T, >= {C + H * dv}]")
    _check(H % Hk == 0 and 0 < dk <= DELTA_MAX_DIM and 0 < dv <= DELTA_MAX_DIM and 1 <= taps <= DELTA_MAX_TAPS,
           f"delta rule: head sizes up to {DELTA_MAX_DIM}, up to {DELTA_MAX_TAPS} taps")
    _check(conv_w.dtype == torch.float32 and conv_w.shape == (C, taps), f"conv_w must be fp32 [{C}, {taps}]")
    _check(ba.dtype == torch.float32 and ba.shape == (T, 2 * H), f"ba must be fp32 [T, {2 * H}]")
    _f32vec(A_log, H, "A_log")
    _f32vec(dt_bias, H, "dt_bias")
    _f32vec(norm_w, dv, "norm weight")
    need = H * dk * dv + (taps - 1) * C
    _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= need,
           f"state rows must be fp32 with at least {need} entries")
    _check(y.shape == (T, H * dv) and y.dtype == z.dtype, "y must be [T, H dv] in z's dtype")
    _i32(ctx.seg_of_token, T, "seg_of_token")
    _i32(ctx.cu_q, B + 1, "cu_q")
    _i32(ctx.state_slots, B, "state_slots")
    lib = load_library("delta_rule")
    lib.sa_delta_rule_work_floats.restype = ctypes.c_longlong
    work = torch.empty(int(lib.sa_delta_rule_work_floats(c_int(T), c_int(H), c_int(Hk), c_int(dk), c_int(dv))),
                       dtype=torch.float32, device=z.device)
    _ret(lib.sa_delta_rule(_ptr(z), c_int(_code(z)), c_int(z.shape[1]), _ptr(conv_w), _ptr(ba), _ptr(A_log),
                           _ptr(dt_bias), _ptr(norm_w), _ptr(state), ctypes.c_longlong(state.shape[1]),
                           _ptr(ctx.seg_of_token), _ptr(ctx.cu_q), _ptr(ctx.state_slots), _ptr(work), _ptr(y),
                           c_float(eps), c_int(T), c_int(B), c_int(int(getattr(ctx, "max_q_len", T) or T)), c_int(H), c_int(Hk), c_int(dk),
                           c_int(dv), c_int(taps),
                           _stream()), "delta_rule")
    return y


# ---------------------------------------------------------------------------------------------
# latent attention
# ---------------------------------------------------------------------------------------------

def latent_kv_write(z: torch.Tensor, norm_w: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                    slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, eps: float, rank: int,
                    rot_dim: int, magnitude: float = 1.0) -> None:
    """z [T, rank + rot_dim] -> the token's cache rows: k_pages [P, 1, page, Dp] gets
    [normed latent | rotated key part | 0], v_pages [P, 1, Dp, page] the normed latent (and zeros).
    `magnitude` multiplies the rotation's sine and cosine."""
    _dev(z, norm_w, positions, inv_freq, slots, k_pages, v_pages)
    T = z.shape[0]
    _check(z.dim() == 2 and z.shape[1] == rank + rot_dim, f"z must be [T, {rank + rot_dim}]")
    P, one, page_size, Dp = k_pages.shape
    _check(one == 1 and Dp >= rank + rot_dim and v_pages.shape == (P, 1, Dp, page_size),
           "latent pages must be [P, 1, page, Dp] and [P, 1, Dp, page]")
    _check(k_pages.dtype == z.dtype and v_pages.dtype == z.dtype, "cache dtype must match activations")
    _f32vec(norm_w, rank, "latent norm weight")
    _f32vec(inv_freq, rot_dim // 2, "inv_freq")
    _i32(positions, T, "positions")
    _i32(slots, T, "slots")
    lib = load_library("latent")
    _ret(lib.sa_latent_kv_write(_ptr(z), c_int(_code(z)), _ptr(norm_w), _ptr(positions), _ptr(inv_freq), _ptr(slots),
                                _ptr(k_pages), _ptr(v_pages), c_float(eps), c_int(T), c_int(rank), c_int(rot_dim),
                                c_int(Dp), c_int(page_size), c_float(magnitude), _stream()), "latent_kv_write")


def head_linear(x: torch.Tensor, in_stride: int, in_head_stride: int, w: torch.Tensor, out: torch.Tensor,
                out_stride: int, out_head_stride: int, T: int, positions: Optional[torch.Tensor] = None,
                inv_freq: Optional[torch.Tensor] = None, rot: int = 0, tail: int = 0,
                magnitude: float = 1.0) -> torch.Tensor:
    """out[t, h, :N] = x[t, h, :K] @ w[h] for w [H, K, N]: head h's K inputs of token t start at element
    t * in_stride + h * in_head_stride of x, its N outputs at t * out_stride + h * out_head_stride of out.
    With `positions`: behind the N outputs come the `rot` inputs that lie behind the head's K inputs, rotated by
    the token's position (dimension i with i + rot / 2, angles positions[t] * inv_freq[i], sine and cosine times
    `magnitude`), then zeros up to `tail` places in all."""
    _dev(x, w, out, positions, inv_freq)
    _check(w.dim() == 3 and x.dtype == w.dtype == out.dtype, "head_linear: w must be [H, K, N], one dtype throughout")
    H, K, N = w.shape
    if T:
        _check(x.numel() >= (T - 1) * in_stride + (H - 1) * in_head_stride + K, "head_linear: input too short")
        _check(out.numel() >= (T - 1) * out_stride + (H - 1) * out_head_stride + N + tail, "head_linear: output too short")
    if positions is not None:
        _i32(positions, T, "positions")
        _check(rot % 2 == 0 and 0 <= rot <= tail and in_head_stride >= K + rot and out_head_stride >= N + tail,
               "head_linear: the rotated inputs lie behind a head's K inputs, the tail behind its N outputs")
        _f32vec(inv_freq, rot // 2, "inv_freq")
        if T:
            _check(x.numel() >= (T - 1) * in_stride + (H - 1) * in_head_stride + K + rot, "head_linear: input too short")
    lib = load_library("latent")
    _ret(lib.sa_head_linear(_ptr(x), c_int(in_stride), c_int(in_head_stride), _ptr(w), _ptr(out), c_int(out_stride),
                            c_int(out_head_stride), c_int(_code(x)), c_int(T), c_int(H), c_int(K), c_int(N),
                            _ptr(positions), _ptr(inv_freq), c_int(rot), c_int(tail), c_float(magnitude),
                            _stream()), "head_linear")
    return out


# ---------------------------------------------------------------------------------------------
# attention with normed queries and keys
# ---------------------------------------------------------------------------------------------

def qk_norm_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor, slots: Optional[torch.Tensor],
                     k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], q_weight: torch.Tensor,
                     k_weight: torch.Tensor, eps: float, num_heads: int, num_kv_heads: int, dim: int, vdim: int,
                     temp_coef: float = 0.0, temp_every: int = 0, v_first: Optional[torch.Tensor] = None,
                     v_blend: float = 0.0) -> torch.Tensor:
    """From rows qkv [T, Hq D | Hk D | Hk Dv]: every query and key head over its root mean square (eps inside
    the root) times `q_weight` / `k_weight` (fp32 [D]); queries at position p times
    1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) (temp_every 0: not); values blended as
    (1 - v_blend) v + v_blend v_first (v_first [T, >= Hk Dv] rows, may be a view with a row stride; None: not).
    Queries go to q_out [T, Hq Dp], keys and values to the token's slot of k_pages [P, Hk, page, Dp] and
    v_pages [P, Hk, Dp, page], each padded with zeros up to the cache's head size Dp.  `slots` None: queries only."""
    _dev(q_out, positions, slots, k_pages, v_pages, q_weight, k_weight)
    Hq, Hk, D, Dv = num_heads, num_kv_heads, dim, vdim
    T = qkv.shape[0]
    _check(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= Hq * D + Hk * (D + Dv),
           f"qkv must be rows of at least {Hq * D + Hk * (D + Dv)} on the GPU")
    _check(q_out.dim() == 2 and q_out.shape[0] == T and q_out.shape[1] % Hq == 0 and q_out.dtype == qkv.dtype,
           "q_out must be [T, Hq Dp] in the dtype of qkv")
    Dp = q_out.shape[1] // Hq
    _check(Dp >= D and Dp >= Dv, f"the padded head size {Dp} is below dim {D} or vdim {Dv}")
    _f32vec(q_weight, D, "q norm weight")
    _f32vec(k_weight, D, "k norm weight")
    _i32(positions, T, "positions")
    page_size = 1
    if slots is not None:
        _i32(slots, T, "slots")
        P, _, page_size, _ = k_pages.shape
        _check(k_pages.shape == (P, Hk, page_size, Dp) and v_pages.shape == (P, Hk, Dp, page_size),
               f"the cache must be k [P, {Hk}, page, {Dp}] and v [P, {Hk}, {Dp}, page]")
        _check(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype must match activations")
    vf_stride = 0
    if v_first is not None:
        _check(v_first.is_cuda and v_first.device == qkv.device and v_first.dim() == 2 and v_first.shape[0] == T
               and v_first.stride(1) == 1 and v_first.shape[1] >= Hk * Dv and v_first.dtype == qkv.dtype,
               f"v_first must be [T, >= {Hk * Dv}] rows in the dtype of qkv")
        vf_stride = v_first.stride(0)
    _check(temp_every >= 0, "temp_every must not be negative")
    lib = load_library("qk_norm")
    _ret(lib.sa_qk_norm_kv_write(_ptr(qkv), c_int(qkv.stride(0)), _ptr(q_out), c_int(_code(qkv)), _ptr(positions),
                                 _ptr(slots), _ptr(k_pages if slots is not None else None),
                                 _ptr(v_pages if slots is not None else None), _ptr(q_weight), _ptr(k_weight),
                                 c_float(eps), c_float(temp_coef), c_int(temp_every), _ptr(v_first), c_int(vf_stride),
                                 c_float(v_blend), c_int(T), c_int(Hq), c_int(Hk), c_int(D), c_int(Dv), c_int(Dp),
                                 c_int(page_size), _stream()), "qk_norm_kv_write")
    return q_out


def row_norm_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                           slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                           v_pages: Optional[torch.Tensor], q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float,
                           inv_freq: Optional[torch.Tensor], rot_dim: int, num_heads: int, num_kv_heads: int, dim: int,
                           vdim: int) -> torch.Tensor:
    """From rows qkv [T, Hq D | Hk D | Hk Dv | ...]: all queries of a token over their common root mean square (eps
    inside the root) times `q_weight` (fp32 [Hq D]), all its keys likewise with `k_weight` (fp32 [Hk D]); then in every
    head the first `rot_dim` dims rotated by position * inv_freq[i] (dim i paired with i + rot_dim / 2).  Queries go
    to q_out [T, Hq Dp], keys and values to the token's slot of k_pages [P, Hk, page, Dp] and v_pages
    [P, Hk, Dp, page], each head padded with zeros up to Dp.  `slots` None: queries only."""
    _dev(q_out, positions, slots, k_pages, v_pages, q_weight, k_weight, inv_freq)
    Hq, Hk, D, Dv = num_heads, num_kv_heads, dim, vdim
    T = qkv.shape[0]
    _check(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= Hq * D + Hk * (D + Dv),
           f"qkv must be rows of at least {Hq * D + Hk * (D + Dv)} on the GPU")
    _check(q_out.dim() == 2 and q_out.shape[0] == T and q_out.shape[1] % Hq == 0 and q_out.dtype == qkv.dtype,
           "q_out must be [T, Hq Dp] in the dtype of qkv")
    Dp = q_out.shape[1] // Hq
    _check(Dp >= D and Dp >= Dv, f"the padded head size {Dp} is below dim {D} or vdim {Dv}")
    _f32vec(q_weight, Hq * D, "q norm weight")
    _f32vec(k_weight, Hk * D, "k norm weight")
    _check(rot_dim >= 0 and rot_dim % 2 == 0 and rot_dim <= D, "rot_dim must be even and within dim")
    if rot_dim:
        _f32vec(inv_freq, rot_dim // 2, "inv_freq")
    _i32(positions, T, "positions")
    page_size = 1
    if slots is not None:
        _i32(slots, T, "slots")
        P, _, page_size, _ = k_pages.shape
        _check(k_pages.shape == (P, Hk, page_size, Dp) and v_pages.shape == (P, Hk, Dp, page_size),
               f"the cache must be k [P, {Hk}, page, {Dp}] and v [P, {Hk}, {Dp}, page]")
        _check(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype must match activations")
    lib = load_library("qk_norm")
    _ret(lib.sa_row_norm_rope_kv_write(_ptr(qkv), ctypes.c_longlong(qkv.stride(0)), _ptr(q_out), c_int(_code(qkv)),
                                       _ptr(positions), _ptr(slots), _ptr(k_pages if slots is not None else None),
                                       _ptr(v_pages if slots is not None else None), _ptr(q_weight), _ptr(k_weight),
                                       c_float(eps), _ptr(inv_freq if rot_dim else None), c_int(rot_dim), c_int(T),
                                       c_int(Hq), c_int(Hk), c_int(D), c_int(Dv), c_int(Dp), c_int(page_size),
                                       _stream()), "row_norm_rope_kv_write")
    return q_out


def bias_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                       slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                       v_pages: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                       inv_freq: Optional[torch.Tensor], rot_dim: int, adjacent_pairs: bool, magnitude: float,
                       num_heads: int, num_kv_heads: int, dim: int, vdim: int) -> torch.Tensor:
    """From rows qkv [T, Hq D | Hk D | Hk Dv | ...]: plus `bias` (fp32 over the Hq D + Hk (D + Dv) columns, or None); in
    every query and key head the first `rot_dim` dims rotated by position * inv_freq[j] (pair j = (j, j + rot_dim / 2), or
    (2j, 2j + 1) with `adjacent_pairs`), sine and cosine times `magnitude`.  Queries go to q_out [T, Hq Dp], keys and
    values to the token's slot of k_pages [P, Hk, page, Dp] and v_pages [P, Hk, Dp, page], each head padded with
    zeros up to Dp.  `slots` None: queries only."""
    _dev(q_out, positions, slots, k_pages, v_pages, bias, inv_freq)
    Hq, Hk, D, Dv = num_heads, num_kv_heads, dim, vdim
    T = qkv.shape[0]
    cols = Hq * D + Hk * (D + Dv)
    _check(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= cols,
           f"qkv must be rows of at least {cols} on the GPU")
    _check(q_out.dim() == 2 and q_out.shape[0] == T and q_out.shape[1] % Hq == 0 and q_out.dtype == qkv.dtype
           and q_out.is_contiguous(), "q_out must be contiguous [T, Hq Dp] in the dtype of qkv")
    Dp = q_out.shape[1] // Hq
    _check(Dp >= D and Dp >= Dv, f"the padded head size {Dp} is below dim {D} or vdim {Dv}")
    if bias is not None:
        _f32vec(bias, cols, "bias")
    _check(rot_dim >= 0 and rot_dim % 2 == 0 and rot_dim <= D, "rot_dim must be even and within dim")
    if rot_dim:
        _f32vec(inv_freq, rot_dim // 2, "inv_freq")
    _i32(positions, T, "positions")
    page_size = 1
    if slots is not None:
        _i32(slots, T, "slots")
        P, _, page_size, _ = k_pages.shape
        _check(k_pages.shape == (P, Hk, page_size, Dp) and v_pages.shape == (P, Hk, Dp, page_size),
               f"the cache must be k [P, {Hk}, page, {Dp}] and v [P, {Hk}, {Dp}, page]")
        _check(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype must match activations")
    lib = load_library("qk_norm")
    _ret(lib.sa_bias_rope_kv_write(_ptr(qkv), ctypes.c_longlong(qkv.stride(0)), _ptr(q_out), c_int(_code(qkv)),
                                   _ptr(positions), _ptr(slots), _ptr(k_pages if slots is not None else None),
                                   _ptr(v_pages if slots is not None else None), _ptr(bias),
                                   _ptr(inv_freq if rot_dim else None), c_int(rot_dim), c_int(1 if adjacent_pairs else 0),
                                   c_float(magnitude), c_int(T), c_int(Hq), c_int(Hk), c_int(D), c_int(Dv), c_int(Dp),
                                   c_int(page_size), _stream()), "bias_rope_kv_write")
    return q_out


def head_gate(a: torch.Tensor, rows: torch.Tensor, col: int, num_heads: int) -> torch.Tensor:
    """a[t, h, :] *= sigmoid(rows[t, col + h]) in place: a [T, H Dp], the heads' gate logits in the columns
    col .. col + H - 1 of `rows` (which may be a wider product's output)."""
    _dev(a)
    T = a.shape[0]
    _check(a.dim() == 2 and a.shape[1] % num_heads == 0, "a must be [T, H Dp]")
    _check(rows.is_cuda and rows.device == a.device and rows.dim() == 2 and rows.stride(1) == 1 and rows.shape[0] == T
           and rows.dtype == a.dtype and 0 <= col and col + num_heads <= rows.shape[1],
           "the gate logits must be columns of [T, >= col + H] rows in a's dtype")
    lib = load_library("qk_norm")
    _ret(lib.sa_head_gate(_ptr(a), _ptr(rows), c_int(_code(a)), ctypes.c_longlong(rows.stride(0)), c_int(col), c_int(T),
                          c_int(num_heads), c_int(a.shape[1] // num_heads), _stream()), "head_gate")
    return a


# ---------------------------------------------------------------------------------------------
# around the residual stream
# ---------------------------------------------------------------------------------------------

def _parts_of(y: torch.Tensor, T: int, d: int, what: str):
    if y.dim() == 3:
        _check(y.dtype == torch.float32 and y.shape[1:] == (T, d), f"{what}: partial sums must be fp32 [parts, T, d]")
        return y.shape[0]
    _check(y.shape == (T, d), f"{what} must be [T, d]")
    return 1


def stream_add(x: torch.Tensor, y: Optional[torch.Tensor], vec: Optional[torch.Tensor] = None,
               h: Optional[torch.Tensor] = None, extra: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x += y + vec + extra on the fp32 residual stream x [T, d], in place (y: [T, d] or fp32 [parts, T, d] partial sums,
    added in order; vec fp32 [d]; extra fp32 [T, d]; each may be None), and `h` ([T, d], any kernel dtype) receives a
    copy of the new x."""
    _dev(x, y, vec, h, extra)
    _check(x.dtype == torch.float32 and x.dim() == 2, "residual stream must be fp32 [T, d]")
    T, d = x.shape
    parts, ycode = 1, F32
    if y is not None:
        parts, ycode = _parts_of(y, T, d, "y"), _code(y)
    if vec is not None:
        _f32vec(vec, d, "the row vector")
    if h is not None:
        _check(h.shape == (T, d), "the stream's copy must be [T, d]")
    if extra is not None:
        _check(extra.dtype == torch.float32 and extra.shape == (T, d) and extra.is_contiguous(),
               "the second array must be contiguous fp32 [T, d]")
    lib = load_library("stream_ops")
    _ret(lib.sa_stream_add(_ptr(x), _ptr(y), c_int(ycode), c_int(parts), _ptr(vec), _ptr(extra), _ptr(h),
                           c_int(_code(h) if h is not None else F32), c_int(T), c_int(d), _stream()), "stream_add")
    return h


def pair_embed(table: torch.Tensor, pair_table: torch.Tensor, ctx, last: torch.Tensor, out: torch.Tensor,
               mul_prev: int, mul_cur: int, keep: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = table[tok_t] + pair_table[(prev_t * mul_prev + tok_t * mul_cur) mod buckets] as fp32, with
    pair_table [buckets + 1, d] whose last row serves a sequence's first token (position 0).  prev_t is the token
    before t in its segment, or what `last` (int32 [slots, 1], by the segment's state slot) holds for the segment's
    first token; afterwards `last` holds every segment's last token.  `ctx`: the step (token_ids, positions,
    seg_of_token, cu_q, state_slots, src_row / prev_tokens for tokens sampled on the device).  `keep`: a second
    copy of the result (fp32 [T, d])."""
    _dev(table, pair_table, last, out, keep, ctx.token_ids, ctx.positions, ctx.seg_of_token, ctx.cu_q, ctx.state_slots,
         ctx.src_row, ctx.prev_tokens)
    T, B = ctx.token_ids.numel(), ctx.state_slots.numel()
    _check(table.dim() == 2 and pair_table.dim() == 2 and pair_table.shape[1] == table.shape[1]
           and pair_table.shape[0] >= 2 and table.dtype == pair_table.dtype and table.is_contiguous()
           and pair_table.is_contiguous(), "the tables must be [V, d] and [buckets + 1, d] of one dtype")
    V, d = table.shape
    _check(out.dtype == torch.float32 and out.shape == (T, d) and out.is_contiguous(), "the output must be fp32 [T, d]")
    if keep is not None:
        _check(keep.dtype == torch.float32 and keep.shape == (T, d) and keep.is_contiguous(), "the copy must be fp32 [T, d]")
    _check(last.dtype == torch.int32 and last.is_contiguous() and last.dim() == 2 and last.shape[1] == 1,
           "the previous tokens must be int32 [slots, 1]")
    _check(mul_prev >= 0 and mul_cur >= 0, "the multipliers must not be negative")
    for name in ("token_ids", "positions", "seg_of_token"):
        _i32(getattr(ctx, name), T, name)
    _i32(ctx.cu_q, B + 1, "cu_q")
    _i32(ctx.state_slots, B, "state_slots")
    if ctx.src_row is not None:
        _i32(ctx.src_row, T, "src_row")
        _check(ctx.prev_tokens is not None and ctx.prev_tokens.dtype == torch.int32, "sampled tokens must be int32")
    lib = load_library("stream_ops")
    _ret(lib.sa_pair_embed(_ptr(table), _ptr(pair_table), c_int(_code(table)), _ptr(ctx.token_ids), _ptr(ctx.src_row),
                           _ptr(ctx.prev_tokens), _ptr(ctx.positions), _ptr(ctx.seg_of_token), _ptr(ctx.cu_q),
                           _ptr(ctx.state_slots), _ptr(last), _ptr(out), _ptr(keep), c_int(T), c_int(B), c_int(d),
                           c_int(V), c_int(pair_table.shape[0] - 1), ctypes.c_longlong(mul_prev),
                           ctypes.c_longlong(mul_cur), _stream()), "pair_embed")
    return out


def dual_norm_mix(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, ca: float, cb: float,
                  eps: float, out: torch.Tensor) -> torch.Tensor:
    """out = ca N(a) wa + cb N(b) wb per row, N(y) = y / sqrt(mean(y^2) + eps); a and b [T, d] or fp32 [parts, T, d]
    partial sums; wa, wb fp32 [d]; out fp32 [T, d]."""
    _dev(a, b, wa, wb, out)
    _check(out.dtype == torch.float32 and out.dim() == 2, "the mixed output must be fp32 [T, d]")
    T, d = out.shape
    pa, pb = _parts_of(a, T, d, "a"), _parts_of(b, T, d, "b")
    _f32vec(wa, d, "the first norm's weight")
    _f32vec(wb, d, "the second norm's weight")
    lib = load_library("stream_ops")
    _ret(lib.sa_dual_norm_mix(_ptr(a), c_int(_code(a)), c_int(pa), _ptr(b), c_int(_code(b)), c_int(pb), _ptr(wa), _ptr(wb),
                              c_float(ca), c_float(cb), c_float(eps), _ptr(out), c_int(T), c_int(d), _stream()),
         "dual_norm_mix")
    return out


def gelu_mul_rows(z: torch.Tensor, table: torch.Tensor, col: int, tokens: torch.Tensor, out: torch.Tensor,
                  src_row: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, j] = gelu_tanh(z[t, j]) * table[token_t, col + j] for z [T, n]; the token of row t is tokens[t], or
    prev[src_row[t]] where src_row[t] >= 0 (a token sampled on the device by an earlier step)."""
    _dev(z, table, tokens, out, src_row, prev)
    _check(z.dim() == 2 and out.shape == z.shape and out.dtype == z.dtype, "z and out must be [T, n] of one dtype")
    T, n = z.shape
    _check(table.dim() == 2 and 0 <= col and col + n <= table.shape[1], "the table must be [V, >= col + n]")
    _i32(tokens, T, "tokens")
    if src_row is not None:
        _i32(src_row, T, "src_row")
        _check(prev is not None and prev.dtype == torch.int32, "prev must be int32")
    lib = load_library("stream_ops")
    _ret(lib.sa_gelu_mul_rows(_ptr(z), c_int(_code(z)), _ptr(table), c_int(_code(table)),
                              ctypes.c_longlong(table.shape[1]), c_int(col), _ptr(tokens), _ptr(src_row), _ptr(prev),
                              _ptr(out), c_int(T), c_int(n), c_int(table.shape[0]), _stream()), "gelu_mul_rows")
    return out


# ---------------------------------------------------------------------------------------------
# recurrences S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t
# ---------------------------------------------------------------------------------------------
SCAN_MAX_DIM = 256
SCAN_MAX_TAPS = 16
SCAN_BLOCK_MIN_TOKENS = 6        # csrc/recurrent_scan.hip: RS_BLOCK_MIN_TOKENS
SCAN_PIECE_MIN = 64              # the shortest piece that a long segment is cut into
SCAN_PIECE_BUSY = 256            # segments are cut where a step's longest ones have fewer workgroups than this (a CU each) ...
SCAN_PIECE_GROUPS = 512          # ... into so many pieces that they have this many (with 256 and more, cutting lost: 288 -> 389 us)
SCAN_PIECE_SCRATCH_BYTES = 1 << 30


def _pow2_rows(dk: int) -> int:
    """16 x a power of two that holds dk rows, over 16: the recurrence kernels' padding of the key size."""
    rpt = 1
    while 16 * rpt < dk:
        rpt *= 2
    return rpt


def decay_scan_state_floats(heads: int, dk: int, dv: int) -> int:
    """Floats of a request's state row that `decay_scan` keeps for `heads` matrices [dk, dv]: the kernel's own
    layout, rows padded to 16 x a power of two and columns to whole tiles (csrc/recurrent_scan.hip)."""
    if not (heads > 0 and 0 < dk <= SCAN_MAX_DIM and dv > 0):
        raise KernelError(f"decay_scan takes key sizes up to {SCAN_MAX_DIM}; got heads {heads}, dk {dk}, dv {dv}")
    rpt = _pow2_rows(dk)
    cpt = 4 if dv >= 64 else (2 if dv >= 32 else 1)
    tiles = -(-dv // (16 * cpt))
    return heads * tiles * rpt * 256 * cpt


def _rows(t: torch.Tensor, T: int, width: int, name: str) -> None:
    _check(t.is_cuda and t.dim() == 2 and t.shape[0] == T and t.stride(1) == 1 and t.shape[1] >= width,
           f"{name} must be rows [T, >= {width}] on the GPU")


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
               state_offset: int, ctx, out: torch.Tensor, heads: int, qk_heads: int, dk: int, dv: int,
               q_scale: float = 1.0, piece_ok: bool = True) -> torch.Tensor:
    """Per segment of the step and head h, from the request's state S (fp32, zeros for a new request), token by token:
    S = diag(a) S + k v^T, out = S^T (q_scale q).  q, k: rows [T, >= qk_heads dk] (views with a row stride are fine;
    head h reads q/k head h // (heads / qk_heads)); v rows [T, >= heads dv]; all three of one dtype.  decay: ln a, fp32
    [T, heads, dk] (one per key channel) or [T, heads] (one per head).  A step whose longest segment has
    `SCAN_BLOCK_MIN_TOKENS` tokens or more takes sixteen tokens a pass on the matrix cores (keys up to 128 wide),
    any other goes token by token; long segments of a step that would leave most of the chip idle are cut into pieces
    that run side by side (`piece_ok` False: never).  state fp32 [slots, row]: the matrices live at
    `state_offset` of a request's row (ctx.state_slots, -1: none) in the kernel's own layout
    (`decay_scan_state_floats` floats).  out fp32 [T, heads dv]."""
    T, B = ctx.num_tokens, ctx.num_segments
    _dev(decay, out, ctx.cu_q, ctx.state_slots)
    _check(heads % qk_heads == 0 and 0 < dk <= SCAN_MAX_DIM and dv > 0, "decay_scan: heads must be a multiple of qk_heads, dk <= 256")
    _rows(q, T, qk_heads * dk, "q")
    _rows(k, T, qk_heads * dk, "k")
    _rows(v, T, heads * dv, "v")
    _check(q.dtype == k.dtype == v.dtype and q.device == k.device == v.device == out.device, "q, k and v must share dtype and device")
    per_channel = decay.dim() == 3
    _check(decay.dtype == torch.float32 and tuple(decay.shape) in ((T, heads, dk), (T, heads)),
           "decay must be fp32 [T, H, dk] or [T, H]")
    _check(out.dtype == torch.float32 and out.shape == (T, heads * dv), "out must be fp32 [T, H dv]")
    need = decay_scan_state_floats(heads, dk, dv)
    _check(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
           and 0 <= state_offset and state_offset + need <= state.shape[1],
           f"state rows must be fp32 with {need} floats from offset {state_offset}")
    _i32(ctx.cu_q, B + 1, "cu_q")
    _i32(ctx.state_slots, B, "state_slots")
    lib = load_library("recurrent_scan")
    LL = ctypes.c_longlong
    max_q = int(getattr(ctx, "max_q_len", 0) or T)
    # a step of few long segments has too few (segment, head, 64 columns) for the chip: its segments are cut into
    # pieces that run side by side (each piece's own contribution to the state first, a chain through them, then the
    # pieces again from their true states), through a scratch row per piece
    piece, scratch = 0, None
    q_lens = list(getattr(ctx, "q_lens", None) or [max_q] * B)       # (bounds, where the step is replayed from a graph)
    busy = sum(1 for n in q_lens if 2 * n >= max_q) * heads * -(-dv // 64)     # what the longest segments have to run on
    if max_q >= 2 * SCAN_PIECE_MIN and busy < SCAN_PIECE_BUSY and dk <= 128 and piece_ok:
        want = -(-SCAN_PIECE_GROUPS // busy)
        piece = max(SCAN_PIECE_MIN, -(-(-(-max_q // want)) // 16) * 16)
        cut = sum(1 for n in q_lens if n > piece)
        rows = cut * -(-max_q // piece)
        row = need + heads * 16 * _pow2_rows(dk)
        if max_q > piece and cut > 0 and rows * row * 4 <= SCAN_PIECE_SCRATCH_BYTES:
            scratch = torch.zeros((rows, row), dtype=torch.float32, device=out.device)
        else:
            piece = 0
    _ret(lib.sa_decay_scan(_ptr(q), _ptr(k), _ptr(v), c_int(_code(q)), LL(q.stride(0)), LL(k.stride(0)), LL(v.stride(0)),
                           _ptr(decay), c_int(1 if per_channel else 0), c_float(q_scale),
                           c_void_p(state.data_ptr() + 4 * state_offset), LL(state.stride(0)), _ptr(ctx.cu_q),
                           _ptr(ctx.state_slots), _ptr(out), c_int(B), c_int(heads), c_int(qk_heads), c_int(dk), c_int(dv),
                           c_int(max_q), c_int(piece), _ptr(scratch), LL(scratch.stride(0) if scratch is not None else 0),
                           _stream()), "decay_scan")
    return out


def gla_decay(z: torch.Tensor, bias: Optional[torch.Tensor], tau: float, out: torch.Tensor) -> torch.Tensor:
    """out = ln(sigmoid(z + bias)^(1 / tau)) = ln sigmoid(z + bias) / tau, the decay's logarithm that `decay_scan` takes:
    z, out fp32 [T, C], bias fp32 [C]."""
    _dev(z, bias, out)
    _check(z.dtype == torch.float32 and z.dim() == 2 and out.shape == z.shape and out.dtype == torch.float32,
           "decay logits and decays must be fp32 [T, C]")
    if bias is not None:
        _f32vec(bias, z.shape[1], "the decay's bias")
    _check(tau > 0, "tau must be positive")
    lib = load_library("recurrent_scan")
    _ret(lib.sa_gla_decay(_ptr(z), _ptr(bias), c_float(tau), _ptr(out), c_int(z.shape[0]), c_int(z.shape[1]), _stream()),
         "gla_decay")
    return out


def ssm_prepare(zx: torch.Tensor, col: int, conv_w: torch.Tensor, conv_b: Optional[torch.Tensor], state: torch.Tensor,
                conv_offset: int, dt_raw: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, ctx,
                xbc: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, heads: int, head_dim: int, taps: int) -> None:
    """The state-space mixer's inputs.  zx rows [T, >= col + C]: columns col .. col + C - 1 are the convolution's
    channels [x: H P | B | C]; conv_w fp32 [C, taps] (last column on the current token), conv_b fp32 [C] or None;
    inputs before a segment come from its request's state row at `conv_offset` ([taps - 1, C] fp32, oldest first).
    xbc fp32 [T, C] = silu(conv); dt = softplus(dt_raw + dt_bias) (dt_raw fp32 [T, H]); decay fp32 [T, H] =
    -exp(A_log) dt, the decay's logarithm; v fp32 [T, H P] = dt x."""
    T, B = ctx.num_tokens, ctx.num_segments
    _dev(conv_w, conv_b, dt_raw, A_log, dt_bias, xbc, v, decay, ctx.seg_of_token, ctx.cu_q, ctx.state_slots)
    H, P = heads, head_dim
    _check(xbc.dtype == torch.float32 and xbc.dim() == 2 and xbc.shape[0] == T, "xbc must be fp32 [T, C]")
    C = xbc.shape[1]
    _check(C >= H * P and 1 <= taps <= SCAN_MAX_TAPS, f"channels must cover H P = {H * P}; up to {SCAN_MAX_TAPS} taps")
    _rows(zx, T, col + C, "zx")
    _check(conv_w.dtype == torch.float32 and conv_w.shape == (C, taps), f"conv_w must be fp32 [{C}, {taps}]")
    if conv_b is not None:
        _f32vec(conv_b, C, "conv bias")
    _check(dt_raw.dtype == torch.float32 and dt_raw.shape == (T, H), "dt_raw must be fp32 [T, H]")
    _f32vec(A_log, H, "A_log")
    _f32vec(dt_bias, H, "dt_bias")
    _check(v.dtype == torch.float32 and v.shape == (T, H * P) and decay.dtype == torch.float32 and decay.shape == (T, H),
           "v must be fp32 [T, H P] and decay fp32 [T, H]")
    _check(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
           and 0 <= conv_offset and conv_offset + (taps - 1) * C <= state.shape[1], "state rows are too short for the convolution")
    _i32(ctx.seg_of_token, T, "seg_of_token")
    _i32(ctx.cu_q, B + 1, "cu_q")
    _i32(ctx.state_slots, B, "state_slots")
    lib = load_library("recurrent_scan")
    LL = ctypes.c_longlong
    _ret(lib.sa_ssm_prepare(_ptr(zx), c_int(_code(zx)), LL(zx.stride(0)), c_int(col), _ptr(conv_w), _ptr(conv_b),
                            _ptr(state), LL(state.stride(0)), LL(conv_offset), _ptr(dt_raw), _ptr(A_log), _ptr(dt_bias),
                            _ptr(ctx.seg_of_token), _ptr(ctx.cu_q), _ptr(ctx.state_slots), _ptr(xbc), _ptr(v), _ptr(decay),
                            c_int(T), c_int(H), c_int(P), c_int(C), c_int(taps), _stream()), "ssm_prepare")


def conv_state_update(zx: torch.Tensor, col: int, channels: int, state: torch.Tensor, conv_offset: int, ctx,
                      taps: int) -> None:
    """After a step: the last taps - 1 inputs of every channel (columns col .. col + channels - 1 of zx rows) into the
    requests' state rows at `conv_offset`, oldest first; a segment shorter than taps - 1 keeps the newest of its old ones."""
    T, B = ctx.num_tokens, ctx.num_segments
    _dev(ctx.cu_q, ctx.state_slots)
    _rows(zx, T, col + channels, "zx")
    _check(1 <= taps <= SCAN_MAX_TAPS, f"up to {SCAN_MAX_TAPS} taps")
    _check(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
           and 0 <= conv_offset and conv_offset + (taps - 1) * channels <= state.shape[1], "state rows are too short for the convolution")
    _i32(ctx.cu_q, B + 1, "cu_q")
    _i32(ctx.state_slots, B, "state_slots")
    lib = load_library("recurrent_scan")
    LL = ctypes.c_longlong
    _ret(lib.sa_conv_state_update(_ptr(zx), c_int(_code(zx)), LL(zx.stride(0)), c_int(col), _ptr(state), LL(state.stride(0)),
                                  LL(conv_offset), _ptr(ctx.cu_q), _ptr(ctx.state_slots), c_int(B), c_int(channels),
                                  c_int(taps), _stream()), "conv_state_update")


def gated_group_norm(o: torch.Tensor, gate_rows: torch.Tensor, gate_col: int, weight: torch.Tensor, group: int,
                     gate_first: bool, eps: float, out: torch.Tensor, skip_x: Optional[torch.Tensor] = None,
                     skip_d: Optional[torch.Tensor] = None, head_dim: int = 1) -> torch.Tensor:
    """What follows a recurrence's read-out o fp32 [T, n]: u = o + skip_d[i // head_dim] skip_x[t, i] (skip_x fp32 rows
    [T, >= n], or None); with g = silu(gate_rows[t, gate_col + i]): `gate_first`: out = N(u g) w, else out = N(u) w g,
    where N divides every run of `group` values by its root mean square (eps inside the root) and w = weight[i % len]."""
    _dev(o, weight, out, skip_d)
    _check(o.dtype == torch.float32 and o.dim() == 2, "o must be fp32 [T, n]")
    T, n = o.shape
    _check(group > 0 and n % group == 0, f"groups of {group} do not divide {n}")
    _check(out.shape == (T, n) and out.dtype == gate_rows.dtype, "out must be [T, n] in the gate's dtype")
    _rows(gate_rows, T, gate_col + n, "gate rows")
    _check(weight.dtype == torch.float32 and weight.dim() == 1 and weight.numel() > 0, "the norm's weight must be an fp32 vector")
    skip_stride = 0
    if skip_x is not None:
        _rows(skip_x, T, n, "skip_x")
        _check(skip_x.dtype == torch.float32 and skip_d is not None and head_dim > 0 and n % head_dim == 0, "skip_x must be fp32 rows with skip_d")
        _f32vec(skip_d, n // head_dim, "skip_d")
        skip_stride = skip_x.stride(0)
    lib = load_library("recurrent_scan")
    LL = ctypes.c_longlong
    _ret(lib.sa_gated_group_norm(_ptr(o), _ptr(skip_x), LL(skip_stride), _ptr(skip_d), c_int(head_dim), _ptr(gate_rows),
                                 c_int(_code(gate_rows)), LL(gate_rows.stride(0)), c_int(gate_col), _ptr(weight),
                                 c_int(weight.numel()), c_int(group), c_int(1 if gate_first else 0), c_float(eps), _ptr(out),
                                 c_int(T), c_int(n), _stream()), "gated_group_norm")
    return out


# ---------------------------------------------------------------------------------------------
# routed experts
# ---------------------------------------------------------------------------------------------

ROUTER_MODES = {"chosen": 0, "all": 1, "sigmoid": 2}


def _router_mode(over_all) -> int:
    """The kernels' number for a way of weighting the chosen experts: a name of ROUTER_MODES, or the older flag
    (True = "all", False = "chosen")."""
    if isinstance(over_all, str):
        _check(over_all in ROUTER_MODES, f"unknown router mode {over_all!r}; known: {sorted(ROUTER_MODES)}")
        return ROUTER_MODES[over_all]
    return 1 if over_all else 0


def moe_route(logits: torch.Tensor, experts: int, top: int, ids: torch.Tensor, weights: torch.Tensor,
              over_all=False, scale: float = 1.0) -> None:
    """Per row of logits fp32 [T, >= experts]: the `top` experts with the largest logits (ids int32
    [T, top]) and their weights fp32 [T, top]: the softmax over those logits alone ("chosen"), or (`over_all` True
    or "all") their shares of the softmax over all experts divided by the sum of the chosen shares + 1e-20, or
    ("sigmoid") the sigmoid of each chosen logit, not normalised; times `scale`."""
    _dev(logits, ids, weights)
    T = logits.shape[0]
    _check(logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[1] >= experts, "router logits must be fp32 [T, >= E]")
    _check(0 < top <= experts, "top must be within the number of experts")
    _check(ids.dtype == torch.int32 and ids.shape == (T, top) and weights.dtype == torch.float32 and weights.shape == (T, top),
           "ids int32 [T, top], weights fp32 [T, top]")
    lib = load_library("moe")
    _ret(lib.sa_moe_route(_ptr(logits), c_int(logits.shape[1]), _ptr(ids), _ptr(weights), c_int(T), c_int(experts),
                          c_int(top), c_int(_router_mode(over_all)), c_float(scale), _stream()), "moe_route")


MOE_ROUTE_INSIDE = 16      # up to this many tokens the experts' call does the routing itself (one kernel less)
MOE_WIDE_MIN_ROWS = 1024   # more (token, k) rows than this take the products with both operands through LDS


def moe_wide_available(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> bool:
    """bf16, widths that are whole stages of 64, and the gates' and ups' matrices one behind the other in memory
    (`w_up` is the second half of the tensor whose first half is `w_gate`: [2, E, F, d])."""
    E, F, d = w_gate.shape
    return (h.dtype == torch.bfloat16 and d % 64 == 0 and F % 64 == 0 and _aligned16(h, w_gate, w_down)
            and w_up.data_ptr() == w_gate.data_ptr() + w_gate.numel() * w_gate.element_size())


def moe_experts(h: torch.Tensor, ids: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                yk: torch.Tensor, logits: Optional[torch.Tensor] = None,
                weights: Optional[torch.Tensor] = None, over_all=False, scale: float = 1.0,
                gate: str = "silu", limit: float = 0.0, weight_inputs: bool = False) -> torch.Tensor:
    """yk[t * top + k] = expert ids[t, k] applied to h[t]: down(gate(gate h, up h)), fp32 [T top, d], with
    one of GATES (silu(g) u unless said otherwise).
    w_gate, w_up [E, F, d], w_down [E, d, F] in h's dtype.  With `logits` (fp32 [T, >= E], at most
    MOE_ROUTE_INSIDE tokens) `ids` and `weights` are made here as `moe_route` makes them (`over_all`, `scale`).
    `weight_inputs`: expert ids[t, k] is applied to weights[t, k] * h[t] (the weight enters where the gate is applied,
    gate and up being linear), for designs whose weights multiply the experts' inputs and not their outputs."""
    _dev(h, ids, w_gate, w_up, w_down, yk, logits, weights)
    T, d = h.shape
    top = ids.shape[1]
    E, F, d2 = w_gate.shape
    _check(d2 == d and w_up.shape == (E, F, d) and w_down.shape == (E, d, F), "expert matrices must be [E, F, d], [E, F, d], [E, d, F]")
    _check(w_gate.dtype == h.dtype and w_up.dtype == h.dtype and w_down.dtype == h.dtype, "experts and activations must share a dtype")
    _check(ids.dtype == torch.int32 and ids.shape == (T, top), "ids must be int32 [T, top]")
    _check(yk.dtype == torch.float32 and yk.shape == (T * top, d), "yk must be fp32 [T top, d]")
    _check(gate in GATES and (gate != "clamped_swish" or limit > 0.0), f"gate must be one of {sorted(GATES)}, "
           "the clamped one with a positive limit")
    lib = load_library("moe")
    n = T * top
    tiles = int(lib.sa_moe_max_tiles(c_int(n), c_int(E)))
    ints = torch.empty(2 * E + 1 + n + 2 * tiles + 1, dtype=torch.int32, device=h.device)
    act = torch.empty((n, F), dtype=h.dtype, device=h.device)
    if weight_inputs:
        _check(weights is not None and weights.dtype == torch.float32 and weights.shape == (T, top)
               and weights.is_contiguous(), "weights on the experts' inputs must be contiguous fp32 [T, top]")
    if n > MOE_WIDE_MIN_ROWS and logits is None and moe_wide_available(h, w_gate, w_up, w_down):
        # prompt portions: the grouping here, the two products over tiles of 128 rows with both operands through LDS
        wide = load_library("gemm_mfma")
        rows = int(wide.sa_moe_wide_tile_rows())
        _ret(lib.sa_moe_group(_ptr(ids), _ptr(ints), c_int(T), c_int(top), c_int(E), c_int(rows), c_void_p(0), c_int(0),
                              c_void_p(0), c_int(0), c_float(1.0), _stream()), "moe_group")
        base, o = ints.data_ptr(), 4
        offsets, perm = base, base + o * (2 * E + 1)
        tile_expert = perm + o * n
        tile_row0, num_tiles = tile_expert + o * tiles, tile_expert + o * 2 * tiles
        _ret(wide.sa_moe_wide(_ptr(h), _ptr(w_gate), _ptr(w_down), _ptr(act), _ptr(yk), c_int(E), c_int(d), c_int(F),
                              c_int(-(-n // rows) + E), c_void_p(offsets), c_void_p(perm), c_void_p(tile_expert),
                              c_void_p(tile_row0), c_void_p(num_tiles), c_int(top), c_int(GATES[gate]), c_float(limit),
                              _ptr(weights if weight_inputs else None), _stream()), "moe_wide")
        return yk
    ldz = 0
    if logits is not None:
        _check(T <= MOE_ROUTE_INSIDE and logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[0] == T
               and logits.shape[1] >= E and 0 < top <= E, "moe_experts: logits fp32 [T, >= E] of at most "
               f"{MOE_ROUTE_INSIDE} tokens")
        _check(weights is not None and weights.dtype == torch.float32 and weights.shape == (T, top), "weights fp32 [T, top]")
        ldz = logits.shape[1]
    _ret(lib.sa_moe_experts(_ptr(h), c_int(_code(h)), _ptr(ids), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(ints),
                            _ptr(act), _ptr(yk), c_int(T), c_int(top), c_int(E), c_int(d), c_int(F), _ptr(logits),
                            c_int(ldz), _ptr(weights), c_int(_router_mode(over_all)), c_float(scale), c_int(GATES[gate]),
                            c_float(limit), _ptr(weights if weight_inputs else None), _stream()), "moe_experts")
    return yk


def moe_combine(yk: torch.Tensor, weights: Optional[torch.Tensor], shared: Optional[torch.Tensor],
                logits: Optional[torch.Tensor], gate_col: int, y: torch.Tensor) -> torch.Tensor:
    """y[t] = sum_k weights[t, k] yk[t top + k] (+ sigmoid(logits[t, gate_col]) * shared[t]);
    shared [T, d] or fp32 [parts, T, d]; logits None: the shared rows are added as they are; weights None: the
    experts' rows are added as they are."""
    _dev(yk, weights, shared, logits, y)
    T, d = y.shape
    _check(T > 0 and yk.dim() == 2 and yk.shape[0] % T == 0, "moe_combine: yk must be [T top, d]")
    top = yk.shape[0] // T
    _check(y.dtype == torch.float32 and yk.shape == (T * top, d) and yk.dtype == torch.float32
           and (weights is None or (weights.dtype == torch.float32 and weights.shape == (T, top))),
           "moe_combine: fp32 y [T, d], yk [T top, d], weights [T, top]")
    parts, scode = 1, F32
    if shared is not None:
        if shared.dim() == 3:
            parts = shared.shape[0]
            _check(shared.dtype == torch.float32 and shared.shape[1:] == (T, d), "shared partial sums must be fp32 [parts, T, d]")
        else:
            _check(shared.shape == (T, d), "shared rows must be [T, d]")
        scode = _code(shared)
    gate, ldz = c_void_p(0), 0
    if logits is not None:
        _check(logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[0] == T
               and 0 <= gate_col < logits.shape[1], "gate logits must be a column of fp32 [T, n]")
        gate, ldz = c_void_p(logits.data_ptr() + 4 * gate_col), logits.shape[1]
    lib = load_library("moe")
    _ret(lib.sa_moe_combine(_ptr(yk), _ptr(weights), _ptr(shared), c_int(scode), c_int(parts), gate,
                            c_int(ldz), _ptr(y), c_int(T), c_int(top), c_int(d), _stream()), "moe_combine")
    return y


_SINKS = {}


def read_bytes(t: torch.Tensor, workgroups: int = 0) -> None:
    """Read the whole tensor with plain 16-byte loads and keep nothing (a measurement of the
    memory's read rate with a kernel of our own)."""
    _dev(t)
    nbytes = t.numel() * t.element_size()
    _check(nbytes % 16 == 0 and t.data_ptr() % 16 == 0, "read_bytes needs 16-byte alignment and size")
    sink = _SINKS.get(t.device)
    if sink is None:
        sink = _SINKS[t.device] = torch.zeros(4, dtype=torch.int32, device=t.device)
    lib = load_library("membench")
    lib.sa_read_bytes.argtypes = [c_void_p, ctypes.c_size_t, c_int, c_void_p, c_void_p]
    _ret(lib.sa_read_bytes(_ptr(t), nbytes, workgroups or 16 * compute_units(), _ptr(sink), _stream()), "read_bytes")


def copy_bytes(dst: torch.Tensor, src: torch.Tensor, workgroups: int = 0) -> None:
    """dst = src with plain 16-byte loads and stores (a measurement of the memory's copy rate)."""
    _dev(dst, src)
    nbytes = src.numel() * src.element_size()
    _check(dst.numel() * dst.element_size() == nbytes and nbytes % 16 == 0 and dst.data_ptr() % 16 == 0
           and src.data_ptr() % 16 == 0, "copy_bytes needs two buffers of one size, 16-byte aligned")
    lib = load_library("membench")
    lib.sa_copy_bytes.argtypes = [c_void_p, c_void_p, ctypes.c_size_t, c_int, c_void_p]
    _ret(lib.sa_copy_bytes(_ptr(dst), _ptr(src), nbytes, workgroups or 16 * compute_units(), _stream()), "copy_bytes")


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor], keys: Optional[torch.Tensor],
           out: torch.Tensor) -> torch.Tensor:
    """One token per row of fp32 logits: argmax where temperature is 0 (or None), else the
    draw argmax(logits / T - log q), q ~ Exp(1) from the row's 64-bit key."""
    _dev(logits, temperature, keys, out)
    _check(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be fp32 [R, V]")
    R, V = logits.shape
    _i32(out, R, "sample output")
    if temperature is not None:
        _check(temperature.dtype == torch.float32 and temperature.numel() == R, "temperature must be fp32 [R]")
        _check(keys is not None and keys.dtype == torch.int64 and keys.numel() == R, "keys must be int64 [R]")
    lib = load_library("sampling")
    _check(R <= 65535, "at most 65535 rows are sampled in one call")
    nchunks = lib.sa_sample_chunks(c_int(V))
    part_v = torch.empty((R, nchunks), dtype=torch.float32, device=logits.device)
    part_i = torch.empty((R, nchunks), dtype=torch.int32, device=logits.device)
    _ret(lib.sa_sample(_ptr(logits), _ptr(temperature), _ptr(keys), _ptr(out), _ptr(part_v), _ptr(part_i),
                       c_int(R), c_int(V), _stream()), "sample")
    return out


# ---------------------------------------------------------------------------------------------
# bf16 matrix-core kernels
# ---------------------------------------------------------------------------------------------
# a product with more than 64 rows and this many outputs (the head over the vocabulary) is the
# library's: the few-row kernel would read its 128 rows of activations once per 64 weight rows
WIDE_OUTPUT = 65536
SKINNY_MAX_ROWS = 128         # above this the weights would be streamed more than once per product
WIDE_MAX_ROWS = 256           # ... but for the kernel with both operands in LDS, where it is ahead of the library


def _aligned16(*tensors: torch.Tensor) -> bool:
    return all(t.data_ptr() % 16 == 0 for t in tensors)


def mfma_gemm_available(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether the bf16 matrix-core products take these operands: bf16 in, bf16 or fp32 out,
    inner size a multiple of 8 (16-byte rows)."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and out.dtype in (torch.bfloat16, torch.float32) and a.shape[1] % 8 == 0 and _aligned16(a, w, out))


def gemm_bf16_skinny(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = a @ w^T on the matrix cores, weights streamed once per 128 rows of a.

    `out` [M, N] bf16 or fp32; or fp32 [parts, M, N]: the inner dimension is cut into `parts`
    slices over workgroups and slice p's partial sums go to out[p] (the consumer adds them)."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    parts = 1
    if out.dim() == 3:
        parts = out.shape[0]
        _check(out.dtype == torch.float32 and out.shape[1:] == (M, N), "partial sums must be fp32 [parts, M, N]")
    else:
        _check(out.shape == (M, N), "gemm_bf16_skinny: shapes do not match")
    _check(w.shape == (N, K), "gemm_bf16_skinny: shapes do not match")
    _check(mfma_gemm_available(a, w, out), "gemm_bf16_skinny needs bf16 operands, K % 8 == 0 and 16-byte alignment")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), c_int(_code(out)), c_int(M), c_int(N), c_int(K),
                                 c_int(parts), _stream()), "gemm_bf16_skinny")
    return out


@functools.lru_cache(maxsize=4096)
def gemm_takes_wide(M: int, N: int, K: int, parts: int = 1, swiglu: bool = False) -> bool:
    """Whether the few-row product of these sizes runs as the kernel that keeps both operands in LDS
    (for SwiGLU, N is the number of gate rows)."""
    lib = load_library("gemm_mfma")
    return bool(lib.sa_gemm_bf16_takes_wide(c_int(1 if swiglu else 0), c_int(M), c_int(N), c_int(K), c_int(parts)))


@functools.lru_cache(maxsize=4096)
def split_k_parts(M: int, N: int, K: int) -> int:
    """Into how many slices the inner dimension of a few-row product is cut across workgroups so
    that a matrix with few rows still fills the chip: 1 means no cut.  Where the kernel with both
    operands in LDS takes the product (64 weight rows a workgroup): as many as one round of workgroups
    over the chip allows, slices of at least twelve stages of 64 columns.  Else, for one or two rows, a
    workgroup takes 16 weight rows (about four workgroups per compute unit wanted, slices of at least
    256); from three rows on it takes 32 (one workgroup per compute unit wanted, slices of at least 512)."""
    if N >= 8192:
        return 1
    cus = compute_units()
    if M <= WIDE_MAX_ROWS and K % 64 == 0:
        groups = -(-N // 64)
        parts = 1
        while parts < 8 and groups * parts * 2 <= cus and K // (64 * parts * 2) >= 12 and (K // 64) % (parts * 2) == 0:
            parts *= 2
        if gemm_takes_wide(M, N, K, parts):
            return parts
    parts = 1
    if M > 2:
        groups = -(-N // 32)
        while parts < 8 and groups * parts < cus and K // (parts * 2) >= 512:
            parts *= 2
        return parts
    tiles = -(-N // 16)
    while parts < 4 and tiles * parts < 4 * cus and K // (parts * 2) >= 512:
        parts *= 2
    return parts


BLASLT_WORKSPACE_BYTES = 64 << 20
_BLASLT_WORKSPACE = {}


def blaslt_workspace(device) -> torch.Tensor:
    """The scratch memory of the BLAS library's products, one buffer per device (the products run
    in one stream).  Made at the first call: the parts ask for it when they load, so that it
    does not come out of the memory pool of a graph capture."""
    dev = torch.device(device)
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _BLASLT_WORKSPACE.get(key)
    if ws is None:
        ws = _BLASLT_WORKSPACE[key] = torch.empty(BLASLT_WORKSPACE_BYTES, dtype=torch.uint8, device=dev)
    return ws


def gemm_bf16_library(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = a @ w^T by the BLAS library (hipBLASLt, called directly: the descriptors and the
    algorithm of a shape are kept after its first call, so a call costs the host a few
    microseconds).  bf16 operands, bf16 or fp32 output."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _check(w.shape == (N, K) and out.shape == (M, N), "gemm_bf16_library: shapes do not match")
    _check(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32)
           and _aligned16(a, w, out), "gemm_bf16_library needs bf16 operands, a bf16 or fp32 result and 16-byte alignment")
    ws = blaslt_workspace(a.device)
    lib = load_library("blaslt")
    _ret(lib.sa_blaslt_mm(_ptr(a), _ptr(w), _ptr(out), c_int(_code(out)), c_int(M), c_int(N), c_int(K), _ptr(ws),
                          ctypes.c_size_t(ws.numel()), _stream()), "gemm_bf16_library")
    return out


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """bf16 product: the weight-streaming kernels for few rows, the BLAS library for many (the
    reference leaves all of its products to the library, serve/model.py:80-82,95,97,159); both
    write bf16 or fp32."""
    M = a.shape[0]
    if M <= SKINNY_MAX_ROWS and not (M > 64 and w.shape[0] >= WIDE_OUTPUT):
        return gemm_bf16_skinny(a, w, out)
    if M <= WIDE_MAX_ROWS and gemm_takes_wide(M, w.shape[0], a.shape[1], 1):
        return gemm_bf16_skinny(a, w, out)
    return gemm_bf16_library(a, w, out)


def swiglu_bf16(a: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, gate: str = "silu",
                limit: float = 0.0) -> torch.Tensor:
    """out[M, I] = silu(a @ Wg^T) * (a @ Wu^T) for w_gate_up = [Wg; Wu] ([2 I, K]), one kernel; or with another
    of GATES in place of silu(g) u."""
    _dev(a, w_gate_up, out)
    _check(gate in GATES and (gate != "clamped_swish" or limit > 0.0), f"gate must be one of {sorted(GATES)}, "
           "the clamped one with a positive limit")
    M, K = a.shape
    I = w_gate_up.shape[0] // 2
    _check(w_gate_up.shape == (2 * I, K) and out.shape == (M, I), "swiglu_bf16: shapes do not match")
    _check(a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
           and K % 8 == 0 and _aligned16(a, w_gate_up, out), "swiglu_bf16 needs bf16 operands and K % 8 == 0")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_skinny_swiglu(_ptr(a), _ptr(w_gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                        c_int(GATES[gate]), c_float(limit), _stream()), "swiglu_bf16")
    return out


def qkv_rope_available(a: torch.Tensor, w_qkv: torch.Tensor, k_pages: torch.Tensor, head_dim: int,
                       rot_dim: int, adjacent_pairs: bool) -> bool:
    """Whether projection, rotation and cache write can run as one kernel: bf16, few rows, all
    dims of a head rotated in (j, j + D/2) pairs, head size a multiple of 16."""
    return (a.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16
            and a.shape[0] <= SKINNY_MAX_ROWS and a.shape[1] % 8 == 0 and head_dim % 16 == 0
            and rot_dim == head_dim and not adjacent_pairs and _aligned16(a, w_qkv))


def qkv_rope_bf16(a: torch.Tensor, w_qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                  inv_freq: torch.Tensor, slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                  bias: Optional[torch.Tensor] = None, magnitude: float = 1.0) -> torch.Tensor:
    """q, k, v = a @ w_qkv^T (w_qkv = [Wq; Wk; Wv]) (+ bias, fp32 over the (Hq + 2 Hk) D outputs, added to the fp32
    sums); q and k rotated by position (sine and cosine times `magnitude`); q to q_out [M, Hq D], rotated k and v
    into the cache pages at each token's slot.  One kernel."""
    _dev(a, w_qkv, q_out, positions, inv_freq, slots, k_pages, v_pages, bias)
    if bias is not None:
        _f32vec(bias, (num_heads + 2 * num_kv_heads) * head_dim, "bias")
    M, K = a.shape
    Hq, Hk, D = num_heads, num_kv_heads, head_dim
    _check(qkv_rope_available(a, w_qkv, k_pages, D, D, False), "qkv_rope_bf16 does not take these operands")
    _check(w_qkv.shape == ((Hq + 2 * Hk) * D, K), f"w_qkv must be [{(Hq + 2 * Hk) * D}, {K}]")
    _check(q_out.shape == (M, Hq * D) and q_out.dtype == torch.bfloat16, "q_out must be bf16 [M, Hq D]")
    _i32(positions, M, "positions")
    _i32(slots, M, "slots")
    _check(inv_freq.dtype == torch.float32 and inv_freq.numel() == D // 2, f"inv_freq must be fp32 [{D // 2}]")
    P = k_pages.shape[0]
    _check(k_pages.shape == (P, Hk, page_size, D) and v_pages.shape == (P, Hk, D, page_size)
           and v_pages.dtype == torch.bfloat16, "cache pages must be bf16 [P, Hk, page, D] and [P, Hk, D, page]")
    lib = load_library("gemm_mfma")
    _ret(lib.sa_gemm_bf16_qkv_rope(_ptr(a), _ptr(w_qkv), _ptr(q_out), _ptr(positions), _ptr(inv_freq), _ptr(slots),
                                   _ptr(k_pages), _ptr(v_pages), c_int(M), c_int(K), c_int(Hq), c_int(Hk),
                                   c_int(D), c_int(page_size), _ptr(bias), c_float(magnitude), _stream()),
         "qkv_rope_bf16")
    return q_out


MFMA_ATTENTION_HEAD_DIMS = tuple(range(16, 129, 16))


def mfma_attention_available(q: torch.Tensor, k_pages: torch.Tensor, q_row_stride: int,
                             scale: float = 1.0) -> bool:
    """bf16, head sizes 16..128 in steps of 16, page sizes that are multiples of 4, and a positive
    score scale (the kernels take row maxima of the raw scores and scale afterwards)."""
    P, Hk, page_size, D = k_pages.shape
    return (q.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and D in MFMA_ATTENTION_HEAD_DIMS
            and page_size % 4 == 0 and q_row_stride % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0.0)


def attention_splits(max_q_len: int, num_segments: int, num_kv_heads: int, max_ctx_len: int,
                     group_size: int = 1) -> int:
    """Into how many parts the key range of a launch is cut so that the chip is filled.
    Single decoded tokens: about two waves per compute unit in all (more cost more in the merge than they gain), and
    no part shorter than 64 keys.  Prompt portions that are at most a quarter of their context (a
    long prompt taken in portions): about one workgroup of 128 rows per compute unit, parts of at
    least 1024 keys; portions that are most of their context are never cut, the causal mask makes
    their parts too unequal."""
    if max_q_len > 1:
        if max_ctx_len < 4 * max_q_len:
            return 1
        groups = -(-max_q_len * group_size // 128)
        workgroups = groups * num_kv_heads * num_segments
        splits = 1
        while splits < 8 and workgroups * splits < compute_units() and max_ctx_len // (splits * 2) >= 1024:
            splits *= 2
        return splits
    # both inputs are rounded up to powers of two, so that a step run eagerly and the same step
    # replayed from a graph (padded batch, context bucket) cut the keys alike
    ctx = 256
    while ctx < max_ctx_len:
        ctx *= 2
    segs = 1
    while segs < num_segments:
        segs *= 2
    by_length = max(1, ctx // 64)
    by_waves = max(1, 2 * compute_units() // (segs * num_kv_heads))
    return max(1, min(by_length, by_waves, 64))


IN_WORKGROUP_MAX_CTX = 512
IN_WORKGROUP_MAX_SEGMENTS = 32


def attention_in_workgroup(max_q_len: int, num_segments: int, max_ctx_len: int, group_size: int = 1) -> bool:
    """Whether single decoded tokens have their keys cut inside a workgroup (four waves that merge
    through LDS, no merge kernel) instead of across workgroups: for few requests with short
    contexts, where the launch is a chain of latencies and the merge kernel one more link (batch 1
    to 32 at 384 keys: 5.5 to 7.8 us against 5.9 to 8.5 us; at 64 requests or 1,024 keys the cut
    across workgroups, or none, is faster; with 64 requests at 4,096 keys it gained 7 % over shuffled
    pages by itself and lost 2 % in the decode step).  Batch and context are rounded up to powers
    of two first, so that a step run eagerly and the same step replayed from a graph (which rounds
    both) decide alike."""
    if max_q_len * group_size > 16:
        return False
    segs = 1
    while segs < num_segments:
        segs *= 2
    ctx = 256
    while ctx < max_ctx_len:
        ctx *= 2
    return segs <= IN_WORKGROUP_MAX_SEGMENTS and ctx <= IN_WORKGROUP_MAX_CTX


def paged_attention_mfma(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                         v_pages: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                         ctx_len: torch.Tensor, num_tokens: int, max_q_len: int, num_heads: int, scale: float,
                         window: Optional[int], num_splits: int = 1, seg_begin: int = 0,
                         seg_count: Optional[int] = None, in_workgroup: bool = False,
                         sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 attention on the matrix cores (head sizes 16..128 in steps of 16, page sizes that are
    multiples of 4).  `in_workgroup` (segments of at most 16 rows per KV head, num_splits 1): the
    key range is cut four ways over the waves of a workgroup, which merges the parts itself.  `seg_begin`, `seg_count`: run only these segments of the step (their
    tokens' rows of `out` are written, the others left alone); `num_tokens` then is the number of
    tokens up to the end of the last of them."""
    _dev(q, out, k_pages, v_pages, block_table, cu_q, ctx_len)
    _check_sinks(sinks, num_heads)
    P, Hk, page_size, D = k_pages.shape
    _check(mfma_attention_available(q, k_pages, q_row_stride, scale),
           f"paged_attention_mfma takes bf16, head sizes {MFMA_ATTENTION_HEAD_DIMS}, page sizes that are "
           f"multiples of 4 and a positive scale; got head size {D}, page size {page_size}, scale {scale}")
    _check(v_pages.shape == (P, Hk, D, page_size) and v_pages.dtype == torch.bfloat16,
           "v_pages must be bf16 [P, Hk, D, page_size]")
    _check(num_heads % Hk == 0, "query heads must be a multiple of KV heads")
    T = num_tokens
    _check(out.dim() == 2 and out.shape[0] >= T and out.shape[1] == num_heads * D and out.dtype == torch.bfloat16,
           "attention output must be bf16 [T, Hq D]")
    _check(q.numel() >= (T - 1) * q_row_stride + num_heads * D if T else True, "q is too short")
    _check(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 [B, pages]")
    B_all = block_table.shape[0]
    _i32(cu_q, B_all + 1, "cu_q")
    _i32(ctx_len, B_all, "ctx_len")
    B = B_all - seg_begin if seg_count is None else seg_count
    _check(0 <= seg_begin and B >= 0 and seg_begin + B <= B_all, "segment range out of bounds")
    if B == 0:
        return out
    if seg_begin or B != B_all:
        block_table = block_table[seg_begin: seg_begin + B]
        cu_q = cu_q[seg_begin: seg_begin + B + 1]
        ctx_len = ctx_len[seg_begin: seg_begin + B]
    _check(1 <= max_q_len <= max(T, 1) and num_splits >= 1, "max_q_len / num_splits out of range")
    _check(not in_workgroup or (num_splits == 1 and max_q_len * (num_heads // Hk) <= 16),
           "the cut inside a workgroup is for segments of at most 16 rows per KV head and takes no other cut")
    part_o = part_ml = None
    if num_splits > 1:
        # the parts are indexed by token, and the merge runs over tokens 0 .. T-1
        _check(seg_begin == 0, "a split key range needs the segments to start at token 0")
        part_o = torch.empty((T * num_heads * num_splits, D), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * num_splits, 2), dtype=torch.float32, device=q.device)
    lib = load_library("attention_mfma", {"HEAD_DIM": D})
    _check(lib.sa_attention_mfma_head_dim() == D, "the attention library was built for another head size")
    _ret(lib.sa_paged_attention_mfma(
        _ptr(q), c_int(q_row_stride), _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(ctx_len), c_int(B), c_int(T), c_int(max_q_len),
        c_int(num_heads), c_int(Hk), c_int(D), c_int(page_size), c_float(scale), c_int(window or 0),
        c_int(num_splits), _ptr(part_o), _ptr(part_ml), c_int(1 if in_workgroup else 0), _ptr(sinks), _stream()),
        "paged_attention_mfma")
    return out


# ---------------------------------------------------------------------------------------------
# dispatch between kernels of the same operation
# ---------------------------------------------------------------------------------------------

@dataclass
class AttentionStep:
    """What `paged_attention` needs to know of a step: the segments' token offsets and context lengths
    on the device, and the same facts on the host so that choosing kernels and grids needs no
    read-back.  The engine's `StepContext` has these attributes and is passed as it is; a mixer that
    brings its own segment layout (tokens of its own, another notion of a request) fills one of these."""

    num_segments: int
    num_tokens: int
    cu_q: torch.Tensor               # int32 [B + 1]: first token of every segment, and the end
    ctx_len: torch.Tensor            # int32 [B]: keys a segment's last token sees (its context after the step)
    seg_of_token: torch.Tensor       # int32 [T]
    q_lens: Sequence[int]            # the host's copies
    ctx_lens: Sequence[int]
    max_q_len: int
    max_ctx_len: int
    decode_only: bool = False


def _attention_launches(ctx):
    """How a step's segments go to the matrix-core attention kernels.  Single decoded tokens take
    the one-wave kernel and a split key range, prompt portions the kernel that shares keys and
    values across a workgroup: a step that begins with decoding requests and goes on with prompt
    portions (the order the scheduler gives) is run as two launches, one of each kind.  Computed
    once per step and kept on `ctx`."""
    plan = getattr(ctx, "_attention_launches", None)
    if plan is not None:
        return plan
    B, T = ctx.num_segments, ctx.num_tokens
    if ctx.decode_only or not ctx.q_lens:
        plan = [(0, B, T, ctx.max_q_len, ctx.max_ctx_len)]
    else:
        nd = 0
        while nd < B and ctx.q_lens[nd] == 1:
            nd += 1
        if nd < 4 or nd == B:
            plan = [(0, B, T, ctx.max_q_len, ctx.max_ctx_len)]
        else:
            plan = [(0, nd, nd, 1, max(ctx.ctx_lens[:nd])),
                    (nd, B - nd, T, max(ctx.q_lens[nd:]), max(ctx.ctx_lens[nd:]))]
    ctx._attention_launches = plan
    return plan


def paged_attention(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, k_pages: torch.Tensor,
                    v_pages: torch.Tensor, block_table: torch.Tensor, ctx, num_heads: int, scale: float,
                    window: Optional[int], sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention over the paged cache for all tokens of the step described by `ctx` (an `AttentionStep`,
    or anything with its attributes: the engine passes its `StepContext`): the matrix-core kernel for
    bf16 where it takes the sizes, else the general fp32-arithmetic kernel.  The plan of launches is
    kept on `ctx`, so that the layers of a step share it.  `sinks` (fp32 [Hq]): one more term exp(sinks[h])
    in the denominator of head h's softmax, in every kernel."""
    if mfma_attention_available(q, k_pages, q_row_stride, scale):
        Hk = k_pages.shape[1]
        # (first segment, segments, tokens up to their end, longest portion, longest context)
        for s0, n, t_end, max_q, max_ctx in _attention_launches(ctx):
            # (the parts of a split key range are indexed by token, from the step's first)
            inside = max_q == 1 and attention_in_workgroup(max_q, n, max_ctx, num_heads // Hk)
            splits = 1
            if not inside and (max_q == 1 or s0 == 0):
                splits = attention_splits(max_q, n, Hk, max_ctx, num_heads // Hk)
            paged_attention_mfma(q, q_row_stride, out, k_pages, v_pages, block_table, ctx.cu_q, ctx.ctx_len,
                                 t_end, max_q, num_heads, scale, window, splits, s0, n, in_workgroup=inside,
                                 sinks=sinks)
        return out
    Hk = k_pages.shape[1]
    if tiled_attention_available(q, k_pages, q_row_stride):
        G = num_heads // Hk
        launches = _attention_launches(ctx)
        if len(launches) > 1 or ctx.max_q_len == 1 or ctx.max_q_len * G > TILED_MIN_ROWS \
                or ctx.max_ctx_len >= TILED_MIN_CONTEXT:
            # decoding requests and prompt portions as two launches, as on the matrix-core path
            for s0, n, t_end, max_q, max_ctx in launches:
                whole = s0 == 0 and n == ctx.num_segments
                bt = block_table if whole else block_table[s0: s0 + n]
                cu = ctx.cu_q if whole else ctx.cu_q[s0: s0 + n + 1]
                cl = ctx.ctx_len if whole else ctx.ctx_len[s0: s0 + n]
                if max_q == 1 and s0 == 0 and n <= 65535:
                    # one token a segment: a wave per (segment, up to four heads of a KV head, part of the
                    # keys); about FP32_DECODE_WAVES waves, parts of at least 128 keys
                    waves = n * Hk * -(-G // 4)
                    splits = max(1, min(64, FP32_DECODE_WAVES // max(waves, 1), max_ctx // 128))
                    paged_attention_decode_f32(q, q_row_stride, out, k_pages, v_pages, bt, cu, cl, num_heads, scale,
                                               window, splits, sinks=sinks)
                    continue
                splits = 1
                if max_q * G <= TILED_MIN_ROWS and max_ctx >= TILED_MIN_CONTEXT and s0 == 0:
                    # few rows over many keys: about two workgroups per compute unit, parts of at least 256 keys
                    splits = max(1, min(64, 2 * compute_units() // max(n * Hk, 1), max_ctx // 256))
                paged_attention_tiled_f32(q, q_row_stride, out, k_pages, v_pages, bt, cu, cl, t_end, max_q,
                                          num_heads, scale, window, splits, sinks=sinks)
            return out
    return paged_attention_simple(q, q_row_stride, out, k_pages, v_pages, block_table, ctx.cu_q,
                                  ctx.ctx_len, ctx.seg_of_token, ctx.num_tokens, num_heads, scale, window, sinks)
