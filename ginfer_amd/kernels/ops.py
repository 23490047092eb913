"""Python faces of the HIP kernels.

Every function checks on the host what its kernel and launch grid assume (devices, dtypes,
contiguity, matching sizes) and raises a clear error instead of launching with operands that do not
fit; a kernel never sees a shape it was not written for.  Tensors are torch tensors on the GPU;
kernels run on torch's current stream.
"""
import ctypes

import torch

from . import build
from .tuning import TUNING

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float


class KernelError(RuntimeError):
    pass


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else _vp(0)


def _stream():
    """The raw handle of torch's current stream on the current device (the recording stream while a step is
    being recorded)."""
    return _vp(_raw_stream(_current_device()))


_raw_stream = torch._C._cuda_getCurrentRawStream
_current_device = torch.cuda.current_device


def _check(rc, name):
    if rc != 0:
        raise KernelError("kernel %s failed to launch (code %d)" % (name, rc))


def _need(cond, msg, *args):
    """Raises KernelError(msg % args) unless cond holds; the message is put together only then."""
    if not cond:
        raise KernelError(msg % args if args else msg)


def _dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU (got a %s tensor)" % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands lie on different devices")


def _is_bf16(dtype):
    if dtype is torch.bfloat16:
        return 1
    _need(dtype is torch.float32, "compute dtype must be float32 or bfloat16, got %s", dtype)
    return 0


def embedding_gather(table, ids, out=None):
    """table [V, H] (float32 or bfloat16), ids [T] int32 in [0, V) -> float32 [T, H]."""
    _dev(table, ids, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    _need(ids.dtype == torch.int32 and ids.dim() == 1 and ids.is_contiguous(), "ids must be contiguous int32 [T]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (T, H) and out.is_contiguous(), "out must be contiguous float32 [T, H]")
    lib = build.load("embedding")
    _check(lib.ga_embedding_gather(_ptr(out), _ptr(table), _ptr(ids), _i(T), _i(H),
                                   _i(_is_bf16(table.dtype)), _stream()), "embedding_gather")
    return out


def add_rmsnorm(residual, delta, gain, eps, dtype, rows=None, out=None):
    """residual float32 [T, H] (updated in place with + delta unless rows is given); delta [T, H] in
    `dtype`, or float32 [parts, T, H] (partial sums of a K-split product, added in order), or None;
    gain [H] in `dtype` (or float32); rows int32 [R] or None -> normed [R or T, H]."""
    _dev(residual, delta, gain, rows, out)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    T, H = residual.shape
    parts = 0
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == (T, H) and delta.is_contiguous() and delta.shape[0] >= 1,
              "partial sums must be contiguous float32 [parts, %d, %d], got %s %s",
              T, H, delta.dtype, tuple(delta.shape))
        parts = delta.shape[0]
    elif delta is not None:
        _need(delta.dtype == dtype and delta.shape == (T, H) and delta.is_contiguous(),
              "delta must be contiguous %s [%d, %d], got %s %s",
              dtype, T, H, delta.dtype, tuple(delta.shape))
    _need(gain.shape == (H,) and gain.is_contiguous() and gain.dtype in (dtype, torch.float32),
          "gain must be contiguous [%d] in %s or float32",
          H, dtype)
    R = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be contiguous int32 [R]")
        R = rows.shape[0]
    if out is None:
        out = torch.empty((R, H), dtype=dtype, device=residual.device)
    _need(out.dtype == dtype and out.shape == (R, H) and out.is_contiguous(), "out must be contiguous [R, H]")
    lib = build.load("norm")
    _check(lib.ga_add_rmsnorm(_ptr(out), _ptr(residual), _ptr(delta), _i(parts), _i(T), _ptr(gain), _ptr(rows), _i(R), _i(H),
                              _f(eps), _i(_is_bf16(dtype)),
                              _i(1 if (gain.dtype == torch.float32 and dtype != torch.float32) else 0),
                              _stream()), "add_rmsnorm")
    return out


def silu_mul(gate_up, out=None):
    """gate_up [T, 2I] -> [T, I]: silu(gate) * up with gate = [:, :I], up = [:, I:]."""
    _dev(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0,
          "gate_up must be contiguous [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.dtype == gate_up.dtype and out.shape == (T, I) and out.is_contiguous(), "out must be contiguous [T, I]")
    lib = build.load("activation")
    _check(lib.ga_silu_mul(_ptr(out), _ptr(gate_up), _i(T), _i(I), _i(_is_bf16(gate_up.dtype)), _stream()),
           "silu_mul")
    return out


def silu_mul_transposed(gate_up_t, out=None):
    """gate_up_t [2I, T] (the gate-up product lying transposed) -> [T, I]: silu(gate) * up."""
    _dev(gate_up_t, out)
    _need(gate_up_t.dim() == 2 and gate_up_t.is_contiguous() and gate_up_t.dtype == torch.bfloat16
          and gate_up_t.shape[0] % 16 == 0 and gate_up_t.shape[1] % 8 == 0,
          "gate_up_t must be contiguous bfloat16 [2I, T] with I and T multiples of 8")
    I, T = gate_up_t.shape[0] // 2, gate_up_t.shape[1]
    if out is None:
        out = torch.empty((T, I), dtype=torch.bfloat16, device=gate_up_t.device)
    _need(out.dtype == torch.bfloat16 and out.shape == (T, I) and out.is_contiguous(), "out must be contiguous bfloat16 [T, I]")
    lib = build.load("activation")
    _check(lib.ga_silu_mul_transposed(_ptr(out), _ptr(gate_up_t), _i(T), _i(I), _stream()), "silu_mul_transposed")
    return out


def rope_kv_write(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads,
                  head_dim, write_kv=True):
    """Rotates q and k inside qkv [T, (nh + 2 nkv) hd] in place and writes k, v to the paged cache
    (k [pages, nkv, page_size, hd], v [pages, nkv, hd, page_size]) at slot_mapping [T] int64 (-1: skip).  cos, sin: float32
    [positions, rotary_dim / 2]."""
    _dev(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages)
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == width and qkv.is_contiguous(),
          "qkv must be contiguous [T, %d]",
          width)
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be contiguous int32 [T]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2
          and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
    rotary_dim = 2 * cos.shape[1]
    _need(0 < rotary_dim <= head_dim,
          "rotary_dim %d must lie in (0, head_dim %d]",
          rotary_dim, head_dim)
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        page_size = _check_pages(k_pages, v_pages, qkv.dtype, num_kv_heads, head_dim)
    lib = build.load("rope_kv")
    _check(lib.ga_rope_kv_write(_ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                                _ptr(k_pages), _ptr(v_pages), _i(T), _i(num_heads), _i(num_kv_heads),
                                _i(head_dim), _i(rotary_dim), _i(page_size), _i(1 if write_kv else 0),
                                _i(_is_bf16(qkv.dtype)), _stream()), "rope_kv_write")


def rope_kv_from_parts(parts, bias, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads, head_dim,
                       write_kv=True):
    """The epilogue of a q|k|v projection that arrives as float32 partial sums [parts, T, (nh + 2 nkv) hd] of a product
    whose K was split over workgroups: the parts added in order, the bias (bfloat16 [width] or None), q and k rotated on
    the 32-bit sums; returns q [T, nh*hd] in bfloat16 and writes k and v into the paged cache at slot_mapping."""
    _dev(parts, bias, positions, cos, sin, slot_mapping, k_pages, v_pages)
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[2] == width and parts.is_contiguous(),
          "parts must be contiguous float32 [parts, T, %d]",
          width)
    T = parts.shape[1]
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be contiguous int32 [T]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2
          and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
    rotary_dim = 2 * cos.shape[1]
    _need(0 < rotary_dim <= head_dim and (rotary_dim // 2) % 4 == 0 and (head_dim - rotary_dim) % 4 == 0 and head_dim % 4 == 0,
          "this kernel takes rotary_dim / 2, head_dim - rotary_dim and head_dim in multiples of 4; got %d of %d",
          rotary_dim, head_dim)
    _need(1 <= parts.shape[0] <= 8, "this kernel adds up to 8 parts, got %d", parts.shape[0])
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (width,) and bias.is_contiguous(),
              "qkv bias must be bfloat16 [%d]",
              width)
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        page_size = _check_pages(k_pages, v_pages, torch.bfloat16, num_kv_heads, head_dim)
    q = torch.empty((T, num_heads * head_dim), dtype=torch.bfloat16, device=parts.device)
    lib = build.load("rope_kv")
    _check(lib.ga_rope_kv_from_parts(_ptr(q), _ptr(parts), _i(parts.shape[0]), _ptr(bias), _ptr(positions), _ptr(cos),
                                     _ptr(sin), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), _i(T), _i(num_heads),
                                     _i(num_kv_heads), _i(head_dim), _i(rotary_dim), _i(page_size),
                                     _i(1 if write_kv else 0), _stream()), "rope_kv_from_parts")
    return q


def _check_pages(k_pages, v_pages, dtype, nkv, hd):
    """k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, hd, page_size] (values transposed)."""
    _need(k_pages is not None and v_pages is not None, "cache pages are missing")
    for p in (k_pages, v_pages):
        _need(p.dtype == dtype and p.dim() == 4 and p.is_contiguous() and p.shape[1] == nkv,
              "cache pages must be contiguous %s with %d kv heads",
              dtype, nkv)
    ps = k_pages.shape[2]
    _need(k_pages.shape[3] == hd and tuple(v_pages.shape) == (k_pages.shape[0], nkv, hd, ps),
          "cache pages must be k [pages, %d, page_size, %d] and v [pages, %d, %d, page_size], got %s and %s",
          nkv, hd, nkv, hd, tuple(k_pages.shape), tuple(v_pages.shape))
    return ps


def _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, nh, nkv, hd):
    _dev(q, k_pages, v_pages, block_table, token_entry, positions)
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd, "q must be [T, >= nh*hd] with unit inner stride")
    _need(nkv > 0 and nh % nkv == 0,
          "num_heads %d is not a multiple of num_kv_heads %d",
          nh, nkv)
    _check_pages(k_pages, v_pages, q.dtype, nkv, hd)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [entries, width]")
    for name, x in (("token_entry", token_entry), ("positions", positions)):
        _need(x.dtype == torch.int32 and x.shape == (T,) and x.is_contiguous(),
              "%s must be contiguous int32 [T]",
              name)
    return T


def _check_sinks(sinks, num_heads, device):
    """sinks: None, or float32 [num_heads]: a score that every query of a head sees beside its keys' and that has no
    value (it enters the softmax's denominator only)."""
    if sinks is not None:
        _need(sinks.dtype == torch.float32 and sinks.shape == (num_heads,) and sinks.is_contiguous()
              and sinks.device == device, "sinks must be contiguous float32 [%d] on the queries' device", num_heads)
    return sinks


def paged_attention_generic(q, k_pages, v_pages, block_table, token_entry, positions, num_heads, num_kv_heads,
                            head_dim, scale, window=None, out=None, tokens_per_workgroup=0, sinks=None):
    """q: rows of the fused projection ([T, >= nh*hd]; the first nh*hd columns are the queries).
    Token t attends to the keys of request token_entry[t] at positions
    [max(0, p - window + 1), p], p = positions[t] (window may be any value of `mask_parameter`: negative for chunks).  Returns [T, nh*hd].  tokens_per_workgroup: how many neighbouring
    tokens share a workgroup and (where they are of one request) its tiles of keys and values; 1 suits steps of
    single tokens, 0 leaves it to the library (from 32 tokens on: the matrix cores for a request's 8 tokens and more,
    a second kernel for the requests with fewer), -1 says besides that every request has at least 8 tokens in the
    step; no token's result depends on it."""
    T = _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, num_heads,
                                  num_kv_heads, head_dim)
    _check_sinks(sinks, num_heads, q.device)
    _need(0 < head_dim <= 256,
          "head_dim %d is not supported by the general attention kernel (up to 256)",
          head_dim)
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.dtype == q.dtype and out.shape == (T, num_heads * head_dim) and out.stride(1) == 1, "out must be [T, nh*hd]")
    lib = build.load("attention_generic")
    _check(lib.ga_paged_attention_generic(
        _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        _i(block_table.shape[1]), _ptr(token_entry), _ptr(positions), _i(T), _i(num_heads), _i(num_kv_heads),
        _i(head_dim), _i(k_pages.shape[2]), _i(int(window) if window else 0), _f(scale), _i(_is_bf16(q.dtype)),
        _i(int(tokens_per_workgroup)), _i(TUNING.generic_few_tokens_workgroups), _i(TUNING.generic_fill_workgroups),
        _ptr(sinks), _stream()), "paged_attention_generic")
    return out


def gemm_nt(a, w, bias=None, out=None, out_dtype=None):
    """a [M, K] . w [N, K]^T (+ bias [N]) -> [M, N]; 32-bit accumulation, plain FMA.  a and w share a
    dtype (float32 or bfloat16); out is that dtype or float32."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          "gemm_nt: a [M, K] and w [N, K] do not agree: %s, %s",
          tuple(a.shape), tuple(w.shape))
    _need(a.dtype == w.dtype and a.stride(1) == 1 and w.is_contiguous(), "gemm_nt: a and w must share a dtype; w contiguous")
    M, K = a.shape
    N = w.shape[0]
    if bias is not None:
        _need(bias.dtype == w.dtype and bias.shape == (N,) and bias.is_contiguous(), "gemm_nt: bias must be [N] in w's dtype")
    out_dtype = out_dtype or (out.dtype if out is not None else a.dtype)
    _need(out_dtype in (a.dtype, torch.float32), "gemm_nt: out dtype must be the operands' or float32")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm_nt: out must be [M, N]")
    lib = build.load("gemm")
    _check(lib.ga_gemm_nt(_ptr(out), _i64(out.stride(0)), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N),
                          _i(K), _i(_is_bf16(a.dtype)), _i(1 if out_dtype == torch.bfloat16 else 0), _stream()),
           "gemm_nt")
    return out


def sample_rows(logits, temperature=None, uniform=None, out=None):
    """logits float32 [R, V] -> int32 [R].  Rows with temperature 0 (or all rows, without
    temperature) take the argmax with the lowest index among equals; others draw by inverse CDF from
    softmax(logits / temperature) with the given uniform numbers in [0, 1)."""
    _dev(logits, temperature, uniform, out)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1, "logits must be float32 [R, V]")
    R, V = logits.shape
    if temperature is not None:
        _need(uniform is not None, "temperature sampling needs uniform numbers")
        for name, x in (("temperature", temperature), ("uniform", uniform)):
            _need(x.dtype == torch.float32 and x.shape == (R,) and x.is_contiguous(),
                  "%s must be contiguous float32 [R]",
                  name)
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.shape == (R,) and out.is_contiguous(), "out must be contiguous int32 [R]")
    _need(R <= 65535, "at most 65535 rows a call")
    lib = build.load("sampling")
    lib.ga_sample_scratch_floats.restype = ctypes.c_int64
    scratch = torch.empty((max(1, lib.ga_sample_scratch_floats(_i(R), _i(V))),), dtype=torch.float32, device=logits.device)
    _check(lib.ga_sample_rows(_ptr(out), _ptr(logits), _i64(logits.stride(0)), _i(R), _i(V), _ptr(temperature),
                              _ptr(uniform), _ptr(scratch), _stream()), "sample_rows")
    return out


def random_normal_fill(out, key, mean, std):
    """out[i] = mean + std * normal(key, i) over out's elements in memory order (float32 or bfloat16, contiguous): the
    counter-based generator that the host shares, so the same key gives the same bits there."""
    _dev(out)
    _need(out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16), "random fill takes a contiguous float32 or "
          "bfloat16 tensor")
    lib = build.load("random_fill")
    _check(lib.ga_random_normal_fill(_ptr(out), _i64(out.numel()), ctypes.c_uint64(int(key)), _f(mean), _f(std),
                                     _i(_is_bf16(out.dtype)), _stream()), "random_normal_fill")
    return out


SKINNY_MAX_ROWS = 64
FOLDED_NORM_MAX_ROWS = 16


class ScaledRows:
    """The rows of a root-mean-square norm in two factors, as the products around a folded norm hand them on:
    `scaled` = h * g (bfloat16 [M, H]) and `sumsq` (float32 [M, parts]), partial sums of h^2 over the columns;
    the normalised row is scaled / sqrt(sum(sumsq) / H + eps).  A product that takes them multiplies its
    32-bit sums by the rows' factors, which gives what the normalised rows would."""

    __slots__ = ("scaled", "sumsq", "eps")

    def __init__(self, scaled, sumsq, eps):
        self.scaled, self.sumsq, self.eps = scaled, sumsq, float(eps)

    @property
    def shape(self):
        return self.scaled.shape

    @property
    def dtype(self):
        return self.scaled.dtype

    def rows(self):
        """The normalised rows themselves (for checks; the kernels never build them)."""
        rstd = torch.rsqrt(self.sumsq.double().sum(dim=1, keepdim=True) / self.scaled.shape[1] + self.eps)
        return (self.scaled.double() * rstd).float()


class _SkinnyNorm(ctypes.Structure):
    _fields_ = [("in_sumsq", _vp), ("in_parts", _i), ("inv_width", _f), ("eps", _f), ("residual", _vp), ("ldr", _i64),
                ("gain", _vp), ("gain_f32", _i), ("scaled", _vp), ("lds", _i64), ("out_sumsq", _vp)]


def _norm_in(norm, a):
    """Fills the in_ fields from ScaledRows; returns the rows the product runs on."""
    _need(a.scaled.dtype == torch.bfloat16 and a.scaled.dim() == 2 and a.scaled.shape[0] <= FOLDED_NORM_MAX_ROWS,
          "rows of a folded norm are bfloat16 [M <= %d, H]",
          FOLDED_NORM_MAX_ROWS)
    M, H = a.scaled.shape
    _need(a.sumsq.dtype == torch.float32 and a.sumsq.dim() == 2 and a.sumsq.shape[0] == M and a.sumsq.is_contiguous()
          and 1 <= a.sumsq.shape[1] <= 512, "partial sums of a folded norm are contiguous float32 [M, parts <= 512]")
    norm.in_sumsq, norm.in_parts = a.sumsq.data_ptr(), a.sumsq.shape[1]
    norm.inv_width, norm.eps = 1.0 / H, a.eps
    return a.scaled


def folded_norm_supported(a, w, residual, gain):
    """Whether a [M, K] . w [N, K]^T can add itself to `residual` and hand on the rows of the norm with `gain`
    in two factors (ScaledRows)."""
    x = a.scaled if isinstance(a, ScaledRows) else a
    N = w.shape[0]
    return (gemm_skinny_supported(x, w) and x.shape[0] <= FOLDED_NORM_MAX_ROWS and N % 8 == 0
            and build.load("gemm_skinny").ga_skinny_norm_parts(_i(x.shape[0]), _i(N)) <= 512
            and residual.dtype == torch.float32 and residual.shape == (x.shape[0], N) and residual.stride(1) == 1
            and gain.dtype in (torch.bfloat16, torch.float32) and gain.shape == (N,) and gain.is_contiguous())


def gemm_skinny_supported(a, w):
    """Whether the matrix-core kernel for few rows takes these operands."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and 0 < a.shape[0] <= SKINNY_MAX_ROWS
            and a.shape[1] % 8 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0)


def gemm_skinny(a, w, bias=None, out=None, out_dtype=None, nt=0, ks=0, grid_splits=1, gated=False, into_norm=None,
                pack=0, gate_bounds=None):
    """a [M <= 64, K] . w [N, K]^T (+ bias) -> [M, N] in bfloat16 (or float32): the decode step's products,
    weights streamed once through the matrix cores.  grid_splits > 1: K is split over workgroups too and
    the result is float32 [grid_splits, M, N], parts for the consumer to add.  gated: w is [2N, K] (gate
    over up) and the result is silu(a.gate^T) * (a.up^T); with gate_bounds = (limit, alpha, shift) it is
    g * sigmoid(alpha g) * (u + shift) with g = min(a.gate^T, limit) and u = clamp(a.up^T, -limit, limit).
    pack = 2 (at most 8 rows): a tile of the matrix cores holds 8 rows of w twice, for the two halves of K,
    so that twice the workgroups stream the weights.
    a may be ScaledRows (at most 16 rows): the rows of a norm in two factors.  into_norm = (residual, gain, eps):
    the product is added to the float32 residual [M, N] in place and the rows of the norm that follows come
    back as ScaledRows instead of the product."""
    norm = None
    if isinstance(a, ScaledRows):
        norm = _SkinnyNorm()
        a = _norm_in(norm, a)
    if into_norm is not None:
        residual, gain, eps = into_norm
        _need(folded_norm_supported(a, w, residual, gain) and not gated and grid_splits == 1 and out is None,
              "a product folds the norm after it for at most %d bfloat16 rows, a float32 residual [M, N] and a "
              "gain [N], N a multiple of 8 with at most 512 partial sums a row",
              FOLDED_NORM_MAX_ROWS)
        _dev(residual, gain)
        norm = norm or _SkinnyNorm()
        M, N = residual.shape
        lib = build.load("gemm_skinny")
        scaled = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
        sumsq = torch.empty((M, lib.ga_skinny_norm_parts(_i(M), _i(N))), dtype=torch.float32, device=a.device)
        norm.residual, norm.ldr = residual.data_ptr(), residual.stride(0)
        norm.gain, norm.gain_f32 = gain.data_ptr(), 1 if gain.dtype == torch.float32 else 0
        norm.scaled, norm.lds, norm.out_sumsq = scaled.data_ptr(), scaled.stride(0), sumsq.data_ptr()
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          "gemm_skinny: a [M, K] and w [N, K] do not agree: %s, %s",
          tuple(a.shape), tuple(w.shape))
    _need(gemm_skinny_supported(a, w),
          "gemm_skinny takes bfloat16, at most %d rows, K a multiple of 8 and 16-byte "
          "aligned rows; got a %s %s, w %s %s",
          SKINNY_MAX_ROWS, a.dtype, tuple(a.shape), w.dtype, tuple(w.shape))
    M, K = a.shape
    N = w.shape[0]
    if gated:       # w stacks gate over up: the result has half as many columns
        _need(N % 2 == 0 and bias is None and grid_splits == 1, "gated product: w must be [2N, K], without bias or split")
        N //= 2
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be bfloat16 [N]")
    if into_norm is not None:
        _check(lib.ga_gemm_skinny(_vp(0), _i64(0), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N), _i(K),
                                  _i(0), _i(1), _i(8), _i(1), _i(0), _i(0), ctypes.byref(norm), _stream()), "gemm_skinny")
        return ScaledRows(scaled, sumsq, eps)
    out_dtype = out_dtype or (out.dtype if out is not None else torch.bfloat16)
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_skinny: out dtype must be bfloat16 or float32")
    if grid_splits > 1:
        _need(out_dtype == torch.float32, "gemm_skinny: parts of a split product are float32")
        if out is None:
            out = torch.empty((grid_splits, M, N), dtype=torch.float32, device=a.device)
        _need(out.shape == (grid_splits, M, N) and out.dtype == torch.float32 and out.is_contiguous(),
              "gemm_skinny: parts must be contiguous float32 [splits, M, N]")
        ldc = N
    else:
        if out is None:
            out = torch.empty((M, N), dtype=out_dtype, device=a.device)
        _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm_skinny: out must be [M, N]")
        ldc = out.stride(0)
    lib = build.load("gemm_skinny")
    if gate_bounds is not None:
        _need(gated and float(gate_bounds[0]) > 0, "gate bounds belong to a gated product, and the limit is positive")
        limit, alpha, shift = gate_bounds
        _check(lib.ga_gemm_skinny_bounded_gate(_ptr(out), _i64(ldc), _ptr(a), _i64(a.stride(0)), _ptr(w), _i(M), _i(N), _i(K),
                                               _i(1 if out_dtype == torch.float32 else 0), _i(ks), _i(pack), _f(limit), _f(alpha),
                                               _f(shift), ctypes.byref(norm) if norm is not None else _vp(0), _stream()),
               "gemm_skinny_bounded_gate")
        return out
    _check(lib.ga_gemm_skinny(_ptr(out), _i64(ldc), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N),
                              _i(K), _i(1 if out_dtype == torch.float32 else 0), _i(nt), _i(ks), _i(grid_splits),
                              _i(1 if gated else 0), _i(pack), ctypes.byref(norm) if norm is not None else _vp(0),
                              _stream()), "gemm_skinny")
    return out


def qkv_rope_skinny_supported(x, w, head_dim, rotary_dim):
    """Whether the fused projection + rotation + cache-write kernel takes these operands."""
    if isinstance(x, ScaledRows):
        x = x.scaled
    return gemm_skinny_supported(x, w) and head_dim % 32 == 0 and rotary_dim == head_dim


def qkv_rope_skinny(x, w, bias, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads, head_dim,
                    write_kv=True, pack=0):
    """The decode step's q|k|v projection with its epilogue in one kernel: x [M <= 64, K] . w^T + bias, NeoX
    rotation of q and k, q returned as [M, nh*hd], k and v written into the paged cache at slot_mapping.
    x may be ScaledRows."""
    norm = None
    if isinstance(x, ScaledRows):
        norm = _SkinnyNorm()
        x = _norm_in(norm, x)
    _dev(x, w, bias, positions, cos, sin, slot_mapping, k_pages, v_pages)
    M, K = x.shape
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(w.shape == (width, K),
          "qkv weight must be [%d, %d], got %s",
          width, K, tuple(w.shape))
    _need(qkv_rope_skinny_supported(x, w, head_dim, 2 * cos.shape[1]),
          "the fused q|k|v kernel takes bfloat16, at most %d "
          "rows, head sizes that are multiples of 32 and a rotation of the whole head",
          SKINNY_MAX_ROWS)
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (width,) and bias.is_contiguous(),
              "qkv bias must be bfloat16 [%d]",
              width)
    _need(positions.dtype == torch.int32 and positions.shape == (M,) and positions.is_contiguous(), "positions must be int32 [M]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.is_contiguous()
          and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, head_dim/2]")
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (M,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [M]")
        page_size = _check_pages(k_pages, v_pages, torch.bfloat16, num_kv_heads, head_dim)
    q = torch.empty((M, num_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    lib = build.load("gemm_skinny")
    _check(lib.ga_qkv_rope_skinny(_ptr(q), _ptr(x), _i64(x.stride(0)), _ptr(w), _ptr(bias), _ptr(positions), _ptr(cos),
                                  _ptr(sin), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), _i(M), _i(K), _i(num_heads),
                                  _i(num_kv_heads), _i(head_dim), _i(page_size), _i(1 if write_kv else 0), _i(pack),
                                  ctypes.byref(norm) if norm is not None else _vp(0), _stream()), "qkv_rope_skinny")
    return q


# ----------------------------------------------------------------------------- attention on the matrix cores

MFMA_HEAD_DIMS = tuple(range(16, 257, 16))


def mask_parameter(window=None, chunk=None):
    """The attention kernels' one mask parameter: a sliding window of w keys as w, chunks of c positions counted from
    position 0 as -c, every earlier key as 0."""
    _need(not (window and chunk), "a window and chunks at once: %r, %r", window, chunk)
    if chunk:
        _need(int(chunk) > 0, "chunks of %r positions", chunk)
        return -int(chunk)
    _need(not window or int(window) > 0, "a window of %r keys", window)
    return int(window) if window else 0


def first_visible_key(pos, mask):
    """The first key that a query at position `pos` sees under the mask parameter (csrc/common.h has the kernels' twin)."""
    if mask > 0:
        return max(0, pos - mask + 1)
    if mask < 0:
        return pos - pos % (-mask)
    return 0


def attention_mfma_supported(dtype, head_dim, page_size):
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size >= 8
            and page_size & (page_size - 1) == 0)


def plan_rows(q_len, q_start, tile_rows):
    """How a step's rows go to the attention kernels: (rows, positions, entries of the single new tokens,
    tiles of the prompt portions as (entry, first row of the step, rows, first position), heaviest first)."""
    decode_rows, decode_pos, decode_entries, tiles = [], [], [], []
    o = 0
    for e, (n, start) in enumerate(zip(q_len, q_start)):
        if n == 1:
            decode_rows.append(o)
            decode_pos.append(start)
            decode_entries.append(e)
        else:
            for r in range(0, n, tile_rows):
                tiles.append((e, o + r, min(tile_rows, n - r), start + r))
        o += n
    tiles.sort(key=lambda t: -(t[3] + t[2]))      # the tiles with the most keys first
    return decode_rows, decode_pos, decode_entries, tiles


PLAN_TILE_ROWS = 16       # rows of a prompt portion per wavefront in steps of fewer than TUNING.prefill_wide_tiles_from tokens


def _attention_plan(step, tile_rows, device, split_for=None):
    """Which rows of the step are single new tokens and how the rows of prompt portions fall into tiles;
    made once per step and shared by all layers.  A recorded step brings its plan along (`static_plan` in the
    step's extra: device arrays of fixed size that the runner refills, counts that include padding).  split_for:
    (window, workgroups per tile, streams of a workgroup) where the kernel takes tiles whose keys are in parts."""
    key = ("attention_plan", tile_rows, split_for)
    plan = step.extra.get(key)
    if plan is not None:
        return plan
    static = step.extra.get("static_plan")
    if static is not None:
        _need(tile_rows == static["tile_rows"], "a recorded step was planned for tiles of %d rows, not %d",
              static["tile_rows"], tile_rows)
        plan = dict(n_decode=static["n_decode"], decode_pos=None, n_tiles=static["n_tiles"],
                    decode_span=step.extra.get("decode_span"), decode_info=step.extra.get("decode_info"),
                    tiles=static["tiles"], parts=None, part_rows=None, n_part_rows=0, num_parts=1)
        step.extra[key] = plan
        return plan
    import numpy as np
    decode_rows, decode_pos, entries, tiles = plan_rows(step.host_q_len, step.host_q_start, tile_rows)
    # (row, position, entry, -) of every single new token; the runner uploads it with the step's other inputs
    decode_info = step.extra.get("decode_info")
    if decode_info is None and decode_rows:
        decode_info = torch.tensor([[r, p, e, 0] for r, p, e in zip(decode_rows, decode_pos, entries)], dtype=torch.int32,
                                   device=device)
    plan = dict(n_decode=len(decode_rows), decode_pos=decode_pos, n_tiles=len(tiles), decode_span=step.extra.get("decode_span"),
                decode_info=decode_info, tiles=None, parts=None, part_rows=None, n_part_rows=0, num_parts=1)
    if tiles:
        split = key_parts(tiles, tile_rows, *split_for) if split_for is not None else None
        if split is None:
            plan["tiles"] = torch.tensor(np.asarray(tiles, dtype=np.int32).reshape(-1, 4), device=device)
        else:
            # the tiles, their parts and the rows that come in parts, in one transfer
            pieces, parts, rows, num_parts = split
            both = np.concatenate([np.asarray(pieces, dtype=np.int32).reshape(-1), np.asarray(parts, dtype=np.int32).reshape(-1),
                                   np.asarray(rows, dtype=np.int32).reshape(-1)])
            dev_all = torch.tensor(both, device=device)
            n, r = len(pieces), len(rows)
            plan.update(n_tiles=n, tiles=dev_all[:4 * n].view(n, 4), parts=dev_all[4 * n:8 * n].view(n, 4),
                        part_rows=dev_all[8 * n:].view(r, 4), n_part_rows=r, num_parts=num_parts)
    step.extra[key] = plan
    return plan


def key_parts(tiles, tile_rows, window, workgroups_per_tile, streams, compute_units=256):
    """Whether the keys of a step's heaviest tiles should be dealt to several workgroups, and how.  A short prompt alone
    in a step makes about as many workgroups as there are compute units, one round, so the kernel lasts as long as its
    heaviest tile's walk over the keys, twice the mean of a causal prompt's tiles.  tiles: (entry, first row, rows, first
    position), heaviest first.  None: leave the tiles whole.  Else (tiles with one entry per part, parts as the kernel takes
    them, the rows that come in parts as int32 x 4, number of parts): the tiles with more than the mean share of keys per
    compute unit fall into equal parts of at most that share.  Switched off in the table of thresholds
    (`prefill_split_imbalance` 0): measured on MI355X it does not pay (a 2,048-token prompt of 12 heads in 2 groups, head
    size 128: 40.8 us whole, 45.6 in parts: the workgroups beyond one round of the chip pay a workgroup's fixed part, some
    8 us, a second time, and the merge and 10 MB of partial results cost what the shorter walks save)."""
    def key_tiles(t):
        lo = first_visible_key(t[3], window or 0)
        return (t[3] + t[2] - 1) // 32 + 1 - lo // 32, (lo // 32) * 32
    counts = [key_tiles(t)[0] for t in tiles]
    heaviest = max(counts)
    share = sum(counts) * workgroups_per_tile / float(compute_units)          # tiles of 32 keys per compute unit, on average
    if (TUNING.prefill_split_imbalance <= 0 or len(tiles) * workgroups_per_tile > TUNING.prefill_split_max_workgroups
            or heaviest < TUNING.prefill_split_min_key_tiles * streams or heaviest <= TUNING.prefill_split_imbalance * share):
        return None
    share = max(share, 1.0)
    num_parts = min(8, -(-heaviest // int(share)))
    if num_parts < 2:
        return None
    out, rows_in_parts = [], []
    for t, k in zip(tiles, counts):
        first = key_tiles(t)[1]
        if k <= 1.15 * share:
            out.append((k, t, (first, first + 32 * k, -1, 1 << 16)))
            continue
        at = len(rows_in_parts)
        rows_in_parts += [(t[1] + j, 0, 0, 0) for j in range(t[2])]
        per = -(-k // num_parts)
        per = -(-per // streams) * streams                    # whole rounds of the workgroup's streams
        for part in range(num_parts):
            b, e = min(part * per, k), min((part + 1) * per, k)
            # a part without keys still writes its rows' (empty) results, which the merge expects
            out.append((e - b, t, (first + 32 * b, first + 32 * e, at, part | (num_parts << 16))))
    out.sort(key=lambda x: -x[0])                             # the longest walks first
    return [x[1] for x in out], [x[2] for x in out], rows_in_parts, num_parts


def _decode_splits(plan, window, nkv, head_blocks):
    span = 0
    if plan.get("decode_span"):             # a recorded step: the split must fit every context of its bucket
        span = plan["decode_span"] if not window else min(plan["decode_span"], (abs(window) + 62) // 32 * 32)
    else:
        for pos in plan["decode_pos"]:
            lo = first_visible_key(pos, window or 0)
            span = max(span, pos + 1 - (lo // 32) * 32)
    per_split = plan["n_decode"] * nkv * head_blocks
    splits = max(1, min(TUNING.decode_target_workgroups // max(per_split, 1), -(-span // TUNING.decode_min_split_keys),
                        TUNING.decode_max_splits))
    split_keys = -(-(-(-span // splits)) // 32) * 32
    return split_keys, -(-span // split_keys)


def paged_attention_mfma(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale,
                         window=None, out=None, sinks=None):
    """bfloat16 attention of every token of the step on the matrix cores: single new tokens through the
    split-key kernel, rows of prompt portions through the tiled kernel."""
    T = _check_attention_operands(q, k_pages, v_pages, block_table, step.token_entry, step.positions, num_heads,
                                  num_kv_heads, head_dim)
    page_size = k_pages.shape[2]
    _check_sinks(sinks, num_heads, q.device)
    _need(attention_mfma_supported(q.dtype, head_dim, page_size),
          "the matrix-core attention kernels take bfloat16, head sizes in steps of 16 up to 256 and page sizes that "
          "are powers of two from 8; got %s, head %d, page %d",
          q.dtype, head_dim, page_size)
    _need(q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0, "q rows must be 16-byte aligned")
    _need(k_pages.shape[0] * num_kv_heads * max(page_size, head_dim) < 2 ** 31,
          "the matrix-core attention kernels count the rows of a layer's cache in 32 bits: %d pages x %d kv heads x "
          "%d is too many",
          k_pages.shape[0], num_kv_heads, max(page_size, head_dim))
    lib = build.load("attention_mfma", {"HEAD_DIM": head_dim})
    _need(lib.ga_attn_head_dim() == head_dim, "attention library was built for another head size")
    # rows of a prompt portion per wavefront: 32 where the kernel has it and the step is long, else 16
    wide = T >= TUNING.prefill_wide_tiles_from
    tile_rows = lib.ga_attn_prefill_max_tile_rows() if wide else 16
    plan = _attention_plan(step, tile_rows, q.device,
                           split_for=_prefill_workgroups(step, tile_rows, num_heads // num_kv_heads, num_kv_heads, head_dim,
                                                         int(window) if window else 0))
    _need(sum(step.host_q_len) == T, "the step's entries do not add up to its tokens")
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.dtype == q.dtype and out.shape == (T, num_heads * head_dim) and out.is_contiguous(), "out must be [T, nh*hd]")
    w = int(window) if window else 0
    if plan["n_decode"]:
        group = num_heads // num_kv_heads
        split_keys, num_splits = _decode_splits(plan, w, num_kv_heads, -(-group // 16))
        n = plan["n_decode"] * num_heads * num_splits
        ws_o = torch.empty((n * head_dim,), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((n * 2,), dtype=torch.float32, device=q.device)
        _check(lib.ga_attn_decode(
            _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            _i(block_table.shape[1]), _ptr(plan["decode_info"]), _i(plan["n_decode"]), _i(num_heads), _i(num_kv_heads), _i(page_size), _i(w), _f(scale), _i(split_keys),
            _i(num_splits), _ptr(ws_o), _ptr(ws_ml), _ptr(sinks), _stream()), "attn_decode")
    if plan["n_tiles"]:
        part_o = part_ml = None
        if plan["n_part_rows"]:
            n = plan["n_part_rows"] * num_heads * plan["num_parts"]
            part_o = torch.empty((n * head_dim,), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((n * 2,), dtype=torch.float32, device=q.device)
        _check(lib.ga_attn_prefill(
            _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            _i(block_table.shape[1]), _ptr(plan["tiles"]), _i(plan["n_tiles"]), _i(tile_rows), _i(num_heads), _i(num_kv_heads),
            _i(page_size), _i(w), _f(scale), _i(TUNING.prefill_fill_workgroups), _i(TUNING.prefill_prefer_workgroups),
            _ptr(plan["parts"]), _ptr(plan["part_rows"]),
            _i(plan["n_part_rows"]), _i(plan["num_parts"]), _ptr(part_o), _ptr(part_ml), _ptr(sinks), _stream()), "attn_prefill")
    return out


def _prefill_workgroups(step, tile_rows, group, nkv, head_dim, window):
    """(window, workgroups per tile, streams of tiles in a workgroup) as the prefill launcher will choose them for this
    step, or None where the step brings its plan along (a recorded step) or has no prompt portion: what `key_parts`
    needs to know.  Follows ga_attn_prefill's choice of heads per workgroup (csrc/attention_mfma.hip)."""
    if "static_plan" in (step.extra or {}):
        return None
    n_tiles = sum(-(-n // tile_rows) for n in step.host_q_len if n > 1)
    if n_tiles == 0:
        return None
    fill, waves = TUNING.prefill_fill_workgroups, 8
    if head_dim in (64, 128, 256):
        heads = 1
        for d in range(waves - 1, 1, -1):
            if group % d == 0 and n_tiles * nkv * (group // d) >= fill:
                heads = d
                if n_tiles * nkv * (group // d) >= TUNING.prefill_prefer_workgroups:
                    break
        if heads >= 2:
            return window, nkv * (group // heads), max(1, waves // (heads + 1))
    hpw = 1
    for d in range(2, waves + 1):
        if group % d == 0 and n_tiles * nkv * (group // d) >= fill:
            hpw = d
    splits = waves // hpw
    if hpw > 1 and splits > 4:
        splits = 4
    return window, nkv * (group // hpw), splits


def paged_attention(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale, window=None,
                    sinks=None, chunk=None):
    """Attention of every token of the step over its request's pages.  window: the last `window` keys; chunk: the keys of
    the query's own chunk of `chunk` positions, counted from position 0 (neither: every earlier key).  Chooses the kernel: the general
    one in 32-bit (fixed order of every sum: bit-identical however the work is cut); in bfloat16 the
    matrix-core kernels where they take the shape.  sinks: None, or float32 [num_heads], a score per head that
    enters every denominator of the softmax and has no value."""
    window = mask_parameter(window, chunk) or None
    if attention_mfma_supported(q.dtype, head_dim, k_pages.shape[2]):
        return paged_attention_mfma(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale,
                                    window, sinks=sinks)
    if step.max_q_len == 1:
        grouping = 1
    elif "static_plan" not in (step.extra or {}) and min(step.host_q_len) >= 8:
        grouping = -1          # the step's own sizes are known here (a recorded step of padded sizes serves many)
    else:
        grouping = 0
    return paged_attention_generic(q, k_pages, v_pages, block_table, step.token_entry, step.positions, num_heads,
                                   num_kv_heads, head_dim, scale, window, tokens_per_workgroup=grouping, sinks=sinks)


# ---------------------------------------------------------------------------------------------------------------------
# norm with one gain, embedding with sinusoidal positions, short convolution, gated recurrence, latent attention

def _f32(t, shape, name):
    _need(t is not None and t.dtype == torch.float32 and tuple(t.shape) == tuple(shape) and t.is_contiguous(),
          "%s must be contiguous float32 %s", name, tuple(shape))


def _scalar_gain(gain):
    _need(gain.numel() == 1 and gain.dtype in (torch.float32, torch.bfloat16), "the gain must be one float32 or bfloat16 number")
    return 1 if gain.dtype == torch.bfloat16 else 0


def clamped_glu(gate_up, limit, alpha, shift, out=None):
    """gate_up [T, 2I] -> [T, I]: g * sigmoid(alpha g) * (u + shift) with g = min(gate, limit), u = clamp(up, -limit, limit)."""
    _dev(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.dtype == gate_up.dtype and out.shape == (T, I) and out.is_contiguous(), "out must be contiguous [T, I]")
    lib = build.load("activation")
    _check(lib.ga_clamped_glu(_ptr(out), _ptr(gate_up), _i(T), _i(I), _f(limit), _f(alpha), _f(shift),
                              _i(_is_bf16(gate_up.dtype)), _stream()), "clamped_glu")
    return out


def scalar_rmsnorm_rows(x, gain, eps, dtype, rows=None):
    """x float32 [T, H]; gain: one number; rows int32 [R] or None -> [R or T, H] in `dtype`: g * x / sqrt(mean(x^2) + eps)."""
    _dev(x, gain, rows)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "x must be contiguous float32 [T, H]")
    T, H = x.shape
    R = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be contiguous int32 [R]")
        R = rows.shape[0]
    out = torch.empty((R, H), dtype=dtype, device=x.device)
    lib = build.load("scalar_norm")
    _check(lib.ga_scalar_rmsnorm_rows(_ptr(out), _ptr(x), _ptr(gain), _ptr(rows), _i(R), _i(H), _f(eps), _i(_is_bf16(dtype)),
                                      _i(_scalar_gain(gain)), _stream()), "scalar_rmsnorm_rows")
    return out


def add_scalar_rmsnorm(residual, y, gain, eps, copy=False):
    """residual float32 [T, H] += g * y / sqrt(mean(y^2) + eps), in place; y [T, H] float32 or bfloat16.  With copy the
    new residual also comes back in y's dtype (what the next product reads); for a float32 y that is the residual itself."""
    _dev(residual, y, gain)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    _need(y.shape == residual.shape and y.is_contiguous(), "y must be contiguous %s, got %s", tuple(residual.shape), tuple(y.shape))
    T, H = residual.shape
    out = None
    if copy and y.dtype != torch.float32:
        out = torch.empty((T, H), dtype=y.dtype, device=y.device)
    lib = build.load("scalar_norm")
    _check(lib.ga_add_scalar_rmsnorm(_ptr(residual), _ptr(y), _ptr(gain), _ptr(out), _i(T), _i(H), _f(eps), _i(_is_bf16(y.dtype)),
                                     _i(_scalar_gain(gain)), _stream()), "add_scalar_rmsnorm")
    if not copy:
        return None
    return out if out is not None else residual


def embedding_sinusoid_norm(table, ids, positions, freq, gain, eps):
    """table [V, H], ids and positions int32 [T], freq float32 [(H + 1) // 2], gain: one number or None -> float32 [T, H]."""
    _dev(table, ids, positions, freq, gain)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    T, H = ids.shape[0], table.shape[1]
    for name, a in (("ids", ids), ("positions", positions)):
        _need(a.dtype == torch.int32 and a.shape == (T,) and a.is_contiguous(), "%s must be contiguous int32 [T]", name)
    _f32(freq, ((H + 1) // 2,), "freq")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    lib = build.load("embedding_sinusoid")
    _check(lib.ga_embedding_sinusoid_norm(_ptr(out), _ptr(table), _ptr(ids), _ptr(positions), _ptr(freq), _ptr(gain), _i(T),
                                          _i(H), _f(eps), _i(_is_bf16(table.dtype)),
                                          _i(_scalar_gain(gain) if gain is not None else 0), _stream()), "embedding_sinusoid_norm")
    return out


SHORT_CONV_MAX_TAPS = 16


def short_conv(x, weight, state, slots, step, dtype, add_input=True, update=True, bias=None):
    """x float32 [T, W] (the residual stream, or columns of a wider 32-bit tensor); weight float32 [W, taps]; state float32
    [slots, taps - 1, W] (None for one tap); slots int64 [entries]; bias float32 [W] or None.  Returns (x +) the causal
    convolution (+ bias) in `dtype`, the inputs before the step's tokens taken from the state, and moves the state on by the
    step's tokens."""
    _dev(x, weight, state, slots, bias)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1, "x must be float32 [T, W] with unit inner stride")
    T, W = x.shape
    if bias is not None:
        _f32(bias, (W,), "bias")
    _need(weight.dim() == 2 and weight.shape[0] == W and 1 <= weight.shape[1] <= SHORT_CONV_MAX_TAPS,
          "the convolution's weight must be [%d, taps <= %d], got %s", W, SHORT_CONV_MAX_TAPS, tuple(weight.shape))
    taps = weight.shape[1]
    _f32(weight, (W, taps), "weight")
    E = step.cu_tokens.shape[0] - 1
    for name, a, n in (("token_entry", step.token_entry, T), ("cu_tokens", step.cu_tokens, E + 1), ("q_start", step.q_start, E)):
        _need(a.dtype == torch.int32 and a.shape == (n,) and a.is_contiguous(), "%s must be contiguous int32 [%d]", name, n)
    if taps > 1:
        _need(state is not None and state.dtype == torch.float32 and state.dim() == 3 and state.is_contiguous()
              and tuple(state.shape[1:]) == (taps - 1, W), "state must be contiguous float32 [slots, %d, %d]", taps - 1, W)
        _need(slots.dtype == torch.int64 and slots.shape == (E,) and slots.is_contiguous(), "slots must be contiguous int64 [%d]", E)
    out = torch.empty((T, W), dtype=dtype, device=x.device)
    lib = build.load("short_conv")
    _check(lib.ga_short_conv_apply(_ptr(out), _ptr(x), _ptr(weight), _ptr(state), _ptr(slots), _ptr(step.token_entry),
                                   _ptr(step.cu_tokens), _ptr(step.q_start), _i(T), _i(W), _i(taps), _i(1 if add_input else 0),
                                   _i(_is_bf16(dtype)), _i64(x.stride(0)), _ptr(bias), _stream()), "short_conv_apply")
    if update and taps > 1:
        _check(lib.ga_short_conv_update(_ptr(state), _ptr(x), _ptr(slots), _ptr(step.cu_tokens), _ptr(step.q_start), _i(E), _i(W),
                                        _i(taps), _i64(x.stride(0)), _stream()), "short_conv_update")
    return out


HGRN2_MAX_DIM = 256


def hgrn2_scan(proj, f_bias, lower, state, slots, step, heads, dim, vdim, update=True):
    """proj float32 [T, 2 heads dim + heads vdim]: (q before its SiLU | forget-gate logits | v); f_bias, lower float32
    [heads dim]; state float32 [slots, heads, dim, vdim], advanced in place.  Returns float32 [T, heads, vdim]."""
    _dev(proj, f_bias, lower, state, slots)
    T = proj.shape[0]
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] == 2 * heads * dim + heads * vdim,
          "proj must be float32 [T, %d] with unit inner stride, got %s %s", 2 * heads * dim + heads * vdim, proj.dtype, tuple(proj.shape))
    _need(0 < dim <= HGRN2_MAX_DIM, "the recurrence kernel takes up to %d key channels per head, got %d", HGRN2_MAX_DIM, dim)
    _f32(f_bias, (heads * dim,), "f_bias")
    _f32(lower, (heads * dim,), "lower")
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dim, vdim),
          "state must be contiguous float32 [slots, %d, %d, %d]", heads, dim, vdim)
    E = step.cu_tokens.shape[0] - 1
    _need(slots.dtype == torch.int64 and slots.shape == (E,) and slots.is_contiguous(), "slots must be contiguous int64 [%d]", E)
    _need(update, "the recurrence always advances its state")
    out = torch.empty((T, heads, vdim), dtype=torch.float32, device=proj.device)
    lib = build.load("gated_recurrence")
    _check(lib.ga_hgrn2_scan(_ptr(out), _ptr(proj), _i64(proj.stride(0)), _ptr(f_bias), _ptr(lower), _ptr(state), _ptr(slots),
                             _ptr(step.cu_tokens), _ptr(step.q_start), _i(E), _i(heads), _i(dim), _i(vdim), _stream()), "hgrn2_scan")
    return out


def headwise_rmsnorm(x, weight, eps, dtype):
    """x float32 [..., V] -> the same shape in `dtype`: every row of V normalised by its root mean square, times weight [V]."""
    _dev(x, weight)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous float32")
    V = x.shape[-1]
    _f32(weight, (V,), "weight")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    lib = build.load("gated_recurrence")
    _check(lib.ga_headwise_rmsnorm(_ptr(out), _ptr(x), _ptr(weight), _i64(x.numel() // V), _i(V), _f(eps), _i(_is_bf16(dtype)),
                                   _stream()), "headwise_rmsnorm")
    return out


LATENT_MAX_RANK = 512


def latent_prepare(proj, q_norm, kv_norm, slot_mapping, c_pages, q_rank, kv_rank, heads, eps, dtype, write=True, gated=True,
                   ct_pages=None):
    """proj float32 [T, q_rank + kv_rank (+ heads)]: the down-projections (and gate logits).  Returns (cq [T, q_rank] in
    `dtype`: the normed query latent; gate float32 [T, heads] or None); writes the normed latent c of every token into its
    slot of c_pages [pages, page_size * kv_rank] (slot -1: no write) and, where ct_pages is given, into the copy that
    lies transposed inside each page ([pages, kv_rank * page_size])."""
    _dev(proj, q_norm, kv_norm, slot_mapping, c_pages, ct_pages)
    T = proj.shape[0]
    cols = q_rank + kv_rank + (heads if gated else 0)
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] == cols,
          "proj must be float32 [T, %d], got %s %s", cols, proj.dtype, tuple(proj.shape))
    _f32(q_norm, (q_rank,), "q_norm")
    _f32(kv_norm, (kv_rank,), "kv_norm")
    _need(slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,) and slot_mapping.is_contiguous(),
          "slot_mapping must be contiguous int64 [T]")
    for pages in (c_pages, ct_pages):
        _need(pages is None or (pages.dtype == dtype and pages.dim() == 2 and pages.is_contiguous() and pages.shape[1] % kv_rank == 0
                                and pages.shape == c_pages.shape),
              "the latent's pages must be contiguous %s [pages, page_size * %d]", dtype, kv_rank)
    cq = torch.empty((T, q_rank), dtype=dtype, device=proj.device)
    gate = torch.empty((T, heads), dtype=torch.float32, device=proj.device) if gated else None
    lib = build.load("latent_attention")
    _check(lib.ga_latent_prepare(_ptr(cq), _ptr(c_pages), _ptr(ct_pages), _i(c_pages.shape[1] // kv_rank), _ptr(gate), _ptr(proj),
                                 _i64(proj.stride(0)), _ptr(q_norm), _ptr(kv_norm), _ptr(slot_mapping), _i(T), _i(q_rank),
                                 _i(kv_rank), _i(heads), _f(eps), _i(1 if write else 0), _i(_is_bf16(dtype)), _stream()),
           "latent_prepare")
    return cq, gate


def latent_attention_mfma_supported(dtype, rank, page_size):
    """The matrix-core kernels take bfloat16, ranks that are multiples of 8 up to 512 and page sizes that are powers of two
    from 8."""
    return dtype == torch.bfloat16 and rank % 8 == 0 and 0 < rank <= 512 and page_size >= 8 and page_size & (page_size - 1) == 0


def latent_attention(qa, c_pages, block_table, step, sink, gate, heads, rank, page_size, scale, window, dtype, ct_pages=None):
    """qa float32 [heads, T, rank]: the queries in the latent space.  Every token attends to the latent rows of its request's
    pages at positions [max(0, p - window + 1), p] (window None: from 0); sink float32 [heads] or None joins the softmax's
    denominator; gate float32 [T, heads] or None scales each head's result.  Returns [heads, T, rank] in `dtype`.
    With ct_pages (the copy transposed inside each page) and sizes that `latent_attention_mfma_supported` takes, the matrix
    cores do it: prompt portions with 16 tokens side by side, single tokens with 16 heads side by side and their keys
    dealt to several workgroups; else the general kernel."""
    _dev(qa, c_pages, ct_pages, block_table, sink, gate)
    T = step.token_entry.shape[0]
    _f32(qa, (heads, T, rank), "qa")
    _need(0 < rank <= LATENT_MAX_RANK, "the latent attention kernel takes ranks up to %d, got %d", LATENT_MAX_RANK, rank)
    _need(c_pages.dtype == dtype and c_pages.dim() == 2 and c_pages.is_contiguous() and c_pages.shape[1] == page_size * rank,
          "the latent's pages must be contiguous %s [pages, %d]", dtype, page_size * rank)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [entries, width]")
    for name, a in (("token_entry", step.token_entry), ("positions", step.positions)):
        _need(a.dtype == torch.int32 and a.shape == (T,) and a.is_contiguous(), "%s must be contiguous int32 [T]", name)
    if sink is not None:
        _f32(sink, (heads,), "sink")
    if gate is not None:
        _f32(gate, (T, heads), "gate")
    out = torch.empty((heads, T, rank), dtype=dtype, device=qa.device)
    lib = build.load("latent_attention")
    w = int(window) if window else 0
    if ct_pages is not None and latent_attention_mfma_supported(dtype, rank, page_size):
        _need(ct_pages.dtype == dtype and ct_pages.shape == c_pages.shape and ct_pages.is_contiguous(),
              "the transposed copy must have the shape of the latent's pages")
        info = (step.extra or {}).get("decode_info") if getattr(step, "extra", None) is not None else None
        _need(info is not None and info.dtype == torch.int32 and info.dim() == 2 and info.shape[1] == 4 and info.is_contiguous(),
              "the step must bring its single tokens as int32 [n, 4] (row, position, entry, 0)")
        E = step.cu_tokens.shape[0] - 1
        _need(step.cu_tokens.dtype == torch.int32 and step.cu_tokens.is_contiguous(), "cu_tokens must be contiguous int32")
        n_single = info.shape[0]
        if n_single < T:      # the step holds prompt portions (in a recorded step of padded sizes: may hold)
            _check(lib.ga_latent_attention_rows(
                _ptr(out), _i64(rank), _i64(T * rank), _ptr(qa), _i64(rank), _i64(T * rank), _ptr(c_pages), _ptr(ct_pages),
                _ptr(block_table), _i(block_table.shape[1]), _ptr(step.token_entry), _ptr(step.positions), _ptr(step.cu_tokens),
                _ptr(sink), _ptr(gate), _i(T), _i(heads), _i(rank), _i(page_size), _i(w), _f(scale), _i(1), _stream()),
                "latent_attention_rows")
        if n_single > 0:
            # the longest walk in tiles of 32: over the window, or over the longest context of the step's bucket
            span = int(step.extra.get("decode_span") or step.max_kv_len)
            if w:
                span = min(span, w)
            tiles = (span + 31) // 32 + 1
            workgroups = n_single * (-(-(-(-heads // 16)) // 4))
            splits = max(1, min(tiles, TUNING.latent_decode_workgroups // max(workgroups, 1), TUNING.latent_decode_max_splits, 64))
            per = -(-tiles // splits)
            splits = -(-tiles // per)
            ws_o = ws_ml = None
            if splits > 1:
                rp = lib.ga_latent_attention_mfma_padded_rank(_i(rank))
                ws_o = torch.empty((n_single * heads * splits * rp,), dtype=torch.float32, device=qa.device)
                ws_ml = torch.empty((n_single * heads * splits * 2,), dtype=torch.float32, device=qa.device)
            _check(lib.ga_latent_attention_heads(
                _ptr(out), _i64(rank), _i64(T * rank), _ptr(ws_o), _ptr(ws_ml), _ptr(qa), _i64(rank), _i64(T * rank), _ptr(c_pages),
                _ptr(ct_pages), _ptr(block_table), _i(block_table.shape[1]), _ptr(info), _i(n_single), _ptr(sink), _ptr(gate),
                _i(heads), _i(rank), _i(page_size), _i(w), _f(scale), _i(splits), _i(per), _stream()), "latent_attention_heads")
        return out
    _check(lib.ga_latent_attention(_ptr(out), _i64(rank), _i64(T * rank), _ptr(qa), _i64(rank), _i64(T * rank), _ptr(c_pages),
                                   _ptr(block_table), _i(block_table.shape[1]), _ptr(step.token_entry), _ptr(step.positions),
                                   _ptr(sink), _ptr(gate), _i(T), _i(heads), _i(rank), _i(page_size), _i(w),
                                   _f(scale), _i(_is_bf16(dtype)), _stream()), "latent_attention")
    return out


# ---------------------------------------------------------------------------------------------------------------------
# norm on a sublayer's output with a factor per channel, routing to experts, activations of feed-forwards without a gate

def output_norm_add(residual, y, gain, scale, eps, next_gain=None, next_eps=None, dtype=None):
    """residual float32 [T, H] += scale * gain * y / sqrt(mean(y^2) + eps), in place; y [T, H] float32 or bfloat16, or
    float32 [parts, T, H]: partial sums of a product whose K was split, added in order first; gain float32 [H]; scale
    float32 [H] or None.  With next_gain (float32 [H]) the rows next_gain * r / sqrt(mean(r^2) +
    next_eps) of the new residual r come back in `dtype`: what the sublayer after this one reads."""
    _dev(residual, y, gain, scale, next_gain)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    parts = 1
    if y.dim() == 3:
        _need(y.dtype == torch.float32 and tuple(y.shape[1:]) == tuple(residual.shape) and y.is_contiguous() and y.shape[0] >= 1,
              "partial sums must be contiguous float32 [parts, %d, %d], got %s %s", residual.shape[0], residual.shape[1], y.dtype,
              tuple(y.shape))
        parts = y.shape[0]
    else:
        _need(y.shape == residual.shape and y.is_contiguous() and y.dtype in (torch.float32, torch.bfloat16),
              "y must be contiguous float32 or bfloat16 %s, got %s %s", tuple(residual.shape), y.dtype, tuple(y.shape))
    T, H = residual.shape
    _f32(gain, (H,), "gain")
    if scale is not None:
        _f32(scale, (H,), "scale")
    out = None
    if next_gain is not None:
        _f32(next_gain, (H,), "next_gain")
        _need(next_eps is not None and dtype is not None, "the following norm needs its eps and the dtype of its rows")
        out = torch.empty((T, H), dtype=dtype, device=residual.device)
    lib = build.load("output_norm")
    _check(lib.ga_output_norm_add(_ptr(residual), _ptr(y), _ptr(gain), _ptr(scale), _f(eps), _ptr(next_gain),
                                  _f(next_eps if next_eps is not None else 0.0), _ptr(out), _i(T), _i(H), _i(_is_bf16(y.dtype)),
                                  _i(_is_bf16(dtype)) if out is not None else _i(0), _i(parts), _stream()), "output_norm_add")
    return out


ROUTE_MAX_EXPERTS = 256


def route_topk(scores, top):
    """scores float32 [T, E] -> (ids int32 [T, top], weights float32 [T, top], dense float32 [T, E]): the `top` largest of
    every row (the lowest index among equals), the softmax over the chosen scores alone, and the same weights as a row
    over all experts with zeros at the others."""
    _dev(scores)
    _need(scores.dtype == torch.float32 and scores.dim() == 2 and scores.is_contiguous(), "scores must be contiguous float32 [T, E]")
    T, E = scores.shape
    _need(1 <= E <= ROUTE_MAX_EXPERTS and 1 <= top <= E, "routing takes 1 to %d experts and 1 <= top <= experts; got %d, top %d",
          ROUTE_MAX_EXPERTS, E, top)
    ids = torch.empty((T, top), dtype=torch.int32, device=scores.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=scores.device)
    dense = torch.empty((T, E), dtype=torch.float32, device=scores.device)
    lib = build.load("routing")
    _check(lib.ga_route_topk(_ptr(ids), _ptr(weights), _ptr(dense), _ptr(scores), _i(T), _i(E), _i(top), _stream()), "route_topk")
    return ids, weights, dense


def route_sigmoid_groups(logits, top, correction=None, groups=1, keep=1, group_top=2, normalise=True, floor=0.0, scale=1.0):
    """logits float32 [T, E] -> (ids, weights, dense) as `route_topk` gives them, from sigmoid scores s = sigmoid(logits): the
    choice goes by s + correction (float32 [E] or None); the experts fall into `groups` equal groups of neighbours, a group's
    score is the sum of its `group_top` largest choice scores, and only experts of the `keep` best groups can be chosen; the
    weights are the chosen experts' s, divided by their sum + floor where `normalise`, times scale."""
    _dev(logits, correction)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "logits must be contiguous float32 [T, E]")
    T, E = logits.shape
    _need(1 <= E <= ROUTE_MAX_EXPERTS and 1 <= top <= E, "routing takes 1 to %d experts and 1 <= top <= experts; got %d, top %d",
          ROUTE_MAX_EXPERTS, E, top)
    _need(groups >= 1 and E % groups == 0 and 1 <= keep <= groups and top <= keep * (E // groups) and 1 <= group_top <= 4,
          "%d experts in %d groups of which %d are kept (scored by their %d largest) cannot give %d choices", E, groups, keep,
          group_top, top)
    if correction is not None:
        _f32(correction, (E,), "correction")
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    dense = torch.empty((T, E), dtype=torch.float32, device=logits.device)
    lib = build.load("routing")
    _check(lib.ga_route_sigmoid_groups(_ptr(ids), _ptr(weights), _ptr(dense), _ptr(logits), _ptr(correction), _i(T), _i(E), _i(top),
                                       _i(groups), _i(keep), _i(group_top), _i(1 if normalise else 0), _f(floor), _f(scale),
                                       _stream()), "route_sigmoid_groups")
    return ids, weights, dense


def router_scores(x, weight, bias):
    """x [T, H] (bfloat16 or float32), weight float32 [E, H], bias float32 [E] or None -> float32 [T, E] = x . weight^T + bias,
    summed in 32-bit, a wavefront per score."""
    _dev(x, weight, bias)
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.float32, torch.bfloat16), "x must be contiguous float32 or bfloat16 [T, H]")
    T, H = x.shape
    E = weight.shape[0]
    _need(1 <= E <= ROUTE_MAX_EXPERTS, "1 to %d experts, got %d", ROUTE_MAX_EXPERTS, E)
    _f32(weight, (E, H), "router weight")
    if bias is not None:
        _f32(bias, (E,), "router bias")
    scores = torch.empty((T, E), dtype=torch.float32, device=x.device)
    lib = build.load("routing")
    _check(lib.ga_router_scores(_ptr(scores), _ptr(x), _ptr(weight), _ptr(bias), _i(T), _i(H), _i(E), _i(_is_bf16(x.dtype)),
                                _stream()), "router_scores")
    return scores


def route_sort(ids, experts):
    """ids int32 [T, top] -> (offsets int32 [experts + 1], pair_of_row int32 [T * top], row_of_pair int32 [T * top]): the
    token-expert pairs (pair p = token p // top, its choice p % top) grouped by expert; expert e owns the rows
    [offsets[e], offsets[e + 1])."""
    _dev(ids)
    _need(ids.dtype == torch.int32 and ids.dim() == 2 and ids.is_contiguous(), "ids must be contiguous int32 [T, top]")
    _need(1 <= experts <= ROUTE_MAX_EXPERTS, "1 to %d experts, got %d", ROUTE_MAX_EXPERTS, experts)
    P = ids.numel()
    offsets = torch.empty((experts + 1,), dtype=torch.int32, device=ids.device)
    pair_of_row = torch.empty((P,), dtype=torch.int32, device=ids.device)
    row_of_pair = torch.empty((P,), dtype=torch.int32, device=ids.device)
    lib = build.load("routing")
    _check(lib.ga_route_sort(_ptr(ids), _ptr(offsets), _ptr(pair_of_row), _ptr(row_of_pair), _i(P), _i(experts), _stream()), "route_sort")
    return offsets, pair_of_row, row_of_pair


def gather_pair_rows(x, pair_of_row, ids, offsets, capacity):
    """x [T, H]; pair_of_row int32 [P], ids int32 [T, top], offsets int32 [E + 1] as route_sort gives them -> [E, capacity,
    H]: expert e's rows side by side from [e, 0] on (what lies behind them holds anything)."""
    _dev(x, pair_of_row, ids, offsets)
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.float32, torch.bfloat16), "x must be contiguous [T, H]")
    _need(pair_of_row.dtype == torch.int32 and pair_of_row.shape == (ids.numel(),) and pair_of_row.is_contiguous(), "pair_of_row must be int32 [P]")
    _need(ids.dtype == torch.int32 and ids.dim() == 2 and ids.shape[0] == x.shape[0] and ids.is_contiguous(), "ids must be contiguous int32 [T, top]")
    _need(offsets.dtype == torch.int32 and offsets.dim() == 1 and offsets.is_contiguous(), "offsets must be int32 [E + 1]")
    E, P, H = offsets.shape[0] - 1, pair_of_row.shape[0], x.shape[1]
    _need(capacity >= 1, "an expert's group must hold at least a row")
    out = torch.empty((E, capacity, H), dtype=x.dtype, device=x.device)
    lib = build.load("routing")
    _check(lib.ga_gather_pair_rows(_ptr(out), _ptr(x), _ptr(pair_of_row), _ptr(ids), _ptr(offsets), _i(capacity), _i(P), _i(H),
                                   _i(ids.shape[1]), _i(_is_bf16(x.dtype)), _stream()), "gather_pair_rows")
    return out


def combine_pairs(y, shared, weights, row_of_pair, ids, offsets):
    """y [E, capacity, H]: the experts' results, laid as gather_pair_rows lays their rows; weights float32 [T, top];
    shared [T, H] or None -> [T, H]: sum_j weights[t, j] * (the result of pair t * top + j) + shared[t], added in 32-bit in
    the order of the choice."""
    _dev(y, shared, weights, row_of_pair, ids, offsets)
    T, top = weights.shape
    _need(y.dim() == 3 and y.is_contiguous() and y.shape[0] == offsets.shape[0] - 1, "y must be contiguous [E, capacity, H]")
    capacity, H = y.shape[1], y.shape[2]
    _f32(weights, (T, top), "weights")
    _need(row_of_pair.dtype == torch.int32 and row_of_pair.shape == (T * top,) and row_of_pair.is_contiguous(), "row_of_pair must be int32 [%d]", T * top)
    _need(ids.dtype == torch.int32 and ids.shape == (T, top) and ids.is_contiguous(), "ids must be contiguous int32 [%d, %d]", T, top)
    _need(offsets.dtype == torch.int32 and offsets.is_contiguous(), "offsets must be int32 [E + 1]")
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == y.dtype and shared.is_contiguous(), "shared must be contiguous [%d, %d]", T, H)
    out = torch.empty((T, H), dtype=y.dtype, device=y.device)
    lib = build.load("routing")
    _check(lib.ga_combine_pairs(_ptr(out), _ptr(y), _ptr(shared), _ptr(weights), _ptr(row_of_pair), _ptr(ids), _ptr(offsets),
                                _i(capacity), _i(T), _i(H), _i(top), _i(_is_bf16(y.dtype)), _stream()), "combine_pairs")
    return out


def weighted_silu_mul(gate_up, dense, ff):
    """gate_up [T, 2 I]: for every expert its ff gate columns, then its ff up columns, the experts one after the other, and
    behind them a shared expert's gates and ups -> [T, I]: w * silu(gate) * up, the columns [e * ff, (e + 1) * ff) weighted
    by dense[t, e], the columns behind the last expert's by 1."""
    _dev(gate_up, dense)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    _need(dense.dtype == torch.float32 and dense.dim() == 2 and dense.shape[0] == T and dense.is_contiguous(),
          "the experts' weights must be contiguous float32 [%d, E]", T)
    E = dense.shape[1]
    _need(ff >= 1 and E * ff <= I, "%d experts of %d columns do not fit %d", E, ff, I)
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    lib = build.load("routing")
    _check(lib.ga_weighted_silu_mul(_ptr(out), _ptr(gate_up), _ptr(dense), _i(T), _i(I), _i(E), _i(ff),
                                    _i(_is_bf16(gate_up.dtype)), _stream()), "weighted_silu_mul")
    return out


def relu_square(x):
    """max(x, 0)^2, in place; x contiguous float32 or bfloat16."""
    _dev(x)
    _need(x.is_contiguous() and x.data_ptr() % 16 == 0, "x must be contiguous at a 16-byte address")
    lib = build.load("activation")
    _check(lib.ga_relu_square(_ptr(x), _ptr(x), _i64(x.numel()), _i(_is_bf16(x.dtype)), _stream()), "relu_square")
    return x


def scaled_sum(a, b, sa, sb, dtype):
    """sa * a + sb * b in 32-bit, [T, W] in `dtype`.  Each of a and b is [T, W] in `dtype`, or float32 [parts, T, W]: the
    partial sums of a product whose K was split, added in order first."""
    _dev(a, b)
    shape = tuple(a.shape[-2:])
    parts = []
    for name, t in (("a", a), ("b", b)):
        _need(t.is_contiguous() and tuple(t.shape[-2:]) == shape and t.dim() in (2, 3), "%s must be contiguous [T, W] or [parts, T, W]", name)
        _need(t.dtype == (torch.float32 if t.dim() == 3 else dtype), "%s: partial sums are float32, a whole result is %s", name, dtype)
        parts.append(t.shape[0] if t.dim() == 3 else 0)
    out = a if a.dim() == 2 else (b if b.dim() == 2 else torch.empty(shape, dtype=dtype, device=a.device))
    lib = build.load("activation")
    _check(lib.ga_scaled_sum(_ptr(out), _ptr(a), _i(parts[0]), _ptr(b), _i(parts[1]), _f(sa), _f(sb), _i64(out.numel()),
                             _i(_is_bf16(dtype)), _stream()), "scaled_sum")
    return out


def conv_rope_kv(proj, weight, state, slots, step, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads, head_dim,
                 value_dim, padded, dtype, write_kv=True, update_state=True, qk_gain=None, qk_eps=0.0):
    """Behind a fused q|k|v projection whose channels pass a short causal convolution: proj [T, (nh + nkv) hd + nkv vd] in
    the compute dtype `dtype` or in float32; weight float32 [channels, taps] (None: no convolution); state float32 [slots, taps - 1, channels]
    (None for one tap) and slots int64 [entries]; cos, sin float32 [positions, rotary_dim / 2] (None: no rotation).
    qk_gain float32 [(nh + nkv) hd] (no convolution then): q and k are divided by the root mean square of the token's WHOLE q
    (k) projection (eps qk_eps) and multiplied by the gain, before the rotation.
    Returns q [T, nh * padded], heads padded with zeros, and writes k and v (padded alike) into the pages at slot_mapping;
    moves the state on by the step's tokens."""
    _dev(proj, weight, state, slots, cos, sin, slot_mapping, k_pages, v_pages)
    T = proj.shape[0]
    C = (num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim
    _need(proj.dim() == 2 and proj.shape[1] == C and proj.is_contiguous() and proj.dtype in (torch.float32, torch.bfloat16),
          "proj must be contiguous float32 or bfloat16 [T, %d], got %s %s", C, proj.dtype, tuple(proj.shape))
    _need(head_dim <= padded <= 256 and value_dim <= padded, "heads padded to %d (at most 256) do not hold %d / %d", padded,
          head_dim, value_dim)
    _need(num_heads + 2 * num_kv_heads <= 65535, "too many heads for one launch: %d", num_heads + 2 * num_kv_heads)
    taps = 1
    if weight is not None:
        _need(weight.dim() == 2 and weight.shape[0] == C and 1 <= weight.shape[1] <= SHORT_CONV_MAX_TAPS,
              "the convolution's weight must be [%d, taps <= %d], got %s", C, SHORT_CONV_MAX_TAPS, tuple(weight.shape))
        taps = weight.shape[1]
        _f32(weight, (C, taps), "weight")
    E = step.cu_tokens.shape[0] - 1
    for name, a, n in (("token_entry", step.token_entry, T), ("cu_tokens", step.cu_tokens, E + 1), ("q_start", step.q_start, E),
                       ("positions", step.positions, T)):
        _need(a.dtype == torch.int32 and a.shape == (n,) and a.is_contiguous(), "%s must be contiguous int32 [%d]", name, n)
    if taps > 1:
        _need(state is not None and state.dtype == torch.float32 and state.dim() == 3 and state.is_contiguous()
              and tuple(state.shape[1:]) == (taps - 1, C), "state must be contiguous float32 [slots, %d, %d]", taps - 1, C)
        _need(slots.dtype == torch.int64 and slots.shape == (E,) and slots.is_contiguous(), "slots must be contiguous int64 [%d]", E)
    rotary_dim = 0
    if cos is not None:
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
        rotary_dim = 2 * cos.shape[1]
        _need(0 < rotary_dim <= head_dim, "rotary_dim %d must lie in (0, head_dim %d]", rotary_dim, head_dim)
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        page_size = _check_pages(k_pages, v_pages, dtype, num_kv_heads, padded)
    _need(proj.dtype in (dtype, torch.float32), "proj must be %s or float32", dtype)
    q = torch.empty((T, num_heads * padded), dtype=dtype, device=proj.device)
    row_scale = None
    if qk_gain is not None:
        _need(weight is None, "the norm over the whole projection stands in front of no convolution")
        _f32(qk_gain, ((num_heads + num_kv_heads) * head_dim,), "qk_gain")
        _need(qk_gain.device == proj.device, "qk_gain lies on another device")
        row_scale = torch.empty((T, 2), dtype=torch.float32, device=proj.device)
    lib = build.load("conv_rope_kv")
    _check(lib.ga_conv_rope_kv(_ptr(q), _ptr(proj), _ptr(weight), _ptr(state), _ptr(slots), _ptr(step.token_entry),
                               _ptr(step.cu_tokens), _ptr(step.q_start), _ptr(step.positions), _ptr(cos), _ptr(sin),
                               _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), _i(T), _i(E), _i(num_heads), _i(num_kv_heads),
                               _i(head_dim), _i(value_dim), _i(padded), _i(rotary_dim), _i(taps), _i(page_size),
                               _i(1 if write_kv else 0), _i(1 if update_state else 0), _i(_is_bf16(dtype)),
                               _i(_is_bf16(proj.dtype)), _ptr(row_scale), _ptr(qk_gain), _f(qk_eps), _stream()),
           "conv_rope_kv")
    return q


DECAY_SCAN_MAX_DIM = 256
GLA_DECAY_MAX_RANK = 768       # 16 tokens' narrow rows in 48 KB of LDS


def _step_entries(step, slots):
    E = step.cu_tokens.shape[0] - 1
    for name, a, n in (("cu_tokens", step.cu_tokens, E + 1), ("q_start", step.q_start, E)):
        _need(a.dtype == torch.int32 and a.shape == (n,) and a.is_contiguous(), "%s must be contiguous int32 [%d]", name, n)
    _need(slots.dtype == torch.int64 and slots.shape == (E,) and slots.is_contiguous(), "slots must be contiguous int64 [%d]", E)
    return E


def _rows_of(proj, start, width, name):
    """A block of columns of a 32-bit projection as (view, row stride)."""
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and 0 <= start and start + width <= proj.shape[1],
          "%s: columns %d .. %d of a float32 projection with unit inner stride, got %s %s", name, start, start + width, proj.dtype,
          tuple(proj.shape))
    return proj[:, start:start + width]


def gla_decay(proj, low_start, a2t, bias, tau):
    """sigmoid(a2 low + bias)^(1 / tau) in 32-bit: low = proj[:, low_start : low_start + rank] (float32 rows), a2t the widening
    matrix transposed, float32 [rank, channels], bias float32 [channels].  Returns float32 [T, channels]."""
    _dev(proj, a2t, bias)
    _need(a2t.dim() == 2, "a2t must be [rank, channels]")
    R, C = a2t.shape
    _f32(a2t, (R, C), "a2t")
    _f32(bias, (C,), "bias")
    _need(R <= GLA_DECAY_MAX_RANK, "the decay's narrow projection may be up to %d wide, got %d", GLA_DECAY_MAX_RANK, R)
    low = _rows_of(proj, low_start, R, "low")
    _need(tau > 0, "tau must be positive, got %r", tau)
    T = proj.shape[0]
    out = torch.empty((T, C), dtype=torch.float32, device=proj.device)
    lib = build.load("decay_scan")
    _check(lib.ga_gla_decay(_ptr(out), _ptr(low), _i64(proj.stride(0)), _ptr(a2t), _ptr(bias), _i(T), _i(C), _i(R), _f(tau),
                            _stream()), "gla_decay")
    return out


def decay_scan(proj, q_start, k_start, v_start, state, slots, step, heads, dim, vdim, decay=None, head_decay=None, cos=None,
               sin=None, q_scale=1.0, k_scale=1.0, silu_inputs=False):
    """Linear attention with a decay as a recurrence over per-request state: S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T
    q_t per head.  q, k, v are column blocks of the float32 projection `proj` (starting at q_start, k_start, v_start; heads *
    dim, heads * dim, heads * vdim wide).  a: `decay` float32 [T, heads * dim], or `head_decay` float32 [heads].  cos, sin
    float32 [positions, r / 2]: q and k are turned on their first r coordinates (pairs i, i + r / 2) by the tokens' positions,
    then multiplied by q_scale and k_scale.  state float32 [slots, heads, dim, vdim] is advanced in place (zeros where an
    entry's q_start is 0).  silu_inputs: the recurrence reads silu(q), silu(k) and silu(v).  Returns float32 [T, heads, vdim]."""
    _dev(proj, state, slots, decay, head_decay, cos, sin)
    T = proj.shape[0]
    q = _rows_of(proj, q_start, heads * dim, "q")
    k = _rows_of(proj, k_start, heads * dim, "k")
    v = _rows_of(proj, v_start, heads * vdim, "v")
    _need(0 < dim <= DECAY_SCAN_MAX_DIM, "the recurrence kernel takes up to %d key channels per head, got %d", DECAY_SCAN_MAX_DIM, dim)
    _need((decay is None) != (head_decay is None), "the decay comes per token and channel, or per head: exactly one of the two")
    if decay is not None:
        _f32(decay, (T, heads * dim), "decay")
    else:
        _f32(head_decay, (heads,), "head_decay")
    rot = 0
    if cos is not None:
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, r/2]")
        rot = 2 * cos.shape[1]
        _need(0 < rot <= dim, "the rotation covers %d coordinates of a head of %d", rot, dim)
        _need(step.max_kv_len <= cos.shape[0], "positions up to %d, tables for %d", step.max_kv_len, cos.shape[0])
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dim, vdim),
          "state must be contiguous float32 [slots, %d, %d, %d]", heads, dim, vdim)
    E = _step_entries(step, slots)
    out = torch.empty((T, heads, vdim), dtype=torch.float32, device=proj.device)
    lib = build.load("decay_scan")
    _check(lib.ga_decay_scan(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _i64(proj.stride(0)), _ptr(decay), _ptr(head_decay),
                             _ptr(cos), _ptr(sin), _i(rot), _f(q_scale), _f(k_scale), _ptr(state), _ptr(slots),
                             _ptr(step.cu_tokens), _ptr(step.q_start), _i(E), _i(heads), _i(dim), _i(vdim),
                             _i(1 if silu_inputs else 0), _stream()), "decay_scan")
    return out


def head_norm_gate(x, weight, eps, dtype, proj=None, gate_start=0, sigmoid_gate=False):
    """x float32 [T, heads, V] -> [T, heads * V] in `dtype`: every head's row divided by its root mean square, times weight
    [V] (None: no weight), times silu of the gate (its sigmoid where sigmoid_gate), the columns gate_start .. gate_start +
    heads * V of the float32 projection `proj` (None: no gate).  A norm over all heads together is the case heads = 1."""
    _dev(x, weight, proj)
    _need(x.dtype == torch.float32 and x.dim() == 3 and x.is_contiguous(), "x must be contiguous float32 [T, heads, V]")
    T, H, V = x.shape
    if weight is not None:
        _f32(weight, (V,), "weight")
    gate = None
    if proj is not None:
        _need(proj.shape[0] == T, "the gate has %d rows, x has %d", proj.shape[0], T)
        gate = _rows_of(proj, gate_start, H * V, "gate")
    out = torch.empty((T, H * V), dtype=dtype, device=x.device)
    lib = build.load("decay_scan")
    _check(lib.ga_head_norm_gate(_ptr(out), _ptr(x), _ptr(weight), _ptr(gate), _i64(proj.stride(0) if proj is not None else 0),
                                 _i64(T), _i(H), _i(V), _f(eps), _i(_is_bf16(dtype)), _i(1 if sigmoid_gate else 0),
                                 _stream()), "head_norm_gate")
    return out


POOLED_ATTENTION_MAX_DIM = 256


def _token_rows(t, width, name, dtype=None):
    """How many slots a paged tensor of `width` elements a slot holds (keys lie a slot a row; values transposed inside a page)."""
    _need(t is not None and t.is_contiguous() and t.numel() % width == 0 and (dtype is None or t.dtype == dtype),
          "%s must be contiguous%s and hold whole rows of %d", name, "" if dtype is None else " " + str(dtype), width)
    return t.numel() // width


def pooled_attention_prepare(proj, positions, cos, sin, slot_mapping, k_rows, v_rows, num_heads, num_kv_heads, dim, vdim, eps,
                             page_size, unit_norm=True, write=True):
    """Behind a float32 projection whose first columns are [q heads | k heads | v heads]: q and k turned by position on their
    first r coordinates (pairs 2i, 2i + 1; cos, sin float32 [positions, r / 2], None: no rotation), then divided by their
    root mean square per head (unit_norm); k and v are written into their pages (keys [page][slot][kv head][dim], values
    transposed inside a page [page][kv head][vdim][slot]; float32 or bfloat16) at slot_mapping.  Returns q float32 [T,
    num_heads * dim]."""
    _dev(proj, positions, cos, sin, slot_mapping, k_rows, v_rows)
    T = proj.shape[0]
    _rows_of(proj, 0, (num_heads + num_kv_heads) * dim + num_kv_heads * vdim, "q | k | v")
    _need(0 < dim <= POOLED_ATTENTION_MAX_DIM and 0 < vdim <= POOLED_ATTENTION_MAX_DIM, "heads of %d / %d are not supported: up to %d",
          dim, vdim, POOLED_ATTENTION_MAX_DIM)
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(), "positions must be contiguous int32 [T]")
    rot = 0
    if cos is not None:
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, r/2]")
        rot = 2 * cos.shape[1]
        _need(0 < rot <= dim, "the rotation covers %d coordinates of a head of %d", rot, dim)
    cache_bf16 = 0
    if write:
        _need(slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,) and slot_mapping.is_contiguous(),
              "slot_mapping must be contiguous int64 [T]")
        _need(k_rows.dtype == v_rows.dtype, "keys and values are cached in one number format")
        cache_bf16 = _is_bf16(k_rows.dtype)
        _need(_token_rows(k_rows, num_kv_heads * dim, "k_rows") == _token_rows(v_rows, num_kv_heads * vdim, "v_rows"),
              "keys and values must hold the same number of rows")
    q = torch.empty((T, num_heads * dim), dtype=torch.float32, device=proj.device)
    lib = build.load("pooled_attention")
    _check(lib.ga_pwa_prepare(_ptr(q), _ptr(proj), _i64(proj.stride(0)), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                              _ptr(k_rows), _ptr(v_rows), _i(T), _i(num_heads), _i(num_kv_heads), _i(dim), _i(vdim), _i(rot),
                              _i(1 if unit_norm else 0), _f(eps), _i(1 if write else 0), _i(page_size), _i(cache_bf16), _stream()),
           "pwa_prepare")
    return q


def pooled_attention_mfma_supported(dtype, cache_dtype, num_heads, num_kv_heads, dim, page_size):
    """Whether the matrix-core kernels take these sizes: bfloat16, at most 16 heads to a kv head, keys whose width is a
    multiple of 8 (a lane's 16 bytes), pages of a multiple of 8 tokens (8 consecutive tokens of a value column lie in one)."""
    return (dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 and num_heads // num_kv_heads <= 16 and dim % 8 == 0
            and page_size % 8 == 0)


def _table(t, entries, name):
    _need(t.dtype == torch.int32 and t.dim() == 2 and t.shape[0] == entries and t.shape[1] >= 1 and t.is_contiguous(),
          "%s must be contiguous int32 [%d, width]", name, entries)
    return t.shape[1]


def pooled_attention_pool(pk_rows, pv_rows, k_rows, v_rows, step, table, pool_slots, num_kv_heads, dim, vdim, pool, page_size):
    """For every token of the step that ends a block of `pool` positions: the means of the block's cached keys and values
    (read through the entries' block `table`) into the float32 pages pk_rows, pv_rows (laid out as the tokens' pages, a block for
    a token) at pool_slots[token] (-1: none)."""
    _dev(pk_rows, pv_rows, k_rows, v_rows, table, pool_slots)
    T = step.positions.shape[0]
    E = step.cu_tokens.shape[0] - 1
    width = _table(table, E, "table")
    _need(pool_slots.dtype == torch.int64 and pool_slots.shape == (T,) and pool_slots.is_contiguous(), "pool_slots must be contiguous int64 [T]")
    _need(step.token_entry.dtype == torch.int32 and step.token_entry.shape == (T,), "token_entry must be int32 [T]")
    _need(k_rows.dtype == v_rows.dtype, "keys and values are cached in one number format")
    _token_rows(k_rows, num_kv_heads * dim, "k_rows")
    _token_rows(v_rows, num_kv_heads * vdim, "v_rows")
    _token_rows(pk_rows, num_kv_heads * dim, "pk_rows", torch.float32)
    _token_rows(pv_rows, num_kv_heads * vdim, "pv_rows", torch.float32)
    _need(pool >= 1 and page_size >= 1, "pool and page_size must be positive")
    lib = build.load("pooled_attention")
    _check(lib.ga_pwa_pool(_ptr(pk_rows), _ptr(pv_rows), _ptr(k_rows), _ptr(v_rows), _ptr(step.positions), _ptr(step.token_entry),
                           _ptr(table), _i(width), _ptr(pool_slots), _i(T), _i(num_kv_heads), _i(dim), _i(vdim), _i(pool),
                           _i(page_size), _i(_is_bf16(k_rows.dtype)), _stream()), "pwa_pool")


def pooled_attention(q, k_rows, v_rows, pk_rows, pv_rows, step, table, pool_table, head_bias, num_heads, num_kv_heads, dim, vdim,
                     size, pool, page_size, scale, dtype, proj=None, gate_start=0):
    """q float32 [T, num_heads * dim]; k_rows, v_rows: the tokens' pages (keys [page][slot][kv head][dim], values [page][kv head][vdim]
    [slot]), pk_rows, pv_rows: the blocks' means, float32, laid out alike.  Token i sees the tokens j with 0 <= i - j < size and the
    means of the blocks of `pool` tokens that end before them; the weight of a key is sigmoid(scale q . k + head_bias[head]) (head_bias float32 [heads] or
    None), not normalised.  The result is multiplied by sigmoid of the gate, the columns gate_start .. of the float32 projection
    `proj` (None: no gate).  Returns [T, num_heads * vdim] in `dtype`."""
    _dev(q, k_rows, v_rows, pk_rows, pv_rows, table, pool_table, head_bias, proj)
    T = q.shape[0]
    _f32(q, (T, num_heads * dim), "q")
    E = step.cu_tokens.shape[0] - 1
    width, pool_width = _table(table, E, "table"), _table(pool_table, E, "pool_table")
    _need(num_heads % num_kv_heads == 0, "num_heads %d is not a multiple of num_kv_heads %d", num_heads, num_kv_heads)
    _need(0 < dim <= POOLED_ATTENTION_MAX_DIM and 0 < vdim <= POOLED_ATTENTION_MAX_DIM, "heads of %d / %d are not supported: up to %d",
          dim, vdim, POOLED_ATTENTION_MAX_DIM)
    _need(k_rows.dtype == v_rows.dtype, "keys and values are cached in one number format")
    _token_rows(k_rows, num_kv_heads * dim, "k_rows")
    _token_rows(v_rows, num_kv_heads * vdim, "v_rows")
    _token_rows(pk_rows, num_kv_heads * dim, "pk_rows", torch.float32)
    _token_rows(pv_rows, num_kv_heads * vdim, "pv_rows", torch.float32)
    for name, a in (("positions", step.positions), ("token_entry", step.token_entry)):
        _need(a.dtype == torch.int32 and a.shape == (T,) and a.is_contiguous(), "%s must be contiguous int32 [T]", name)
    if head_bias is not None:
        _f32(head_bias, (num_heads,), "head_bias")
    gate = None
    if proj is not None:
        _need(proj.shape[0] == T, "the gate has %d rows, q has %d", proj.shape[0], T)
        gate = _rows_of(proj, gate_start, num_heads * vdim, "gate")
    _need(size >= 1 and pool >= 1 and page_size >= 1, "size, pool and page_size must be positive")
    out = torch.empty((T, num_heads * vdim), dtype=dtype, device=q.device)
    lib = build.load("pooled_attention")
    if pooled_attention_mfma_supported(dtype, k_rows.dtype, num_heads, num_kv_heads, dim, page_size):
        # the matrix cores: prompt portions by the step's tiles of 16 rows, single tokens with a kv group's heads side by side
        plan = _attention_plan(step, PLAN_TILE_ROWS, q.device)
        n_tiles, n_single = plan["n_tiles"], plan["n_decode"]
        splits, partial = 1, None
        if n_single:
            # the longest walk in tiles of 32: the window and the blocks of the longest context of the step's bucket
            span = int(plan.get("decode_span") or step.max_kv_len)
            tiles = (min(size, span) + 31) // 32 + 1 + (span // pool + 31) // 32
            splits = max(1, min(tiles // TUNING.pooled_decode_tiles_per_split,
                                TUNING.pooled_decode_workgroups // max(n_single * num_kv_heads, 1), 64))
            if splits > 1:
                partial = torch.empty((splits, n_single, num_heads * vdim), dtype=torch.float32, device=q.device)
        _check(lib.ga_pwa_attend_mfma(_ptr(out), _ptr(partial), _ptr(q), _ptr(k_rows), _ptr(v_rows), _ptr(pk_rows), _ptr(pv_rows),
                                      _ptr(plan["tiles"]), _i(n_tiles), _ptr(plan["decode_info"]), _i(n_single), _i(splits),
                                      _ptr(table), _i(width), _ptr(pool_table), _i(pool_width), _ptr(head_bias), _ptr(gate),
                                      _i64(proj.stride(0) if proj is not None else 0), _i(num_heads), _i(num_kv_heads), _i(dim),
                                      _i(vdim), _i(size), _i(pool), _i(page_size), _f(scale), _stream()), "pwa_attend_mfma")
        return out
    _check(lib.ga_pwa_attend(_ptr(out), _ptr(q), _ptr(k_rows), _ptr(v_rows), _ptr(pk_rows), _ptr(pv_rows), _ptr(step.positions),
                             _ptr(step.token_entry), _ptr(table), _i(width), _ptr(pool_table), _i(pool_width), _ptr(head_bias),
                             _ptr(gate), _i64(proj.stride(0) if proj is not None else 0), _i(T), _i(num_heads), _i(num_kv_heads),
                             _i(dim), _i(vdim), _i(size), _i(pool), _i(page_size), _f(scale), _i(_is_bf16(k_rows.dtype)),
                             _i(_is_bf16(dtype)), _stream()), "pwa_attend")
    return out


def gated_residual_add(residual, z, y1, y2=None, next_gain=None, next_eps=0.0, dtype=None):
    """residual float32 [T, H] += sigmoid(z[:, :H]) * y1 (+ sigmoid(z[:, H:]) * y2), the gated results added to each other
    first; z float32 [T, H] or [T, 2H] (rows may have a stride: columns of a wider projection); y1, y2 [T, H] in float32 or
    bfloat16.  With next_gain (float32 [H]) the rows of the norm
    that is read next, rmsnorm(residual) * next_gain in `dtype`, come back; else None."""
    _dev(residual, z, y1, y2, next_gain)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(), "residual must be contiguous float32 [T, H]")
    T, H = residual.shape
    gates = 1 if y2 is None else 2
    _need(z.dtype == torch.float32 and tuple(z.shape) == (T, gates * H) and z.stride(1) == 1,
          "z must be float32 [%d, %d] with unit inner stride (it may be columns of a wider projection)", T, gates * H)
    for name, y in (("y1", y1), ("y2", y2)):
        _need(y is None or (y.shape == (T, H) and y.is_contiguous() and y.dtype == y1.dtype), "%s must be contiguous [%d, %d] in one dtype", name, T, H)
    nxt = None
    if next_gain is not None:
        _f32(next_gain, (H,), "next_gain")
        nxt = torch.empty((T, H), dtype=dtype, device=residual.device)
    lib = build.load("gated_residual")
    _check(lib.ga_gated_residual_add(_ptr(residual), _ptr(z), _i64(z.stride(0)), _ptr(y1), _ptr(y2), _i(T), _i(H), _i(_is_bf16(y1.dtype)),
                                     _ptr(next_gain), _f(next_eps), _ptr(nxt), _i(_is_bf16(dtype) if nxt is not None else 0),
                                     _stream()), "gated_residual_add")
    return nxt


# ---------------------------------------------------------------------------------------------------------------------
# hyper-connections: the residual stream as several streams side by side

HYPER_MAX_STREAMS = 16
HYPER_MAX_WIDTH = 15360          # a token's row of 32-bit sums lies in LDS


def _streams(X):
    _need(X.dtype == torch.float32 and X.dim() == 3 and X.is_contiguous(), "the streams must be contiguous float32 [T, S, W]")
    T, S, W = X.shape
    _need(1 <= S <= HYPER_MAX_STREAMS and 1 <= W <= HYPER_MAX_WIDTH, "1 to %d streams of up to %d channels, got %d of %d",
          HYPER_MAX_STREAMS, HYPER_MAX_WIDTH, S, W)
    return T, S, W


def hyper_open(x, streams):
    """x float32 [T, W] -> float32 [T, streams, W]: every stream a copy of x."""
    _dev(x)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "x must be contiguous float32 [T, W]")
    X = torch.empty((x.shape[0], int(streams), x.shape[1]), dtype=torch.float32, device=x.device)
    T, S, W = _streams(X)
    _check(build.load("hyper_connection").ga_hc_open(_ptr(X), _ptr(x), _i(T), _i(W), _i(S), _stream()), "hc_open")
    return X


def hyper_read(X, in_weights, gain, eps, dtype):
    """rows [T, W] in `dtype` = gain * u / sqrt(mean(u^2) + eps), u = sum_s in_weights[s] X[:, s]."""
    _dev(X, in_weights, gain)
    T, S, W = _streams(X)
    _f32(in_weights, (S,), "in_weights")
    _f32(gain, (W,), "gain")
    rows = torch.empty((T, W), dtype=dtype, device=X.device)
    _check(build.load("hyper_connection").ga_hc_read(_ptr(rows), _ptr(X), _ptr(in_weights), _ptr(gain), _f(eps), _i(T), _i(W), _i(S),
                                                     _i(_is_bf16(dtype)), _stream()), "hc_read")
    return rows


def hyper_write(X, mix, out_weights, y, next_in=None, next_gain=None, next_eps=0.0, dtype=None):
    """X[:, j] <- sum_s mix[s, j] X[:, s] + out_weights[j] * y for all j at once, in place.  y [T, W] in float32 or bfloat16, or
    float32 [parts, T, W] (partial sums, added in order).  With next_in (float32 [S]) and next_gain (float32 [W]) the rows that
    the sublayer which runs next reads of the new streams (`hyper_read`) come back in `dtype`; else None."""
    _dev(X, mix, out_weights, y, next_in, next_gain)
    T, S, W = _streams(X)
    _f32(mix, (S, S), "mix")
    _f32(out_weights, (S,), "out_weights")
    parts, part_stride = 1, 0
    if y.dim() == 3:
        _need(y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape[1:]) == (T, W), "partial sums must be contiguous float32 [parts, %d, %d]", T, W)
        parts, part_stride = y.shape[0], T * W
    else:
        _need(tuple(y.shape) == (T, W) and y.is_contiguous() and y.dtype in (torch.float32, torch.bfloat16),
              "y must be contiguous float32 or bfloat16 [%d, %d], got %s %s", T, W, y.dtype, tuple(y.shape))
    rows = None
    _need((next_in is None) == (next_gain is None), "the next sublayer's weights and its norm's gain come together")
    if next_in is not None:
        _f32(next_in, (S,), "next_in")
        _f32(next_gain, (W,), "next_gain")
        rows = torch.empty((T, W), dtype=dtype, device=X.device)
    _check(build.load("hyper_connection").ga_hc_write(
        _ptr(X), _ptr(mix), _ptr(out_weights), _ptr(y), _i(_is_bf16(y.dtype)), _i(parts), _i64(part_stride), _ptr(next_in),
        _ptr(next_gain), _f(next_eps), _ptr(rows), _i(_is_bf16(dtype) if rows is not None else 0), _i(T), _i(W), _i(S), _stream()),
        "hc_write")
    return rows


def hyper_sum(X, rows=None):
    """float32 [R, W]: the sum of the streams at the rows `rows` (int32 [R]; None: at every row)."""
    _dev(X, rows)
    T, S, W = _streams(X)
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be contiguous int32 [R]")
    R = T if rows is None else rows.shape[0]
    out = torch.empty((R, W), dtype=torch.float32, device=X.device)
    _check(build.load("hyper_connection").ga_hc_sum_rows(_ptr(out), _ptr(X), _ptr(rows), _i(R), _i(W), _i(S), _stream()), "hc_sum_rows")
    return out


# ---------------------------------------------------------------------------------------------------------------------
# the real-gated linear recurrent unit

RGLRU_MAX_BLOCK = 15360          # one token's channels of a block lie in LDS (narrower blocks: up to 16 tokens a thread)


def rglru_gates(u, ra_t, ra_bias, ri_t, ri_bias, lam, blocks, rate, y):
    """u float32 [T, C] -> (a, b, g) float32 [T, C]: per block of C / blocks channels r = sigmoid(Ra u + ra), i = sigmoid(Ri u +
    ri); a = exp(-rate * r * softplus(lam)); b = sqrt(1 - a^2) * i * u; g = gelu_tanh(y), y float32 [T, C] with unit inner
    stride (columns of a projection, before their activation).  ra_t, ri_t: the blocks' square matrices transposed, float32
    [blocks, in, out]; the biases and lam float32 [C]."""
    _dev(u, ra_t, ra_bias, ri_t, ri_bias, lam, y)
    _need(u.dtype == torch.float32 and u.dim() == 2 and u.is_contiguous(), "u must be contiguous float32 [T, C]")
    T, C = u.shape
    _need(blocks >= 1 and C % blocks == 0 and C // blocks <= RGLRU_MAX_BLOCK, "%d channels in %d blocks (a block may hold up to %d)",
          C, blocks, RGLRU_MAX_BLOCK)
    bw = C // blocks
    for name, t in (("ra_t", ra_t), ("ri_t", ri_t)):
        _f32(t, (blocks, bw, bw), name)
    for name, t in (("ra_bias", ra_bias), ("ri_bias", ri_bias), ("lam", lam)):
        _f32(t, (C,), name)
    _need(y.dtype == torch.float32 and tuple(y.shape) == (T, C) and y.stride(1) == 1, "y must be float32 [%d, %d] with unit inner stride", T, C)
    a, b, g = (torch.empty((T, C), dtype=torch.float32, device=u.device) for _ in range(3))
    _check(build.load("rglru").ga_rglru_gates(_ptr(a), _ptr(b), _ptr(u), _ptr(ra_t), _ptr(ra_bias), _ptr(ri_t), _ptr(ri_bias), _ptr(lam),
                                              _ptr(y), _i64(y.stride(0)), _ptr(g), _i(T), _i(C), _i(blocks), _f(rate), _stream()),
           "rglru_gates")
    return a, b, g


def rglru_scan(a, b, g, state, slots, step, dtype):
    """S_t = a_t S_(t-1) + b_t per channel over the step's entries, from the state float32 [slots, C] (zeros where an entry's
    q_start is 0), which moves on in place; returns S * g in `dtype`, [T, C].  a, b, g float32 [T, C]."""
    _dev(a, b, g, state, slots)
    _need(a.dtype == torch.float32 and a.dim() == 2 and a.is_contiguous(), "a must be contiguous float32 [T, C]")
    T, C = a.shape
    _f32(b, (T, C), "b")
    _f32(g, (T, C), "g")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == C and state.is_contiguous(),
          "state must be contiguous float32 [slots, %d]", C)
    E = _step_entries(step, slots)
    _need(E <= 65535, "too many entries for one launch: %d", E)
    out = torch.empty((T, C), dtype=dtype, device=a.device)
    _check(build.load("rglru").ga_rglru_scan(_ptr(out), _ptr(a), _ptr(b), _ptr(g), _ptr(state), _ptr(slots), _ptr(step.cu_tokens),
                                             _ptr(step.q_start), _i(E), _i(T), _i(C), _i(_is_bf16(dtype)), _stream()),
           "rglru_scan")
    return out
