"""Python faces of the HIP kernels: each checks its operands on the host (device, dtype, shape,
contiguity) and launches on torch's current stream.  Tensors are torch tensors used as plain
device memory; no torch arithmetic happens here.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

from functools import lru_cache
from typing import Optional

import torch

from . import library

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "gi_embed": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gi_embed_handing": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "gi_rmsnorm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_long, c_long, c_void_p],
    "gi_rope_cos_sin": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gi_rope_store": [c_void_p, c_void_p, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_int, c_void_p, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gi_silu_mul": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "gi_gather_rows": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gi_scale_rows": [c_void_p, c_int, c_int, c_long, c_float, c_void_p],
    "gi_softcap_rows": [c_void_p, c_int, c_int, c_long, c_float, c_void_p],
    "gi_gemm_exact": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gi_attention_exact": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "gi_gemm_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p, c_long, c_void_p],
    "gi_attention_prompt_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_void_p, c_void_p, c_int, c_void_p, c_long, c_void_p],
    "gi_attention_decode_bf16": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_long, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_long, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_int, c_void_p],
    "gi_random_normal": [c_void_p, c_int, c_long, ctypes.c_ulonglong, ctypes.c_double, ctypes.c_double, c_void_p],
    "gi_probe_stream": [c_void_p, c_void_p, c_long, c_void_p, c_int, c_int, c_void_p],
    "gi_probe_mfma": [c_int, c_void_p, c_int, c_void_p],
    "gi_gemm_bf16_handing": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p, c_long,
                             c_void_p, c_int, c_float, c_void_p, c_void_p, c_long, c_void_p, c_void_p],
    "gi_gemm_bf16_qkv_rope_store": [c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p],
    "gi_argmax": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
    "gi_sample_temperature": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
    "gi_sample_filtered": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        l = library.load()
        for name, sig in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = sig
            fn.restype = c_int
        l.gi_argmax_chunks.argtypes = [c_int]
        l.gi_argmax_chunks.restype = c_int
        l.gi_sample_filtered_histogram_bytes.argtypes = []
        l.gi_sample_filtered_histogram_bytes.restype = c_int
        l.gi_attention_exact_max_head_size.argtypes = []
        l.gi_attention_exact_max_head_size.restype = c_int
        l.gi_attention_decode_workgroups_per_unit.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_attention_decode_workgroups_per_unit.restype = c_int
        l.gi_attention_bf16_supports.argtypes = [c_int, c_int, c_int]
        l.gi_attention_bf16_supports.restype = c_int
        l.gi_gemm_bf16_scratch_floats.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_scratch_floats.restype = c_long
        l.gi_gemm_bf16_norm_parts.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_norm_parts.restype = c_int
        l.gi_gemm_bf16_takes_norm.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_gemm_bf16_takes_norm.restype = c_int
        l.gi_gemm_bf16_qkv_rope_store_takes.argtypes = [c_int, c_int, c_int, c_int]
        l.gi_gemm_bf16_qkv_rope_store_takes.restype = c_int
        l.gi_compute_units.argtypes = []
        l.gi_compute_units.restype = c_int
        l.gi_gemm_bf16_qkv_rope_store_max_parts.argtypes = [c_int, c_int, c_int]
        l.gi_gemm_bf16_qkv_rope_store_max_parts.restype = c_int
        l.gi_probe_mfma_flops.argtypes = [c_int, c_int]
        l.gi_probe_mfma_flops.restype = c_long
        _lib = l
    return _lib


_FUNCTIONS = {}


def _call(name, *args):
    fn = _FUNCTIONS.get(name)
    if fn is None:
        fn = _FUNCTIONS[name] = getattr(lib(), name)
    if _profile is not None:
        return _profile.timed(name, fn, args)
    if fn(*args) != 0:
        raise KernelError(lib().gi_last_error().decode())


_PROFILE_LABEL = {"gi_gemm_bf16_handing": "gemm_bf16", "gi_gemm_bf16_qkv_rope_store": "gemm_bf16"}        # the same products, with a norm's share on top


class KernelProfile:
    """Time per kernel entry point, with the device waited for before and after every call (so the times add up, and
    a step takes longer than it does unobserved).  What the reference's device model reports with --profile
    (src/gpu/gpu_transformer.cpp:178-224), by entry point and weight shape instead of a fixed list of sections.
    Matrix products are kept apart by the weight's shape, which tells the projections from one another, and count the
    weight bytes they read."""

    def __init__(self):
        self.seconds, self.calls, self.weight_bytes = {}, {}, {}
        self.note = None                        # (label suffix, weight bytes) of the product about to be launched

    def timed(self, name, fn, args):
        import time
        label, nbytes = _PROFILE_LABEL.get(name, name[3:]), 0
        if self.note is not None:
            label, nbytes = f"{label} {self.note[0]}", self.note[1]
            self.note = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rc = fn(*args)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if rc != 0:
            raise KernelError(lib().gi_last_error().decode())
        self.seconds[label] = self.seconds.get(label, 0.0) + dt
        self.calls[label] = self.calls.get(label, 0) + 1
        self.weight_bytes[label] = self.weight_bytes.get(label, 0) + nbytes

    def report(self, positions: int, steps: int, wall_seconds: float) -> str:
        if not self.seconds or positions <= 0:
            return ""
        inside = sum(self.seconds.values())
        lines = [f"device profile: {positions} positions in {steps} steps, {wall_seconds * 1e3 / positions:.3f} ms per position "
                 "(the device waits before and after every kernel)",
                 f"  {'kernel':<34} {'calls':>8} {'ms/position':>12} {'share':>7} {'weights GB/s':>13}"]
        for label in sorted(self.seconds, key=self.seconds.get, reverse=True):
            sec, nbytes = self.seconds[label], self.weight_bytes[label]
            rate = f"{nbytes / sec / 1e9:.1f}" if nbytes and sec > 0 else ""
            lines.append(f"  {label:<34} {self.calls[label]:>8} {sec * 1e3 / positions:>12.4f} {100 * sec / wall_seconds:>6.1f}% {rate:>13}")
        rest = max(wall_seconds - inside, 0.0)
        lines.append(f"  {'host work, uploads, downloads':<34} {'':>8} {rest * 1e3 / positions:>12.4f} {100 * rest / wall_seconds:>6.1f}%")
        return "\n".join(lines) + "\n"


_profile: Optional[KernelProfile] = None


def set_profiling(on: bool) -> Optional[KernelProfile]:
    """Switches the per-kernel timing on (a fresh KernelProfile, which is returned) or off.  While it is on, steps are
    not replayed from captured graphs: a replay has no kernel boundaries to wait at."""
    global _profile
    _profile = KernelProfile() if on else None
    return _profile


def profiling() -> bool:
    return _profile is not None


# The current stream's handle, asked for at every launch (it changes under graph capture).  torch's
# public way costs several microseconds a call, and a step makes over a hundred launches.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what} has dtype {t.dtype}; float32 or bfloat16 is needed") from None


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must lie in device memory")


def _i32(t, what, n=None):
    if not (t.dtype == torch.int32 and t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous int32 tensor")
    if n is not None:
        if not (t.numel() >= n):
            raise KernelError(f"{what} holds {t.numel()} entries, {n} are needed")


def _ptr(t):
    return None if t is None else t.data_ptr()


def device_arch() -> str:
    buf = ctypes.create_string_buffer(64)
    l = lib()
    if l.gi_device_arch(buf, 64) != 0:
        raise KernelError(l.gi_last_error().decode())
    return buf.value.decode()


# ------------------------------------------------------------------------------------------------
def embed(table, tokens, out):
    """out[t, :] = table[tokens[t], :] widened to float32."""
    _dev(table, tokens, out)
    n, dim = out.shape
    if not (table.dim() == 2 and table.shape[1] == dim and table.is_contiguous()):
        raise KernelError("embed: table must be [vocab, dim], contiguous")
    if not (out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("embed: out must be contiguous float32")
    _i32(tokens, "embed: tokens", n)
    _call("gi_embed", table.data_ptr(), _code(table, "embed: table"), tokens.data_ptr(), out.data_ptr(), n, dim, _stream())
    return out


def embed_handing(table, tokens, out, g, scaled, squares):
    """`embed`, and on the way the first half of an RMS norm of the rows for a product that finishes it (`gemm_bf16(..., norm_in=...)`):
    scaled = bfloat16(g * out) and squares [n, 1] = the rows' sums of out^2."""
    _dev(table, tokens, out, g, scaled, squares)
    n, dim = out.shape
    if not (table.dim() == 2 and table.shape[1] == dim and table.is_contiguous() and out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("embed: table must be [vocab, dim], contiguous, and out contiguous float32")
    if not (g.dtype == torch.float32 and g.is_contiguous() and g.numel() == dim and scaled.dtype == torch.bfloat16 and scaled.shape == (n, dim)
            and scaled.is_contiguous() and squares.dtype == torch.float32 and squares.is_contiguous() and squares.shape == (n, 1)):
        raise KernelError("embed: handing a norm on needs float32 weights [dim], bfloat16 [n, dim] for the scaled rows and float32 [n, 1] for the sums of squares")
    _i32(tokens, "embed: tokens", n)
    _call("gi_embed_handing", table.data_ptr(), _code(table, "embed: table"), tokens.data_ptr(), out.data_ptr(), n, dim, g.data_ptr(), scaled.data_ptr(),
          squares.data_ptr(), _stream())
    return out


def rmsnorm_can_gather(x, weight, out) -> bool:
    dim = x.shape[1]
    return (dim % 4 == 0 and dim <= 4096 and x.stride(0) % 4 == 0 and out.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0
            and weight.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0)


def rmsnorm(x, weight, eps, out, rows=None):
    """out = weight * (x * rsqrt(mean(x^2) + eps)) per row; x float32 [n, dim].  rows: int32 indices, out[i] = norm(x[rows[i]])."""
    _dev(x, weight, out, rows)
    dim = x.shape[1]
    n = x.shape[0] if rows is None else rows.numel()
    if not (x.dtype == torch.float32 and x.stride(1) == 1):
        raise KernelError("rmsnorm: x must be float32 with unit inner stride")
    if not (out.shape == (n, dim) and out.stride(1) == 1):
        raise KernelError("rmsnorm: out must be [rows, dim] with unit inner stride")
    if not (weight.shape == (dim,) and weight.is_contiguous()):
        raise KernelError("rmsnorm: weight must be [dim]")
    if rows is not None:
        _i32(rows, "rmsnorm: rows", n)
        if not (rmsnorm_can_gather(x, weight, out)):
            raise KernelError("rmsnorm: these operands cannot be gathered in the kernel")
    _call("gi_rmsnorm", x.data_ptr(), _ptr(rows), weight.data_ptr(), _code(weight, "rmsnorm: weight"), out.data_ptr(), _code(out, "rmsnorm: out"),
          n, dim, float(eps), x.stride(0), out.stride(0), _stream())
    return out


def rope_cos_sin(positions, inv_freq, cos_out, sin_out):
    """cos/sin of positions[t] * inv_freq[k] with 64-bit angles; outputs float32 [n, half]."""
    _dev(positions, inv_freq, cos_out, sin_out)
    n, half = cos_out.shape
    _i32(positions, "rope_cos_sin: positions", n)
    if not (inv_freq.dtype == torch.float64 and inv_freq.shape == (half,) and inv_freq.is_contiguous()):
        raise KernelError("rope_cos_sin: inv_freq must be float64 [half]")
    for t in (cos_out, sin_out):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.shape == (n, half)):
            raise KernelError("rope_cos_sin: outputs must be float32 [n, half]")
    _call("gi_rope_cos_sin", positions.data_ptr(), inv_freq.data_ptr(), cos_out.data_ptr(), sin_out.data_ptr(), n, half, _stream())


def _check_cache(cache, table, page_size, n_kv, hd, what):
    # the last two axes of the value half hold [hd][place]: values are stored transposed
    if not (cache.dim() == 5 and tuple(cache.shape[1:]) == (2, n_kv, page_size, hd) and cache.is_contiguous()):
        raise KernelError( f"{what}: the cache must be [pages, 2, {n_kv}, {page_size}, {hd}], contiguous; it is {tuple(cache.shape)}")
    if not (table.dim() == 2 and table.dtype == torch.int32 and table.stride(1) == 1):
        raise KernelError(f"{what}: the page table must be int32 [slots, pages]")


def rope_store(q, k, v, cos, sin, positions, slots, table, q_out, cache, n_heads, n_kv, hd):
    """Rotates q into q_out and, if k is given, rotates k and writes k and v into the cache pages.
    q, k, v are float32 views [n, heads*hd] with unit inner stride (columns of one product are fine)."""
    _dev(q, k, v, cos, sin, positions, slots, table, q_out, cache)
    n = q.shape[0]
    if not (q.dtype == torch.float32 and q.shape[1] == n_heads * hd and q.stride(1) == 1):
        raise KernelError("rope_store: q must be float32 [n, heads*hd]")
    if not (q_out.shape == (n, n_heads * hd) and q_out.is_contiguous()):
        raise KernelError("rope_store: q_out must be [n, heads*hd], contiguous")
    if cos is not None:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (n, hd // 2) and t.is_contiguous()):
                raise KernelError("rope_store: cos/sin must be float32 [n, hd/2]")
    page_size = page_stride = 0
    cache_code = _code(q_out, "rope_store: q_out")
    if k is not None:
        for t, name in ((k, "k"), (v, "v")):
            if not (t.dtype == torch.float32 and t.shape == (n, n_kv * hd) and t.stride(1) == 1):
                raise KernelError(f"rope_store: {name} must be float32 [n, kv_heads*hd]")
        page_size = cache.shape[3]
        _check_cache(cache, table, page_size, n_kv, hd, "rope_store")
        page_stride = cache.stride(0)
        cache_code = _code(cache, "rope_store: cache")
        _i32(positions, "rope_store: positions", n)
        _i32(slots, "rope_store: slots", n)
    _call("gi_rope_store", q.data_ptr(), _ptr(k), _ptr(v), q.stride(0), k.stride(0) if k is not None else 0,
          v.stride(0) if v is not None else 0, _ptr(cos), _ptr(sin), _ptr(positions), _ptr(slots),
          _ptr(table) if k is not None else None, table.stride(0) if k is not None else 0, q_out.data_ptr(),
          _code(q_out, "rope_store: q_out"), _ptr(cache) if k is not None else None, cache_code, page_stride, page_size,
          n, n_heads, n_kv, hd, _stream())


def silu_mul(gate_up, out):
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, inter + i]."""
    _dev(gate_up, out)
    n, inter = out.shape
    if not (gate_up.dtype == torch.float32 and gate_up.shape == (n, 2 * inter) and gate_up.is_contiguous()):
        raise KernelError("silu_mul: gate_up must be float32 [n, 2*inter]")
    if not (out.is_contiguous()):
        raise KernelError("silu_mul: out must be contiguous")
    _call("gi_silu_mul", gate_up.data_ptr(), out.data_ptr(), _code(out, "silu_mul: out"), n, inter, _stream())
    return out


def gather_rows(x, rows, out):
    _dev(x, rows, out)
    k, dim = out.shape
    if not (x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == dim):
        raise KernelError("gather_rows: x must be contiguous float32 [n, dim]")
    if not (out.dtype == torch.float32 and out.is_contiguous()):
        raise KernelError("gather_rows: out must be contiguous float32")
    _i32(rows, "gather_rows: rows", k)
    _call("gi_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(), k, dim, _stream())
    return out


def _rows_in_place(name, x, c):
    _dev(x)
    if not (x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1):
        raise KernelError(f"{name}: x must be float32 [n, dim] with unit inner stride")
    _call("gi_" + name, x.data_ptr(), x.shape[0], x.shape[1], x.stride(0), float(c), _stream())
    return x


def scale_rows(x, factor):
    """x *= factor, in place."""
    return _rows_in_place("scale_rows", x, factor)


def softcap_rows(x, cap):
    """x = cap * tanh(x / cap), in place."""
    return _rows_in_place("softcap_rows", x, cap)


def random_normal(out, key: int, offset: float, scale: float):
    """out[i] = offset + scale * z_i, z_i the standard normal number that (key, i) give (`weights.random_init` states the formula);
    out is a contiguous float32 or bfloat16 tensor of any shape, filled in the order of its memory."""
    _dev(out)
    if not out.is_contiguous():
        raise KernelError("random_normal: out must be contiguous")
    _call("gi_random_normal", out.data_ptr(), _code(out, "random_normal: out"), out.numel(), int(key) & 0xFFFFFFFFFFFFFFFF, float(offset), float(scale), _stream())
    return out


def gemm_exact(a, w, out, accumulate=False):
    """out (=|+=) a @ w.T in 32-bit arithmetic with one summation order for every batch size."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    if not (w.shape == (n, k)):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, activations are {tuple(a.shape)}")
    if not (out.shape == (m, n)):
        raise KernelError(f"gemm: out is {tuple(out.shape)}, ({m}, {n}) is needed")
    if not (a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1):
        raise KernelError("gemm: operands need unit inner stride")
    if _profile is not None:
        _profile.note = (f"{n}x{k}", n * k * w.element_size())
    _call("gi_gemm_exact", a.data_ptr(), _code(a, "gemm: a"), w.data_ptr(), _code(w, "gemm: w"), out.data_ptr(), _code(out, "gemm: out"),
          1 if accumulate else 0, m, n, k, a.stride(0), w.stride(0), out.stride(0), _stream())
    return out


def attention_max_head_size() -> int:
    """The largest head the attention kernels take (the exact kernel's limit; the matrix-core kernels take fewer sizes and
    leave the others to it)."""
    return lib().gi_attention_exact_max_head_size()


def attention_exact(q, cache, out, positions, slots, table, n_heads, n_kv, hd, window=None, scale=None):
    """Each row attends over its request's cached keys up to its own position."""
    _dev(q, cache, out, positions, slots, table)
    n = q.shape[0]
    if not (q.shape == (n, n_heads * hd) and q.is_contiguous() and out.shape == q.shape and out.is_contiguous()):
        raise KernelError( "attention: q and out must be [n, heads*hd], contiguous")
    page_size = cache.shape[3]
    _check_cache(cache, table, page_size, n_kv, hd, "attention")
    _i32(positions, "attention: positions", n)
    _i32(slots, "attention: slots", n)
    _call("gi_attention_exact", q.data_ptr(), _code(q, "attention: q"), cache.data_ptr(), _code(cache, "attention: cache"), out.data_ptr(),
          _code(out, "attention: out"), positions.data_ptr(), slots.data_ptr(), table.data_ptr(), table.stride(0), cache.stride(0),
          page_size, n, n_heads, n_kv, hd, int(window or 0), float(scale if scale is not None else hd ** -0.5), _stream())
    return out


class AttentionPlan:
    """How a step's rows are shared between the two bfloat16 attention kernels: requests that bring
    one row go to the decode kernel, portions of prompts are cut into tiles of up to 128 rows for
    the prompt kernel.  Short portions go to the decode kernel too, row by row (every row attends
    over its own prefix, which the cache holds by then): a tile's workgroup walks the whole context
    in sequence, however few its rows, while the decode kernel cuts each row's context into pieces
    for the whole chip (break-even near 90 rows at the Llama-3.2-1B shape; above SHORT_TOTAL rows
    in all, the rows' repeated reading of the context costs more than the tiles' sequence).
    Made once per step and used by every layer."""
    TILE = 0                             # rows of a prompt tile, 64 or 128; 0: by the step's size
    SMALL_STEP = 768                     # up to this many tiled rows in a step, tiles of 64 rows fill the chip better (measured at 32 heads)
    PAIRS = True                         # a portion's late tiles share workgroups with its early ones
    SHORT, SHORT_TOTAL = 64, 64          # portions of up to SHORT rows count as short; they go row by row while they sum to at most SHORT_TOTAL

    @classmethod
    def all_decode(cls, n_rows, max_context, device):
        """Every row is a request's single new row (what a captured decode step uses: nothing in it depends on the step)."""
        plan = cls.__new__(cls)
        plan.n_decode, plan.n_tiles, plan.max_decode_context, plan.single_rows = n_rows, 0, max_context, True
        plan.decode_rows = None                                  # rows 0 .. n_rows-1
        plan.tiles = torch.empty(0, dtype=torch.int32, device=device)
        plan.n_tile_rows, plan.max_tile_context, plan.tile_first, plan.tile_rows, plan.paired, plan.tile = 0, 0, None, None, False, 128
        return plan

    def __init__(self, seg_start, seg_len, seg_pos0, seg_slot, device, to_device=None):
        dec, tiles, portions, self.max_decode_context = [], [], [], 0
        short_rows = sum(n for n in seg_len if 1 < n <= self.SHORT)
        row_by_row = self.SHORT if short_rows <= self.SHORT_TOTAL else 1
        self.single_rows = all(n == 1 for n in seg_len)          # every row is a request's only new row
        self.tile = self.TILE or (64 if sum(n for n in seg_len if n > row_by_row) <= self.SMALL_STEP else 128)
        for start, n, pos0, slot in zip(seg_start, seg_len, seg_pos0, seg_slot):
            if n <= row_by_row:
                dec.extend(range(start, start + n))
                self.max_decode_context = max(self.max_decode_context, pos0 + n)
            else:
                portions.append([(start + off, min(self.tile, n - off), pos0 + off, slot) for off in range(0, n, self.tile)])
        # Tile i of a portion sees the keys of the tiles before it: the last tile goes with the first, the last but
        # one with the second, ... so that every pair has about the same number of keys to visit and reads them once
        # for both (a tile of no rows fills the middle pair of an odd number).  Without a portion of two tiles, no pairs.
        self.paired = self.PAIRS and any(len(p) > 1 for p in portions)
        for p in portions:
            if not self.paired:
                tiles.extend(p)
                continue
            for i in range((len(p) + 1) // 2):
                late, early = p[len(p) - 1 - i], p[i]
                tiles.extend((late, early if early is not late else (late[0], 0, late[2], late[3])))
        self.n_decode, self.n_tiles = len(dec), len(tiles)
        self.n_tile_rows = sum(t[1] for t in tiles)
        self.max_tile_context = max((t[2] + t[1] for t in tiles), default=0)
        # for sharing a tile's keys out over workgroups: rows before each tile, and the tiles' rows in order
        firsts, count = [], 0
        for t in tiles:
            firsts.append(count)
            count += t[1]
        put = to_device if to_device is not None else (lambda *lists: tuple(torch.tensor(values, dtype=torch.int32).to(device) for values in lists))
        self.decode_rows = self.tile_first = self.tile_rows = None      # no prompt rows: the decode rows are all rows, in order
        self.tiles = torch.empty(0, dtype=torch.int32, device=device)
        if tiles:                            # (every piece starts at a multiple of 16 bytes: the kernel reads a tile's four numbers at once)
            self.tiles, self.tile_first, self.tile_rows, *rest = put([v for t in tiles for v in t], firsts, [r for t in tiles for r in range(t[0], t[0] + t[1])],
                                                                     *([dec] if dec else []))
            self.decode_rows = rest[0] if rest else None


@lru_cache(maxsize=None)
def attention_bf16_supports(hd, page_size, prompt: bool) -> bool:
    return bool(lib().gi_attention_bf16_supports(hd, page_size, 1 if prompt else 0))


PAIRED_TARGET_GROUPS = 256


def prompt_attention_splits(n_groups, n_heads, span, target_groups=512):
    """Workgroups the keys of a tile (or pair of tiles) are shared out over: none while the tiles alone fill the chip
    (two workgroups a compute unit) or the context is short; every share keeps at least 256 keys."""
    groups = n_groups * n_heads
    if groups >= target_groups // 2:
        return 1
    return max(1, min(-(-target_groups // groups), span // 256, 64))


def _decode_piece(span, n_pieces):
    """Positions a wave of the decode kernel takes when a context of `span` is cut into `n_pieces` (multiples of 32, as the kernel cuts)."""
    return (-(-span // n_pieces) + 31) & ~31


@lru_cache(maxsize=None)
def _decode_places(hd, fused, n_waves, gh):
    """Workgroups of `n_waves` waves of the decode kernel that the chip holds at once."""
    per_unit = lib().gi_attention_decode_workgroups_per_unit(hd, 1 if fused else 0, n_waves, gh)
    return lib().gi_compute_units() * (per_unit if per_unit > 0 else max(1, 16 // n_waves))


def _decode_plain_shape(groups, span, max_waves, target_waves=4096, small=False):
    """About `target_waves` waves in all, pieces of at least 64 positions; one split when a workgroup's waves cover them.
    small (a few rows, heads of up to 64 channels, the kernel with rotation inside): pieces down to 32 positions, and workgroups
    of 8 waves while there are few of them (up to 64 groups of heads: half the partial results for the second kernel to merge)."""
    if small:
        target_waves //= 2          # (its waves ask for the next keys while they multiply: half as many, twice as long, measured faster at 4 to 12 rows)
    pieces = max(1, min(-(-target_waves // groups), -(-span // (32 if small else 64))))
    if pieces <= max_waves:
        return (1, pieces)
    n_waves = min(8 if small and groups <= 64 else 4, max_waves)
    return (min(-(-pieces // n_waves), 256), n_waves)


# What the decode kernel's workgroups reach (measured at heads of 64 and 128 channels, 17 to 128 rows, contexts of 1,100 to
# 16,384): a compute unit pulls about 31 GB/s for one workgroup and 27 GB/s for several, however many waves they have (from
# four up), the chip 5.9 TB/s, and a second kernel that merges splits costs about 6 us with the partial results it reads.
_DECODE_UNIT_MB_PER_S, _DECODE_SHARED_UNIT_MB_PER_S, _DECODE_CHIP_MB_PER_S, _DECODE_MERGE_US = 31e3, 27e3, 5.9e6, 6.0


def _decode_single_split(groups, span, hd, max_waves):
    """(1, waves) if one workgroup per (row, group of heads) over the whole context, which needs no second kernel, is expected
    to be no slower than a context cut over several; else None.  Without splits the compute unit with the most workgroups sets
    the time (`groups` over the units, rounded up, each pulling its share of the bytes at a unit's rate); with them the chip's
    rate does, plus the merge.  Of a bracket of contexts three quarters are taken as read.  Four waves where a wave's share
    stays under 200 KB and there is a workgroup for every unit, else eight."""
    units = lib().gi_compute_units()
    mbytes = groups * 0.75 * span * hd * 4 / 1e6
    most = -(-groups // units)                       # workgroups of the busiest compute unit
    single_us = max(most * (mbytes / groups) / (_DECODE_UNIT_MB_PER_S if most == 1 else _DECODE_SHARED_UNIT_MB_PER_S), mbytes / _DECODE_CHIP_MB_PER_S) * 1e6
    if groups < units // 2 or single_us > mbytes / _DECODE_CHIP_MB_PER_S * 1e6 + _DECODE_MERGE_US:
        return None
    n_waves = 8 if groups < units or 0.75 * span / 4 * hd * 4 > 200e3 else 4
    return (1, min(n_waves, max_waves))


@lru_cache(maxsize=None)
def decode_attention_shape(n_decode, n_heads, n_kv, hd, span, target_waves=4096, fused=False):
    """(splits, waves per workgroup) of the decode kernel: about `target_waves` waves in all and pieces of
    at least 64 positions; a single split (no combine kernel) when a workgroup's waves cover them.

    The chip holds so many workgroups of the kernel at once (the runtime's answer for this head size: 16 waves a compute
    unit at 64 channels, 12 at 128); workgroups beyond that run as a further round, and a round with a few workgroups in it
    costs as much as a full one (65 requests of 8 key/value heads: 520 workgroups of 8 waves on 512 places took 73 us a layer
    against 50 at 64).  So where the plain rule leaves a last round less than half full (less than a third where it has one
    split: there is no combine kernel to save then, and fewer pieces mean longer waves), or workgroups of 5 to 7 waves (which
    measured slower than either neighbour), the context is cut into as many pieces as fit in one round instead, in workgroups
    of 8 or 4 waves (of 3 or 2 where those leave fewer than 6 pieces), with as few splits as that allows: 65 rows 73 -> 57 us a layer, 96 rows 90 -> 74, 40 rows 46 -> 38,
    56 rows 2.10 -> 1.92 ms a step (heads of 64 channels); 65 rows 127 -> 111 us (heads of 128).  The small batches whose kernel
    also rotates and stores the new key keep the plain rule at heads of 64 channels: their workgroups are short, and 8 and 16 rows
    measured 5 and 3 % slower with one round.  What helps them is more and shorter pieces in fewer, larger workgroups (`small` in
    `_decode_plain_shape`; attention and combine kernel together, context 2,100: 1 row 11.4 -> 9.9 us a layer, 4 rows 13.8 -> 12.2,
    6 rows 15.8 -> 14.8, 8 rows 17.5 -> 17.0; context 1,100: 8 rows 12.9 -> 11.8).  At 128 channels that kernel's registers leave room for 8 waves a compute unit, and
    there one round is the faster cut whenever the plain rule needs more (8 rows: 30 -> 27 us a layer at a context of 2,100, 35 ->
    29 at 3,000; the step of the 8B shape 4.82 -> 4.79 ms at 8 rows, 5.47 -> 5.31 at 16).

    Since the kernel's waves ask for the next keys while they multiply (page numbers through the scalar unit, no wait for loads
    that are not needed yet), a wave is cheap to run for long, and from 17 rows on a context that is not cut at all is often the
    faster one: no partial results, no second kernel (`_decode_single_split` says when: 24 rows 27 -> 21 us a layer at a context
    of 2,100, 32 rows 31 -> 25, 64 rows 50 -> 47 with four waves instead of eight, 96 rows 76 -> 69; 24 rows at heads of 128
    channels 48 -> 38).  The rules above decide the rest."""
    group = n_heads // n_kv
    groups = n_decode * n_kv * ((group + 15) // 16)
    max_waves = min(8, lib().gi_attention_decode_max_waves(hd))
    base = _decode_plain_shape(groups, span, max_waves, target_waves, small=fused and hd <= 64)
    if target_waves != 4096:
        return base
    if not fused or n_decode > 16:                   # (more than 16 rows: whichever kernel serves them)
        single = _decode_single_split(groups, span, hd, max_waves)
        if single is not None:
            return single
    if fused and hd < 128:
        return base
    gh = min(group, 16)
    units = lib().gi_compute_units()
    places = lambda n_waves: min(_decode_places(hd, fused, n_waves, gh), units) if fused else _decode_places(hd, fused, n_waves, gh)
    rounds = groups * base[0] / places(base[1])
    if fused:                        # (heads of 128 channels: 8 waves a compute unit, and a second round costs what it brings; with the
        if rounds <= 1:              # waves asking ahead, a workgroup for every compute unit is enough: 4 rows 17.2 -> 14.7 us a layer)
            return base
    else:
        short_last_round = rounds > 1 and 0 < rounds - int(rounds) < (0.5 if base[0] > 1 else 0.3)
        if not (short_last_round or 5 <= base[1] <= 7):
            return base
    def most_pieces(widths):
        best = None
        for n_waves in widths:
            if n_waves > max_waves:
                continue
            splits = min(places(n_waves) // groups, 256)         # as many as still fit in one round
            while splits > 1 and _decode_piece(span, splits * n_waves) < 64:
                splits -= 1
            if splits >= 1 and (best is None or splits * n_waves > best[0] * best[1] or (splits * n_waves == best[0] * best[1] and splits < best[0])):
                best = (splits, n_waves)
        return best
    best = most_pieces((8, 4))
    if best is None or best[0] * best[1] < 6:        # narrow workgroups only where wide ones leave few pieces: many small ones run slower than the same pieces in wide ones
        best = most_pieces((8, 4, 3, 2))
    return best or base


def attention_bf16(q, cache, out, plan: AttentionPlan, positions, slots, table, n_heads, n_kv, hd, window=None, scale=None,
                   target_waves: int = 4096, products=None):
    """Attention of a step's rows with the matrix-core kernels (bfloat16 cache and out).

    `q` holds the rotated queries in bfloat16 and the cache the rows' keys and values; or, for a step
    of single decoded rows only, `q` is None and `products = (q, k, v, cos, sin)` holds the unrotated
    float32 products and the rotation's tables (k, v None: the pages are another layer's; cos, sin
    None: no rotation): the decode kernel then rotates, writes the cache and attends in one launch."""
    n = out.shape[0]
    _dev(q, cache, out, positions, slots, table)
    for t, name in ((q, "q"), (cache, "cache"), (out, "out")):
        if not (t is None or t.dtype == torch.bfloat16):
            raise KernelError(f"attention_bf16: {name} must be bfloat16")
    if not (out.shape == (n, n_heads * hd) and out.is_contiguous() and (q is None or (q.shape == out.shape and q.is_contiguous()))):
        raise KernelError( "attention: q and out must be [n, heads*hd], contiguous")
    page_size = cache.shape[3]
    _check_cache(cache, table, page_size, n_kv, hd, "attention")
    _i32(positions, "attention: positions", n)
    _i32(slots, "attention: slots", n)
    window = int(window or 0)
    scale = float(scale if scale is not None else hd ** -0.5)
    if not ((q is None) != (products is None)):
        raise KernelError("attention_bf16: give rotated queries or the unrotated products")
    qf = kf = vf = cos = sin = None
    if products is not None:
        if not (plan.n_tiles == 0):
            raise KernelError("attention_bf16: unrotated products serve steps of single decoded rows only")
        qf, kf, vf, cos, sin = products
        _dev(qf, kf, vf, cos, sin)
        if not (qf.dtype == torch.float32 and qf.shape == (n, n_heads * hd) and qf.stride(1) == 1):
            raise KernelError("attention: q must be float32 [n, heads*hd]")
        for t, name in ((kf, "k"), (vf, "v")):
            if not (t is None or (t.dtype == torch.float32 and t.shape == (n, n_kv * hd) and t.stride(1) == 1)):
                raise KernelError( f"attention: {name} must be float32 [n, kv_heads*hd]")
        for t in (cos, sin):
            if not (t is None or (t.dtype == torch.float32 and t.shape == (n, hd // 2) and t.is_contiguous())):
                raise KernelError("attention: cos/sin must be float32 [n, hd/2]")
    if plan.n_tiles:
        n_splits = prompt_attention_splits(plan.n_tiles // 2 if plan.paired else plan.n_tiles, n_heads,
                                           plan.max_tile_context if not window else min(plan.max_tile_context, window + plan.tile),
                                           target_groups=PAIRED_TARGET_GROUPS if plan.paired else 512)      # a pair's workgroup has twice the waves
        n_part = plan.n_tile_rows * n_heads * n_splits * (hd + 2) if n_splits > 1 else 0
        part = torch.empty(n_part, dtype=torch.float32, device=out.device) if n_part else None
        _call("gi_attention_prompt_bf16", q.data_ptr(), cache.data_ptr(), out.data_ptr(), plan.tiles.data_ptr(), plan.n_tiles, plan.tile,
              1 if plan.paired else 0, table.data_ptr(), table.stride(0), cache.stride(0), page_size, n_heads, n_kv, hd, window, scale, n_splits,
              _ptr(plan.tile_first), _ptr(plan.tile_rows), plan.n_tile_rows, _ptr(part), n_part, _stream())
    if plan.n_decode:
        span = plan.max_decode_context if not window else min(plan.max_decode_context, window + 31)
        n_splits, n_waves = decode_attention_shape(plan.n_decode, n_heads, n_kv, hd, span, target_waves, products is not None)
        n_part = plan.n_decode * n_heads * n_splits * (hd + 2) if n_splits > 1 else 0
        part = torch.empty(n_part, dtype=torch.float32, device=out.device) if n_part else None
        _call("gi_attention_decode_bf16", _ptr(q), _ptr(qf), _ptr(kf), _ptr(vf), qf.stride(0) if qf is not None else 0,
              kf.stride(0) if kf is not None else 0, vf.stride(0) if vf is not None else 0, _ptr(cos), _ptr(sin), cache.data_ptr(),
              out.data_ptr(), _ptr(part), n_part, _ptr(plan.decode_rows), plan.n_decode, positions.data_ptr(), slots.data_ptr(),
              table.data_ptr(), table.stride(0), cache.stride(0), page_size, n_heads, n_kv, hd, window, scale, n_splits, n_waves, _stream())
    return out


def _plan_of(ctx):
    if "attention_plan" not in ctx.memo:
        ctx.memo["attention_plan"] = AttentionPlan(ctx.seg_start, ctx.seg_len, ctx.seg_pos0, ctx.seg_slot, ctx.device, ctx.to_device)
    return ctx.memo["attention_plan"]


def attention(q, cache, out, ctx, table, n_heads, n_kv, hd, window=None):
    """Attention of a step's rows; the kernel is chosen by the storage dtype and the batch's shape."""
    page_size = cache.shape[3]
    if q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16:
        plan = _plan_of(ctx)
        if (not plan.n_tiles or attention_bf16_supports(hd, page_size, True)) and (not plan.n_decode or attention_bf16_supports(hd, page_size, False)):
            return attention_bf16(q, cache, out, plan, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window)
    return attention_exact(q, cache, out, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window)


# Up to so many rows the decode kernel rotates and writes the pages itself.  It saves the rotation kernel's launch wherever the
# q/k/v product does not rotate and store in its own epilogue (which it does from 33 rows on, and for long k from 17): +2..3 % a
# step at 1 and 8 rows, and at 17 to 32 rows of the Llama-3.2-1B shape (24 rows 1.323 -> 1.290 ms).
FUSED_DECODE_MAX_ROWS = 32


def attention_from_products(q, k, v, cos, sin, cache, out, ctx, table, n_heads, n_kv, hd, window=None) -> bool:
    """Rotation, cache write and attention in one launch, from the unrotated float32 products, when
    every row of the step is a request's single new row, the rows are few and the matrix-core decode
    kernel takes the sizes.  Returns False (nothing done) otherwise: the caller then rotates and stores first."""
    if not (cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and q.dtype == torch.float32):
        return False
    plan = _plan_of(ctx)
    if plan.n_tiles or not plan.single_rows or not attention_bf16_supports(hd, cache.shape[3], False):      # rows of one portion need each other's keys in the cache
        return False
    if plan.n_decode > FUSED_DECODE_MAX_ROWS:
        return False
    if q.stride(0) % 4 or q.data_ptr() % 16 or (k is not None and (k.stride(0) % 4 or k.data_ptr() % 16)):
        return False
    attention_bf16(None, cache, out, plan, ctx.row_pos, ctx.row_slot, table, n_heads, n_kv, hd, window, products=(q, k, v, cos, sin))
    return True


def gemm_bf16_supports(a, w, out) -> bool:
    """Shapes and alignments the matrix-core kernels take; the exact kernel serves the rest."""
    k = a.shape[1]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and k % 8 == 0 and a.stride(1) == 1 and w.stride(1) == 1
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and (out.dtype == torch.float32 or out.dtype == torch.bfloat16) and out.stride(1) == 1)


# What the library says about a shape does not change while the process lives, and a step asks it some hundred times: the answers
# are kept (a question costs a call through ctypes, about a microsecond of the host's time each).
@lru_cache(maxsize=None)
def _scratch_floats(m, n, k) -> int:
    return lib().gi_gemm_bf16_scratch_floats(m, n, k)


@lru_cache(maxsize=None)
def gemm_bf16_norm_parts(m, n, k) -> int:
    """The pieces per row in which a product [m, k] x [n, k] that adds onto rows writes their sums of squares when it hands
    the next norm on (`gemm_bf16(..., norm_out=...)`); 0 if a product of these sizes cannot."""
    return lib().gi_gemm_bf16_norm_parts(m, n, k)


@lru_cache(maxsize=None)
def gemm_bf16_takes_norm(m, n, k, gated=False) -> bool:
    """Whether a product of these sizes can read rows whose norm was handed on (`gemm_bf16(..., norm_in=...)`) by a product
    of as many rows."""
    return bool(lib().gi_gemm_bf16_takes_norm(m, n, k, 1 if gated else 0))


def gemm_bf16(a, w, out, accumulate=False, gated=False, checked=False, norm_in=None, norm_out=None):
    """out (=|+=) a @ w.T with bfloat16 operands on the matrix cores, float32 sums.
    gated: w is [gate; up] interleaved in groups of 16 rows and out = silu(a @ gate.T) * (a @ up.T), bfloat16 [m, n/2].

    An RMS norm between two products of a few rows, without a kernel of its own:
    norm_out = (g, scaled, squares), with accumulate: beside out += a @ w.T, scaled = bfloat16(g * out) and squares
    [m, gemm_bf16_norm_parts(m, n, k)] = the pieces of the rows' sums of out^2;
    norm_in = (squares, eps): a is such a `scaled`, and the results are multiplied by rsqrt(sum of the row's pieces / k + eps)."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    if not (w.shape == (n, k)):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, activations are {tuple(a.shape)}")
    if not (out.shape == (m, n // 2 if gated else n)):
        raise KernelError(f"gemm: out is {tuple(out.shape)}, ({m}, {n // 2 if gated else n}) is needed")
    if not (checked or gemm_bf16_supports(a, w, out)):
        raise KernelError("gemm_bf16: operands must be bfloat16 with K and row strides multiples of 8, 16-byte aligned")
    n_scratch = _scratch_floats(m, n, k)                             # partial sums where k is split over workgroups
    scratch = torch.empty(n_scratch, dtype=torch.float32, device=a.device) if n_scratch else None
    if _profile is not None:
        _profile.note = (f"{n}x{k}{' gated' if gated else ''}", n * k * w.element_size())
    if norm_in is not None or norm_out is not None:
        squares_in, eps = norm_in if norm_in is not None else (None, 0.0)
        g, scaled, squares_out = norm_out if norm_out is not None else (None, None, None)
        if squares_in is not None and not (squares_in.dtype == torch.float32 and squares_in.is_contiguous() and squares_in.dim() == 2 and squares_in.shape[0] == m):
            raise KernelError("gemm: the pieces of the sums of squares must be float32 [m, pieces]")
        if norm_out is not None:
            parts = gemm_bf16_norm_parts(m, n, k)
            if not (parts and accumulate and out.dtype == torch.float32 and g.dtype == torch.float32 and g.is_contiguous() and g.numel() == n
                    and scaled.dtype == torch.bfloat16 and scaled.shape == (m, n) and scaled.stride(1) == 1
                    and squares_out.dtype == torch.float32 and squares_out.is_contiguous() and squares_out.shape == (m, parts)):
                raise KernelError("gemm: handing a norm on needs a product of a few rows that adds onto float32 rows, float32 weights of the norm, "
                                  "bfloat16 [m, n] for the scaled rows and float32 [m, gemm_bf16_norm_parts] for the sums of squares")
            _dev(g, scaled, squares_out)
        _call("gi_gemm_bf16_handing", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "gemm: out"), 1 if accumulate else 0, 1 if gated else 0,
              m, n, k, a.stride(0), w.stride(0), out.stride(0), _ptr(scratch), n_scratch, _ptr(squares_in), squares_in.shape[1] if squares_in is not None else 0, float(eps),
              _ptr(g), _ptr(scaled), scaled.stride(0) if scaled is not None else 0, _ptr(squares_out), _stream())
        return out
    _call("gi_gemm_bf16", a.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "gemm: out"), 1 if accumulate else 0, 1 if gated else 0,
          m, n, k, a.stride(0), w.stride(0), out.stride(0), _ptr(scratch), n_scratch, _stream())
    return out


@lru_cache(maxsize=None)
def gemm_bf16_qkv_rope_store_takes(m, n, k, hd) -> bool:
    """Whether `gemm_bf16_qkv_rope_store` takes a q/k/v product of m rows, n = (heads + 2 kv heads) * hd columns and k."""
    return bool(lib().gi_gemm_bf16_qkv_rope_store_takes(m, n, k, hd))


@lru_cache(maxsize=None)
def gemm_bf16_qkv_rope_store_max_parts(m, n, k) -> int:
    """The most pieces of a row's sum of squares (`norm_in`) that `gemm_bf16_qkv_rope_store` reads for these sizes."""
    return lib().gi_gemm_bf16_qkv_rope_store_max_parts(m, n, k)


def gemm_bf16_qkv_rope_store(a, w, cos, sin, positions, slots, table, q_out, cache, n_heads, n_kv, hd, norm_in=None):
    """The q/k/v product a @ w.T of an attention layer whose results do not come back: the queries go, rotated, into q_out
    (bfloat16 [m, heads*hd]), the keys (rotated) and the values into the cache's pages, as `rope_store` puts them.
    cos, sin: float32 [m, hd/2] or None; norm_in as for `gemm_bf16`."""
    _dev(a, w, cos, sin, positions, slots, table, q_out, cache)
    m, k = a.shape
    n = w.shape[0]
    if not (gemm_bf16_supports(a, w, q_out) and w.shape == (n, k) and n == (n_heads + 2 * n_kv) * hd and gemm_bf16_qkv_rope_store_takes(m, n, k, hd)):
        raise KernelError(f"gemm (q/k/v): a product of {m} x {n} x {k} with heads of {hd} is not taken")
    if not (q_out.dtype == torch.bfloat16 and q_out.shape == (m, n_heads * hd) and q_out.is_contiguous() and cache.dtype == torch.bfloat16):
        raise KernelError("gemm (q/k/v): q_out must be bfloat16 [m, heads*hd], contiguous, and the cache bfloat16")
    if cos is not None:
        for t in (cos, sin):
            if not (t.dtype == torch.float32 and t.shape == (m, hd // 2) and t.is_contiguous()):
                raise KernelError("gemm (q/k/v): cos/sin must be float32 [m, hd/2]")
    page_size = cache.shape[3]
    _check_cache(cache, table, page_size, n_kv, hd, "gemm (q/k/v)")
    _i32(positions, "gemm (q/k/v): positions", m)
    _i32(slots, "gemm (q/k/v): slots", m)
    squares_in, eps = norm_in if norm_in is not None else (None, 0.0)
    if squares_in is not None and not (squares_in.dtype == torch.float32 and squares_in.is_contiguous() and squares_in.dim() == 2 and squares_in.shape[0] == m):
        raise KernelError("gemm: the pieces of the sums of squares must be float32 [m, pieces]")
    n_scratch = _scratch_floats(m, n, k)
    scratch = torch.empty(n_scratch, dtype=torch.float32, device=a.device) if n_scratch else None
    if _profile is not None:
        _profile.note = (f"{n}x{k}", n * k * w.element_size())
    _call("gi_gemm_bf16_qkv_rope_store", a.data_ptr(), w.data_ptr(), m, n, k, a.stride(0), w.stride(0), _ptr(scratch), n_scratch,
          _ptr(squares_in), squares_in.shape[1] if squares_in is not None else 0, float(eps), _ptr(cos), _ptr(sin), positions.data_ptr(),
          slots.data_ptr(), table.data_ptr(), table.stride(0), q_out.data_ptr(), cache.data_ptr(), cache.stride(0), page_size, n_heads, n_kv, hd, _stream())
    return q_out


def interleave_gate_up(gate, up):
    """[gate; up] in groups of 16 rows: 16 gate rows, the 16 up rows of the same outputs, and so on."""
    i, d = gate.shape
    if not (i % 16 == 0 and up.shape == gate.shape):
        raise KernelError("interleave_gate_up: the intermediate size must be a multiple of 16")
    return torch.stack([gate.view(i // 16, 16, d), up.view(i // 16, 16, d)], dim=1).reshape(2 * i, d).contiguous()


def argmax(logits, out):
    _dev(logits, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("argmax: logits must be float32 with unit inner stride")
    _i32(out, "argmax: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_v = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_i = torch.empty(n * chunks, dtype=torch.int32, device=logits.device)
    _call("gi_argmax", logits.data_ptr(), out.data_ptr(), part_v.data_ptr(), part_i.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


def sample_temperature(logits, temperature, uniform, out):
    _dev(logits, temperature, uniform, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("sample: logits must be float32 with unit inner stride")
    for t, name in ((temperature, "temperature"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"sample: {name} must be float32 [n]")
    _i32(out, "sample: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_m = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_s = torch.empty(n * chunks, dtype=torch.float64, device=logits.device)
    _call("gi_sample_temperature", logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), out.data_ptr(), part_m.data_ptr(),
          part_s.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


def sample_filtered(logits, temperature, top_k, top_p, uniform, out):
    """Top-k, then top-p, then the draw, for rows that each have one of the two filters (top_k in 1..vocab-1, or
    top_p < 1): a row without a filter is drawn in index order, which `sample_temperature` does."""
    _dev(logits, temperature, top_k, top_p, uniform, out)
    n, vocab = logits.shape
    if not (logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise KernelError("sample: logits must be float32 with unit inner stride")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"sample: {name} must be float32 [n]")
    _i32(top_k, "sample: top_k", n)
    _i32(out, "sample: out", n)
    chunks = lib().gi_argmax_chunks(vocab)
    part_m = torch.empty(n * chunks, dtype=torch.float32, device=logits.device)
    part_s = torch.empty(n * chunks, dtype=torch.float64, device=logits.device)
    kept = torch.empty(n * vocab, dtype=torch.float32, device=logits.device)
    tops = torch.empty(n * lib().gi_sample_filtered_histogram_bytes() // 8, dtype=torch.int64, device=logits.device)
    _call("gi_sample_filtered", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), uniform.data_ptr(),
          out.data_ptr(), part_m.data_ptr(), part_s.data_ptr(), kept.data_ptr(), tops.data_ptr(), n, vocab, logits.stride(0), _stream())
    return out


# ------------------------------------------------------------------------------------------------ probes
def _timed_ms(launch, repeats):
    """Median time of `launch()` over `repeats` runs, by device events, after one run that is not timed."""
    launch()
    times = []
    for _ in range(repeats):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        launch()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    return sorted(times)[len(times) // 2]


# (workgroups of 256 threads per compute unit, loads of 16 bytes in flight per thread) of the plain read.  On an MI355X few
# waves with many loads each read fastest (measured over 1 to 64 workgroups a unit and 4, 8, 16 loads: 6.3 TB/s with one
# workgroup and 8 loads, 6.2 with two and 4; 5.3 to 5.8 with 4 to 16 workgroups; 6.0 with 32 and 64); a copy reaches 5.1 to 5.3.
STREAM_SHAPES = ((1, 8), (2, 4), (1, 16), (64, 4))


def measured_read_bandwidth(device="cuda:0", n_bytes: int = 2 << 30, repeats: int = 5, copy: bool = False, shapes=STREAM_SHAPES) -> float:
    """GB/s at which a plain kernel of this library reads `n_bytes` of device memory (much more than the caches hold);
    with `copy`, reads and writes them (bytes moved = 2 * n_bytes): the best of a few shapes of the kernel (`STREAM_SHAPES`)."""
    src = torch.empty(n_bytes // 4, dtype=torch.int32, device=device).fill_(1)
    dst = torch.empty_like(src) if copy else None
    best = 0.0
    for blocks_per_unit, in_flight in shapes:
        n_blocks = lib().gi_compute_units() * blocks_per_unit
        sink = torch.empty(n_blocks * 256, dtype=torch.int32, device=device)
        ms = _timed_ms(lambda: _call("gi_probe_stream", src.data_ptr(), _ptr(dst), n_bytes, sink.data_ptr(), n_blocks, in_flight, _stream()), repeats)
        best = max(best, (2 if copy else 1) * n_bytes / (ms * 1e-3) / 1e9)
    return best


def measured_mfma_rate(device="cuda:0", iters: int = 20000, repeats: int = 5) -> float:
    """TFLOP/s of a loop of bfloat16 matrix instructions (32x32x16, eight independent sums a wave, eight waves a compute unit)."""
    n_blocks = 256 * 2
    sink = torch.empty(n_blocks * 256, dtype=torch.float32, device=device)
    ms = _timed_ms(lambda: _call("gi_probe_mfma", iters, sink.data_ptr(), n_blocks, _stream()), repeats)
    return lib().gi_probe_mfma_flops(iters, n_blocks) / (ms * 1e-3) / 1e12
