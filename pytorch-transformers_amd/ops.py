"""Python face of the HIP kernel library: loading, argument checks, one function per kernel.

There is no CPU fallback.  A function given a tensor that is not on a GPU, or
called when the library cannot be loaded, raises.  Shapes, strides and types are
checked here, before a pointer reaches a kernel.  Kernels run on torch's current
stream, so they order with torch's own work and are recorded by a HIP graph
capture like it.
"""
from __future__ import annotations

import ctypes
import functools
import importlib.util
import os
import threading
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
F32, BF16 = 0, 1
QKV_LAYOUT_CODES = {"grouped": 0, "tail": 1, "interleaved": 2}
# activations by the reference's names (src/transformers/activations.py:200-220) -> codes of csrc/common.h
ACT_CODES = {None: 0, "none": 0, "linear": 0, "gelu": 1, "gelu_python": 1, "gelu_new": 2, "gelu_pytorch_tanh": 2,
             "gelu_fast": 2, "gelu_accurate": 2, "quick_gelu": 3, "relu": 4, "relu2": 5, "relu6": 6, "silu": 7, "swish": 7,
             "sigmoid": 8, "tanh": 9, "leaky_relu": 10, "mish": 11, "gelu_10": 12, "laplace": 13}
ABI_VERSION = 14
PAIRING_CODES = {"half": 0, "interleaved": 1}  # PtaPairing: elements (i, i + rotary_dim / 2) or (2i, 2i + 1)
BIAS_OF_CODES = {"key": 0, "distance": 1}  # PtaBiasOf: the slope times the key's position, or times key - query position


class _PtaRotation(ctypes.Structure):
    _fields_ = [("inv_freq", ctypes.c_void_p), ("inv_freq_ld", ctypes.c_int), ("cs_scale", ctypes.c_float),
                ("rotary_dim", ctypes.c_int), ("pairing", ctypes.c_int)]


class _PtaGate(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("alpha", ctypes.c_float), ("limit", ctypes.c_float)]


class _PtaScoreBias(ctypes.Structure):
    _fields_ = [("slopes", ctypes.c_void_p), ("of", ctypes.c_int), ("bf16", ctypes.c_int), ("scale", ctypes.c_float)]

_lib = None
_lock = threading.Lock()


class KernelError(RuntimeError):
    pass


from . import tuning  # noqa: E402  the timed choices; it calls the faces below back, so each refers to the other by module


def __getattr__(name: str):
    """Names of ``tuning`` (``decode_plan``, ``live_tuning``, ``tuning_table`` ...) are reachable here too."""
    if name.startswith("__"):
        raise AttributeError(name)
    try:
        return getattr(tuning, name)
    except AttributeError:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}") from None


def _build_module():
    spec = importlib.util.spec_from_file_location("_pta_csrc_build", os.path.join(_HERE, "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load_library(build_if_missing: bool = True):
    """Load libpta_kernels.so, compiling it first if no current build exists."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        b = _build_module()
        path = b.find_library(require_current=True)
        if path is None:
            if not build_if_missing:
                raise KernelError("libpta_kernels.so is not built (run __graft_entry__.build())")
            path = b.build(verbose=True)
        lib = ctypes.CDLL(path)
        lib.pta_last_error.restype = ctypes.c_char_p
        if lib.pta_abi_version() != ABI_VERSION:
            raise KernelError(f"{path} has ABI {lib.pta_abi_version()}, this package needs {ABI_VERSION}; rebuild it")
        _lib = lib
        return lib


def _call(name: str, *args) -> None:
    lib = load_library()
    if _timing is None or name in _HOST_ENTRIES:
        rc = getattr(lib, name)(*args)
    else:
        with timed(name, *_entry_cost(name, args)):
            rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.pta_last_error().decode("utf-8", "replace"))


# ---- per-kernel timings for measurements ----------------------------------------------------------------------
# With ``start_timing()`` every launch through this module (and the library products that ``timed`` wraps) is
# bracketed by two events; ``stop_timing()`` returns, per entry point, calls, microseconds, the bytes it has to
# read and the arithmetic it does.  Steps must then be launched directly (``model.use_graphs = False``): events
# cannot be recorded into a captured step.  ``timing_hint`` carries what an entry point's arguments do not say
# (how many cached keys and values an attention launch reads, the arithmetic of a prompt's attention).
_timing = None
_HOST_ENTRIES = ("pta_gemm_splitk_pair_parts", "pta_gemm_stationary_rule")  # entry points that launch nothing
timing_hint = {"attn_bytes": 0, "attn_flops": 0}


class timed:
    def __init__(self, name: str, nbytes: float = 0.0, flops: float = 0.0):
        self.name, self.nbytes, self.flops = name, nbytes, flops

    def __enter__(self):
        if _timing is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if _timing is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _timing.append((self.name, self.start, end, self.nbytes, self.flops))
        return False


def start_timing() -> None:
    global _timing
    _timing = []


def stop_timing() -> dict:
    """``{entry point: {"calls", "us", "bytes", "flops"}}`` of everything launched since ``start_timing``."""
    global _timing
    records, _timing = _timing or [], None
    torch.cuda.synchronize()
    out: dict = {}
    for name, start, end, nbytes, flops in records:
        r = out.setdefault(name, {"calls": 0, "us": 0.0, "bytes": 0.0, "flops": 0.0})
        r["calls"] += 1
        r["us"] += start.elapsed_time(end) * 1e3
        r["bytes"] += nbytes
        r["flops"] += flops
    return out


def _entry_cost(name: str, a) -> tuple:
    """(bytes a launch has to read, arithmetic it does), from the entry point's own arguments: matrices count
    once, activations and results of a few rows are left out."""
    gemm = lambda M, N, K, elem=2: (float(N) * K * elem, 2.0 * M * N * K)
    both = lambda x, y: (x[0] + y[0], x[1] + y[1])
    if name == "pta_gemm_skinny_bf16":
        return gemm(a[6], a[7], a[8])
    if name == "pta_gemm_skinny_pair_bf16":
        return both(gemm(a[12], a[4], a[13]), gemm(a[12], a[10], a[13]))
    if name == "pta_gemm_skinny_pair_qkv_bf16":
        return both(gemm(a[22], (a[11] + 2 * a[12]) * a[13], a[23]), gemm(a[22], a[20], a[23]))
    if name == "pta_gemm_splitk_bf16":
        return gemm(a[7], a[8], a[9])
    if name == "pta_gemm_splitk_pair_bf16":
        return both(gemm(a[10], a[3], a[4]), gemm(a[10], a[8], a[9]))
    if name == "pta_gemm_splitk_pair_reduced_bf16":
        return both(gemm(a[16], a[5], a[6]), gemm(a[16], a[13], a[14]))
    if name == "pta_gemm_splitk_pair_reduced_qkv_bf16":
        return both(gemm(a[26], (a[13] + 2 * a[14]) * a[15], a[5]), gemm(a[26], a[23], a[24]))
    if name == "pta_gemm_splitk_reduced_qkv_bf16":
        return gemm(a[18], (a[13] + 2 * a[14]) * a[15], a[5])
    if name == "pta_gemm_f32":
        return gemm(a[6], a[7], a[8], 4)
    if name == "pta_layernorm_sum":
        return ((a[4] + a[7]) * float(a[17]) * a[19] * 4, 0.0)
    if name in ("pta_attn_mfma", "pta_attn_generic", "pta_attn_latent_mfma", "pta_attn_latent", "pta_attn_talk",
                "pta_attn_talk_mfma"):
        # (a model with two kinds of attention says each kind's figures under the entry point's name)
        return (float(timing_hint.get("attn_bytes:" + name, timing_hint.get("attn_bytes", 0))),
                float(timing_hint.get("attn_flops:" + name, timing_hint.get("attn_flops", 0))))
    val = lambda i: float(getattr(a[i], "value", a[i]) or 0)
    given = lambda i: 1.0 if getattr(a[i], "value", a[i]) else 0.0
    if name == "pta_rmsnorm":  # what it reads and writes: x (and gate), the residual, the two results
        M, H, e = val(19), val(20), (4.0 if a[21] == F32 else 2.0)
        return (M * H * ((4.0 if a[3] else e) + given(5) * e + given(12) * 4.0 + given(1) * 4.0 + given(0) * e
                         + given(14) * 4.0 * a[17]), 0.0)
    if name == "pta_depth_mix":
        return (val(6) * ((a[5] + 1) * 4.0 + given(1) * 2.0), 0.0)
    if name == "pta_widen":
        return (val(2) * 6.0, 0.0)
    if name == "pta_gated_scan":
        return (float(timing_hint.get("rows", 0)) * a[12] * 4 * (4.0 if a[15] == F32 else 2.0), 0.0)
    if name == "pta_conv_silu":
        return (float(a[11]) * a[12] * ((4.0 if a[14] == F32 else 2.0) + 4.0), 0.0)
    if name == "pta_ssm_scan":  # the convolution's output in, y out, both 32-bit
        M, inner = float(timing_hint.get("rows", 0)), float(a[14] * a[15])
        return (M * (2 * inner + 2 * a[17] * a[16]) * 4.0, 4.0 * M * inner * a[16])
    if name == "pta_head_project":
        M, H, K, O = float(a[9]), a[10], a[11], a[12]
        return (H * K * O * (4.0 if a[13] == F32 else 2.0) + M * H * (K + O) * 4.0, 2.0 * M * H * K * O)
    if name == "pta_latent_prep":
        return (float(a[13]) * (a[14] * (a[15] + a[16]) + a[17] + a[16]) * (4.0 if a[19] == F32 else 2.0), 0.0)
    el = lambda code: 4.0 if code == F32 else 2.0
    if name == "pta_shift_norm":  # the stream in and out (32-bit), the terms in, the two norms out
        M, H, e = float(a[16]), float(a[17]), el(a[20])
        return (M * H * (4.0 + given(2) * 4.0 + (given(4) + given(5)) * e + (1.0 + given(1)) * e), 0.0)
    if name == "pta_wide_sum":
        return (val(4) * (8.0 + (1.0 + given(3)) * el(a[5])), 0.0)
    if name == "pta_head_norm_rope_cache":  # the heads in, the queries' frames and the pages' rows out
        M, e = float(a[16]), el(a[23])
        return (M * e * ((a[17] + a[18]) * (a[19] + a[21]) + a[18] * (a[20] + a[21])), 0.0)
    if name == "pta_gated_heads":
        M, N, e = float(a[9]), float(a[10] * a[11]), el(a[13])
        return (M * N * ((4.0 if a[2] else e) + 2 * e), 0.0)
    if name == "pta_xielu":
        return (float(a[3]) * a[4] * 2 * el(a[6]), 0.0)
    if name == "pta_glu":
        return (float(a[4]) * a[5] * 3 * el(a[9]), 0.0)
    if name == "pta_decay_scan":  # q, k, v in, o out in 32-bit; two multiply-adds per state element and token
        M, heads, P, N, e = float(timing_hint.get("rows", 0)), a[12], a[13], a[14], el(a[18])
        return (M * heads * ((2 * N + P) * e + P * 4.0), 4.0 * M * heads * N * P)
    if name == "pta_moe_route":
        return (float(a[6]) * a[7] * el(a[18]) + float(a[7]) * a[8] * 4.0, 2.0 * a[6] * a[7] * a[8])
    if name == "pta_layernorm_stream":  # what it reads and writes: the stream, a sublayer's output, a second tensor, the results
        M, H, e = float(a[14]), float(a[15]), el(a[16])
        return (M * H * ((given(2) + given(8) + given(1)) * 4.0 + (given(3) + given(0)) * e), 0.0)
    if name == "pta_polynorm":
        return (float(a[5]) * a[6] * 2.0 * el(a[7]), 0.0)
    if name == "pta_embed_pos":
        return (float(a[6]) * a[7] * (2.0 * el(a[9]) + 4.0), 0.0)
    if name == "pta_moe_up":  # at most every (token, expert) pair's matrices once, and no more than all experts'
        M, H, Fe, top, e, mats = float(a[5]), a[6], a[7], a[8], el(a[12]), (2 if a[11] else 1)
        pairs = min(M * top, float(timing_hint.get("experts", M * top)))
        return (pairs * mats * Fe * H * e, 2.0 * mats * M * top * Fe * H)
    if name == "pta_moe_down":
        M, H, Fe, top, e = float(a[5]), a[6], a[7], a[8], el(a[12])
        pairs = min(M * top, float(timing_hint.get("experts", M * top)))
        return (pairs * Fe * H * e, 2.0 * M * top * Fe * H)
    if name == "pta_moe_grouped":  # every expert's three matrices once; the arithmetic of the pairs
        M, H, Fe, E, top, mats = float(a[12]), a[13], a[14], a[15], a[16], (3.0 if a[19] else 2.0)
        return (min(E, M * top) * mats * Fe * H * 2.0, 2.0 * mats * M * top * Fe * H)
    return (0.0, 0.0)


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"dtype {dt} is not supported; use torch.float32 or torch.bfloat16")


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise KernelError(f"{name} is on {t.device}; the kernels run on the GPU only and there is no CPU fallback")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def _need_rows(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    """Like ``_need`` for a matrix whose rows may lie apart (a block of columns of a wider matrix)."""
    if isinstance(t, torch.Tensor) and t.dim() == 2 and t.is_cuda and not t.is_contiguous() and t.stride(1) == 1 \
            and t.stride(0) >= t.shape[1]:
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
        return
    _need(t, name, dtype, shape)


def _need_pools(k_pool, v_pool, dtype, nkv: int, d: int) -> None:
    """Key pages are [pages, kv_heads, 64, d]; value pages are transposed, [pages, kv_heads, d, 64]."""
    _need(k_pool, "k_pool", dtype)
    _need(v_pool, "v_pool", dtype)
    if tuple(k_pool.shape[1:]) != (nkv, 64, d) or k_pool.dim() != 4:
        raise KernelError(f"k_pool must be [pages, {nkv}, 64, {d}], got {tuple(k_pool.shape)}")
    if tuple(v_pool.shape) != (k_pool.shape[0], nkv, d, 64):
        raise KernelError(f"v_pool must be [{k_pool.shape[0]}, {nkv}, {d}, 64], got {tuple(v_pool.shape)}")


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[m] = table[ids[m]].  The caller has checked that ids lie in [0, rows)."""
    _need(table, "table")
    V, H = table.shape
    _need(ids, "ids", torch.int32)
    M = ids.numel()
    if out is None:
        out = torch.empty((M, H), dtype=table.dtype, device=table.device)
    _need(out, "out", table.dtype, (M, H))
    _call("pta_embed", _ptr(out), _ptr(table), _ptr(ids), M, H, dtype_code(table.dtype), _stream())
    return out


def embed_pos(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0, pos_table: Optional[torch.Tensor] = None,
              token_pos: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[m] = table[ids[m]] * scale + pos_table[token_pos[m]]`` in 32-bit: the start of a stream that is held so.
    The caller has checked ids and positions against the tables' rows."""
    _need(table, "table")
    V, H = table.shape
    _need(ids, "ids", torch.int32)
    M = ids.numel()
    P = 0
    if pos_table is not None:
        P = pos_table.shape[0]
        _need(pos_table, "pos_table", table.dtype, (P, H))
        _need(token_pos, "token_pos", torch.int32, (M,))
    out = torch.empty((M, H), dtype=torch.float32, device=table.device)
    if M:
        _call("pta_embed_pos", _ptr(out), _ptr(table), _ptr(ids), _ptr(pos_table), _ptr(token_pos), ctypes.c_float(scale),
              M, H, P, dtype_code(table.dtype), _stream())
    return out


def layernorm_stream(dtype: torch.dtype, *, x: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None,
                     post=None, mult: float = 1.0, add: Optional[torch.Tensor] = None, vec: Optional[torch.Tensor] = None,
                     pre=None, eps: float = 0.0, rows: Optional[torch.Tensor] = None, want_wide: bool = True,
                     want_narrow: bool = False):
    """LayerNorm around a stream held in 32-bit, one launch: ``s = x + mult * LN_post(y) + add + vec`` (each term if
    given: ``x``, ``add`` ``[tokens, H]`` 32-bit, ``y`` ``[tokens, H]`` in ``dtype`` with rows that may lie apart, ``vec``
    ``[H]`` 32-bit, ``post = (weight, bias)``), then ``LN_pre(s)`` in ``dtype`` if ``pre = (weight, bias)`` is given.
    LN is ``(v - mean) / sqrt(var + eps) * weight + bias`` with the biased variance.  ``rows`` takes those rows of the
    inputs alone.  Without ``pre``, ``want_narrow`` asks for s itself in ``dtype`` beside the 32-bit one (what the next
    matrix product reads).  Returns ``(narrow or None, s or None)``; s is returned only if ``want_wide``."""
    ref = x if x is not None else y
    if ref is None:
        raise KernelError("layernorm_stream needs a stream or a sublayer's output")
    H = ref.shape[1]
    y_ld = 0
    if x is not None:
        _need(x, "x", torch.float32, (x.shape[0], H))
    if y is not None:
        y_ld = _rows_of(y, "y", H, dtype)
        if post is None:
            raise KernelError("a sublayer's output needs the norm that stands on it")
        _need(post[0], "post weight", torch.float32, (H,))
        _need(post[1], "post bias", torch.float32, (H,))
        if x is not None and y.shape[0] != x.shape[0]:
            raise KernelError("x and y differ in their number of rows")
    if add is not None:
        _need(add, "add", torch.float32, (ref.shape[0], H))
    if vec is not None:
        _need(vec, "vec", torch.float32, (H,))
    if pre is not None:
        _need(pre[0], "pre weight", torch.float32, (H,))
        _need(pre[1], "pre bias", torch.float32, (H,))
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = ref.shape[0]
    wide = torch.empty((M, H), dtype=torch.float32, device=ref.device) if (want_wide or pre is None) else None
    narrow = torch.empty((M, H), dtype=dtype, device=ref.device) if (pre is not None or want_narrow) else None
    if M:
        _call("pta_layernorm_stream", _ptr(narrow), _ptr(wide), _ptr(x), _ptr(y), ctypes.c_long(y_ld),
              _ptr(post[0]) if y is not None else None, _ptr(post[1]) if y is not None else None, ctypes.c_float(mult),
              _ptr(add), _ptr(vec), _ptr(rows), _ptr(pre[0]) if pre is not None else None,
              _ptr(pre[1]) if pre is not None else None, ctypes.c_float(eps), M, H, dtype_code(dtype), _stream())
    return narrow, wide


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """``a N(z) + b N(z^2) + c N(z^3) + e`` row by row, with powers element by element, ``N(v) = v / sqrt(mean(v^2) +
    eps)`` and ``coef = (a, b, c, e)`` 32-bit; sums in 32-bit."""
    M, F = z.shape
    ld = _rows_of(z, "z", F)
    _need(coef, "coef", torch.float32, (4,))
    out = torch.empty((M, F), dtype=z.dtype, device=z.device)
    if M:
        _call("pta_polynorm", _ptr(out), _ptr(z), ctypes.c_long(ld), _ptr(coef), ctypes.c_float(eps), M, F,
              dtype_code(z.dtype), _stream())
    return out


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, *, w2=None, b2=None,
              rows: Optional[torch.Tensor] = None):
    """LayerNorm of the rows of x (or of x[rows]); with (w2, b2) a second affine output of the same pass."""
    _need(x, "x")
    H = x.shape[-1]
    _need(w, "weight", torch.float32, (H,))
    _need(b, "bias", torch.float32, (H,))
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = x.shape[0]
    if x.dim() != 2:
        raise KernelError(f"x must be [tokens, features], got {tuple(x.shape)}")
    out1 = torch.empty((M, H), dtype=x.dtype, device=x.device)
    out2 = None
    if w2 is not None:
        _need(w2, "weight2", torch.float32, (H,))
        _need(b2, "bias2", torch.float32, (H,))
        out2 = torch.empty((M, H), dtype=x.dtype, device=x.device)
    if M == 0:
        return (out1, out2) if w2 is not None else out1
    _call("pta_layernorm", _ptr(out1), _ptr(out2), _ptr(x), _ptr(rows), _ptr(w), _ptr(b), _ptr(w2), _ptr(b2), M, H,
          ctypes.c_float(eps), dtype_code(x.dtype), _stream())
    return (out1, out2) if w2 is not None else out1


def epilogue_(y: torch.Tensor, bias=None, act=None, add1=None, add2=None) -> torch.Tensor:
    """In place: y = act(round(y + bias)) + add1 + add2.  The rows of y may lie apart."""
    _need_rows(y, "y")
    M, N = y.shape
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, a in (("add1", add1), ("add2", add2)):
        if a is not None:
            _need(a, name, y.dtype, (M, N))
    _call("pta_epilogue", _ptr(y), int(y.stride(0)), _ptr(bias), _ptr(add1), _ptr(add2), M, N, ACT_CODES[act],
          dtype_code(y.dtype), _stream())
    return y


def _rotation_arg(inv_freq, cs_scale: float, d: int, n_seqs: Optional[int] = None, rotary_dim: Optional[int] = None,
                  pairing: str = "half"):
    """The rotation of queries and keys as the kernels take it (a ``PtaRotation`` by reference; None: no rotation).
    ``inv_freq`` is one table ``[rotary_dim / 2]`` for all tokens or one per sequence of the step, ``[sequences,
    rotary_dim / 2]``; the first ``rotary_dim`` elements of a head (default: all of them) are rotated in pairs
    ``(i, i + rotary_dim / 2)`` (``"half"``) or ``(2i, 2i + 1)`` (``"interleaved"``)."""
    if inv_freq is None:
        return None
    r = int(d if rotary_dim is None else rotary_dim)
    problem = rotation_problem(d, rotary_dim, pairing)
    if problem is not None:
        raise KernelError(problem)
    _need(inv_freq, "inv_freq", torch.float32)
    if inv_freq.dim() == 1 and inv_freq.shape[0] == r // 2:
        ld = 0
    elif inv_freq.dim() == 2 and inv_freq.shape[1] == r // 2 and (n_seqs is None or inv_freq.shape[0] == n_seqs):
        ld = r // 2
    else:
        raise KernelError(f"inv_freq must be [{r // 2}] or [sequences, {r // 2}], got {tuple(inv_freq.shape)}")
    return ctypes.byref(_PtaRotation(inv_freq.data_ptr(), ld, float(cs_scale), r, PAIRING_CODES[pairing]))


def rotation_problem(d: int, rotary_dim: Optional[int] = None, pairing: str = "half") -> Optional[str]:
    """None if the launches that rotate take this arrangement, else why not (for refusing a model early)."""
    r = int(d if rotary_dim is None else rotary_dim)
    if pairing not in PAIRING_CODES:
        return f"a rotation with pairing {pairing!r} is not built; built: {sorted(PAIRING_CODES)}"
    if r < 2 or r % 2 or r > d:
        return f"rotary_dim must be even, from 2 up to the head size {d}; got {r}"
    return None


def score_bias_problem(bias_of: str, bf16: bool) -> Optional[str]:
    """None if the attention kernels form this bias on scores, else why not."""
    if bias_of not in BIAS_OF_CODES:
        return (f"a score bias of {bias_of!r} is not built; built: slopes per head times {sorted(BIAS_OF_CODES)} "
                "(the key's position, or its distance from the query)")
    if bf16 and bias_of != "key":
        return "rounding to bfloat16 as the reference rounds is built for slopes times the key's position only"
    return None


def _score_bias_arg(slopes, nh: int, bias_of: str = "key", bias_bf16: bool = True, bias_scale: float = 1.0):
    """A bias on attention scores as the kernels take it (a ``PtaScoreBias`` by reference; None: no bias):
    ``slopes[head] * x * bias_scale`` with x the key's position (``"key"``; ``bias_bf16``: position and product
    rounded to bfloat16 as the reference rounds them) or the key's position minus the query's (``"distance"``)."""
    if slopes is None:
        return None
    problem = score_bias_problem(bias_of, False)
    if problem is not None:
        raise KernelError(problem)
    _need(slopes, "slopes", torch.float32, (nh,))
    return ctypes.byref(_PtaScoreBias(slopes.data_ptr(), BIAS_OF_CODES[bias_of], int(bool(bias_bf16) and bias_of == "key"),
                                      float(bias_scale)))


def rope_dynamic_table(seq_start: torch.Tensor, cu_tokens: torch.Tensor, d: int, theta: float, factor: float,
                       max_pos: int) -> torch.Tensor:
    """A frequency table per sequence of the step, [sequences, d/2], for frequencies that follow the sequence's
    length after the step: the trained ones up to ``max_pos`` tokens, beyond that those of a base stretched by
    ``(factor * length / max_pos - (factor - 1)) ** (d / (d - 2))``."""
    n = seq_start.numel()
    _need(seq_start, "seq_start", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    out = torch.empty((n, d // 2), dtype=torch.float32, device=seq_start.device)
    _call("pta_rope_dynamic_table", _ptr(out), _ptr(seq_start), _ptr(cu_tokens), n, int(d), ctypes.c_float(theta),
          ctypes.c_float(factor), int(max_pos), _stream())
    return out


def qkv_rope_cache(fused: torch.Tensor, bias, inv_freq, cs_scale: float, token_pos, token_seq, block_table,
                   k_pool, v_pool, nh: int, nkv: int, d: int, layout: str, write_cache: bool = True,
                   rotary_dim: Optional[int] = None, pairing: str = "half") -> torch.Tensor:
    """Queries [M, nh, d] from the fused rows (which may lie apart); keys and values go to the cache pages.
    ``inv_freq``, ``rotary_dim`` and ``pairing`` say how queries and keys are rotated (``_rotation_arg``)."""
    M = fused.shape[0]
    _need_rows(fused, "fused", None, (M, (nh + 2 * nkv) * d))
    dt = fused.dtype
    if bias is not None:
        _need(bias, "bias", torch.float32, ((nh + 2 * nkv) * d,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, dt, nkv, d)
    q = torch.empty((M, nh, d), dtype=dt, device=fused.device)
    _call("pta_qkv_rope_cache", _ptr(q), _ptr(fused), int(fused.stride(0)), _ptr(bias), rot,
          _ptr(token_pos), _ptr(token_seq), _ptr(block_table), block_table.shape[1], _ptr(k_pool), _ptr(v_pool), M,
          nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), dtype_code(dt), _stream())
    return q


def attention_sizes_problem(nh: int, nkv: int, d: int, rotated: bool) -> Optional[str]:
    """None if the attention kernels take these head counts and this head size (``rotated``: queries and keys are
    rotated by position), else the reason.  Launches nothing: for refusing a model before its weights are read."""
    lib = load_library()
    if lib.pta_attention_sizes_ok(int(nh), int(nkv), int(d), int(bool(rotated))) == 0:
        return None
    return lib.pta_last_error().decode("utf-8", "replace")


def attn_generic(q: torch.Tensor, k_pool, v_pool, block_table, token_seq, token_pos, slopes, scale: float,
                 window: int = 0, alibi_exact: bool = False, bias_of: str = "key", bias_scale: Optional[float] = None,
                 chunk: int = 0):
    """Causal attention of every token over its sequence's cache (the last ``window`` positions of it, itself
    included, if ``window`` > 0; the positions of its own block of ``chunk``, counted from the sequence's start, if
    ``chunk`` > 0); out [M, nh*d].  ``slopes`` (None: no bias), ``bias_of``, ``alibi_exact`` (no
    rounding to bfloat16) and ``bias_scale`` (None: 1 / sqrt(head size), as the reference folds its bias into the
    mask) describe a bias on the scores (``_score_bias_arg``)."""
    _need(q, "q")
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    bias = _score_bias_arg(slopes, nh, bias_of, not alibi_exact, d ** -0.5 if bias_scale is None else bias_scale)
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    _call("pta_attn_generic", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
          block_table.shape[1], _ptr(token_seq), _ptr(token_pos), bias, M, nh, nkv, d,
          ctypes.c_float(scale), int(window), int(chunk), dtype_code(q.dtype), _stream())
    return out


def attn_talk_sizes_problem(nh: int, nkv: int, d: int) -> Optional[str]:
    """Why ``attn_talk`` does not take these sizes, or None."""
    lib = load_library()
    if lib.pta_attn_talk_sizes_ok(int(nh), int(nkv), int(d)):
        return lib.pta_last_error().decode("utf-8", "replace")
    return None


WEIGHTS_CODES = {"softmax": 0, "sigmoid": 1}


def _head_numbers(nh: int, head_scale, head_bias, weights: str):
    if weights not in WEIGHTS_CODES:
        raise KernelError(f"attention weights of kind {weights!r} are not built; built: {sorted(WEIGHTS_CODES)}")
    for name, t in (("head_scale", head_scale), ("head_bias", head_bias)):
        if t is not None:
            _need(t, name, torch.float32, (nh,))
    return _ptr(head_scale), _ptr(head_bias), WEIGHTS_CODES[weights]


def attn_talk(q: torch.Tensor, k_pool, v_pool, block_table, token_seq, token_pos, scale: float, *,
              talk: Optional[torch.Tensor] = None, softcap: float = 0.0, window: int = 0, chunk: int = 0,
              head_scale: Optional[torch.Tensor] = None, head_bias: Optional[torch.Tensor] = None, weights: str = "softmax"):
    """Causal attention as ``attn_generic`` (no bias) whose scores are, before the softmax, multiplied by a number per
    head (``head_scale`` ``[nh]`` 32-bit), capped (``softcap * tanh(score / softcap)`` if ``softcap`` > 0) and mixed over
    the heads (``score_h <- sum_g talk[h, g] score_g`` if ``talk`` ``[nh, nh]`` 32-bit is given).  ``weights``
    ``"sigmoid"``: a key's weight is ``sigmoid(score + head_bias[h])``, not normalised over the keys, in place of the
    softmax.  32-bit arithmetic; out [M, nh*d]."""
    _need(q, "q")
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    if talk is not None:
        _need(talk, "talk", torch.float32, (nh, nh))
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    if M:
        _call("pta_attn_talk", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), block_table.shape[1],
              _ptr(token_seq), _ptr(token_pos), _ptr(talk), ctypes.c_float(softcap), M, nh, nkv, d, ctypes.c_float(scale),
              int(window), int(chunk), *_head_numbers(nh, head_scale, head_bias, weights), dtype_code(q.dtype), _stream())
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None) -> torch.Tensor:
    """act(a @ w.T + bias) + add1 + add2 in true 32-bit with a fixed summation order."""
    _need(a, "a", torch.float32)
    _need(w, "w", torch.float32)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"a is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.float32, (M, N))
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    _call("pta_gemm_f32", _ptr(out), _ptr(a), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K, ACT_CODES[act],
          _stream())
    return out


# The smallest range of keys that one wave of a split decode launch walks (PTA_ATTN_SPLIT and PTA_ATTN_TILES
# pin the cut of a decode launch for tuning: keys per wave, column tiles per wave).
ATTN_SPLIT_KEYS = 128
ATTN_FORCE_SPLIT = int(os.environ.get("PTA_ATTN_SPLIT", "0"))
ATTN_FORCE_TILES = int(os.environ.get("PTA_ATTN_TILES", "0"))
ATTN_FORCE_WIDE = int(os.environ.get("PTA_ATTN_WIDE", "-1"))  # eight-wave workgroups for prompts: 1 always, 0 never

def attn_mfma_ok(q: torch.Tensor) -> bool:
    """Whether the matrix-core attention kernel takes these queries (bfloat16, head size built)."""
    return q.dtype == torch.bfloat16 and bool(load_library().pta_attn_mfma_supported(int(q.shape[2])))


SHARED_KEYS = 0  # as the waves of a decode cut: the heads of a KV head share its keys in one workgroup


def attn_decode_shared_ok(head_dim: int, heads_per_kv_head: int) -> bool:
    """Whether a decode launch with keys shared through LDS is built for this shape (many heads on a KV head)."""
    return bool(load_library().pta_attn_decode_shared_ok(int(head_dim), int(heads_per_kv_head)))


def attn_mfma(q: torch.Tensor, k_pool, v_pool, block_table, cu_tokens, seq_start, slopes, scale: float, *,
              max_new: int, n_splits: int = 1, split_size: int = ATTN_SPLIT_KEYS, window: int = 0,
              decode_tiles: int = 0, decode_waves: int = 1, alibi_exact: bool = False,
              prompt_wide: Optional[bool] = None, bias_of: str = "key", bias_scale: Optional[float] = None,
              chunk: int = 0) -> torch.Tensor:
    """Causal attention of a step's tokens over the cache on the matrix cores; out [M, nh*d].

    ``max_new`` bounds the new tokens of any sequence of the step; with ``n_splits > 1`` the keys
    are split into ranges of ``split_size`` and ``n_splits * split_size`` bounds every context.
    ``decode_tiles``: groups of sixteen heads of one KV head that a wave holds when ``max_new`` is 1
    (0: as many as the head size allows).  ``decode_waves``: waves of a workgroup that divide its keys among
    them, or ``SHARED_KEYS``: the heads of a KV head on the waves of one workgroup, which share its keys through
    LDS (``attn_decode_shared_ok``).  ``prompt_wide``: workgroups of eight waves (True) or four (False) for prompts
    with heads up to 64 (None: eight where the launch has workgroups enough).  ``slopes``, ``alibi_exact``,
    ``bias_of`` and ``bias_scale``: the bias on the scores, as in ``attn_generic``."""
    _need(q, "q", torch.bfloat16)
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    n_seqs = block_table.shape[0]
    _need(cu_tokens, "cu_tokens", torch.int32, (n_seqs + 1,))
    _need(seq_start, "seq_start", torch.int32, (n_seqs,))
    bias = _score_bias_arg(slopes, nh, bias_of, not alibi_exact, d ** -0.5 if bias_scale is None else bias_scale)
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    po = pm = pl = None
    if n_splits > 1:
        po = torch.empty((M, nh, n_splits, d), dtype=torch.float32, device=q.device)
        pm = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
        pl = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
    _call("pta_attn_mfma", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), block_table.shape[1],
          _ptr(cu_tokens), _ptr(seq_start), bias, n_seqs, int(max_new), M, nh, nkv, d,
          ctypes.c_float(scale),
          int(split_size), int(n_splits), _ptr(po), _ptr(pm), _ptr(pl), int(window), int(chunk), int(decode_tiles), int(decode_waves),
          ATTN_FORCE_WIDE if prompt_wide is None else int(bool(prompt_wide)), _stream())
    return out



def attention(q: torch.Tensor, k_pool, v_pool, block_table, ctx, slopes, scale: float, window: int = 0,
              alibi_exact: bool = False, bias_of: str = "key", bias_scale: Optional[float] = None,
              chunk: int = 0) -> torch.Tensor:
    """Attention of a step's tokens over the cache: picks the kernel for the step's shape and type.
    ``chunk`` > 0: a token sees the keys of its own block of so many positions only (``attn_generic``).

    bfloat16 with a head size the matrix-core kernel is built for: that kernel, with the context
    split over several waves when every sequence brings one token; anything else: the 32-bit
    kernel."""
    if attn_mfma_ok(q):
        n_splits, size, tiles, waves = 1, ATTN_SPLIT_KEYS, 0, 1
        if ctx.is_decode:
            shape = (ctx.n_seqs, q.shape[1], k_pool.shape[1], q.shape[2], ctx.max_len, getattr(ctx, "mean_len", 0))
            if window == 0 and chunk == 0:
                tuning.note_decode_launch(*shape)
            tiles, size, waves = tuning.decode_plan(*shape)
            n_splits = (ctx.max_len + size - 1) // size
        return attn_mfma(q, k_pool, v_pool, block_table, ctx.cu_tokens, ctx.seq_start, slopes, scale,
                         max_new=max(ctx.new_tokens), n_splits=n_splits, split_size=size, window=window,
                         decode_tiles=tiles, decode_waves=waves, alibi_exact=alibi_exact, bias_of=bias_of,
                         bias_scale=bias_scale, chunk=chunk)
    return attn_generic(q, k_pool, v_pool, block_table, ctx.token_seq, ctx.token_pos, slopes, scale, window, alibi_exact,
                        bias_of, bias_scale, chunk)


def attn_talk_mfma_ok(q: torch.Tensor, nkv: int, mixed: bool = True) -> bool:
    """Whether the matrix-core kernel for capped, mixed scores takes these queries (bfloat16, sizes built); ``mixed``:
    whether the scores are mixed over the heads (without a mix a token's heads need not share a workgroup)."""
    return q.dtype == torch.bfloat16 and bool(
        load_library().pta_attn_talk_mfma_supported(int(q.shape[1]), int(nkv), int(q.shape[2]), int(bool(mixed))))


def attn_talk_mfma(q: torch.Tensor, k_pool, v_pool, block_table, cu_tokens, seq_start, scale: float, *, max_new: int,
                   talk: Optional[torch.Tensor] = None, softcap: float = 0.0, window: int = 0, chunk: int = 0,
                   n_splits: int = 1, split_size: int = ATTN_SPLIT_KEYS, head_scale: Optional[torch.Tensor] = None,
                   head_bias: Optional[torch.Tensor] = None, weights: str = "softmax") -> torch.Tensor:
    """``attn_talk`` on the matrix cores (bfloat16 in, 32-bit scores, mix and softmax); out [M, nh*d].  ``max_new``
    bounds the new tokens of any sequence of the step; with one token per sequence and ``n_splits`` > 1 the keys are
    cut into ranges of ``split_size`` (``n_splits * split_size`` bounds every context), merged by a second launch;
    ``split_size`` 0: every tile of sixteen tokens cuts the keys it sees into ``n_splits`` equal runs (prompts)."""
    _need(q, "q", torch.bfloat16)
    M, nh, d = q.shape
    nkv = k_pool.shape[1]
    _need_pools(k_pool, v_pool, q.dtype, nkv, d)
    _need(block_table, "block_table", torch.int32)
    n_seqs = block_table.shape[0]
    _need(cu_tokens, "cu_tokens", torch.int32, (n_seqs + 1,))
    _need(seq_start, "seq_start", torch.int32, (n_seqs,))
    if talk is not None:
        _need(talk, "talk", torch.float32, (nh, nh))
    out = torch.empty((M, nh * d), dtype=q.dtype, device=q.device)
    po = pm = pl = None
    if n_splits > 1:
        po = torch.empty((M, nh, n_splits, d), dtype=torch.float32, device=q.device)
        pm = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
        pl = torch.empty((M, nh, n_splits), dtype=torch.float32, device=q.device)
    _call("pta_attn_talk_mfma", _ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), block_table.shape[1],
          _ptr(cu_tokens), _ptr(seq_start), _ptr(talk), ctypes.c_float(softcap), n_seqs, int(max_new), M, nh, nkv, d,
          ctypes.c_float(scale), int(window), int(chunk), int(split_size), int(n_splits), _ptr(po), _ptr(pm), _ptr(pl),
          *_head_numbers(nh, head_scale, head_bias, weights), _stream())
    return out


def talk_decode_ranges(n_seqs: int, max_len: int, window: int = 0, chunk: int = 0, per_token: int = 1) -> tuple:
    """(runs, 0) for a decode step of ``attn_talk_mfma``: every token cuts the keys it sees into so many equal runs of
    blocks, about two workgroups for every compute unit, a run no shorter than a page at the longest context, at most
    1,024 runs and 65,535 workgroups a launch.  The size 0 says that the runs are each token's own (``attn_talk_mfma``):
    what a window has left behind is in no run, so the partial results do not grow with the context.  The batch counts
    by its next power of two and the longest context by its next multiple of 1,024, so that a captured step, which is
    sized for a padded batch and such a bound, is cut exactly as the same step run directly.  ``per_token``: the
    workgroups that share a token's heads (more than one where the scores are not mixed over the heads)."""
    n_seqs = (1 << max(int(n_seqs) - 1, 0).bit_length()) * max(1, int(per_token))
    max_len = (int(max_len) + 1023) // 1024 * 1024
    seen = max_len
    for bound in (window, chunk):
        if bound > 0:
            seen = min(seen, bound + 31)
    runs = min((seen + 63) // 64, -(-512 // max(n_seqs, 1)), 1024, 65535 // max(n_seqs, 1))
    return max(1, runs), 0


def attention_talk(q: torch.Tensor, k_pool, v_pool, block_table, ctx, scale: float, *, talk=None, softcap: float = 0.0,
                   window: int = 0, chunk: int = 0, head_scale=None, head_bias=None, weights: str = "softmax") -> torch.Tensor:
    """Attention of a step's tokens over the cache with capped scores that are mixed over the heads before the
    softmax: picks the kernel for the step's shape and type.  bfloat16 with sizes the matrix-core kernel is built
    for: that kernel, with the context cut into ranges when every sequence brings one token; anything else: the
    32-bit kernel."""
    if attn_talk_mfma_ok(q, k_pool.shape[1], talk is not None):
        n_splits, size = 1, ATTN_SPLIT_KEYS
        per_token = int(load_library().pta_attn_talk_mfma_workgroups(int(q.shape[1]), int(k_pool.shape[1]), int(q.shape[2]),
                                                                     int(talk is not None)))
        if ctx.is_decode:
            n_splits, size = talk_decode_ranges(ctx.n_seqs, ctx.max_len, window, chunk, per_token)
            n_splits = min(n_splits, 65535 // max(1, ctx.n_seqs))
        else:  # few tiles of sixteen tokens: each cuts its keys into runs, so that no compute unit idles
            seen = min([ctx.max_len] + [b + 15 for b in (window, chunk) if b > 0])
            tiles = sum((n + 15) // 16 for n in ctx.new_tokens) * per_token
            n_splits, size = int(load_library().pta_attn_talk_prompt_ranges(tiles, seen)), 0
        return attn_talk_mfma(q, k_pool, v_pool, block_table, ctx.cu_tokens, ctx.seq_start, scale,
                              max_new=max(ctx.new_tokens), talk=talk, softcap=softcap, window=window, chunk=chunk,
                              n_splits=n_splits, split_size=size, head_scale=head_scale, head_bias=head_bias,
                              weights=weights)
    return attn_talk(q, k_pool, v_pool, block_table, ctx.token_seq, ctx.token_pos, scale, talk=talk, softcap=softcap,
                     window=window, chunk=chunk, head_scale=head_scale, head_bias=head_bias, weights=weights)


def sample(logits: torch.Tensor, *, do_sample: bool, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0,
           min_p: float = 0.0, typical_p: float = 1.0, epsilon_cutoff: float = 0.0, eta_cutoff: float = 0.0,
           penalty: float = 1.0, hist=None, hist_off=None, ban=None, ban_off=None, eos=None, suppress=None,
           remove_invalid: bool = False, renorm: bool = False, seed: int = 0, rng_seq=None, rng_step=None,
           uniforms=None, need_scores: bool = True, bias_tok=None, bias_val=None, bias_off=None, forced=None,
           decay: Optional[float] = None):
    """Processors and choice for every row of ``logits`` [R, V] (32-bit); returns (tokens int32 [R], scores [R, V]).

    ``bias_tok`` / ``bias_val`` / ``bias_off``: per row a list of tokens (each once) whose scores get a value added
    before every other processor.  ``forced``: token ids of which one is forced in this step (every other score
    goes, theirs become 0; a banned token stays gone).  ``decay``: the scores of the ``eos`` tokens gain
    ``|score| * decay`` after the removal of invalid values.

    Without ``need_scores``, a greedy choice that no processor touches is a plain argmax and the scores
    come back as None."""
    _need(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise KernelError(f"logits must be [rows, vocab], got {tuple(logits.shape)}")
    R, V = logits.shape
    if ban is not None and ban.numel() == 0:
        ban = ban_off = None  # no row has a banned token
    if bias_off is not None and (bias_tok is None or bias_tok.numel() == 0):
        bias_tok = bias_val = bias_off = None  # no row has a biased token
    if (not need_scores and not do_sample and penalty == 1.0 and suppress is None and ban_off is None
            and not remove_invalid and not renorm and bias_off is None and forced is None and decay is None):
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        _call("pta_argmax", _ptr(out), _ptr(logits), R, V, _stream())
        return out, None
    for name, t, n in (("hist_off", hist_off, R + 1), ("ban_off", ban_off, R + 1), ("suppress", suppress, R), ("rng_seq", rng_seq, R),
                       ("rng_step", rng_step, R)):
        if t is not None:
            _need(t, name, torch.int32, (n,))
    if hist is not None:
        _need(hist, "hist", torch.int32)
    if ban_off is not None:
        if ban is None:
            raise KernelError("ban_off without ban")
        _need(ban, "ban", torch.int32)
    if eos is not None:
        _need(eos, "eos", torch.int32)
    if uniforms is not None:
        _need(uniforms, "uniforms", torch.float32, (R,))
    if bias_off is not None:
        _need(bias_off, "bias_off", torch.int32, (R + 1,))
        _need(bias_tok, "bias_tok", torch.int32)
        _need(bias_val, "bias_val", torch.float32, tuple(bias_tok.shape))
    if forced is not None:
        _need(forced, "forced", torch.int32)
    if decay is not None and (eos is None or eos.numel() == 0):
        raise KernelError("a bonus on the EOS tokens needs their ids")
    work = torch.empty_like(logits)
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _call("pta_sample", _ptr(out), _ptr(work), _ptr(logits), R, V, int(bool(do_sample)), ctypes.c_float(temperature),
          int(top_k), ctypes.c_float(top_p), ctypes.c_float(min_p), ctypes.c_float(typical_p),
          ctypes.c_float(epsilon_cutoff), ctypes.c_float(eta_cutoff), ctypes.c_float(penalty), _ptr(hist), _ptr(hist_off),
          _ptr(ban), _ptr(ban_off),
          _ptr(eos), 0 if eos is None else int(eos.numel()), _ptr(suppress), int(bool(remove_invalid)),
          int(bool(renorm)), ctypes.c_uint64(int(seed) & (2 ** 64 - 1)), _ptr(rng_seq), _ptr(rng_step), _ptr(uniforms),
          int(bool(need_scores)), _ptr(bias_tok), _ptr(bias_val), _ptr(bias_off), _ptr(forced),
          0 if forced is None else int(forced.numel()), int(decay is not None), ctypes.c_float(decay or 0.0), _stream())
    return out, (work if need_scores else None)



def library_mm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` in bfloat16 through the vendor library, in the pieces along M that were measured fastest."""
    M, N = x.shape[0], w.shape[0]
    with timed("library_mm", float(w.numel()) * 2, 2.0 * M * N * w.shape[1]):
        if not tuning.MM_CHUNKS or M < 512:
            return torch.mm(x, w.t())
        if (N, w.shape[1], (M + 63) // 64) not in tuning.active().mm_plans and not tuning.may_time():
            return torch.mm(x, w.t())
        out = torch.empty((M, N), dtype=x.dtype, device=x.device)
        plan = tuning.mm_plan(x, w, out)
        at = 0
        for rows in plan:
            torch.mm(x[at:at + rows], w.t(), out=out[at:at + rows])
            at += rows
        return out



# ---- the vendor library's product with K cut into a batch ------------------------------------------------
# Where K is long against N (the feed-forward's second matrix) and the rows are a few hundred, the library's
# kernel choice has too few tiles of the result to fill the chip: with K = 18,176 and N = 4,544, 512 rows take 225
# us, and 112 us as a batch of two products over the halves of K (32-bit partial sums, added in order by the kernel
# that also applies bias, activation and additions, so no epilogue launch follows).  Timed once per shape when
# timing is on; without an entry the plain product runs.
MM_KSPLIT = os.environ.get("PTA_MM_KSPLIT", "1") != "0"
MM_KSPLIT_MAX_ROWS = 1536  # at 2,048 rows the batch gained nothing alone and lost 3 % in a model (K = 32,768, N = 8,192)


def _k_batch(x: torch.Tensor, w: torch.Tensor, S: int) -> torch.Tensor:
    M, K = x.shape
    xb = x.unflatten(1, (S, K // S)).transpose(0, 1)   # [S, M, K/S], rows as far apart as x's
    wb = w.unflatten(1, (S, K // S)).permute(1, 2, 0)  # [S, K/S, N]
    return torch.bmm(xb, wb, out_dtype=torch.float32)


def library_mm_ksplit(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None):
    """``act(x @ w.T + bias) + add1 + add2`` through the library's batched product over ranges of K, where that
    was timed faster than its plain product (once per shape, by 64 rows); else None."""
    M, (N, K) = x.shape[0], w.shape
    if (not MM_KSPLIT or K < 2 * N or not (tuning.SPLITK_MAX_ROWS < M <= MM_KSPLIT_MAX_ROWS) or K % 32 or x.stride(1) != 1
            or not w.is_contiguous()):
        return None
    key = (N, K, (M + 63) // 64)
    S = tuning.active().mm_ksplit.get(key)
    if S is None:
        if not tuning.may_time():
            return None
        ways = [(1, lambda: library_mm(x, w))] + [(s, (lambda s=s: _k_batch(x, w, s))) for s in (2, 4) if K % (s * 8) == 0]
        best = tuning.time_ways_cold([run for _, run in ways], x.device)
        pick = min(range(len(ways)), key=lambda i: best[i])
        S = ways[pick][0] if best[pick] < 0.9 * best[0] else 1
        tuning.active().mm_ksplit[key] = S
    if S == 1:
        return None
    with timed("library_mm", float(w.numel()) * 2, 2.0 * M * N * K):
        part = _k_batch(x, w, S)
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, a in (("add1", add1), ("add2", add2)):
        if a is not None:
            _need(a, name, torch.bfloat16, (M, N))
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _call("pta_gemm_reduce_parts", _ptr(y), _ptr(part), _ptr(bias), _ptr(add1), _ptr(add2), M, N, S, ACT_CODES[act], 0,
          _stream())
    return y


def gemm_skinny_pair_bf16(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor, bias1=None, act1=None,
                          bias2=None, act2=None):
    """(act1(x1 @ w1.T + bias1), act2(x2 @ w2.T + bias2)) in one launch: few rows, one K, bfloat16."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M, K = x1.shape
    if tuple(x2.shape) != (M, K) or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != K or w2.shape[1] != K:
        raise KernelError(f"a pair shares M and K: x1 {tuple(x1.shape)}, x2 {tuple(x2.shape)}, w1 {tuple(w1.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    N1, N2 = w1.shape[0], w2.shape[0]
    if bias1 is not None:
        _need(bias1, "bias1", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    y1 = torch.empty((M, N1), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_skinny_pair_bf16", _ptr(y1), _ptr(x1), _ptr(w1), _ptr(bias1), N1, ACT_CODES[act1], _ptr(y2), _ptr(x2),
          _ptr(w2), _ptr(bias2), N2, ACT_CODES[act2], M, K, _stream())
    return y1, y2


def gemm_skinny_pair_qkv_ok(x: torch.Tensor, w_qkv: torch.Tensor, w2: torch.Tensor, d: int) -> bool:
    """Whether the pair launch for few rows can take a fused query_key_value projection to its end (rotation,
    queries, cache pages): bfloat16, at most 16 rows, head sizes that are multiples of 32.  PTA_QKV_TAIL=0
    switches it off."""
    return (QKV_TAIL and gemm_skinny_ok(x, w_qkv) and gemm_skinny_ok(x, w2) and d % 32 == 0 and d <= 256
            and w_qkv.shape[1] == w2.shape[1])


QKV_TAIL = os.environ.get("PTA_QKV_TAIL", "1") != "0"


def gemm_skinny_pair_qkv(x1: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos,
                         token_seq, block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str,
                         write_cache: bool, x2: torch.Tensor, w2: torch.Tensor, bias2=None, act2=None,
                         rotary_dim: Optional[int] = None, pairing: str = "half"):
    """One launch for a decode step's two input products, the first a fused query_key_value projection taken to
    its end: returns (queries [M, nh, d] rotated, act2(x2 @ w2.T + bias2)); keys and values are in the cache pages,
    as ``qkv_rope_cache`` would have left them."""
    for name, t in (("x1", x1), ("w_qkv", w_qkv), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M, K = x1.shape
    N1, N2 = (nh + 2 * nkv) * d, w2.shape[0]
    if tuple(x2.shape) != (M, K) or tuple(w_qkv.shape) != (N1, K) or w2.dim() != 2 or w2.shape[1] != K:
        raise KernelError(f"a pair shares M and K: x1 {tuple(x1.shape)}, x2 {tuple(x2.shape)}, w_qkv {tuple(w_qkv.shape)} "
                          f"(wanted [{N1}, {K}]), w2 {tuple(w2.shape)}")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_skinny_pair_qkv_bf16", _ptr(q), _ptr(x1), _ptr(w_qkv), _ptr(bias_qkv), rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table), block_table.shape[1], _ptr(k_pool),
          _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), _ptr(y2), _ptr(x2), _ptr(w2), _ptr(bias2),
          N2, ACT_CODES[act2], M, K, _stream())
    return q, y2


def gemm_splitk_bf16(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None,
                     out_f32: bool = False, rt: int = 0, parts: int = 0, stage_blocks: int = 0,
                     depth: int = 0) -> torch.Tensor:
    """act(x @ w.T + bias) + add1 + add2 for a batch of at most 128 rows of bfloat16: x shared through LDS,
    K split over workgroups where N gives too few of them."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.bfloat16, (M, N))
    parts = int(load_library().pta_gemm_splitk_parts(N, K, int(parts), int(rt)))
    part = torch.empty((parts, M, N), dtype=torch.float32, device=x.device) if parts > 1 else None
    out = torch.empty((M, N), dtype=torch.float32 if out_f32 else torch.bfloat16, device=x.device)
    _call("pta_gemm_splitk_bf16", _ptr(out), _ptr(part), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K,
          ACT_CODES[act], int(out_f32), int(rt), int(parts), int(stage_blocks), int(depth), 1, _stream())
    return out


def gemm_splitk_partial(x: torch.Tensor, w: torch.Tensor, rt: int = 0, parts: int = 0, stage_blocks: int = 0) -> torch.Tensor:
    """x @ w.T left as 32-bit partial sums over ranges of K, [ranges, M, N]: for a kernel that adds them
    in order while it reads them (``layernorm_sum``)."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.dim() != 2 or w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    parts = int(load_library().pta_gemm_splitk_parts(N, K, int(parts), int(rt)))
    part = torch.empty((parts, M, N), dtype=torch.float32, device=x.device)
    _call("pta_gemm_splitk_bf16", None, _ptr(part), _ptr(x), _ptr(w), None, None, None, M, N, K, 0, 0, int(rt),
          int(parts), int(stage_blocks), 0, 0, _stream())
    return part


def gemm_splitk_pair_parts(N1: int, K1: int, N2: int, K2: int, M: int = 0):
    """How many ranges of K each product of a pair launch of ``M`` rows is cut into (0: by the kernel that walks
    K in stages, whatever the rows; steps of 17 to 128 rows may run with the activations stationary, which has
    ranges of its own)."""
    p1, p2 = ctypes.c_int(0), ctypes.c_int(0)
    _call("pta_gemm_splitk_pair_parts", int(N1), int(K1), int(N2), int(K2), int(M), ctypes.byref(p1), ctypes.byref(p2))
    return p1.value, p2.value


STATIONARY_CLASS_ROWS = (16, 32, 64, 128)  # a pair launch's rows count by the first of these that holds them


def gemm_stationary_rule(N1: int, K1: int, N2: int, K2: int, cls: int):
    """(ranges, ranges) of K of the pair launch with stationary activations for rows of class ``cls`` (the index
    into ``STATIONARY_CLASS_ROWS``), by the rule."""
    q1, q2 = ctypes.c_int(0), ctypes.c_int(0)
    _call("pta_gemm_stationary_rule", int(N1), int(K1), int(N2), int(K2), int(cls), ctypes.byref(q1), ctypes.byref(q2))
    return q1.value, q2.value



def gemm_splitk_pair_partial(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor):
    """(x1 @ w1.T, x2 @ w2.T), both left as 32-bit partial sums, in one launch; the products share M."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    if x2.shape[0] != M or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != x1.shape[1] or w2.shape[1] != x2.shape[1]:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w1 {tuple(w1.shape)}, x2 {tuple(x2.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    (N1, K1), (N2, K2) = w1.shape, w2.shape
    tuning.tune_pair_parts(w1, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    _call("pta_gemm_splitk_pair_bf16", _ptr(part1), _ptr(x1), _ptr(w1), N1, K1, _ptr(part2), _ptr(x2), _ptr(w2), N2, K2,
          M, _stream())
    return part1, part2


def gemm_splitk_pair_bf16(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor, bias1=None, act1=None,
                          bias2=None, act2=None):
    """(act1(x1 @ w1.T + bias1), act2(x2 @ w2.T + bias2)) for a batch of up to 128 rows: one matrix launch for
    both products and one launch that adds their partial sums."""
    for name, t in (("x1", x1), ("w1", w1), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    if x2.shape[0] != M or w1.dim() != 2 or w2.dim() != 2 or w1.shape[1] != x1.shape[1] or w2.shape[1] != x2.shape[1]:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w1 {tuple(w1.shape)}, x2 {tuple(x2.shape)}, "
                          f"w2 {tuple(w2.shape)}")
    lib = load_library()
    (N1, K1), (N2, K2) = w1.shape, w2.shape
    if bias1 is not None:
        _need(bias1, "bias1", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    tuning.tune_pair_parts(w1, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    y1 = torch.empty((M, N1), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_splitk_pair_reduced_bf16", _ptr(y1), _ptr(part1), _ptr(x1), _ptr(w1), _ptr(bias1), N1, K1,
          ACT_CODES[act1], _ptr(y2), _ptr(part2), _ptr(x2), _ptr(w2), _ptr(bias2), N2, K2, ACT_CODES[act2], M, _stream())
    return y1, y2


def gemm_splitk_pair_qkv(x1: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos,
                         token_seq, block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str,
                         write_cache: bool, x2: torch.Tensor, w2: torch.Tensor, bias2=None, act2=None,
                         rotary_dim: Optional[int] = None, pairing: str = "half"):
    """The pair launch of a decode batch (17 to 256 rows) with its first product a fused query_key_value projection
    taken to its end by the launch that adds the partial sums: returns (queries [M, nh, d] rotated,
    act2(x2 @ w2.T + bias2)); keys and values are in the cache pages, as ``qkv_rope_cache`` leaves them."""
    for name, t in (("x1", x1), ("w_qkv", w_qkv), ("x2", x2), ("w2", w2)):
        _need(t, name, torch.bfloat16)
    M = x1.shape[0]
    N1, (N2, K2), K1 = (nh + 2 * nkv) * d, w2.shape, x1.shape[1]
    if x2.shape[0] != M or tuple(w_qkv.shape) != (N1, K1) or x2.shape[1] != K2:
        raise KernelError(f"a pair shares M: x1 {tuple(x1.shape)}, w_qkv {tuple(w_qkv.shape)} (wanted [{N1}, {K1}]), "
                          f"x2 {tuple(x2.shape)}, w2 {tuple(w2.shape)}")
    if d % 2:
        raise KernelError(f"head size {d} must be even")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N1,))
    if bias2 is not None:
        _need(bias2, "bias2", torch.float32, (N2,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    tuning.tune_pair_parts(w_qkv, w2)
    p1, p2 = gemm_splitk_pair_parts(N1, K1, N2, K2, M)
    part1 = torch.empty((p1, M, N1), dtype=torch.float32, device=x1.device)
    part2 = torch.empty((p2, M, N2), dtype=torch.float32, device=x1.device)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x1.device)
    y2 = torch.empty((M, N2), dtype=torch.bfloat16, device=x1.device)
    _call("pta_gemm_splitk_pair_reduced_qkv_bf16", _ptr(q), _ptr(part1), _ptr(x1), _ptr(w_qkv), _ptr(bias_qkv), K1,
          rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table),
          block_table.shape[1], _ptr(k_pool), _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache),
          _ptr(y2), _ptr(part2), _ptr(x2), _ptr(w2), _ptr(bias2), N2, K2, ACT_CODES[act2], M, _stream())
    return q, y2


def gemm_splitk_qkv(x: torch.Tensor, w_qkv: torch.Tensor, bias_qkv, inv_freq, cs_scale: float, token_pos, token_seq,
                    block_table, k_pool, v_pool, nh: int, nkv: int, d: int, layout: str, write_cache: bool,
                    rotary_dim: Optional[int] = None, pairing: str = "half"):
    """A fused query_key_value projection of a decode batch (17 to 256 rows) on its own, taken to its end by the
    launch that adds its partial sums: returns the queries [M, nh, d] rotated; keys and values are in the cache
    pages, as ``qkv_rope_cache`` leaves them."""
    _need(x, "x", torch.bfloat16)
    _need(w_qkv, "w_qkv", torch.bfloat16)
    M, K = x.shape
    N = (nh + 2 * nkv) * d
    if tuple(w_qkv.shape) != (N, K):
        raise KernelError(f"w_qkv {tuple(w_qkv.shape)}: wanted [{N}, {K}] for x {tuple(x.shape)}")
    if d % 2:
        raise KernelError(f"head size {d} must be even")
    if bias_qkv is not None:
        _need(bias_qkv, "bias_qkv", torch.float32, (N,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise KernelError("block_table must be [sequences, pages]")
    rot = _rotation_arg(inv_freq, cs_scale, d, block_table.shape[0], rotary_dim, pairing)
    _need_pools(k_pool, v_pool, torch.bfloat16, nkv, d)
    part = torch.empty((int(load_library().pta_gemm_splitk_parts(N, K, 0, 0)), M, N), dtype=torch.float32, device=x.device)
    q = torch.empty((M, nh, d), dtype=torch.bfloat16, device=x.device)
    _call("pta_gemm_splitk_reduced_qkv_bf16", _ptr(q), _ptr(part), _ptr(x), _ptr(w_qkv), _ptr(bias_qkv), K,
          rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table),
          block_table.shape[1], _ptr(k_pool), _ptr(v_pool), nh, nkv, d, QKV_LAYOUT_CODES[layout], int(write_cache), M,
          _stream())
    return q


def gemm_partial_pair_ok(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor) -> bool:
    """Whether two products onto the same features are best left as partial sums of one launch: up to 128
    rows each, and at least one of them worth leaving so on its own."""
    return (_bf16_rows_ok(x1, w1) and _bf16_rows_ok(x2, w2) and 0 < x1.shape[0] == x2.shape[0] <= tuning.SPLITK_MAX_ROWS
            and tuning.splitk_rows_ok(x1, w1, w2)
            and w1.shape[0] == w2.shape[0] and w1.shape[0] % 8 == 0
            and (gemm_partial_ok(x1, w1) or gemm_partial_ok(x2, w2)))


def gemm_partial_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether leaving x @ w.T as partial sums for the next norm pays: up to 128 rows, and either K long against
    N (any batch: the kernel for few rows has too few row tiles there) or a batch past 16 rows."""
    if not (_bf16_rows_ok(x, w) and 0 < x.shape[0] <= tuning.SPLITK_MAX_ROWS and w.shape[0] % 8 == 0 and tuning.splitk_rows_ok(x, w)):
        return False
    return w.shape[1] >= 2 * w.shape[0] or (x.shape[0] > 16 and w.shape[0] < 2 * w.shape[1])


def layernorm_sum_ok(H: int) -> bool:
    return bool(load_library().pta_layernorm_sum_ok(int(H)))


def layernorm_sum_rows_min() -> int:
    """Rows from which a sum of tensors alone is formed and normalised by a wave per row (the arrangement for prompts)."""
    return int(load_library().pta_layernorm_sum_rows_min())


def layernorm_sum(terms, H: int, *, w=None, b=None, eps: float = 0.0, w2=None, b2=None, rows=None,
                  want_x: bool = True):
    """The sum of ``terms`` rounded to bfloat16 and, with (w, b), its LayerNorm: ``(x, out1, out2)``.

    A term is a bfloat16 tensor [M, H] or a pair (partial sums [P, M, H] in 32-bit, bias or None) of a
    product left unreduced; at most two products and three tensors, products first.  A product is valued as its
    own epilogue would have stored it; the terms are added in 32-bit in the order given, and the sum is rounded."""
    prods = [t for t in terms if isinstance(t, tuple)]
    adds = [t for t in terms if not isinstance(t, tuple)]
    if len(prods) > 2 or len(adds) > 3 or not terms:
        raise KernelError(f"layernorm_sum takes one to five terms, at most two products and three tensors; got {len(terms)}")
    if any(isinstance(t, tuple) for t in terms[len(prods):]):
        raise KernelError("layernorm_sum: products must come before tensors in the list of terms")
    M_in = None
    for part, bias in prods:
        _need(part, "partial sums", torch.float32)
        if part.dim() != 3 or part.shape[2] != H:
            raise KernelError(f"partial sums must be [parts, rows, {H}], got {tuple(part.shape)}")
        if bias is not None:
            _need(bias, "bias", torch.float32, (H,))
        M_in = part.shape[1] if M_in is None else M_in
        if part.shape[1] != M_in:
            raise KernelError("terms differ in their number of rows")
    for a in adds:
        _need(a, "addend", torch.bfloat16)
        M_in = a.shape[0] if M_in is None else M_in
        if tuple(a.shape) != (M_in, H):
            raise KernelError(f"addend must be [{M_in}, {H}], got {tuple(a.shape)}")
    ref = prods[0][0] if prods else adds[0]
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = M_in
    dev = ref.device
    norm = w is not None
    if norm:
        _need(w, "weight", torch.float32, (H,))
        _need(b, "bias", torch.float32, (H,))
    if w2 is not None:
        _need(w2, "weight2", torch.float32, (H,))
        _need(b2, "bias2", torch.float32, (H,))
    out_x = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if want_x else None
    out1 = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if norm else None
    out2 = torch.empty((M, H), dtype=torch.bfloat16, device=dev) if norm and w2 is not None else None
    if M == 0:
        return out_x, out1, out2
    pb, bb = prods[0] if prods else (None, None)  # the kernel adds B first, then A
    pa, ba = prods[1] if len(prods) > 1 else (None, None)
    a1 = adds[0] if adds else None
    a2 = adds[1] if len(adds) > 1 else None
    a3 = adds[2] if len(adds) > 2 else None
    _call("pta_layernorm_sum", _ptr(out_x), _ptr(out1), _ptr(out2), _ptr(pa), 0 if pa is None else pa.shape[0], _ptr(ba),
          _ptr(pb), 0 if pb is None else pb.shape[0], _ptr(bb), _ptr(a1), _ptr(a2), _ptr(a3), _ptr(rows), _ptr(w), _ptr(b),
          _ptr(w2), _ptr(b2), M_in, M, H, ctypes.c_float(eps), _stream())
    return out_x, out1, out2


def _bf16_rows_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the kernel for few rows takes this product and is the faster choice for it: bfloat16 with K a
    multiple of 8 and at most 16 rows (measured on MI355X against the vendor library at K = 4,544 and K = 18,176)."""
    return _bf16_rows_ok(x, w) and 0 < x.shape[0] <= 16


def gemm_splitk_pair_ok(x1: torch.Tensor, w1: torch.Tensor, x2: torch.Tensor, w2: torch.Tensor) -> bool:
    """Whether the two products run as a pair launch of the decode batch kernel (17 to 256 rows; beyond 128 only
    where the pair was timed faster than the library's two products)."""
    return (_bf16_rows_ok(x1, w1) and _bf16_rows_ok(x2, w2) and 16 < x1.shape[0] == x2.shape[0] <= tuning.SPLITK_MAX_ROWS
            and tuning.splitk_rows_ok(x1, w1, w2))


def gemm_splitk_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the kernel for a decode batch of 17 to 128 rows is the faster choice.  Measured at K = 4,544 and
    K = 18,176: it beats the vendor library except where N is long against K (the feed-forward's first matrix
    and the output head), which give the library enough row tiles to fill the chip."""
    return (_bf16_rows_ok(x, w) and 16 < x.shape[0] <= tuning.SPLITK_MAX_ROWS and w.shape[0] < 2 * w.shape[1]
            and tuning.splitk_rows_ok(x, w))


def gemm_skinny_bf16(x: torch.Tensor, w: torch.Tensor, bias=None, act=None, add1=None, add2=None,
                     out_f32: bool = False, variant: int = 0, waves: int = 0) -> torch.Tensor:
    """act(x @ w.T + bias) + add1 + add2 for at most 64 rows of bfloat16, 32-bit accumulation."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"x is [{M}, {K}] but w is {tuple(w.shape)}; w must be [N, {K}]")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    for name, t in (("add1", add1), ("add2", add2)):
        if t is not None:
            _need(t, name, torch.bfloat16, (M, N))
    out = torch.empty((M, N), dtype=torch.float32 if out_f32 else torch.bfloat16, device=x.device)
    _call("pta_gemm_skinny_bf16", _ptr(out), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), _ptr(add2), M, N, K,
          ACT_CODES[act], int(out_f32), int(variant), int(waves), _stream())
    return out


# ---- a residual stream held in 32-bit ---------------------------------------------------------------------------
def _rows_of(t: torch.Tensor, name: str, cols: int, dtype=None):
    """Check a matrix whose rows may lie apart (a block of columns of a wider one) and return its row distance."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dim() != 2 or t.shape[1] != cols or t.stride(1) != 1:
        raise KernelError(f"{name} must be a GPU matrix [rows, {cols}] with adjacent columns, got "
                          f"{tuple(getattr(t, 'shape', ()))} strides {getattr(t, 'stride', lambda: None)()}")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    return int(t.stride(0)) if t.shape[0] > 1 else max(int(t.stride(0)), cols)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, dtype: torch.dtype, *, offset: float = 0.0, groups: int = 1,
            gate: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            residual: Optional[torch.Tensor] = None, mult: float = 1.0, want_wide: bool = False, want_narrow: bool = True,
            out_wide: Optional[torch.Tensor] = None, mix=None):
    """RMS norm in 32-bit: ``n = v / sqrt(mean(v^2) + eps) * (offset + w)`` with ``v = x`` or ``x * silu(gate)``,
    each of ``groups`` equal parts of a row by its own mean square; with ``residual`` (32-bit) the result is
    ``residual + mult * n``.  ``x`` is 32-bit or of the compute type ``dtype`` and its rows may lie apart, as may
    the gate's.  Returns ``(narrow, wide)``: the result in ``dtype`` and in 32-bit (each None unless wanted;
    ``out_wide``: where to write the 32-bit result).  In a 32-bit model the two are one tensor.

    ``mix = (planes, coef, count)``: ``out_wide`` is plane ``count - 1`` of ``planes`` ``[>= count, rows, features]``
    (32-bit), and the launch goes on to ``sum_j coef[j] * planes[j]`` over the first ``count`` planes, in order, as
    ``depth_mix`` forms it; ``(narrow, wide)`` are then that sum's."""
    H = w.numel()
    _need(w, "weight", torch.float32, (H,))
    x_wide = x.dtype == torch.float32
    if not x_wide and x.dtype != dtype:
        raise KernelError(f"x must be 32-bit or {dtype}, got {x.dtype}")
    x_ld = _rows_of(x, "x", H)
    gate_ld = 0 if gate is None else _rows_of(gate, "gate", H, dtype)
    if rows is not None:
        _need(rows, "rows", torch.int32)
        M = rows.numel()
    else:
        M = x.shape[0]
    if gate is not None and gate.shape[0] != x.shape[0]:
        raise KernelError("gate and x differ in their number of rows")
    if residual is not None:
        _need(residual, "residual", torch.float32, (x.shape[0], H))
    if H % groups:
        raise KernelError(f"{H} features do not split into {groups} equal groups")
    f32 = dtype == torch.float32
    if out_wide is not None:
        _need(out_wide, "out_wide", torch.float32, (M, H))
        want_wide = True
    elif want_wide or (f32 and want_narrow):
        out_wide = torch.empty((M, H), dtype=torch.float32, device=x.device)
    narrow = None
    if want_narrow and not f32:
        narrow = torch.empty((M, H), dtype=dtype, device=x.device)
    planes = coef = mix_wide = None
    count = 0
    if mix is not None:
        planes, coef, count = mix
        _need(planes, "planes", torch.float32)
        _need(coef, "coef", torch.float32, (count,))
        if (planes.dim() != 3 or tuple(planes.shape[1:]) != (M, H) or not (0 < count <= planes.shape[0]) or rows is not None
                or out_wide is None or out_wide.data_ptr() != planes[count - 1].data_ptr()):
            raise KernelError("a sum of streams needs planes [at least count, rows, features] whose plane count - 1 is out_wide")
        mix_wide = torch.empty((M, H), dtype=torch.float32, device=x.device)
    if M:
        _call("pta_rmsnorm", _ptr(narrow), _ptr(out_wide), _ptr(x), int(x_wide), ctypes.c_long(x_ld), _ptr(gate),
              ctypes.c_long(gate_ld), _ptr(rows), _ptr(w), ctypes.c_float(offset), int(groups), ctypes.c_float(eps),
              _ptr(residual), ctypes.c_float(mult), _ptr(planes), ctypes.c_long(M * H), _ptr(coef), int(count),
              _ptr(mix_wide), M, H, dtype_code(dtype), _stream())
    if mix is not None:
        return (mix_wide if f32 else narrow), mix_wide
    if f32:
        return (out_wide if want_narrow else None), (out_wide if want_wide else None)
    return narrow, (out_wide if want_wide else None)


def depth_mix(planes: torch.Tensor, coef: torch.Tensor, count: int, dtype: torch.dtype):
    """``sum_j coef[j] * planes[j]`` over the first ``count`` planes of ``[planes, rows, features]`` (32-bit), added
    in that order; returns ``(narrow, wide)``: the sum in ``dtype`` and in 32-bit (one tensor in a 32-bit model)."""
    _need(planes, "planes", torch.float32)
    if planes.dim() != 3 or not (0 < count <= planes.shape[0]):
        raise KernelError(f"planes must be [at least {count}, rows, features], got {tuple(planes.shape)}")
    _need(coef, "coef", torch.float32, (count,))
    _, M, H = planes.shape
    wide = torch.empty((M, H), dtype=torch.float32, device=planes.device)
    narrow = None if dtype == torch.float32 else torch.empty((M, H), dtype=dtype, device=planes.device)
    if M:
        _call("pta_depth_mix", _ptr(wide), _ptr(narrow), _ptr(planes), ctypes.c_long(M * H), _ptr(coef), int(count),
              ctypes.c_long(M * H), dtype_code(dtype), _stream())
    return (wide if narrow is None else narrow), wide


def widen(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x`` (compute type) as 32-bit, into ``out`` if given."""
    _need(x, "x")
    if out is None:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _need(out, "out", torch.float32, tuple(x.shape))
    if x.numel():
        _call("pta_widen", _ptr(out), _ptr(x), ctypes.c_long(x.numel()), dtype_code(x.dtype), _stream())
    return out


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """In place: ``x *= factor`` (32-bit)."""
    _need(x, "x", torch.float32)
    if x.numel() and factor != 1.0:
        _call("pta_scale_f32", _ptr(x), ctypes.c_float(factor), ctypes.c_long(x.numel()), _stream())
    return x


# ---- layers with a state of fixed size per sequence -------------------------------------------------------------
def _need_state(state: torch.Tensor, row: int, name: str = "state") -> int:
    """A state table ``[slots, >= row]`` in 32-bit whose rows may lie apart; returns the row distance."""
    if not (isinstance(state, torch.Tensor) and state.is_cuda and state.dtype == torch.float32 and state.dim() == 2
            and state.stride(1) == 1 and state.shape[1] >= row):
        raise KernelError(f"{name} must be a 32-bit GPU table [slots, at least {row}] with adjacent columns")
    return int(state.stride(0))


SCAN_CHUNK_TOKENS = 64  # a sequence that brings more than twice as many tokens is cut into chunks that run side by side


def gated_scan(zxg: torch.Tensor, bz, bx, state: torch.Tensor, cu_tokens: torch.Tensor, seq_slot: torch.Tensor,
               max_new: int = 1) -> torch.Tensor:
    """The gated recurrence ``S = (1 - z) S + z c`` over every sequence's tokens of the step, from and into its row
    of ``state`` ``[slots, W]``: ``zxg`` ``[tokens, 3 W]`` holds the gate's and the candidate's pre-activations
    (biases ``bz``, ``bx`` still to add) and the output gate; returns ``S * silu(g)`` ``[tokens, W]``."""
    if zxg.dim() != 2 or zxg.shape[1] % 3:
        raise KernelError(f"zxg must be [tokens, 3 * width], got {tuple(zxg.shape)}")
    M, W = zxg.shape[0], zxg.shape[1] // 3
    ld = _rows_of(zxg, "zxg", 3 * W)
    for name, b in (("bz", bz), ("bx", bx)):
        if b is not None:
            _need(b, name, torch.float32, (W,))
    n = seq_slot.numel()
    _need(seq_slot, "seq_slot", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    state_ld = _need_state(state, W)
    y = torch.empty((M, W), dtype=zxg.dtype, device=zxg.device)
    timing_hint["rows"] = M
    chunk, chunks = SCAN_CHUNK_TOKENS, 1
    if max_new > 2 * chunk:  # (``max_new``: the most tokens any sequence brings)
        chunks = (int(max_new) + chunk - 1) // chunk
    chunk_state = chunk_decay = None
    if chunks > 1:
        chunk_state = torch.empty((n * chunks, W), dtype=torch.float32, device=zxg.device)
        chunk_decay = torch.empty((n * chunks, W), dtype=torch.float32, device=zxg.device)
    if M:
        _call("pta_gated_scan", _ptr(y), _ptr(zxg), ctypes.c_long(ld), _ptr(bz), _ptr(bx), _ptr(state),
              ctypes.c_long(state_ld), _ptr(chunk_state), _ptr(chunk_decay), _ptr(cu_tokens), _ptr(seq_slot), n, W, chunk,
              chunks, dtype_code(zxg.dtype), _stream())
    return y


def conv_silu(x: torch.Tensor, w: torch.Tensor, b, tail: torch.Tensor, cu_tokens, token_seq, seq_slot) -> torch.Tensor:
    """``silu`` of a causal convolution per channel over each sequence's tokens: ``w`` ``[channels, taps]`` (the last
    tap is the token's own), ``b`` ``[channels]`` or None; ``tail`` ``[slots, (taps - 1) * channels]`` holds every
    sequence's last inputs from before the step and is moved on.  ``x`` ``[tokens, channels]`` may be a block of
    columns; the result is 32-bit."""
    C, K = w.shape
    _need(w, "w", torch.float32)
    if b is not None:
        _need(b, "b", torch.float32, (C,))
    M = x.shape[0]
    ld = _rows_of(x, "x", C)
    n = seq_slot.numel()
    _need(seq_slot, "seq_slot", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    tail_ld = _need_state(tail, (K - 1) * C, "tail")
    out = torch.empty((M, C), dtype=torch.float32, device=x.device)
    if M:
        _call("pta_conv_silu", _ptr(out), _ptr(x), ctypes.c_long(ld), _ptr(w), _ptr(b), _ptr(tail), ctypes.c_long(tail_ld),
              _ptr(cu_tokens), _ptr(token_seq), _ptr(seq_slot), n, M, C, K, dtype_code(x.dtype), _stream())
    return out


SSM_CHUNK_TOKENS = 128  # a sequence that brings more than twice as many tokens is cut into chunks that run side by side


def ssm_scan(xbc: torch.Tensor, dt: torch.Tensor, dt_bias, a_log, d_skip, state: torch.Tensor, cu_tokens, seq_slot,
             heads: int, head_dim: int, state_rows: int, groups: int, max_new: int = 1) -> torch.Tensor:
    """The state-space recurrence per head over every sequence's tokens, from and into its row of ``state``
    ``[slots, heads * state_rows * head_dim]``: ``xbc`` ``[tokens, heads * head_dim + 2 * groups * state_rows]``
    (32-bit: inputs, then B, then C per group), ``dt`` ``[tokens, heads]`` (compute type, may be a block of
    columns; softplus and ``dt_bias`` are applied here).  ``max_new``: the most tokens any sequence brings; long
    sequences are walked in chunks side by side (the same sums in another order).  Returns y ``[tokens, heads *
    head_dim]`` in 32-bit."""
    inner = heads * head_dim
    C = inner + 2 * groups * state_rows
    M = xbc.shape[0]
    _need(xbc, "xbc", torch.float32, (M, C))
    dt_ld = _rows_of(dt, "dt", heads)
    for name, t in (("dt_bias", dt_bias), ("A_log", a_log), ("D", d_skip)):
        _need(t, name, torch.float32, (heads,))
    n = seq_slot.numel()
    _need(seq_slot, "seq_slot", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    state_ld = _need_state(state, heads * state_rows * head_dim)
    y = torch.empty((M, inner), dtype=torch.float32, device=xbc.device)
    timing_hint["rows"] = M
    chunk, chunks = SSM_CHUNK_TOKENS, 1
    if max_new > 2 * chunk:
        chunks = (int(max_new) + chunk - 1) // chunk
    chunk_state = chunk_decay = None
    if chunks > 1:
        chunk_state = torch.empty((n * chunks, heads, state_rows, head_dim), dtype=torch.float32, device=xbc.device)
        chunk_decay = torch.empty((n * chunks, heads), dtype=torch.float32, device=xbc.device)
    if M:
        _call("pta_ssm_scan", _ptr(y), _ptr(xbc), _ptr(dt), ctypes.c_long(dt_ld), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip),
              _ptr(state), ctypes.c_long(state_ld), _ptr(chunk_state), _ptr(chunk_decay), _ptr(cu_tokens), _ptr(seq_slot),
              n, heads, head_dim, state_rows, groups, chunk, chunks, dtype_code(dt.dtype), _stream())
    return y


# ---- attention over a cache of latents ---------------------------------------------------------------------------
def latent_sizes_problem(heads: int, dim: int, rot_dim: int, rank: int) -> Optional[str]:
    """None if the latent attention launches take these sizes, else why not."""
    lib = load_library()
    if lib.pta_attn_latent_sizes_ok(int(heads), int(dim), int(rot_dim), int(rank)) == 0:
        return None
    return lib.pta_last_error().decode("utf-8", "replace")


def latent_prep(proj: torch.Tensor, w_norm: torch.Tensor, eps: float, inv_freq, cs_scale: float, rotary_dim, pairing: str,
                token_pos, token_seq, block_table, k_pool, heads: int, dim: int, rot_dim: int, rank: int,
                write_cache: bool = True, q: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From ``proj`` ``[tokens, heads * (dim + rot_dim) + rank + rot_dim]`` (the queries, then the down-projection), or
    with the queries ``q`` ``[tokens, heads * (dim + rot_dim)]`` given apart from ``proj`` ``[tokens, rank + rot_dim]``
    (each may be a block of columns): the normed latent and the rotated shared key part go into the token's cache row
    ``[rank + rot_dim]``; returns the queries' frame ``[tokens, heads, rank + rot_dim]`` in 32-bit with the rotated
    parts filled in (the first ``rank`` of each head are for ``head_project``)."""
    M = proj.shape[0]
    q_cols = heads * (dim + rot_dim)
    if q is None:
        ld = _rows_of(proj, "proj", q_cols + rank + rot_dim)
        q_ptr, q_ld, down_ptr = proj.data_ptr(), ld, proj.data_ptr() + q_cols * proj.element_size()
    else:
        ld = _rows_of(proj, "proj", rank + rot_dim)
        q_ld = _rows_of(q, "q", q_cols, proj.dtype)
        q_ptr, down_ptr = q.data_ptr(), proj.data_ptr()
    _need(w_norm, "w_norm", torch.float32, (rank,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(block_table, "block_table", torch.int32)
    D = rank + rot_dim
    _need(k_pool, "k_pool", proj.dtype)
    if k_pool.dim() != 4 or tuple(k_pool.shape[1:]) != (1, 64, D):
        raise KernelError(f"k_pool must be [pages, 1, 64, {D}], got {tuple(k_pool.shape)}")
    rot = _rotation_arg(inv_freq, cs_scale, rot_dim, block_table.shape[0], rotary_dim, pairing) if rot_dim else None
    q_full = torch.empty((M, heads, D), dtype=torch.float32, device=proj.device)
    if M:
        _call("pta_latent_prep", _ptr(q_full), _ptr(k_pool), ctypes.c_void_p(q_ptr), ctypes.c_long(q_ld),
              ctypes.c_void_p(down_ptr), ctypes.c_long(ld), _ptr(w_norm),
              ctypes.c_float(eps), rot, _ptr(token_pos), _ptr(token_seq), _ptr(block_table), block_table.shape[1], M,
              heads, dim, rot_dim, rank, int(write_cache), dtype_code(proj.dtype), _stream())
    return q_full


def head_project(x: torch.Tensor, x_head: int, w: torch.Tensor, heads: int, K: int, O: int,
                 out: Optional[torch.Tensor] = None, out_head: Optional[int] = None, out_dtype=None) -> torch.Tensor:
    """A product per head: ``out[t, h, :O] = x[t, h, :K] @ W_h`` with ``w`` ``[heads, K, O]`` (a head's rows are its
    inputs).  ``x`` is ``[tokens, >= heads * x_head]`` (rows may lie apart; head h starts at column ``h * x_head``),
    32-bit or of w's type.  The result goes to ``out`` ``[tokens, >= heads * out_head]`` if given (32-bit or w's
    type), else to a new ``[tokens, heads * O]`` of ``out_dtype`` (default w's type)."""
    _need(w, "w", None, (heads, K, O))
    M = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1 or not x.is_cuda or x.shape[1] < (heads - 1) * x_head + K:
        raise KernelError(f"x {tuple(x.shape)} does not hold {heads} heads of {K} elements {x_head} apart")
    if x.dtype not in (torch.float32, w.dtype):
        raise KernelError(f"x must be 32-bit or {w.dtype}, got {x.dtype}")
    if out is None:
        out_head = O
        out = torch.empty((M, heads * O), dtype=out_dtype or w.dtype, device=x.device)
    if out.dim() != 2 or out.stride(1) != 1 or out.shape[0] != M or out.shape[1] < (heads - 1) * out_head + O:
        raise KernelError(f"out {tuple(out.shape)} does not hold {heads} heads of {O} elements {out_head} apart")
    if out.dtype not in (torch.float32, w.dtype):
        raise KernelError(f"out must be 32-bit or {w.dtype}, got {out.dtype}")
    if M:
        _call("pta_head_project", _ptr(out), int(out.dtype == torch.float32), ctypes.c_long(out.stride(0)),
              ctypes.c_long(out_head), _ptr(x), int(x.dtype == torch.float32), ctypes.c_long(x.stride(0)),
              ctypes.c_long(x_head), _ptr(w), M, heads, K, O, dtype_code(w.dtype), _stream())
    return out


HEAD_PROJECT_LIBRARY_ROWS = 0  # bfloat16 steps of more tokens run their per-head products in the vendor library


def head_project_library(x3: torch.Tensor, w: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """The same products for many tokens through the vendor library's batched product: ``x3`` ``[tokens, heads, K]``
    (any strides) and ``w`` ``[heads, K, O]``, both bfloat16 -> ``[heads, tokens, O]``."""
    M, H, K = x3.shape
    with timed("library_mm", float(w.numel()) * 2, 2.0 * M * H * K * w.shape[2]):
        if out_dtype is None or out_dtype == x3.dtype:
            return torch.bmm(x3.transpose(0, 1), w)
        return torch.bmm(x3.transpose(0, 1), w, out_dtype=out_dtype)


LATENT_MFMA = os.environ.get("PTA_LATENT_MFMA", "1") != "0"
LATENT_SPLIT_WORKGROUPS = 1024  # a decode launch cuts its keys into ranges until it has about so many workgroups


def attn_latent_mfma_ok(k_pool: torch.Tensor, rank: int) -> bool:
    """Whether the matrix-core kernel takes this cache (bfloat16, a size class built for its rows)."""
    return (LATENT_MFMA and k_pool.dtype == torch.bfloat16
            and bool(load_library().pta_attn_latent_mfma_ok(int(rank), int(k_pool.shape[-1]))))


def latent_decode_split(n_seqs: int, heads: int, max_len: int):
    """(keys per range, ranges) of a decode launch: ranges of a multiple of 64 keys, enough of them to fill the chip."""
    tiles = (heads + 63) // 64
    want = max(1, min((max_len + 63) // 64, LATENT_SPLIT_WORKGROUPS // max(1, n_seqs * tiles)))
    size = ((max_len + want - 1) // want + 63) // 64 * 64
    return size, (max_len + size - 1) // size


def attn_latent(q_full: torch.Tensor, k_pool: torch.Tensor, block_table, token_seq, token_pos, rank: int,
                scale: float, ctx=None) -> torch.Tensor:
    """Causal attention of every token over its sequence's cache rows ``[rank + rot_dim]``, whose first ``rank``
    elements are also the values: ``q_full`` ``[tokens, heads, rank + rot_dim]`` (32-bit) -> ``[tokens, heads,
    rank]`` (32-bit).  With the step's context (``ctx``) and a bfloat16 cache of a size that is built, the kernel on
    the matrix cores runs, its keys cut into ranges when every sequence brings one token; else the 32-bit kernel."""
    _need(q_full, "q_full", torch.float32)
    M, H, D = q_full.shape
    if k_pool.dim() != 4 or tuple(k_pool.shape[1:]) != (1, 64, D) or not k_pool.is_cuda or not k_pool.is_contiguous():
        raise KernelError(f"k_pool must be [pages, 1, 64, {D}], got {tuple(k_pool.shape)}")
    _need(block_table, "block_table", torch.int32)
    _need(token_seq, "token_seq", torch.int32, (M,))
    _need(token_pos, "token_pos", torch.int32, (M,))
    out = torch.empty((M, H, rank), dtype=torch.float32, device=q_full.device)
    if M == 0:
        return out
    if ctx is not None and attn_latent_mfma_ok(k_pool, rank):
        n = block_table.shape[0]
        _need(ctx.cu_tokens, "cu_tokens", torch.int32, (n + 1,))
        _need(ctx.seq_start, "seq_start", torch.int32, (n,))
        size, splits = latent_decode_split(n, H, ctx.max_len) if ctx.is_decode else (0, 1)
        po = pm = pl = None
        if splits > 1:
            po = torch.empty((M, H, splits, rank), dtype=torch.float32, device=q_full.device)
            pm = torch.empty((M, H, splits), dtype=torch.float32, device=q_full.device)
            pl = torch.empty((M, H, splits), dtype=torch.float32, device=q_full.device)
        _call("pta_attn_latent_mfma", _ptr(out), _ptr(po), _ptr(pm), _ptr(pl), _ptr(q_full), _ptr(k_pool), _ptr(block_table),
              block_table.shape[1], _ptr(ctx.cu_tokens), _ptr(ctx.seq_start), n, int(max(ctx.new_tokens)), M, H, int(rank),
              D - int(rank), ctypes.c_float(scale), int(size), int(splits), _stream())
        return out
    _call("pta_attn_latent", _ptr(out), _ptr(q_full), _ptr(k_pool), _ptr(block_table), block_table.shape[1],
          _ptr(token_seq), _ptr(token_pos), M, H, int(rank), D - int(rank), ctypes.c_float(scale),
          dtype_code(k_pool.dtype), _stream())
    return out


# ---- a 32-bit stream with a token-shifted norm at the head of a block ---------------------------------------------
def shift_norm(base: torch.Tensor, terms, w1: torch.Tensor, w2: Optional[torch.Tensor], mu: torch.Tensor, eps: float,
               state: torch.Tensor, ctx, dtype: torch.dtype):
    """The stream ``x = base + sum(terms)`` (32-bit; ``terms``: up to two tensors of the compute type that a block
    left), its norm with ``w1`` mixed with the token before's by ``mu`` (``n1 + (n1' - n1) * mu``; the token before
    a step's first is the sequence's row of ``state``, which is moved on to the step's last), and its norm with
    ``w2`` (None: none).  Returns ``(x, shifted, second norm or None)``, the last two in ``dtype``."""
    M, H = base.shape
    _need(base, "base", torch.float32, (M, H))
    terms = [t for t in terms if t is not None]
    if len(terms) > 2:
        raise KernelError(f"at most two terms are added to the stream, got {len(terms)}")
    for t in terms:
        _need(t, "term", dtype, (M, H))
    for name, t in (("w1", w1), ("mu", mu)) + ((("w2", w2),) if w2 is not None else ()):
        _need(t, name, torch.float32, (H,))
    state_ld = _need_state(state, H)
    n = ctx.seq_slot.numel()
    _need(ctx.token_seq, "token_seq", torch.int32, (M,))
    _need(ctx.token_pos, "token_pos", torch.int32, (M,))
    _need(ctx.cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    x = torch.empty_like(base) if terms else None
    a = torch.empty((M, H), dtype=dtype, device=base.device)
    m = torch.empty((M, H), dtype=dtype, device=base.device) if w2 is not None else None
    _call("pta_shift_norm", _ptr(a), _ptr(m), _ptr(x), _ptr(base), _ptr(terms[0] if terms else None),
          _ptr(terms[1] if len(terms) > 1 else None), _ptr(w1), _ptr(w2), _ptr(mu), _ptr(state), ctypes.c_long(state_ld),
          _ptr(ctx.token_seq), _ptr(ctx.token_pos), _ptr(ctx.cu_tokens), _ptr(ctx.seq_slot), n, M, H, ctypes.c_float(eps),
          int(max(ctx.new_tokens) > 1), dtype_code(dtype), _stream())
    return (x if terms else base), a, m


def wide_sum(base: torch.Tensor, terms) -> torch.Tensor:
    """``base + sum(terms)`` in 32-bit (``terms``: one or two tensors of one type, 32-bit or bfloat16)."""
    terms = [t for t in terms if t is not None]
    if not terms:
        return base
    _need(base, "base", torch.float32)
    for t in terms:
        _need(t, "term", terms[0].dtype, tuple(base.shape))
    out = torch.empty_like(base)
    _call("pta_wide_sum", _ptr(out), _ptr(base), _ptr(terms[0]), _ptr(terms[1] if len(terms) > 1 else None),
          ctypes.c_long(base.numel()), dtype_code(terms[0].dtype), _stream())
    return out


# ---- normed heads into attention ------------------------------------------------------------------------------------
def head_norm_rope_cache(q_in: torch.Tensor, k_in: torch.Tensor, v_in: torch.Tensor, q_w, k_w, eps: float, v_norm: bool,
                         rotation, ctx, block_table, k_pool, v_pool, nh: int, nkv: int, dk: int, dv: int,
                         write_cache: bool = True) -> torch.Tensor:
    """Queries ``[M, nh, D]`` from ``q_in`` ``[M, nh * dk]``; keys (``k_in`` ``[M, nkv * dk]``) and values (``v_in``
    ``[M, nkv * dv]``) go to the cache pages, whose heads have D >= max(dk, dv) elements (what lies past a head's own
    is written as zeros).  The three inputs are blocks of columns of one product.  Every query and key head is
    divided by its root mean square (+ ``eps`` inside the root) and multiplied by ``q_w`` / ``k_w`` ``[dk]`` (None:
    left as it is), then rotated (``rotation``: a ``parts.positions.Rotation`` or None); every value head is
    divided by its root mean square if ``v_norm``."""
    M = q_in.shape[0]
    dt = q_in.dtype
    ld = _rows_of(q_in, "q_in", nh * dk, dt)
    if _rows_of(k_in, "k_in", nkv * dk, dt) != ld or _rows_of(v_in, "v_in", nkv * dv, dt) != ld:
        if M > 1:
            raise KernelError("queries, keys and values must be blocks of columns of one matrix")
    D = k_pool.shape[-1]
    _need_pools(k_pool, v_pool, dt, nkv, D)
    for name, t in (("q_w", q_w), ("k_w", k_w)):
        if t is not None:
            _need(t, name, torch.float32, (dk,))
    _need(block_table, "block_table", torch.int32)
    rot = None
    if rotation is not None:
        rot = _rotation_arg(rotation.inv_freq, rotation.scale, dk, block_table.shape[0], rotation.rotary_dim, rotation.pairing)
    q = torch.empty((M, nh, D), dtype=dt, device=q_in.device)
    _call("pta_head_norm_rope_cache", _ptr(q), _ptr(q_in), _ptr(k_in), _ptr(v_in), ctypes.c_long(ld), _ptr(q_w), _ptr(k_w),
          ctypes.c_float(eps), int(bool(v_norm)), rot, _ptr(ctx.token_pos), _ptr(ctx.token_seq), _ptr(block_table),
          block_table.shape[1], _ptr(k_pool), _ptr(v_pool), M, nh, nkv, dk, dv, D, int(write_cache), dtype_code(dt), _stream())
    return q


# ---- gates between two products -------------------------------------------------------------------------------------
GLU_CODES = {"silu": 0, "clamped": 1}


def gated_heads(x: torch.Tensor, x_head: int, g: torch.Tensor, heads: int, dv: int, dtype: torch.dtype,
                w: Optional[torch.Tensor] = None, eps: float = 0.0, per_head: bool = False) -> torch.Tensor:
    """``n(x) * sigmoid(g)`` ``[M, heads * dv]`` in ``dtype``: ``x`` (32-bit or ``dtype``) holds heads of ``dv``
    elements in frames ``x_head`` apart; n is an RMS norm over the row of all heads with the weight ``w``, or the
    identity (``w`` None); ``g`` ``[M, heads * dv]`` (``dtype``) may be a block of columns.  ``per_head``: the gate is
    one number a head, ``g`` ``[M, heads]``."""
    M = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < (heads - 1) * x_head + dv or x.dtype not in (torch.float32, dtype):
        raise KernelError(f"x must be [M, at least {(heads - 1) * x_head + dv}] in 32-bit or {dtype}")
    g_ld = _rows_of(g, "g", heads if per_head else heads * dv, dtype)
    if w is not None:
        _need(w, "w", torch.float32, (heads * dv,))
    out = torch.empty((M, heads * dv), dtype=dtype, device=x.device)
    if M:
        _call("pta_gated_heads", _ptr(out), _ptr(x), int(x.dtype == torch.float32), ctypes.c_long(x.stride(0)), int(x_head),
              _ptr(g), ctypes.c_long(g_ld), _ptr(w), ctypes.c_float(eps), M, heads, dv, int(bool(per_head)), dtype_code(dtype),
              _stream())
    return out


def xielu(z: torch.Tensor, act: torch.Tensor) -> torch.Tensor:
    """xIELU element by element: with ``ap = softplus(act[0])`` and ``an = 1/2 + softplus(act[1])`` (``act``: two learned
    numbers, 32-bit), ``ap z^2 + z / 2`` for z > 0 and ``an (e^z - 1 - z) + z / 2`` else; ``z`` may be a block of columns."""
    M, F = z.shape
    ld = _rows_of(z, "z", F)
    _need(act, "act", torch.float32, (2,))
    out = torch.empty((M, F), dtype=z.dtype, device=z.device)
    if M:
        _call("pta_xielu", _ptr(out), _ptr(z), ctypes.c_long(ld), M, F, _ptr(act), dtype_code(z.dtype), _stream())
    return out


def glu(gate: torch.Tensor, up: torch.Tensor, kind: str = "silu", alpha: float = 1.0, limit: float = 0.0) -> torch.Tensor:
    """``silu(gate) * up`` (``"silu"``), or with ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``:
    ``g * sigmoid(alpha * g) * (u + 1)`` (``"clamped"``); gate and up are blocks of columns of one product."""
    M, F = gate.shape
    ld = _rows_of(gate, "gate", F)
    if _rows_of(up, "up", F, gate.dtype) != ld and M > 1:
        raise KernelError("gate and up must be blocks of columns of one matrix")
    out = torch.empty((M, F), dtype=gate.dtype, device=gate.device)
    if M:
        _call("pta_glu", _ptr(out), _ptr(gate), _ptr(up), ctypes.c_long(ld), M, F, GLU_CODES[kind], ctypes.c_float(alpha),
              ctypes.c_float(limit), dtype_code(gate.dtype), _stream())
    return out


# ---- linear attention with a decay per head -------------------------------------------------------------------------
DECAY_SCAN_CHUNK_TOKENS = 64  # a sequence that brings more than twice as many tokens is cut into chunks that run side by side


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor, cu_tokens,
               seq_slot, heads: int, key_dim: int, value_dim: int, act: Optional[str] = "silu", max_new: int = 1) -> torch.Tensor:
    """Per head ``S <- decay[h] S + k v^T``, ``o = S^T q`` over every sequence's tokens, from and into its row of
    ``state`` ``[slots, heads * key_dim * value_dim]`` (32-bit); ``q``, ``k`` ``[tokens, heads * key_dim]`` and ``v``
    ``[tokens, heads * value_dim]`` are blocks of columns of one product in the compute type, and ``act`` is applied
    to them on the way in.  Returns o ``[tokens, heads * value_dim]`` in 32-bit."""
    M = q.shape[0]
    ld = _rows_of(q, "q", heads * key_dim)
    if (_rows_of(k, "k", heads * key_dim, q.dtype) != ld or _rows_of(v, "v", heads * value_dim, q.dtype) != ld) and M > 1:
        raise KernelError("q, k and v must be blocks of columns of one matrix")
    _need(decay, "decay", torch.float32, (heads,))
    n = seq_slot.numel()
    _need(seq_slot, "seq_slot", torch.int32, (n,))
    _need(cu_tokens, "cu_tokens", torch.int32, (n + 1,))
    state_ld = _need_state(state, heads * key_dim * value_dim)
    y = torch.empty((M, heads * value_dim), dtype=torch.float32, device=q.device)
    timing_hint["rows"] = M
    chunk, chunks = DECAY_SCAN_CHUNK_TOKENS, 1
    if max_new > 2 * chunk:
        chunks = (int(max_new) + chunk - 1) // chunk
    chunk_state = None
    if chunks > 1:
        chunk_state = torch.empty((n * chunks, heads, key_dim, value_dim), dtype=torch.float32, device=q.device)
    if M:
        _call("pta_decay_scan", _ptr(y), _ptr(q), _ptr(k), _ptr(v), ctypes.c_long(ld), _ptr(decay), _ptr(state),
              ctypes.c_long(state_ld), _ptr(chunk_state), _ptr(cu_tokens), _ptr(seq_slot), n, heads, value_dim, key_dim,
              ACT_CODES[act], chunk, chunks, dtype_code(q.dtype), _stream())
    return y


# ---- routed experts ---------------------------------------------------------------------------------------------------
ROUTE_SCORE_CODES = {"sigmoid": 0, "softmax": 1}


def moe_route(h: torch.Tensor, router: torch.Tensor, top: int, score: str = "sigmoid", normalise: bool = True,
              scale: float = 1.0, bias: Optional[torch.Tensor] = None, groups: int = 1, keep: int = 1,
              extra: Optional[torch.Tensor] = None):
    """Per token the ``top`` experts with the largest scores of ``router @ h`` (+ ``bias``; 32-bit; ``router``
    ``[experts, features]`` and ``bias`` ``[experts]`` 32-bit) and their weights: ``(ids [M, top] int32, weights [M,
    top] 32-bit)``.  With ``groups`` > 1 the experts form that many equal runs of neighbours, a run's score is its
    largest, and only experts of the ``keep`` best runs can be taken.  ``extra`` ``[rows, features]`` (32-bit): the
    launch also forms ``sigmoid(extra @ h)`` ``[M, rows]`` in 32-bit, returned as a third value."""
    M, H = h.shape
    E = router.shape[0]
    _need(router, "router", torch.float32, (E, H))
    if bias is not None:
        _need(bias, "router bias", torch.float32, (E,))
    ld = _rows_of(h, "h", H)
    ids = torch.empty((M, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((M, top), dtype=torch.float32, device=h.device)
    gates, X = None, 0
    if extra is not None:
        X = extra.shape[0]
        _need(extra, "extra", torch.float32, (X, H))
        gates = torch.empty((M, X), dtype=torch.float32, device=h.device)
    if M:
        _call("pta_moe_route", _ptr(ids), _ptr(wts), _ptr(h), ctypes.c_long(ld), _ptr(router), _ptr(bias), M, H, E, int(top),
              ROUTE_SCORE_CODES[score], int(bool(normalise)), ctypes.c_float(scale), int(groups), int(keep), _ptr(extra),
              _ptr(gates), int(X), dtype_code(h.dtype), _stream())
    return (ids, wts) if extra is None else (ids, wts, gates)


MOE_GROUPED_FROM_ROWS = 16  # steps of more tokens run their experts on the matrix cores (bfloat16)


def moe_experts(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor,
                act: str = "silu", gate=None, gated: bool = True, extra: Optional[torch.Tensor] = None,
                extra_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``sum_k wts[m, k] * down[e] (act(gate[e] h) * (up[e] h))`` with ``e = ids[m, k]``: ``gate_up`` ``[experts, 2 F,
    features]`` (an expert's gate rows, then its up rows), ``down`` ``[experts, features, F]``; out ``[M, features]``.
    ``gate = (kind, alpha, limit)`` of ``GLU_CODES``: with ``"clamped"`` an expert's two products meet as ``glu`` says
    in place of ``act(g) * u``.  ``gated=False``: experts without a gate, ``down[e] act(up[e] h)``, with ``gate_up`` their
    one input matrix ``[experts, F, features]``.  ``extra`` ``[M, features]`` with ``extra_gate`` ``[M, 1]`` (32-bit, rows
    may lie apart): ``extra_gate[m] * extra[m]`` is added in the launch that sums the experts."""
    how = None
    if gate is not None:
        how = ctypes.byref(_PtaGate(GLU_CODES[gate[0]], float(gate[1]), float(gate[2])))
    M, H = h.shape
    E, F2, _ = gate_up.shape
    F = F2 // 2 if gated else F2
    top = ids.shape[1]
    _need(gate_up, "gate_up", h.dtype, (E, (2 if gated else 1) * F, H))
    _need(down, "down", h.dtype, (E, H, F))
    _need(ids, "ids", torch.int32, (M, top))
    _need(wts, "wts", torch.float32, (M, top))
    ld = _rows_of(h, "h", H, h.dtype)
    gate_ld = 0
    if extra is not None:
        _need(extra, "extra", h.dtype, (M, H))
        gate_ld = _rows_of(extra_gate, "extra_gate", 1, torch.float32)
    out = torch.empty((M, H), dtype=h.dtype, device=h.device)
    timing_hint["experts"] = E
    if (h.dtype == torch.bfloat16 and M > MOE_GROUPED_FROM_ROWS and H % 64 == 0 and F % 64 == 0 and ld % 8 == 0
            and h.data_ptr() % 16 == 0):
        # many tokens: the pairs sorted by expert, tiles of one expert's tokens on the matrix cores
        slots = load_library().pta_moe_grouped_slots(M * top, E)
        ints = torch.empty(slots + M * top + slots // 64, dtype=torch.int32, device=h.device)
        act_sorted = torch.empty((slots, F), dtype=h.dtype, device=h.device)
        y_sorted = torch.empty((slots, H), dtype=h.dtype, device=h.device)
        _call("pta_moe_grouped", _ptr(out), _ptr(h), ctypes.c_long(ld), _ptr(gate_up), _ptr(down), _ptr(ids), _ptr(wts),
              _ptr(ints[:slots]), _ptr(ints[slots:slots + M * top]), _ptr(ints[slots + M * top:]), _ptr(act_sorted),
              _ptr(y_sorted), M, H, F, E, top, ACT_CODES[act], how, int(bool(gated)), _ptr(extra), _ptr(extra_gate),
              int(gate_ld), _stream())
        return out
    act_buf = torch.empty((M * top, F), dtype=h.dtype, device=h.device)
    if M:
        _call("pta_moe_up", _ptr(act_buf), _ptr(h), ctypes.c_long(ld), _ptr(gate_up), _ptr(ids), M, H, F, top,
              ACT_CODES[act], how, int(bool(gated)), dtype_code(h.dtype), _stream())
        _call("pta_moe_down", _ptr(out), _ptr(act_buf), _ptr(down), _ptr(ids), _ptr(wts), M, H, F, top, _ptr(extra),
              _ptr(extra_gate), int(gate_ld), dtype_code(h.dtype), _stream())
    return out
