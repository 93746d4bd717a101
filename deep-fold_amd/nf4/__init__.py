"""Packed NF4 linear operators on MI355X: the public operator API.

Same names, argument order and error behaviour as the reference wrapper
(``gpu/nf4/__init__.py:151-372``) and the tensor checks of its binding
(``gpu/nf4/bindings.cpp:35-503``), on top of ``libchr_nf4_amd.so`` — a plain C
ABI loaded with ``ctypes``; torch is only used for device memory and streams.

The kernels never allocate.  ``nf4_gemm`` allocates ``y`` and the split-K
workspace from torch's caching allocator (the graph-private pool under capture);
every GEMV-family call writes into a caller-provided ``out``.

There is no CPU fallback: a missing library or a non-GPU tensor raises.
"""

from __future__ import annotations

import ctypes
import os

import torch

from .plan import LIVE_MAX_N, PLAN_MAX_N, k_pad as _k_pad

__all__ = [
    "ATTN_SPLIT",
    "LIVE_MAX_N",
    "PLAN_MAX_N",
    "nf4_gemm",
    "nf4_gemv",
    "nf4_qkv",
    "nf4_swiglu",
    "nf4_rope_kv",
    "nf4_attn",
    "nf4_rms",
    "nf4_plan",
    "nf4_set_tuning",
    "nf4_dequant",
    "nf4_embed_rows",
    "nf4_quantize",
    "dv2_mark_written",
    "dv2_argmax_commit",
    "dv2_argmax_ws_bytes",
    "dv2_begin_step",
    "ATTN_WG_WAVES",
    "ATTN_CHUNK_WAVES",
    "ATTN_PARTS",
    "ATTN_PART_WAVES",
    "dv2_attn_state_floats",
    "dv2_attn_parts",
    "dv2_gemv_attn",
    "dv2_sumsq_ok",
    "dv2_sumsq_parts",
    "dv2_attn",
    "dv2_rms_cols",
    "dv2_sq_blocks",
    "dv2_rope_kv_cols",
    "dv2_attn_chunk",
    "dv2_swiglu_elems",
    "dv2_add_cols",
    "dv2_gemm_qkv",
    "dv2_gemm_swiglu",
    "library_path",
]

#: KV splits of the decode attention (``gpu/nf4/__init__.py:43``).
ATTN_SPLIT = 32

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
_LIB_PATH = os.path.join(_CSRC, "libchr_nf4_amd.so")
_lib = None


class _Dev(ctypes.Structure):
    """``chr_nf4_dev_t`` (``gpu/include/chr_gpu.h:11-17``)."""

    _fields_ = [
        ("M", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("K_pad", ctypes.c_int32),
        ("packed", ctypes.c_void_p),
        ("scale", ctypes.c_void_p),
    ]


class _Plan(ctypes.Structure):
    """``chr_nf4_plan_t`` (``gpu/include/chr_gpu.h:48-60``)."""

    _fields_ = [
        ("path", ctypes.c_int32),
        ("grid_x", ctypes.c_int32),
        ("grid_y", ctypes.c_int32),
        ("block", ctypes.c_int32),
        ("bm", ctypes.c_int32),
        ("bk", ctypes.c_int32),
        ("n_ktiles", ctypes.c_int32),
        ("tiles_per_split", ctypes.c_int32),
        ("ctas", ctypes.c_int32),
        ("smem_bytes", ctypes.c_int32),
        ("ws_floats", ctypes.c_int64),
    ]


_PLAN_KEYS = tuple(name for name, _ in _Plan._fields_)

#: every symbol ``include/chr_nf4_amd.h`` declares: (name, restype, argtypes)
_P = ctypes.c_void_p
_I = ctypes.c_int32
_F = ctypes.c_float
_DP = ctypes.POINTER(_Dev)
EXPORTS = (
    ("chr_nf4_gemm", ctypes.c_int, [_DP, _P, _P, _I, _P]),
    ("chr_nf4_gemm_plan", ctypes.c_int, [_DP, _I, _I, ctypes.POINTER(_Plan)]),
    ("chr_nf4_gemm_ws", ctypes.c_int, [_DP, _P, _P, _I, _P, ctypes.c_int64, _P]),
    ("chr_nf4_gemm_ws_max", ctypes.c_int, [_DP, _P, _P, _I, _P, ctypes.c_int64, _P, _I]),
    ("chr_nf4_gemm_noalloc", ctypes.c_int, [_DP, _P, _P, _I, _P]),
    ("chr_nf4_gemm_noalloc_max_floats", ctypes.c_int64, []),
    ("chr_nf4_set_tuning", None, [_I, _I, _I]),
    ("chr_nf4_gemm_stream_policy", None, [_I]),
    ("chr_nf4_gemv", ctypes.c_int, [_DP, _P, _P, _P, _P, _P, _F]),
    ("chr_nf4_gemv_qkv", ctypes.c_int, [_DP, _DP, _DP, _P, _P, _P, _P, _P, _P, _P, _P, _P, _F]),
    ("chr_nf4_gemv_swiglu", ctypes.c_int, [_DP, _DP, _P, _P, _P, _P, _F]),
    ("chr_nf4_rope_kv", ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    ("chr_nf4_attn", ctypes.c_int,
     [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _P, _P, _P, _P, _P, _P, _I]),
    ("chr_nf4_rms", ctypes.c_int, [_P, _P, _P, _I, _F, _P]),
    ("chr_nf4_dequant", ctypes.c_int, [_DP, _P, _P]),
    ("chr_nf4_embed_rows", ctypes.c_int, [_DP, _P, _I, _P, _P]),
    ("chr_nf4_quantize", ctypes.c_int, [_P, _DP, _P, _P]),
    ("chr_dv2_begin_step", ctypes.c_int, [_DP, _P, _P, _P, _P, _P, _F, _P, _P]),
    ("chr_dv2_begin_step_sumsq", ctypes.c_int, [_DP, _P, _P, _P, _P, _P, _P]),
    ("chr_dv2_sumsq_parts", ctypes.c_int32, []),
    ("chr_dv2_sumsq_ok", ctypes.c_int32, [_I, _I, _I, _I]),
    ("chr_dv2_gemv_sumsq", ctypes.c_int, [_DP, _P, _P, _P, _P, _P, _F, _P, _P]),
    ("chr_dv2_gemv_qkv_sumsq", ctypes.c_int,
     [_DP, _DP, _DP, _P, _P, _P, _P, _P, _P, _P, _P, _P, _F, _P]),
    ("chr_dv2_gemv_swiglu_sumsq", ctypes.c_int, [_DP, _DP, _P, _P, _P, _P, _F, _P]),
    ("chr_dv2_gemv_attn_sumsq", ctypes.c_int, [_DP, _P, _I, _I, _I, _P, _P, _P, _P]),
    ("chr_dv2_attn", ctypes.c_int,
     [_P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _P, _P, _P, _P, _P, _P, _I]),
    ("chr_dv2_attn_state_floats", ctypes.c_int64, [_I, _I, _I]),
    ("chr_dv2_attn_parts", ctypes.c_int,
     [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _P, _P, _P, _P, _P, _P, _I]),
    ("chr_dv2_gemv_attn", ctypes.c_int, [_DP, _P, _I, _I, _I, _P, _P, _P]),
    ("chr_dv2_rms_cols", ctypes.c_int, [_P, _P, _P, _I, _I, _F, _P]),
    ("chr_dv2_rope_kv_cols", ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    ("chr_dv2_attn_chunk", ctypes.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _P, _I, _I, _I]),
    ("chr_dv2_swiglu_elems", ctypes.c_int, [_P, _P, _P, ctypes.c_int64, _P]),
    ("chr_dv2_add_cols", ctypes.c_int, [_P, _P, _P, _I, _I, _P]),
    ("chr_dv2_gemm_add", ctypes.c_int, [_DP, _P, _P, _I, _P, ctypes.c_int64, _P, _P, _P]),
    ("chr_dv2_gemm_add_sq", ctypes.c_int, [_DP, _P, _P, _I, _P, ctypes.c_int64, _P, _P, _P, _P]),
    ("chr_dv2_sq_rows", ctypes.c_int32, [_I]),
    ("chr_dv2_rms_cols_sq", ctypes.c_int, [_P, _P, _P, _I, _I, ctypes.c_float, _P, _I, _P]),
    ("chr_dv2_gemm_qkv_ws", ctypes.c_int64, [_DP, _DP, _DP, _I]),
    ("chr_dv2_gemm_qkv", ctypes.c_int, [_DP, _DP, _DP, _P, _P, _I, _P, ctypes.c_int64, _P, _P]),
    ("chr_dv2_gemm_swiglu_ws", ctypes.c_int64, [_DP, _DP, _I]),
    ("chr_dv2_gemm_swiglu", ctypes.c_int, [_DP, _DP, _P, _P, _I, _P, ctypes.c_int64, _P]),
    ("chr_dv2_mark_written", ctypes.c_int, [_P, _P, _P]),
    ("chr_dv2_argmax_commit", ctypes.c_int, [_P, _I, _P, _P, _P, _P, _P, _I, _P]),
    ("chr_dv2_argmax_ws_bytes", ctypes.c_int64, []),
    ("chr_dv2_argmax_commit_ws", ctypes.c_int, [_P, _I, _P, _P, _P, _P, _P, _I, _P, ctypes.c_int64, _P]),
    ("chr_nf4_abi_version", ctypes.c_int, []),
)


def library_path() -> str:
    return _LIB_PATH


def _load_ext() -> ctypes.CDLL:
    """Load the HIP library.  torch is imported first so that the library binds
    to the HIP runtime torch already loaded (one runtime per process)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"chr_nf4_amd: {_LIB_PATH} is not built. Run `python -m deepfold_amd.build_ext` "
            "(needs hipcc). There is no CPU fallback."
        )
    lib = ctypes.CDLL(_LIB_PATH)
    for name, restype, argtypes in EXPORTS:
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.chr_nf4_abi_version() != 1:
        raise RuntimeError("chr_nf4_amd: library ABI version mismatch; rebuild it")
    _lib = lib
    return lib


_ERR = {
    0: "ok",
    -1: "null pointer",
    -2: "N out of range (live 1..32, plan 1..64)",
    -3: "invalid M/K or null packed/scale",
    -4: "K_pad != 64*ceil(K/64)",
    -5: "packed or x not 16-byte aligned",
    -6: "HIP launch / func attribute failed",
    -7: "split-K workspace smaller than the plan asked for",
    -8: "this launch cannot serve the sum-of-squares hand-over asked for",
}


def _check_rc(what: str, rc: int) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed ({rc}): {_ERR.get(rc, 'unknown error')}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_packed(packed, scale, M: int, K: int, K_pad: int, name: str = "") -> None:
    pre = f"{name} " if name else ""
    _need(packed.is_cuda and scale.is_cuda, f"{pre}packed/scale must be CUDA tensors")
    _need(packed.dtype == torch.uint8, f"{pre}packed must be uint8")
    _need(scale.dtype == torch.float16, f"{pre}scale must be float16")
    _need(M >= 1 and K >= 1, "M and K must be >= 1")
    want = _k_pad(K)
    _need(K_pad == want, f"{pre}K_pad must be 64*ceil(K/64) = {want}, got {K_pad}")
    # The kernels index packed with stride K_pad/2 up to row M-1 and scale with
    # stride K_pad/64; smaller blobs would be read past their end.
    _need(packed.numel() >= M * (K_pad // 2),
          f"{pre}packed has {packed.numel()} bytes, the kernel reads M*K_pad/2 = {M * (K_pad // 2)}")
    _need(scale.numel() >= M * (K_pad // 64),
          f"{pre}scale has {scale.numel()} elements, the kernel reads M*K_pad/64 = {M * (K_pad // 64)}")


def _dev(packed, scale, M: int, K: int, K_pad: int) -> _Dev:
    return _Dev(int(M), int(K), int(K_pad), packed.data_ptr(), scale.data_ptr())


def _as_kvec(x: torch.Tensor, K: int) -> torch.Tensor:
    """``[K]``, ``[K,1]`` or ``[1,K]`` -> contiguous ``[K]`` (``bindings.cpp:219-234``)."""
    x = x.contiguous()
    if x.dim() == 1:
        _need(x.size(0) == K, "x.size(0) must equal K")
        return x
    _need(x.dim() == 2, "x must be [K], [K,1], or [1,K]")
    if (x.size(0) == K and x.size(1) == 1) or (x.size(0) == 1 and x.size(1) == K):
        return x.view(K)
    raise RuntimeError("x must be [K], [K,1], or [1,K]")


def _opt_bf16(t, numel: int, what: str, exact: bool):
    """Optional tensor -> (keepalive, pointer or None)."""
    if t is None or t.numel() == 0:
        return None, None
    _need(t.is_cuda, f"{what} must be CUDA")
    if exact:
        _need(t.numel() == numel, f"{what} numel must equal {numel}")
    else:
        _need(t.numel() >= numel, f"{what} too small")
    keep = t.contiguous()
    if keep.dtype != torch.bfloat16:
        keep = keep.to(torch.bfloat16)
    return keep, keep.data_ptr()


def _out_vec(out: torch.Tensor, M: int) -> torch.Tensor:
    _need(out is not None, "out must be defined")
    _need(out.is_cuda and out.dtype == torch.bfloat16, "out must be CUDA bfloat16")
    _need(out.numel() >= M, "out too small")
    _need(out.is_contiguous(), "out must be contiguous")
    return out


def nf4_plan(M: int, K: int, N: int = 1, *, K_pad: int | None = None,  # noqa: N803
             have_ws: bool = True) -> dict:
    """The grid ``chr_nf4_gemm`` would launch.  No device memory, no launch
    (``gpu/nf4/__init__.py:341-358``)."""
    kp = _k_pad(K) if K_pad is None else int(K_pad)
    w = _Dev(int(M), int(K), kp, None, None)
    p = _Plan()
    rc = _load_ext().chr_nf4_gemm_plan(ctypes.byref(w), int(N), 1 if have_ws else 0,
                                       ctypes.byref(p))
    _check_rc("chr_nf4_gemm_plan", rc)
    return {k: int(getattr(p, k)) for k in _PLAN_KEYS}


def nf4_set_tuning(path: int = 0, split_k: int = 0, one_wave: int = 0) -> None:
    """Override the planner for this process (``gpu/nf4/__init__.py:361-372``):
    ``split_k`` 0 = auto, >0 forced; ``one_wave`` 0 = this GPU's compute units."""
    _load_ext().chr_nf4_set_tuning(int(path), int(split_k), int(one_wave))


def nf4_gemm_stream_policy(policy: int = 0) -> None:
    """Which prefill launches run the tile whose workgroups finish their rows themselves
    (no reduce launch): 0 where the planner's cost model prefers it to the split tiles (the
    default unless ``CHR_NF4_GEMM_STREAM`` says otherwise), 1 wherever it fits, -1 never.  No
    counterpart in the reference."""
    _load_ext().chr_nf4_gemm_stream_policy(int(policy))


def nf4_gemm(packed: torch.Tensor, scale: torch.Tensor, x: torch.Tensor, M: int, K: int,  # noqa: N803
             K_pad: int, max_n: int = LIVE_MAX_N, *, bias: torch.Tensor | None = None,  # noqa: N803
             residual: torch.Tensor | None = None, colsq: torch.Tensor | None = None):
    """Fused NF4 dequant-MFMA GEMM.  ``x`` is bf16 ``[K, N]`` or ``[K]``; returns
    ``y [M, N]`` (``gpu/nf4/__init__.py:151-176``, ``bindings.cpp:35-97``).  With
    ``bias`` (bf16 ``[M]``) and/or ``residual`` (bf16 ``[M, N]``, N >= 2) the result is
    ``residual + (y + bias)``, written over ``residual``, in the same launches.  With
    ``max_n=64`` chunks of 33..64 columns run too (one pass over the weights).

    With ``colsq`` (fp32, at least ``dv2_sq_blocks(M, N) * N`` elements, N >= 2) the return
    value is ``(y, written)``: ``written`` says whether the launch left the column sums of
    squares of ``y`` there for ``dv2_rms_cols(..., colsq=)`` (it does when it has a split-K
    reduction and N divides 256)."""
    n = 1 if x.dim() == 1 else int(x.size(-1))
    cap = int(max_n)
    if cap < 1 or cap > PLAN_MAX_N:
        raise RuntimeError(f"chr_nf4_gemm: max_n={cap} not in 1..{PLAN_MAX_N}")
    if n < 1 or n > cap:
        raise RuntimeError(f"chr_nf4_gemm: N={n} not in 1..{cap} (host must chunk N>{LIVE_MAX_N})")
    wide = n > LIVE_MAX_N  # the 33..64-column tile: launched by chr_dv2_gemm_add only
    _need(packed.is_cuda and scale.is_cuda and x.is_cuda, "packed, scale, and x must be CUDA tensors")
    _need(x.dtype == torch.bfloat16, "x must be bfloat16")
    M, K, K_pad = int(M), int(K), int(K_pad)
    _check_packed(packed, scale, M, K, K_pad)
    packed = packed.contiguous()
    scale = scale.contiguous()
    x = x.contiguous()
    if x.dim() == 1:
        x = x.unsqueeze(1)
    _need(x.dim() == 2, "x must be [K, N] or [K]")
    _need(x.size(0) == K, "x.size(0) must equal K")
    lib = _load_ext()
    y = torch.empty((M, n), dtype=torch.bfloat16, device=x.device)
    w = _dev(packed, scale, M, K, K_pad)
    p = _Plan()
    _check_rc("chr_nf4_gemm_plan", lib.chr_nf4_gemm_plan(ctypes.byref(w), n, 1, ctypes.byref(p)))
    ws = None
    ws_ptr = None
    if p.ws_floats > 0:
        ws = torch.empty(int(p.ws_floats), dtype=torch.float32, device=x.device)
        ws_ptr = ws.data_ptr()
    if bias is None and residual is None and not wide and colsq is None:
        rc = lib.chr_nf4_gemm_ws_max(ctypes.byref(w), x.data_ptr(), y.data_ptr(), n, ws_ptr,
                                     int(p.ws_floats), _stream(), cap)
        _check_rc("chr_nf4_gemm", rc)
        return y
    _need(n >= 2, "bias/residual ride on the N >= 2 tiles")
    for t, numel, name in ((bias, M, "bias"), (residual, M * n, "residual")):
        _need(t is None or (t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous()
                            and t.numel() == numel), f"{name} must be contiguous CUDA bf16 of {numel} elements")
    if residual is not None:
        y = residual.view(M, n)
    if colsq is not None:
        _need(colsq.is_cuda and colsq.dtype == torch.float32 and colsq.is_contiguous()
              and colsq.numel() >= dv2_sq_blocks(M, n) * n, "colsq must be contiguous CUDA fp32 of "
              f"{dv2_sq_blocks(M, n) * n} elements")
        rc = lib.chr_dv2_gemm_add_sq(ctypes.byref(w), x.data_ptr(), y.data_ptr(), n, ws_ptr,
                                     int(p.ws_floats), None if bias is None else bias.data_ptr(),
                                     None if residual is None else residual.data_ptr(),
                                     colsq.data_ptr(), _stream())
        if rc not in (0, 1):
            _check_rc("chr_dv2_gemm_add_sq", rc)
        return y, rc == 0
    rc = lib.chr_dv2_gemm_add(ctypes.byref(w), x.data_ptr(), y.data_ptr(), n, ws_ptr, int(p.ws_floats),
                              None if bias is None else bias.data_ptr(),
                              None if residual is None else residual.data_ptr(), _stream())
    _check_rc("chr_dv2_gemm_add", rc)
    return y


def dv2_sq_blocks(rows: int, n: int) -> int:
    """Row blocks whose column sums of squares ``nf4_gemm(..., colsq=)`` leaves for an
    ``[rows, n]`` result: ``rows`` over 1024 / n rows per block, so ``blocks * n`` is at most
    ``rows * n * n / 1024 + n`` elements; 0 when ``n`` does not divide 1024."""
    per = int(_load_ext().chr_dv2_sq_rows(int(n)))
    return -(-int(rows) // per) if per > 0 else 0


def dv2_sumsq_parts() -> int:
    """Floats of a sum-of-squares hand-over buffer (``sumsq_in`` / ``sumsq_out`` below)."""
    return int(_load_ext().chr_dv2_sumsq_parts())


def dv2_sumsq_ok(M: int, K: int, K_pad: int, merges_attention: bool = False) -> bool:  # noqa: N803
    """Whether a single-matrix GEMV of this shape runs on a kernel that can write
    ``sumsq_out`` (those that stage x in LDS; it reads the environment switches a launch reads)."""
    return bool(_load_ext().chr_dv2_sumsq_ok(int(M), int(K), int(K_pad), int(bool(merges_attention))))


def _opt_sumsq(t: torch.Tensor | None, what: str):
    """Device pointer of a sum-of-squares hand-over buffer, or None."""
    if t is None:
        return None
    _need(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
          and t.numel() >= dv2_sumsq_parts() and t.data_ptr() % 16 == 0,
          f"{what} must be a contiguous, 16-byte aligned CUDA float32 tensor of dv2_sumsq_parts() elements")
    return t.data_ptr()


def nf4_gemv(packed: torch.Tensor, scale: torch.Tensor, x: torch.Tensor, M: int, K: int,  # noqa: N803
             K_pad: int, out: torch.Tensor | None = None, add: torch.Tensor | None = None,  # noqa: N803
             rms_w: torch.Tensor | None = None, rms_eps: float = 1e-6,
             sumsq_in: torch.Tensor | None = None, sumsq_out: torch.Tensor | None = None) -> torch.Tensor:
    """N=1 GEMV.  ``x`` is bf16 ``[K, 1]`` or ``[K]``; ``y`` is ``[M, 1]``.

    Optional ``out`` is the destination (numel >= M).  Optional ``add`` is a
    residual of numel >= M; ``out`` and ``add`` may alias.  Optional ``rms_w``
    applies RMSNorm(x, rms_w, rms_eps) in the same launch
    (``gpu/nf4/__init__.py:179-206``, ``bindings.cpp:127-204``).

    ``sumsq_out``: the launch also leaves the sum of squares of what it stored, in parts, for
    the launch that normalises ``y``; ``sumsq_in`` (with ``rms_w``): mean(x^2) comes from the
    parts the writer of ``x`` left instead of a sum over ``x`` (``chr_dv2_gemv_sumsq``; no
    reference counterpart)."""
    n = 1 if x.dim() == 1 else int(x.size(-1))
    if n != 1:
        raise RuntimeError(f"chr_nf4_gemv is N=1 only, got N={n}")
    _need(packed.is_cuda and scale.is_cuda and x.is_cuda, "packed, scale, and x must be CUDA tensors")
    _need(x.dtype == torch.bfloat16, "x must be bfloat16")
    M, K, K_pad = int(M), int(K), int(K_pad)
    _check_packed(packed, scale, M, K, K_pad)
    packed = packed.contiguous()
    scale = scale.contiguous()
    x = x.contiguous()
    if x.dim() == 1:
        x = x.unsqueeze(1)
    _need(x.dim() == 2, "x must be [K, 1] or [K]")
    _need(x.size(0) == K, "x.size(0) must equal K")
    _need(x.size(1) == 1, "chr_nf4_gemv is N=1 only")
    if out is not None:
        _need(out.is_cuda and out.dtype == torch.bfloat16, "out must be CUDA bfloat16")
        _need(out.is_contiguous(), "out must be contiguous")
        _need(out.numel() >= M, "out too small")
        y = out
    else:
        y = torch.empty((M, 1), dtype=torch.bfloat16, device=x.device)
    add_keep, add_ptr = _opt_bf16(add, M, "add", exact=False)
    rms_keep, rms_ptr = _opt_bf16(rms_w, K, "rms_w", exact=True)
    w = _dev(packed, scale, M, K, K_pad)
    if sumsq_in is None and sumsq_out is None:
        rc = _load_ext().chr_nf4_gemv(ctypes.byref(w), x.data_ptr(), y.data_ptr(), _stream(), add_ptr,
                                      rms_ptr, float(rms_eps))
        _check_rc("chr_nf4_gemv", rc)
    else:
        rc = _load_ext().chr_dv2_gemv_sumsq(ctypes.byref(w), x.data_ptr(), y.data_ptr(), _stream(),
                                            add_ptr, rms_ptr, float(rms_eps),
                                            _opt_sumsq(sumsq_in, "sumsq_in"),
                                            _opt_sumsq(sumsq_out, "sumsq_out"))
        _check_rc("chr_dv2_gemv_sumsq", rc)
    del add_keep, rms_keep
    return y


def nf4_qkv(q_packed, q_scale, k_packed, k_scale, v_packed, v_scale, x, Mq: int, Mk: int,  # noqa: N803
            Mv: int, K: int, K_pad: int, out_q, out_k, out_v, q_bias=None, k_bias=None,  # noqa: N803
            v_bias=None, rms_w=None, rms_eps: float = 1e-6, sumsq_in=None):
    """One launch: q/k/v GEMVs sharing x.  Writes ``out_*`` (numel >= M)
    (``gpu/nf4/__init__.py:209-257``, ``bindings.cpp:281-324``).  ``sumsq_in``: see ``nf4_gemv``."""
    Mq, Mk, Mv, K, K_pad = int(Mq), int(Mk), int(Mv), int(K), int(K_pad)
    _check_packed(q_packed, q_scale, Mq, K, K_pad, "q")
    _check_packed(k_packed, k_scale, Mk, K, K_pad, "k")
    _check_packed(v_packed, v_scale, Mv, K, K_pad, "v")
    _need(x.is_cuda and x.dtype == torch.bfloat16, "x must be CUDA bf16")
    x = _as_kvec(x, K)
    yq, yk, yv = _out_vec(out_q, Mq), _out_vec(out_k, Mk), _out_vec(out_v, Mv)
    q_packed, q_scale = q_packed.contiguous(), q_scale.contiguous()
    k_packed, k_scale = k_packed.contiguous(), k_scale.contiguous()
    v_packed, v_scale = v_packed.contiguous(), v_scale.contiguous()
    qb_keep, bq = _opt_bf16(q_bias, Mq, "bias", exact=True)
    kb_keep, bk = _opt_bf16(k_bias, Mk, "bias", exact=True)
    vb_keep, bv = _opt_bf16(v_bias, Mv, "bias", exact=True)
    rms_keep, rms_ptr = _opt_bf16(rms_w, K, "rms_w", exact=True)
    q = _dev(q_packed, q_scale, Mq, K, K_pad)
    k = _dev(k_packed, k_scale, Mk, K, K_pad)
    v = _dev(v_packed, v_scale, Mv, K, K_pad)
    if sumsq_in is None:
        rc = _load_ext().chr_nf4_gemv_qkv(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v),
                                          x.data_ptr(), yq.data_ptr(), yk.data_ptr(), yv.data_ptr(),
                                          bq, bk, bv, _stream(), rms_ptr, float(rms_eps))
        _check_rc("chr_nf4_gemv_qkv", rc)
    else:
        rc = _load_ext().chr_dv2_gemv_qkv_sumsq(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v),
                                                x.data_ptr(), yq.data_ptr(), yk.data_ptr(),
                                                yv.data_ptr(), bq, bk, bv, _stream(), rms_ptr,
                                                float(rms_eps), _opt_sumsq(sumsq_in, "sumsq_in"))
        _check_rc("chr_dv2_gemv_qkv_sumsq", rc)
    del qb_keep, kb_keep, vb_keep, rms_keep
    return (yq, yk, yv)


def nf4_swiglu(g_packed, g_scale, u_packed, u_scale, x, M: int, K: int, K_pad: int, out,  # noqa: N803
               rms_w=None, rms_eps: float = 1e-6, sumsq_in=None) -> torch.Tensor:
    """One launch: ``silu(gate @ x) * (up @ x)`` into ``out``
    (``gpu/nf4/__init__.py:260-287``, ``bindings.cpp:326-354``).  ``sumsq_in``: see ``nf4_gemv``."""
    M, K, K_pad = int(M), int(K), int(K_pad)
    _check_packed(g_packed, g_scale, M, K, K_pad, "gate")
    _check_packed(u_packed, u_scale, M, K, K_pad, "up")
    _need(x.is_cuda and x.dtype == torch.bfloat16, "x must be CUDA bf16")
    x = _as_kvec(x, K)
    y = _out_vec(out, M)
    g_packed, g_scale = g_packed.contiguous(), g_scale.contiguous()
    u_packed, u_scale = u_packed.contiguous(), u_scale.contiguous()
    rms_keep, rms_ptr = _opt_bf16(rms_w, K, "rms_w", exact=True)
    g = _dev(g_packed, g_scale, M, K, K_pad)
    u = _dev(u_packed, u_scale, M, K, K_pad)
    if sumsq_in is None:
        rc = _load_ext().chr_nf4_gemv_swiglu(ctypes.byref(g), ctypes.byref(u), x.data_ptr(),
                                             y.data_ptr(), _stream(), rms_ptr, float(rms_eps))
        _check_rc("chr_nf4_gemv_swiglu", rc)
    else:
        rc = _load_ext().chr_dv2_gemv_swiglu_sumsq(ctypes.byref(g), ctypes.byref(u), x.data_ptr(),
                                                   y.data_ptr(), _stream(), rms_ptr, float(rms_eps),
                                                   _opt_sumsq(sumsq_in, "sumsq_in"))
        _check_rc("chr_dv2_gemv_swiglu_sumsq", rc)
    del rms_keep
    return y


def _heads(q: torch.Tensor, hd: int) -> int:
    if q.dim() == 3:
        _need(q.size(0) == 1, "q batch must be 1")
        _need(q.size(2) == hd, "q head_dim")
        return int(q.size(1))
    _need(q.dim() == 2, "q must be [n_q,hd] or [1,n_q,hd]")
    _need(q.size(1) == hd, "q head_dim")
    return int(q.size(0))


def nf4_rope_kv(q, k, v, k_cache, v_cache, cos, sin, position) -> None:
    """In-place RoPE on q, k; write k, v into the caches at device ``position``
    (``gpu/nf4/__init__.py:290-300``, ``bindings.cpp:356-411``)."""
    _need(q.is_cuda and k.is_cuda and v.is_cuda, "q/k/v must be CUDA")
    _need(q.dtype == torch.bfloat16, "q must be bf16")
    for t, name in ((q, "q"), (k, "k"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        _need(t.is_contiguous(), f"{name} must be contiguous (it is written in place)")
    v = v.contiguous()
    cos, sin = cos.contiguous(), sin.contiguous()
    position = position.contiguous()
    _need(position.is_cuda, "position must be CUDA")
    _need(position.numel() == 1, "position must be a scalar")
    _need(position.dtype == torch.int64, "position must be int64")
    _need(k_cache.dim() == 3 and v_cache.dim() == 3, "cache must be [max_seq,n_kv,hd]")
    max_seq, n_kv, hd = (int(s) for s in k_cache.shape)
    _need(tuple(v_cache.shape) == (max_seq, n_kv, hd), "v_cache shape mismatch")
    _need(cos.size(0) == max_seq and cos.size(1) == hd, "cos shape")
    _need(sin.size(0) == max_seq and sin.size(1) == hd, "sin shape")
    n_q = _heads(q, hd)
    for t, name in ((k, "k"), (v, "v")):
        if t.dim() == 3:
            _need(t.size(0) == 1 and t.size(1) == n_kv and t.size(2) == hd, name)
        else:
            _need(t.dim() == 2 and t.size(0) == n_kv and t.size(1) == hd, name)
    rc = _load_ext().chr_nf4_rope_kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), k_cache.data_ptr(),
                                     v_cache.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                     position.data_ptr(), n_q, n_kv, hd, max_seq, _stream())
    _check_rc("chr_nf4_rope_kv", rc)


def nf4_attn(q, k, v, out, valid_len, scale: float, ws=None, n_split: int = ATTN_SPLIT,
             k_act=None, v_act=None, cos=None, sin=None, position=None) -> None:
    """GQA flash-decode.  ``k``/``v`` are caches ``[max_seq, n_kv, hd]``.

    Optional ``k_act``/``v_act`` + RoPE tables write the current slot and rotate q
    (``gpu/nf4/__init__.py:303-336``, ``bindings.cpp:413-487``)."""
    _need(q.is_cuda and k.is_cuda and v.is_cuda and out.is_cuda, "q/k/v/out must be CUDA")
    _need(q.dtype == torch.bfloat16, "q must be bf16")
    q = q.contiguous()
    _need(k.is_contiguous() and v.is_contiguous(), "k/v caches must be contiguous")
    _need(out.is_contiguous(), "out must be contiguous")
    _need(out.dtype == torch.bfloat16, "out must be bf16")
    valid_len = valid_len.contiguous()
    _need(valid_len.is_cuda, "valid_len must be CUDA")
    _need(valid_len.numel() == 1, "valid_len must be a scalar")
    _need(valid_len.dtype == torch.int32, "valid_len must be int32")
    _need(k.dim() == 3 and v.dim() == 3, "cache must be [max_seq,n_kv,hd]")
    max_seq, n_kv, hd = (int(s) for s in k.shape)
    _need(tuple(v.shape) == (max_seq, n_kv, hd), "v cache shape mismatch")
    n_q = _heads(q, hd)
    _need(out.numel() >= n_q * hd, "out too small")
    n_split = int(n_split)
    _need(1 <= n_split <= 64, "n_split must be 1..64")
    need = n_q * n_split * (hd + 2)
    if ws is None:
        ws = torch.empty(need, device=q.device, dtype=torch.float32)
    _need(ws.is_cuda and ws.dtype == torch.float32, "ws must be CUDA fp32")
    ws = ws.contiguous()
    _need(ws.numel() >= need, "attn workspace too small")

    def opt(t):
        if t is None or t.numel() == 0:
            return None, None
        keep = t.contiguous()
        return keep, keep.data_ptr()

    ka_keep, ka = opt(k_act)
    va_keep, va = opt(v_act)
    c_keep, cp = opt(cos)
    s_keep, sp = opt(sin)
    p_keep, pp = None, None
    if position is not None and position.numel() == 1:
        _need(position.is_cuda and position.dtype == torch.int64, "position must be CUDA int64")
        p_keep = position.contiguous()
        pp = p_keep.data_ptr()
    if cp is not None:
        _need(tuple(c_keep.shape[-2:]) == (max_seq, hd), "cos shape")
    if sp is not None:
        _need(tuple(s_keep.shape[-2:]) == (max_seq, hd), "sin shape")
    if ka is not None:
        _need(ka_keep.numel() >= n_kv * hd, "k_act too small")
    if va is not None:
        _need(va_keep.numel() >= n_kv * hd, "v_act too small")
    rc = _load_ext().chr_nf4_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                  valid_len.data_ptr(), ws.data_ptr(), n_q, n_kv, hd, n_split,
                                  float(scale), _stream(), ka, va, cp, sp, pp, max_seq)
    _check_rc("chr_nf4_attn", rc)
    del ka_keep, va_keep, c_keep, s_keep, p_keep


def nf4_rms(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, eps: float) -> None:
    """``y = w * x * rsqrt(mean(x^2)+eps)``.  All numel match
    (``gpu/nf4/__init__.py:336-338``, ``bindings.cpp:489-503``)."""
    _need(x.is_cuda and w.is_cuda and y.is_cuda, "x/w/y must be CUDA")
    _need(x.dtype == torch.bfloat16, "x must be bf16")
    _need(w.dtype == torch.bfloat16, "w must be bf16")
    x = x.contiguous()
    w = w.contiguous()
    _need(y.is_contiguous() and y.dtype == torch.bfloat16, "y must be contiguous bf16")
    n = int(x.numel())
    _need(w.numel() == n and y.numel() == n, "rms numel mismatch")
    rc = _load_ext().chr_nf4_rms(x.data_ptr(), w.data_ptr(), y.data_ptr(), n, float(eps), _stream())
    _check_rc("chr_nf4_rms", rc)


# ---- operators whose reference counterpart is Python / CPU code ---------------
def nf4_dequant(packed: torch.Tensor, scale: torch.Tensor, M: int, K: int, K_pad: int,  # noqa: N803
                out: torch.Tensor | None = None) -> torch.Tensor:
    """``W_hat [M, K]`` fp32 = ``LUT[code] * f32(scale)``, bit for bit what the CPU
    codec decodes (``internal/nf4/nf4.go:85-121``).  A verification tool, not a
    step of the hot path."""
    M, K, K_pad = int(M), int(K), int(K_pad)
    _check_packed(packed, scale, M, K, K_pad)
    packed, scale = packed.contiguous(), scale.contiguous()
    if out is None:
        out = torch.empty((M, K), dtype=torch.float32, device=packed.device)
    _need(out.is_cuda and out.dtype == torch.float32 and out.is_contiguous(), "out must be CUDA fp32")
    _need(out.numel() >= M * K, "out too small")
    w = _dev(packed, scale, M, K, K_pad)
    _check_rc("chr_nf4_dequant", _load_ext().chr_nf4_dequant(ctypes.byref(w), out.data_ptr(), _stream()))
    return out


def nf4_embed_rows(packed: torch.Tensor, scale: torch.Tensor, ids: torch.Tensor, K: int,  # noqa: N803
                   out: torch.Tensor | None = None) -> torch.Tensor:
    """Decode rows ``ids`` of a packed table to bf16 ``[len(ids), K]``; only the
    requested rows are touched (``gpu/host/embedding.py:74-107``)."""
    _need(packed.dim() == 2 and packed.dtype == torch.uint8, "packed must be uint8 [M, K_pad/2]")
    _need(scale.dtype == torch.float16, "scale must be float16")
    M = int(packed.size(0))
    K = int(K)
    K_pad = int(packed.size(1)) * 2
    _check_packed(packed, scale, M, K, K_pad)
    _need(ids.is_cuda and ids.dtype == torch.int64, "ids must be CUDA int64")
    ids = ids.reshape(-1).contiguous()
    n = int(ids.numel())
    _need(n >= 1, "ids must be non-empty")
    if out is None:
        out = torch.empty((n, K), dtype=torch.bfloat16, device=packed.device)
    _need(out.is_cuda and out.dtype == torch.bfloat16 and out.is_contiguous(), "out must be CUDA bf16")
    _need(out.numel() >= n * K, "out too small")
    w = _dev(packed.contiguous(), scale.contiguous(), M, K, K_pad)
    rc = _load_ext().chr_nf4_embed_rows(ctypes.byref(w), ids.data_ptr(), n, out.data_ptr(), _stream())
    _check_rc("chr_nf4_embed_rows", rc)
    return out


def nf4_quantize(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 ``[M, K]`` on the GPU -> (packed uint8 ``[M, K_pad/2]``, scale fp16
    ``[M, K_pad/64]``), the same bits the CPU encoder writes
    (``internal/nf4/nf4.go:46-82,129-185``).  Raises on NaN/Inf like the encoder."""
    _need(w.is_cuda and w.dtype == torch.float32 and w.dim() == 2, "w must be CUDA fp32 [M, K]")
    w = w.contiguous()
    M, K = int(w.size(0)), int(w.size(1))
    _need(M >= 1 and K >= 1, "nf4: empty shape")
    K_pad = _k_pad(K)
    packed = torch.empty((M, K_pad // 2), dtype=torch.uint8, device=w.device)
    scale = torch.empty((M, K_pad // 64), dtype=torch.float16, device=w.device)
    status = torch.zeros(1, dtype=torch.int32, device=w.device)
    d = _dev(packed, scale, M, K, K_pad)
    rc = _load_ext().chr_nf4_quantize(w.data_ptr(), ctypes.byref(d), status.data_ptr(), _stream())
    _check_rc("chr_nf4_quantize", rc)
    if int(status.item()) != 0:
        raise ValueError("nf4: non-finite weight")
    return packed, scale


def dv2_mark_written(position: torch.Tensor, valid_len: torch.Tensor) -> None:
    """``valid_len = position + 1`` on the device (``gpu/decodev2/kv.py:118-120``)."""
    _need(position.is_cuda and position.dtype == torch.int64 and position.numel() == 1,
          "position must be a CUDA int64 scalar")
    _need(valid_len.is_cuda and valid_len.dtype == torch.int32 and valid_len.numel() == 1,
          "valid_len must be a CUDA int32 scalar")
    rc = _load_ext().chr_dv2_mark_written(position.data_ptr(), valid_len.data_ptr(), _stream())
    _check_rc("chr_dv2_mark_written", rc)


def dv2_argmax_commit(logits: torch.Tensor, next_token: torch.Tensor, token: torch.Tensor | None = None,
                      position: torch.Tensor | None = None, finished: torch.Tensor | None = None,
                      eos_id: torch.Tensor | None = None, commit: bool = False,
                      ws: torch.Tensor | None = None) -> None:
    """``next_token = argmax(logits)`` (first maximum wins); with ``commit`` also
    ``token = next``, ``position += 1``, ``finished |= next == eos``
    (``gpu/decodev2/step.py:182``, ``gpu/decodev2/state.py:98-103``).  With ``ws``
    (``dv2_argmax_ws_bytes()`` bytes on the GPU) a large vocabulary is searched by 128
    workgroups and a small second launch instead of one workgroup."""
    _need(logits.is_cuda and logits.dtype == torch.bfloat16 and logits.is_contiguous(),
          "logits must be contiguous CUDA bf16")
    _need(next_token.is_cuda and next_token.dtype == torch.int64 and next_token.numel() == 1,
          "next_token must be a CUDA int64 scalar")
    ptrs = [None, None, None, None]
    if commit:
        _need(token is not None and token.is_cuda and token.dtype == torch.int64, "token must be CUDA int64")
        _need(position is not None and position.is_cuda and position.dtype == torch.int64,
              "position must be CUDA int64")
        _need(finished is not None and finished.is_cuda and finished.dtype == torch.uint8,
              "finished must be CUDA uint8")
        _need(eos_id is not None and eos_id.is_cuda and eos_id.dtype == torch.int64,
              "eos_id must be CUDA int64")
        ptrs = [token.data_ptr(), position.data_ptr(), finished.data_ptr(), eos_id.data_ptr()]
    if ws is not None:
        _need(ws.is_cuda and ws.is_contiguous(), "ws must be a contiguous CUDA tensor")
        rc = _load_ext().chr_dv2_argmax_commit_ws(
            logits.data_ptr(), int(logits.numel()), next_token.data_ptr(), ptrs[0], ptrs[1], ptrs[2],
            ptrs[3], 1 if commit else 0, ws.data_ptr(), int(ws.numel() * ws.element_size()), _stream())
        _check_rc("chr_dv2_argmax_commit_ws", rc)
        return
    rc = _load_ext().chr_dv2_argmax_commit(logits.data_ptr(), int(logits.numel()), next_token.data_ptr(),
                                           ptrs[0], ptrs[1], ptrs[2], ptrs[3], 1 if commit else 0,
                                           _stream())
    _check_rc("chr_dv2_argmax_commit", rc)


def dv2_argmax_ws_bytes() -> int:
    return int(_load_ext().chr_dv2_argmax_ws_bytes())


def dv2_begin_step(packed: torch.Tensor, scale: torch.Tensor, K: int, token: torch.Tensor,  # noqa: N803
                   position: torch.Tensor, valid_len: torch.Tensor, x: torch.Tensor,
                   norm_w: torch.Tensor | None = None, eps: float = 1e-6,
                   h: torch.Tensor | None = None, sumsq_out: torch.Tensor | None = None) -> None:
    """First launch of a decode step: ``valid_len = position + 1``, ``x`` = the packed
    embedding row ``token`` and, with ``norm_w``, ``h = RMSNorm(x, norm_w, eps)``; with
    ``sumsq_out`` (and no ``norm_w``) the sum of squares of ``x`` in parts, see ``nf4_gemv``."""
    M, K, K_pad = int(packed.size(0)), int(K), int(packed.size(1)) * 2
    _check_packed(packed, scale, M, K, K_pad, "embed")
    _need(packed.is_contiguous() and scale.is_contiguous(), "embed blobs must be contiguous")
    for t, dt, name in ((token, torch.int64, "token"), (position, torch.int64, "position"),
                        (valid_len, torch.int32, "valid_len")):
        _need(t.is_cuda and t.dtype == dt and t.numel() == 1, f"{name} must be a CUDA {dt} scalar")
    _need((norm_w is None) == (h is None), "norm_w and h go together")
    for t, name in ((x, "x"), (norm_w, "norm_w"), (h, "h")):
        _need(t is None or (t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous()
                            and t.numel() == K), f"{name} must be contiguous CUDA bf16 with K elements")
    w = _dev(packed, scale, M, K, K_pad)
    if sumsq_out is not None:
        _need(norm_w is None, "sumsq_out goes without norm_w")
        rc = _load_ext().chr_dv2_begin_step_sumsq(ctypes.byref(w), token.data_ptr(), position.data_ptr(),
                                                  valid_len.data_ptr(), x.data_ptr(), _stream(),
                                                  _opt_sumsq(sumsq_out, "sumsq_out"))
        _check_rc("chr_dv2_begin_step_sumsq", rc)
        return
    rc = _load_ext().chr_dv2_begin_step(ctypes.byref(w), token.data_ptr(), position.data_ptr(),
                                        valid_len.data_ptr(), x.data_ptr(),
                                        None if norm_w is None else norm_w.data_ptr(), float(eps),
                                        None if h is None else h.data_ptr(), _stream())
    _check_rc("chr_dv2_begin_step", rc)


#: wavefronts per head of the one-launch attention
ATTN_WG_WAVES = 16


def dv2_attn(q, k, v, out, valid_len, scale: float, n_waves: int = ATTN_WG_WAVES,
             k_act=None, v_act=None, cos=None, sin=None, position=None) -> None:
    """``nf4_attn`` as one launch: a workgroup of ``n_waves`` wavefronts per query head
    merges its own partial softmax states in LDS (no workspace)."""
    _need(q.is_cuda and q.dtype == torch.bfloat16 and q.is_contiguous(), "q must be contiguous CUDA bf16")
    _need(k.is_contiguous() and v.is_contiguous() and k.dim() == 3, "caches must be contiguous [max_seq,n_kv,hd]")
    max_seq, n_kv, hd = (int(t) for t in k.shape)
    n_q = _heads(q, hd)
    _need(out.is_contiguous() and out.dtype == torch.bfloat16 and out.numel() >= n_q * hd, "out too small")
    _need(valid_len.is_cuda and valid_len.dtype == torch.int32 and valid_len.numel() == 1,
          "valid_len must be a CUDA int32 scalar")
    _need(1 <= int(n_waves) <= 16, "n_waves must be in 1..16")

    def ptr(t):
        return None if t is None else t.data_ptr()

    for t in (k_act, v_act, cos, sin, position):
        _need(t is None or (t.is_cuda and t.is_contiguous()), "optional inputs must be contiguous CUDA")
    rc = _load_ext().chr_dv2_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                  valid_len.data_ptr(), n_q, n_kv, hd, int(n_waves), float(scale),
                                  _stream(), ptr(k_act), ptr(v_act), ptr(cos), ptr(sin),
                                  ptr(position), max_seq)
    _check_rc("chr_dv2_attn", rc)


#: workgroups per head and wavefronts per workgroup of the attention that leaves its merge
#: to the o projection
ATTN_PARTS = 4
ATTN_PART_WAVES = 8


def dv2_attn_state_floats(n_q: int, hd: int, n_parts: int = ATTN_PARTS) -> int:
    """fp32 elements ``dv2_attn_parts`` writes for ``n_q`` heads of ``hd`` dims."""
    return int(_load_ext().chr_dv2_attn_state_floats(int(n_q), int(hd), int(n_parts)))


def dv2_attn_parts(q, k, v, valid_len, scale: float, state, n_parts: int = ATTN_PARTS,
                   n_waves: int = ATTN_PART_WAVES, k_act=None, v_act=None, cos=None, sin=None,
                   position=None) -> None:
    """Attention that stops before the merge: ``n_parts`` workgroups per query head leave
    their softmax states in ``state`` (fp32); ``dv2_gemv_attn`` merges them."""
    _need(q.is_cuda and q.dtype == torch.bfloat16 and q.is_contiguous(), "q must be contiguous CUDA bf16")
    _need(k.is_contiguous() and v.is_contiguous() and k.dim() == 3, "caches must be contiguous [max_seq,n_kv,hd]")
    max_seq, n_kv, hd = (int(t) for t in k.shape)
    n_q = _heads(q, hd)
    _need(valid_len.is_cuda and valid_len.dtype == torch.int32 and valid_len.numel() == 1,
          "valid_len must be a CUDA int32 scalar")
    _need(1 <= int(n_waves) <= 16 and 1 <= int(n_parts) <= 64, "n_waves in 1..16, n_parts in 1..64")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous()
          and state.numel() >= n_q * int(n_parts) * (hd + 4), "attention state buffer too small")

    def ptr(t):
        return None if t is None else t.data_ptr()

    for t in (k_act, v_act, cos, sin, position):
        _need(t is None or (t.is_cuda and t.is_contiguous()), "optional inputs must be contiguous CUDA")
    rc = _load_ext().chr_dv2_attn_parts(q.data_ptr(), k.data_ptr(), v.data_ptr(), valid_len.data_ptr(),
                                        state.data_ptr(), n_q, n_kv, hd, int(n_parts), int(n_waves),
                                        float(scale), _stream(), ptr(k_act), ptr(v_act), ptr(cos),
                                        ptr(sin), ptr(position), max_seq)
    _check_rc("chr_dv2_attn_parts", rc)


def dv2_gemv_attn(packed: torch.Tensor, scale: torch.Tensor, state: torch.Tensor, n_q: int, hd: int,
                  M: int, K: int, K_pad: int, out: torch.Tensor, add: torch.Tensor | None = None,  # noqa: N803
                  n_parts: int = ATTN_PARTS, sumsq_out: torch.Tensor | None = None) -> torch.Tensor:
    """``out = W @ merge(state) (+ add)``: the o projection that also merges the softmax
    states of ``dv2_attn_parts``.  ``K == n_q * hd`` and a multiple of 64; ``hd % 8 == 0``.
    ``sumsq_out``: see ``nf4_gemv``."""
    M, K, K_pad = int(M), int(K), int(K_pad)
    _check_packed(packed, scale, M, K, K_pad)
    _need(packed.is_contiguous() and scale.is_contiguous(), "blobs must be contiguous")
    _need(K == int(n_q) * int(hd) and K == K_pad and int(hd) % 8 == 0,
          "K must equal n_q*hd, be a multiple of 64, and hd a multiple of 8")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous()
          and state.numel() >= int(n_q) * int(n_parts) * (int(hd) + 4), "attention state buffer too small")
    for t, name in ((out, "out"), (add, "add")):
        _need(t is None or (t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous()
                            and t.numel() >= M), f"{name} must be contiguous CUDA bf16 with M elements")
    w = _dev(packed, scale, M, K, K_pad)
    if sumsq_out is None:
        rc = _load_ext().chr_dv2_gemv_attn(ctypes.byref(w), state.data_ptr(), int(n_q), int(hd),
                                           int(n_parts), out.data_ptr(),
                                           None if add is None else add.data_ptr(), _stream())
        _check_rc("chr_dv2_gemv_attn", rc)
    else:
        rc = _load_ext().chr_dv2_gemv_attn_sumsq(ctypes.byref(w), state.data_ptr(), int(n_q), int(hd),
                                                 int(n_parts), out.data_ptr(),
                                                 None if add is None else add.data_ptr(), _stream(),
                                                 _opt_sumsq(sumsq_out, "sumsq_out"))
        _check_rc("chr_dv2_gemv_attn_sumsq", rc)
    return out


def _bf16_cuda(t: torch.Tensor, what: str) -> None:
    _need(t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous(),
          f"{what} must be a contiguous CUDA bfloat16 tensor")


def dv2_rms_cols(x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor | None = None,
                 colsq: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm of every column of feature-major ``x [rows, N]`` (N <= 64).  ``colsq``: the
    column sums of squares the launch that produced ``x`` left (``nf4_gemm(..., colsq=)``
    returned ``written``); the tile is then not read a second time for them."""
    _bf16_cuda(x, "x")
    _bf16_cuda(w, "w")
    _need(x.dim() == 2 and w.numel() == x.size(0), "x must be [rows, N] and w hold rows elements")
    if out is None:
        out = torch.empty_like(x)
    _bf16_cuda(out, "out")
    _need(out.shape == x.shape, "out must have x's shape")
    if colsq is not None:
        blocks = dv2_sq_blocks(x.size(0), x.size(1))
        _need(blocks > 0 and colsq.is_cuda and colsq.dtype == torch.float32 and colsq.is_contiguous()
              and colsq.numel() >= blocks * x.size(1), "colsq does not cover x")
        rc = _load_ext().chr_dv2_rms_cols_sq(x.data_ptr(), w.data_ptr(), out.data_ptr(), int(x.size(0)),
                                             int(x.size(1)), float(eps), colsq.data_ptr(), blocks, _stream())
        _check_rc("chr_dv2_rms_cols_sq", rc)
        return out
    rc = _load_ext().chr_dv2_rms_cols(x.data_ptr(), w.data_ptr(), out.data_ptr(), int(x.size(0)),
                                      int(x.size(1)), float(eps), _stream())
    _check_rc("chr_dv2_rms_cols", rc)
    return out


def dv2_rope_kv_cols(q, k, v, q_out, k_cache, v_cache, cos, sin, start) -> None:
    """RoPE of feature-major ``q [n_q*hd, N]`` / ``k [n_kv*hd, N]`` at positions
    ``start + n`` (``start``: CUDA int64 scalar); rotated q goes token-major to
    ``q_out [N, n_q*hd]``, rotated k and ``v`` to the cache rows."""
    for t, name in ((q, "q"), (k, "k"), (v, "v"), (q_out, "q_out"), (k_cache, "k_cache"),
                    (v_cache, "v_cache"), (cos, "cos"), (sin, "sin")):
        _bf16_cuda(t, name)
    _need(k_cache.dim() == 3 and v_cache.shape == k_cache.shape, "caches must be [max_seq, n_kv, hd]")
    max_seq, n_kv, hd = (int(t) for t in k_cache.shape)
    _need(q.dim() == 2 and k.dim() == 2 and v.shape == k.shape, "q, k, v must be [features, N]")
    n = int(q.size(1))
    _need(int(k.size(1)) == n and int(k.size(0)) == n_kv * hd and int(q.size(0)) % hd == 0,
          "q, k, v feature counts must match the caches")
    n_q = int(q.size(0)) // hd
    _need(q_out.numel() >= n * n_q * hd, "q_out too small")
    _need(cos.dim() == 2 and cos.size(1) == hd and cos.size(0) >= max_seq and sin.shape == cos.shape,
          "cos/sin must be [>= max_seq, hd]")
    _need(start.is_cuda and start.dtype == torch.int64 and start.numel() == 1,
          "start must be a CUDA int64 scalar")
    rc = _load_ext().chr_dv2_rope_kv_cols(q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(),
                                          k_cache.data_ptr(), v_cache.data_ptr(), cos.data_ptr(),
                                          sin.data_ptr(), start.data_ptr(), n, n_q, n_kv, hd,
                                          max_seq, _stream())
    _check_rc("chr_dv2_rope_kv_cols", rc)


#: wavefronts per (head, token) workgroup of the chunk attention: a chunk launches n_q * N
#: workgroups, so small ones fill the card better than the decode step's 16 (measured at 40
#: heads x 64 tokens: 30 vs 56 us at 256 cached rows, 172 vs 215 us at 2048)
ATTN_CHUNK_WAVES = 4


def dv2_attn_chunk(q, k, v, out, first_len, scale: float, n_waves: int = ATTN_CHUNK_WAVES,
                   feature_major: bool = True) -> None:
    """Causal attention of a chunk: token ``t`` of ``q [N, n_q*hd]`` sees cache rows
    ``0 .. first_len + t - 1``.  ``out`` is ``[n_q*hd, N]`` when ``feature_major`` else
    ``[N, n_q*hd]``."""
    _bf16_cuda(q, "q")
    _bf16_cuda(out, "out")
    _need(k.is_contiguous() and v.is_contiguous() and k.dim() == 3 and k.dtype == torch.bfloat16
          and v.dtype == torch.bfloat16 and v.shape == k.shape, "caches must be contiguous bf16 [max_seq,n_kv,hd]")
    max_seq, n_kv, hd = (int(t) for t in k.shape)
    _need(q.dim() == 2 and int(q.size(1)) % hd == 0, "q must be [N, n_q*hd]")
    n, n_q = int(q.size(0)), int(q.size(1)) // hd
    _need(out.numel() == n * n_q * hd, "out must hold N*n_q*hd elements")
    _need(first_len.is_cuda and first_len.dtype == torch.int32 and first_len.numel() == 1,
          "first_len must be a CUDA int32 scalar")
    _need(1 <= int(n_waves) <= 16, "n_waves must be in 1..16")
    strides = (1, n) if feature_major else (n_q * hd, 1)
    rc = _load_ext().chr_dv2_attn_chunk(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                        first_len.data_ptr(), n, n_q, n_kv, hd, int(n_waves),
                                        float(scale), _stream(), max_seq, strides[0], strides[1])
    _check_rc("chr_dv2_attn_chunk", rc)


def dv2_swiglu_elems(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(gate) * up`` elementwise on bf16 tensors of one shape."""
    _bf16_cuda(gate, "gate")
    _bf16_cuda(up, "up")
    _need(gate.shape == up.shape, "gate and up must have one shape")
    if out is None:
        out = torch.empty_like(gate)
    _bf16_cuda(out, "out")
    _need(out.numel() == gate.numel(), "out must have gate's size")
    rc = _load_ext().chr_dv2_swiglu_elems(gate.data_ptr(), up.data_ptr(), out.data_ptr(),
                                          int(gate.numel()), _stream())
    _check_rc("chr_dv2_swiglu_elems", rc)
    return out


def dv2_add_cols(y: torch.Tensor, a: torch.Tensor | None = None, bias: torch.Tensor | None = None) -> torch.Tensor:
    """In place on feature-major ``y [rows, N]``: ``y += a (+ bias[row])`` or ``y += bias[row]``."""
    _bf16_cuda(y, "y")
    _need(y.dim() == 2, "y must be [rows, N]")
    _need(a is not None or bias is not None, "give a, bias or both")
    if a is not None:
        _bf16_cuda(a, "a")
        _need(a.shape == y.shape, "a must have y's shape")
    if bias is not None:
        _bf16_cuda(bias, "bias")
        _need(bias.numel() == y.size(0), "bias must hold rows elements")
    rc = _load_ext().chr_dv2_add_cols(y.data_ptr(), None if a is None else a.data_ptr(),
                                      None if bias is None else bias.data_ptr(), int(y.size(0)),
                                      int(y.size(1)), _stream())
    _check_rc("chr_dv2_add_cols", rc)
    return y


def dv2_gemm_qkv(q, k, v, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """One launch for q, k and v of a layer: ``q``, ``k``, ``v`` are ``(packed, scale, M)``
    triples over the same ``K``; ``x`` is bf16 ``[K, N]``, N = 2..64.  Returns
    ``[Mq + Mk + Mv, N]`` (q's rows first) with ``bias`` (stacked, bf16) added per row."""
    _bf16_cuda(x, "x")
    _need(x.dim() == 2 and 2 <= x.size(1) <= PLAN_MAX_N, f"x must be [K, N] with N in 2..{PLAN_MAX_N}")
    K, n = int(x.size(0)), int(x.size(1))
    kp = _k_pad(K)
    devs = []
    for name, (packed, scale, M) in (("q", q), ("k", k), ("v", v)):
        _check_packed(packed, scale, int(M), K, kp, name)
        _need(packed.is_contiguous() and scale.is_contiguous(), f"{name} blobs must be contiguous")
        devs.append(_dev(packed, scale, int(M), K, kp))
    m_all = sum(d.M for d in devs)
    if bias is not None:
        _bf16_cuda(bias, "bias")
        _need(bias.numel() == m_all, f"bias must hold {m_all} elements")
    lib = _load_ext()
    need = int(lib.chr_dv2_gemm_qkv_ws(ctypes.byref(devs[0]), ctypes.byref(devs[1]), ctypes.byref(devs[2]), n))
    _need(need >= 0, "chr_dv2_gemm_qkv_ws refused the shapes")
    ws = torch.empty(max(need, 1), dtype=torch.float32, device=x.device)
    y = torch.empty((m_all, n), dtype=torch.bfloat16, device=x.device)
    rc = lib.chr_dv2_gemm_qkv(ctypes.byref(devs[0]), ctypes.byref(devs[1]), ctypes.byref(devs[2]),
                              x.data_ptr(), y.data_ptr(), n, ws.data_ptr() if need else None, need,
                              None if bias is None else bias.data_ptr(), _stream())
    _check_rc("chr_dv2_gemm_qkv", rc)
    return y


def dv2_gemm_swiglu(gate, up, x: torch.Tensor) -> torch.Tensor:
    """``silu(gate @ x) * (up @ x)`` in one GEMM launch and its reduce; ``gate`` and ``up`` are
    ``(packed, scale, M)`` triples of one shape; ``x`` is bf16 ``[K, N]``, N = 2..64."""
    _bf16_cuda(x, "x")
    _need(x.dim() == 2 and 2 <= x.size(1) <= PLAN_MAX_N, f"x must be [K, N] with N in 2..{PLAN_MAX_N}")
    K, n = int(x.size(0)), int(x.size(1))
    kp = _k_pad(K)
    devs = []
    for name, (packed, scale, M) in (("gate", gate), ("up", up)):
        _check_packed(packed, scale, int(M), K, kp, name)
        _need(packed.is_contiguous() and scale.is_contiguous(), f"{name} blobs must be contiguous")
        devs.append(_dev(packed, scale, int(M), K, kp))
    _need(devs[0].M == devs[1].M, "gate and up must have the same number of rows")
    lib = _load_ext()
    need = int(lib.chr_dv2_gemm_swiglu_ws(ctypes.byref(devs[0]), ctypes.byref(devs[1]), n))
    _need(need >= 0, "chr_dv2_gemm_swiglu_ws refused the shapes")
    # (0: the launch pairs gate and up rows inside the tile and stores the activation itself)
    ws = torch.empty(need, dtype=torch.float32, device=x.device) if need > 0 else None
    y = torch.empty((devs[0].M, n), dtype=torch.bfloat16, device=x.device)
    rc = lib.chr_dv2_gemm_swiglu(ctypes.byref(devs[0]), ctypes.byref(devs[1]), x.data_ptr(), y.data_ptr(),
                                 n, None if ws is None else ws.data_ptr(), need, _stream())
    _check_rc("chr_dv2_gemm_swiglu", rc)
    return y
