"""Typed Python faces of the HIP kernels.

Each function checks what the kernel assumes about its operands (device, dtype, contiguity,
shapes) on the host before the launch, and raises `KernelError` with the kernel's own message
when it refuses a size.  Nothing here computes on the CPU or through a tensor library: a missing
library or a CPU tensor is an error.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from .csrc import lib as _libmod

F32 = torch.float32
BF16 = torch.bfloat16
_DT = {torch.float32: 0, torch.bfloat16: 1}
ATT_TILE_TOKENS = 8  # tokens per tile of the prompt-portion attention kernel (ilm_attn_tile_tokens())
ATT_STEP = 128  # keys a workgroup of the chunked attention takes in one step (ilm_attn_mfma_step())
ATT_MAX_CHUNKS = 256  # most chunks a context is cut into (a wave of the merge kernel walks a quarter of them; it takes 512)
BASIC_CHUNK = 512    # keys a chunk of the plain attention kernel (ilm_attn_basic_chunk())
BASIC_SPLIT = os.environ.get("INFINILM_AMD_BASIC_SPLIT", "1") == "1"   # 0: always one wave a (token, head)
BASIC_SPLIT_WAVES = 4096   # (token, head) pairs up to which the plain kernel takes one wave a chunk
F32_ATTN_CHUNK = 128   # keys a chunk of the 32-bit matrix-core attention (ilm_attn_f32_chunk())
F32_ATTN_SPLIT = os.environ.get("INFINILM_AMD_F32_ATTN_SPLIT", "1") == "1"   # 0: always one wave a (token, head group)
F32_ATTN_SPLIT_WAVES = 2048   # (token, head group) pairs up to which it takes one wave a chunk
# INFINILM_AMD_BASIC=1 runs the plain kernels everywhere (for telling a kernel's fault from the engine's)
FORCE_BASIC = os.environ.get("INFINILM_AMD_BASIC", "0") == "1"
SKINNY_VARIANT = int(os.environ.get("INFINILM_AMD_SKINNY_VARIANT", "0"))  # 0: the kernel chooses
USE_KSPLIT = os.environ.get("INFINILM_AMD_KSPLIT", "1") == "1"
USE_LIBRARY_GEMM = os.environ.get("INFINILM_AMD_LIBRARY_GEMM", "1") == "1"


class KernelError(RuntimeError):
    pass


def _lib():
    return _libmod.load()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (the raw lookup costs a tenth of `torch.cuda.current_stream()`,
    which matters with some hundred launches a step)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


# ---- timers per kernel entry point, off unless asked for ------------------------------------------
_TIMES: Optional[dict] = {} if os.environ.get("INFINILM_AMD_KERNEL_TIMES", "0") == "1" else None


def enable_timing(on: bool = True) -> None:
    """Brackets every launch with a pair of events (also: INFINILM_AMD_KERNEL_TIMES=1).  Launches
    inside a graph capture are not timed.  Costs host time; for looking at a step, not for serving."""
    global _TIMES
    _TIMES = {} if on else None


def timing_report(reset: bool = True) -> dict:
    """{entry point: {"calls", "total_ms", "mean_us"}}, after waiting for the device."""
    if _TIMES is None:
        return {}
    torch.cuda.synchronize()
    out = {}
    for name, pairs in _TIMES.items():
        total = sum(a.elapsed_time(b) for a, b in pairs)
        out[name] = {"calls": len(pairs), "total_ms": round(total, 4), "mean_us": round(1e3 * total / max(len(pairs), 1), 2)}
    if reset:
        _TIMES.clear()
    return dict(sorted(out.items(), key=lambda kv: -kv[1]["total_ms"]))


class _timed:
    """Context of one launch; a no-op when timing is off or the stream is being captured."""
    __slots__ = ("name", "start")

    def __init__(self, name: str):
        self.name = name
        self.start = None

    def __enter__(self):
        if _TIMES is not None and not torch.cuda.is_current_stream_capturing():
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if self.start is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _TIMES.setdefault(self.name, []).append((self.start, end))
        return False


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelError("the kernels run on the GPU only; got a CPU tensor")


def _run(name: str, *args, label: Optional[str] = None) -> None:
    """`label`: the name the launch's time is filed under, where one entry point serves uses that are worth telling apart."""
    if _TIMES is None:
        rc = getattr(_lib(), name)(*args)
    else:
        with _timed(label or name):
            rc = getattr(_lib(), name)(*args)
    if rc != 0:
        raise KernelError(_libmod.last_error())


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int) -> int:
    """Keys [pages, nkv, page, d], values transposed [pages, nkv, d, page]; returns the page size."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != d \
            or tuple(v_cache.shape) != (k_cache.shape[0], nkv, d, k_cache.shape[2]) \
            or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError(f"cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} are not "
                          f"[pages, {nkv}, page, {d}] / [pages, {nkv}, {d}, page]")
    return k_cache.shape[2]


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor, got {t.dtype}")


# ------------------------------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """float32 residual rows scale * table[ids]."""
    _dev(ids, table)
    _i32(ids, "ids")
    V, H = table.shape
    if not table.is_contiguous():
        raise KernelError("embedding table must be contiguous")
    T = ids.numel()
    out = torch.empty((T, H), dtype=F32, device=table.device)
    _run("ilm_embed", out.data_ptr(), ids.data_ptr(), table.data_ptr(), T, H, V, float(scale), _dt(table), _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, branch: Optional[torch.Tensor], weight: torch.Tensor,
                alpha: float, eps: float, out_dtype: torch.dtype, frag: bool = False):
    """residual += alpha * branch (in place, float32), then its RMS norm times weight, as out_dtype.
    `frag`: the result comes in fragment order (`FragRows`; bfloat16, at most 64 rows of a multiple of 8 elements),
    for a product that takes it so.

    `branch` is [rows, H] in out_dtype or float32, or [parts, rows, H] (the float32 parts of a K-split
    product, summed in order)."""
    _dev(residual, branch, weight)
    rows, H = residual.shape
    if residual.dtype != F32 or not residual.is_contiguous():
        raise KernelError("the residual stream is a contiguous float32 tensor")
    parts, pstride, h_dt = 1, 0, _DT[out_dtype]
    if branch is not None:
        if branch.dim() == 3:
            parts, pstride = branch.shape[0], branch.stride(0)
        if tuple(branch.shape[-2:]) != (rows, H) or branch.dtype not in (out_dtype, F32) or not branch.is_contiguous():
            raise KernelError(f"branch {tuple(branch.shape)} {branch.dtype} does not match residual "
                              f"{tuple(residual.shape)} / {out_dtype}")
        h_dt = _dt(branch)
    if weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"norm weight has shape {tuple(weight.shape)}, expected ({H},)")
    if frag:
        if out_dtype != BF16 or rows > FRAG_MAX_ROWS or H % 8:
            raise KernelError("a norm's result in fragment order is bfloat16, at most 64 rows of a multiple of 8 elements")
        out = frag_rows_empty(rows, H, residual.device)
        _run("ilm_add_rmsnorm", out.data.data_ptr(), residual.data_ptr(), _ptr(branch), weight.data_ptr(), rows, H,
             float(alpha), float(eps), _DT[out_dtype], _dt(weight), h_dt, parts, pstride, -(-rows // 16), _stream())
        return out
    out = torch.empty((rows, H), dtype=out_dtype, device=residual.device)
    _run("ilm_add_rmsnorm", out.data_ptr(), residual.data_ptr(), _ptr(branch), weight.data_ptr(), rows, H,
         float(alpha), float(eps), _DT[out_dtype], _dt(weight), h_dt, parts, pstride, 0, _stream())
    return out


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                 k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                 slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, rd: int) -> None:
    """Rotates q and k inside the fused projection rows [T, (nh + 2 nkv) d] and writes k, v to the
    paged cache [pages, nkv, page, d] at `slots` (None: no write)."""
    _dev(qkv, positions, cos, sin, k_cache, v_cache, slots)
    _i32(positions, "positions")
    T = qkv.shape[0]
    if qkv.stride(1) != 1 or positions.numel() != T:
        raise KernelError("qkv rows must be dense and positions must have one entry a token")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or (rd > 0 and cos.shape[1] != rd // 2):
        raise KernelError(f"rotation tables must be float32 [positions, {rd // 2}], got {tuple(cos.shape)}")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    _run("ilm_rope_kvwrite", qkv.data_ptr(), positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache),
         _ptr(v_cache), _ptr(slots), T, nh, nkv, d, rd, qkv.stride(0), page, _dt(qkv), _stream())


USE_QKV_ROPE = os.environ.get("INFINILM_AMD_QKV_ROPE", "1") == "1"


def qkv_rope_gemm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                  cos: torch.Tensor, sin: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, rd: int) -> Optional[torch.Tensor]:
    """The fused projection x w^T (+ bias) of a few rows, q and k rotated and k, v written to the cache
    in the product's epilogue.  Returns the rotated q [T, nh*d], or None where the fused kernel does
    not apply (more than 32 rows, float32, a partly rotated or odd-sized head): the caller then
    runs the projection and `rope_kvwrite` one after the other."""
    M, K = x.shape
    if not (USE_QKV_ROPE and not FORCE_BASIC and x.dtype == BF16 and w.dtype == BF16 and _few_rows(M, K) and rd == d and d % 32 == 0
            and K % 8 == 0 and K <= 8192 and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return None
    _dev(x, w, bias, positions, cos, sin, k_cache, v_cache, slots)
    _i32(positions, "positions")
    if w.shape != ((nh + 2 * nkv) * d, K) or positions.numel() != M:
        raise KernelError(f"fused projection {tuple(w.shape)} does not fit {nh}+2*{nkv} heads of {d} over {K}")
    if bias is not None and (bias.shape != (w.shape[0],) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused projection")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or cos.shape[1] != d // 2 \
            or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError(f"rotation tables must be float32 [positions, {d // 2}], got {tuple(cos.shape)}")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != BF16 or v_cache.dtype != BF16:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    q = torch.empty((M, nh * d), dtype=BF16, device=x.device)
    _run("ilm_gemm_qkv_rope", q.data_ptr(), q.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), _ptr(bias),
         M, K, positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache) if slots is not None else None,
         _ptr(v_cache) if slots is not None else None, _ptr(slots), nh, nkv, d, page, _stream())
    return q


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up from rows [gate | up]."""
    _dev(gate_up)
    T, two_i = gate_up.shape
    if two_i % 2 or gate_up.stride(1) != 1:
        raise KernelError("swiglu takes dense rows of even length")
    out = torch.empty((T, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _run("ilm_swiglu", out.data_ptr(), gate_up.data_ptr(), T, two_i // 2, gate_up.stride(0), _dt(gate_up), _stream())
    return out


def gather_rows(x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    _dev(x, idx)
    _i32(idx, "row indices")
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("gather_rows takes a contiguous matrix")
    out = torch.empty((idx.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    _run("ilm_gather_rows", out.data_ptr(), x.data_ptr(), idx.data_ptr(), idx.numel(), x.shape[1], _dt(x), _stream())
    return out


_LIBRARY_F32_OUT = [True]   # cleared when torch.mm refuses out_dtype
KSPLIT_SPAN = 4096  # K range of one part of the K-split few-rows product (ilm_gemm_ksplit_max_k(1))
# Rows up to which the products keep X in registers (16 or 32; 32 only for K up to 4096 a workgroup)
FEW_ROWS = int(os.environ.get("INFINILM_AMD_FEW_ROWS", "32"))


def _few_rows(M: int, K: int) -> bool:
    """Whether the products that keep X in registers take M rows: a wave of eight holds the fragments of K / 8 of one
    group of 16 rows in 4 registers a 32 k, and 256 registers take 16 rows of K up to 8192 or 32 rows of K up to 4096
    beside the W fragments in flight."""
    groups = max(1, min(FEW_ROWS // 16, 8192 // max(K, 4096)))
    return M <= 16 * groups


def _frag_of(frag_w):
    """`frag_w` arguments are a FragWeight, a function that packs one when it is needed, or None."""
    return frag_w() if callable(frag_w) else frag_w


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, alpha: float = 1.0,
         out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
         allow_parts: bool = False, frag_w=None) -> torch.Tensor:
    """alpha * (a w^T + bias); a [M, K] with dense rows, w [N, K]; float accumulation.

    `allow_parts`: the result goes straight into the residual sum (add_rmsnorm), so it may come in
    float32 instead of the activations' dtype, and in parts [P, M, N] that still have to be summed;
    parts are chosen for few rows and long K, where splitting K over workgroups pays."""
    _dev(a, w, bias, out)
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelError(f"gemm shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
    if a.dtype != w.dtype or a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm operands must share a dtype and have dense rows")
    M, K = a.shape
    N = w.shape[0]
    out_dtype = out_dtype or a.dtype
    if bias is not None and (bias.shape != (N,) or bias.dtype != w.dtype or not bias.is_contiguous()):
        raise KernelError(f"bias shape {tuple(bias.shape)} does not fit {N} outputs")
    if out is not None and (out.shape != (M, N) or out.dtype != out_dtype or out.stride(1) != 1):
        raise KernelError("gemm output does not fit")
    fast = a.dtype == BF16 and not FORCE_BASIC
    aligned = K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 \
        and w.data_ptr() % 16 == 0
    plain = bias is None and alpha == 1.0
    # (From 65 rows on the vendor library leaves the chip idle on such products: down projection 68 us at 96 rows, 81
    # at 128, 92 at 160, 114 at 192, 63 at 208; o projection 22, 25, 32 at 192.  Not for small matrices, whose few
    # tiles leave most of the chip idle whatever the split: 0.5B shape at 128 rows 2.22 against 1.96 ms a step with
    # the library.)
    # 17 to 208 rows on their way into the residual sum: chunks of X resident in LDS, two workgroups a compute unit
    # (gemm_tall.hip).  Measured at the 8B shapes against the kernels it took over from: o projection 9.8 us against
    # 10.6 (K ranges of 1024, X in registers) at 32 rows, 11.0 / 12.4 at 64, 12.8 / 17.1 (steps of 64 k, X through LDS, a
    # step's loads waited for before the next step's were issued) at 96, 15.8 / 19.4 at 128, 16.9 / 22.2 at 160; down projection 27.7 / 33.1 (four parts of 4096, X in registers) at
    # 32 rows, 30.3 / 33.3 at 64, 33.7 / 38.1 at 96, 37.1 / 42.0 at 128, 46.2 / 47.1 at 160, 52.0 / 56.7 at 208
    if (fast and aligned and plain and allow_parts and out is None and USE_TALL and TALL_MIN_ROWS <= M <= TALL_MAX_ROWS
            and M > 16 and _tall_fills_the_chip(N, K, a.device)):
        return _gemm_tall(a, w, K, frag_w)
    # 17 to 64 rows on their way into the residual sum: K in ranges of 1024 with the X fragments of all rows
    # in registers (o projection at 64 rows 13.1 against the library's 18.9 us, down projection 33.9
    # against 41.3, of which the sum of its 16 parts takes 5 back; up to 32 rows the down projection
    # stays with the K-split kernel and its 4 parts)
    if (fast and aligned and plain and allow_parts and out is None and 16 < M <= 64
            and -(-K // ROWS64_SPAN) <= ROWS64_MAX_PARTS and (M > FEW_ROWS or K <= KSPLIT_SPAN)):
        kb = -(-K // ROWS64_SPAN)
        parts = torch.empty((kb, M, N), dtype=F32, device=a.device)
        fw = _frag_of(frag_w) if USE_FRAG else None
        if fw is not None:   # W in fragment order: a wave's fragment is 1 KB of consecutive bytes
            _run("ilm_gemm_rows64", parts.data_ptr(), N, M * N, kb, fw.data.data_ptr(), 0, M, N, K, a.data_ptr(),
                 a.stride(0), 1, _stream())
        else:
            _run("ilm_gemm_rows64", parts.data_ptr(), N, M * N, kb, w.data_ptr(), w.stride(0), M, N, K, a.data_ptr(),
                 a.stride(0), 0, _stream())
        return parts
    if fast and aligned and plain and allow_parts and out is None and M <= max(16, FEW_ROWS) and K > KSPLIT_SPAN and USE_KSPLIT:
        kb = -(-K // KSPLIT_SPAN)
        parts = torch.empty((kb, M, N), dtype=F32, device=a.device)
        _run("ilm_gemm_ksplit", parts.data_ptr(), _DT[F32], N, M * N, kb, w.data_ptr(), w.stride(0), None, 1.0,
             M, N, K, a.data_ptr(), a.stride(0), 0, _stream())
        return parts
    few = fast and aligned and _few_rows(M, K)
    if few and allow_parts and out is None:
        out_dtype = F32   # a branch on its way into the float32 residual sum need not be rounded first
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    library_ok = fast and plain and out_dtype == BF16 and USE_LIBRARY_GEMM
    # measured at the 8B shapes: the few-rows kernel with X in registers beats the vendor library (up to
    # 32 rows: gate_up 53 against 62 us, o projection 14 against 18); where X no longer fits the
    # registers it loses (its X fragments are re-read from L2 for every 16 rows of W)
    if (not few and M > 16 and fast and bias is None and out_dtype == F32 and USE_LIBRARY_GEMM and _LIBRARY_F32_OUT[0]
            and M <= 65535):
        # bfloat16 operands, float32 accumulation and result (the output head with many rows)
        try:
            with _timed("library_gemm"):
                torch.mm(a, w.t(), out_dtype=F32, out=out)
        except (TypeError, RuntimeError) as exc:
            if "out_dtype" not in str(exc):
                raise
            _LIBRARY_F32_OUT[0] = False   # this build of the library door has no float32 result
        else:
            if alpha != 1.0:
                _run("ilm_scale_rows", out.data_ptr(), M, N, out.stride(0), float(alpha), _stream())
            return out
    if fast and aligned and M <= 64 and (few or not library_ok):
        _run("ilm_gemm_skinny", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _DT[out_dtype], SKINNY_VARIANT, _stream())
        return out
    if M > 16 and fast and bias is not None and alpha == 1.0 and out_dtype == BF16 and USE_LIBRARY_GEMM:
        # many rows with a bias: the vendor library's product with the bias row as its addend
        with _timed("library_gemm"):
            torch.addmm(bias, a, w.t(), out=out)
        return out
    if M > 16 and library_ok:
        # large products go to the vendor library, as the reference's linear layers do
        # (csrc/layers/quantization/none_quantization.cpp:26-46 calls its library's linear)
        with _timed("library_gemm"):
            torch.matmul(a, w.t(), out=out)
        return out
    if (a.dtype == F32 and out_dtype == F32 and not FORCE_BASIC and M <= F32_FEW_ROWS and K % 4 == 0 and a.stride(0) % 4 == 0
            and w.stride(0) % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        # the 32-bit path's few rows (decoded tokens): W streamed once on the float matrix instruction
        _run("ilm_gemm_f32_skinny", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _stream())
        return out
    if (a.dtype == F32 and out_dtype == F32 and not FORCE_BASIC and F32_FEW_ROWS > 0 and K % 4 == 0 and a.stride(0) % 4 == 0
            and w.stride(0) % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        # the 32-bit path's many rows (portions of prompts): tiles on the float matrix instruction, every
        # output summed in the few-rows kernel's order, so a row's bits do not depend on the rows around it
        _run("ilm_gemm_f32_tile", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _stream())
        return out
    _run("ilm_gemm_basic", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0), w.stride(0),
         out.stride(0), float(alpha), _dt(a), _DT[out_dtype], _stream())
    return out


# Rows up to which the 32-bit products take the few-rows kernel; beyond, the tile kernel that sums in the same
# order (0: neither, always the plain ascending-k kernel)
F32_FEW_ROWS = int(os.environ.get("INFINILM_AMD_F32_FEW_ROWS", "64"))


ROWS64_SPAN = 1024   # K range of one part of the 17-to-64-rows product (ilm_gemm_rows64_span())
ROWS64_MAX_PARTS = int(os.environ.get("INFINILM_AMD_ROWS64_PARTS", "16"))   # 0: never this kernel
TALL_MIN_WGS_PER_CU = 0.25   # the tall product is used where its grid can give more than a quarter of the units a workgroup


def _tall_fills_the_chip(N: int, K: int, device) -> bool:
    """The tall product cuts W into tiles of 128 rows and K into ranges of at least 512: with fewer workgroups
    than a quarter of the compute units whatever the split, the vendor library's product is faster (measured with
    the kernel this one replaced, which cut alike: the 0.5B shape's 1024 x 4096 gives 64 workgroups on 256 units and
    loses, 2.22 against 1.96 ms a step at 128 rows; the 2B-family's 2304 x 2304 gives 72 and wins)."""
    return -(-N // 128) * max(K // 512, 1) > TALL_MIN_WGS_PER_CU * _num_cus(device)


USE_TALL = os.environ.get("INFINILM_AMD_TALL", "1") == "1"
TALL_MIN_ROWS = int(os.environ.get("INFINILM_AMD_TALL_MIN_ROWS", "17"))
TALL_MAX_ROWS = 208   # most rows of X of the products that keep chunks of X in LDS (ilm_gemm_tall_max_rows())
TALL_MAX_PARTS = 16
TALL_GATEUP_MAX_ROWS = 112     # rows up to which the gate/up projection takes that product (beyond: see gateup_swiglu_gemm)


def _tall_plan(M: int, N: int, K: int) -> tuple:
    """(k a chunk, parts, chunks a part) of the tall product with parts: chunks of 128 k and K split so that the launch
    has about a workgroup a compute unit; where a part would then be longer than 1024 k (the down projection), chunks
    of 64 k and two workgroups a unit, up to 128 rows.  Measured at the 8B shapes, down projection: 30.3 us with
    chunks of 64 and 512 workgroups against 32.2 with chunks of 128 and 256 at 64 rows, 33.7 / 35.0 at 96, 37.1 / 42.3
    at 128, 60.7 / 52.0 at 208 (and the step at 160 rows 11.17 against 11.00 ms); o projection 12.5 / 11.0 at 64 rows,
    14.6 / 12.8 at 96."""
    n_tiles = -(-N // 128)

    def split(kc, wgs):
        chunks = -(-K // kc)
        kb = max(1, min(-(-wgs // n_tiles), chunks, TALL_MAX_PARTS))
        cpp = -(-chunks // kb)
        return kc, -(-chunks // cpp), cpp
    plan = split(128, 256)
    if plan[2] > 8 and M <= 128:
        plan = split(64, 512)
    return plan


def _gemm_tall(x: torch.Tensor, w: torch.Tensor, K: int, frag_w=None, plan: Optional[tuple] = None) -> torch.Tensor:
    """17 to 208 rows, result in float32 parts [P, M, N] split over K (see gemm_tall.hip)."""
    M, N = x.shape[0], w.shape[0]
    kc, kb, cpp = plan or _tall_plan(M, N, K)
    parts = torch.empty((kb, M, N), dtype=F32, device=x.device)
    fw = _frag_of(frag_w) if USE_FRAG else None
    if fw is not None:
        _run("ilm_gemm_tall", parts.data_ptr(), N, M * N, kb, cpp, kc, fw.data.data_ptr(), 0, M, N, K, x.data_ptr(), x.stride(0),
             1, _stream())
    else:
        _run("ilm_gemm_tall", parts.data_ptr(), N, M * N, kb, cpp, kc, w.data_ptr(), w.stride(0), M, N, K, x.data_ptr(),
             x.stride(0), 0, _stream())
    return parts


def gemm_tall_swiglu(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], frag_w=None, kc: int = 128) -> torch.Tensor:
    """silu(x Wg^T + bg) * (x Wu^T + bu) for 17 to 208 rows, W = [Wg; Wu] (see gemm_tall.hip)."""
    M, K = x.shape
    inter = w.shape[0] // 2
    act = torch.empty((M, inter), dtype=x.dtype, device=x.device)
    fw = _frag_of(frag_w) if USE_FRAG else None
    if fw is not None:
        _run("ilm_gemm_tall_swiglu", act.data_ptr(), act.stride(0), x.data_ptr(), x.stride(0), fw.data.data_ptr(), 0, _ptr(bias),
             M, inter, K, kc, 1, _stream())
    else:
        _run("ilm_gemm_tall_swiglu", act.data_ptr(), act.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
             _ptr(bias), M, inter, K, kc, 0, _stream())
    return act


USE_GATEUP_SWIGLU = os.environ.get("INFINILM_AMD_GATEUP_SWIGLU", "1") == "1"
# outputs from which the gate/up kernel with X in LDS is used (-1: 48 a compute unit; 0: always, as its tests do)
GATEUP_TALL_MIN_OUTPUTS = int(os.environ.get("INFINILM_AMD_GATEUP_TALL_MIN", "-1"))


# Rows up to which the projection that ends a branch takes the residual sum and the first half of the next
# norm into its epilogue (gemm_tail.hip); 0: never
TAIL_MAX_ROWS = int(os.environ.get("INFINILM_AMD_TAIL_ROWS", "16"))
TAIL_SS_ROWS = 32   # rows of a tile's record of partial sums of squares (ilm_gemm_tail_ss_rows())


def _mfma_operands_ok(x: torch.Tensor, w: torch.Tensor, K: int) -> bool:
    return (x.dtype == BF16 and w.dtype == BF16 and x.is_cuda and w.shape[1] == K and K % 8 == 0 and x.stride(1) == 1
            and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def tail_ok(rows: int, w: torch.Tensor, bias: Optional[torch.Tensor], norm_w: torch.Tensor, dtype: torch.dtype) -> bool:
    """Whether `gemm_tail` takes a product of `rows` rows with the weight w [N, K] (see there)."""
    N, K = w.shape
    return (not FORCE_BASIC and dtype == BF16 and w.dtype == BF16 and 0 < rows <= min(TAIL_MAX_ROWS, 32)
            and (K <= 4096 or (rows <= 16 and K <= 8192)) and K % 8 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0 and norm_w.shape == (N,) and norm_w.dtype in (BF16, F32) and norm_w.is_contiguous()
            and (bias is None or (bias.shape == (N,) and bias.dtype == BF16 and bias.is_contiguous())))


def gemm_tail(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], alpha: float, residual: torch.Tensor,
              norm_w: torch.Tensor):
    """The projection that ends a branch, with the residual sum and the first half of the norm after it
    in its epilogue: residual += alpha * (x w^T + bias) in place (float32 [M, N]); returns (xw, ss) with
    xw = bfloat16(residual * norm_w) [M, N], not yet divided by the rows' root mean square, and ss
    [ceil(N / 16), 32] partial sums of squares of the residual's rows, which the consumer of xw adds up
    (`gateup_swiglu_gemm(..., row_ss=ss, eps=...)`).  For what `tail_ok` accepts."""
    M, K = x.shape
    N = w.shape[0]
    _dev(x, w, bias, residual, norm_w)
    if not (tail_ok(M, w, bias, norm_w, x.dtype) and _mfma_operands_ok(x, w, K)):
        raise KernelError(f"gemm_tail does not take {tuple(x.shape)} x {tuple(w.shape)}^T")
    if residual.dtype != F32 or tuple(residual.shape) != (M, N) or residual.stride(1) != 1:
        raise KernelError("the residual stream is a float32 tensor with dense rows of the product's width")
    xw = torch.empty((M, N), dtype=BF16, device=x.device)
    ss = torch.empty((-(-N // 16), TAIL_SS_ROWS), dtype=F32, device=x.device)
    _run("ilm_gemm_tail", residual.data_ptr(), residual.stride(0), xw.data_ptr(), xw.stride(0), ss.data_ptr(), x.data_ptr(),
         x.stride(0), w.data_ptr(), w.stride(0), _ptr(bias), norm_w.data_ptr(), _dt(norm_w), float(alpha), M, N, K, _stream())
    return xw, ss


def gateup_resident_ok(rows: int, w: torch.Tensor) -> bool:
    """Whether the gate/up kernel that keeps X in registers takes `rows` rows with the weight w [2I, K]."""
    K = w.shape[1]
    return (USE_GATEUP_SWIGLU and not FORCE_BASIC and w.dtype == BF16 and _few_rows(rows, K) and K <= 8192 and K % 8 == 0
            and w.shape[0] % 2 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def gateup_swiglu_gemm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                       row_ss: Optional[torch.Tensor] = None, eps: float = 0.0, frag_w=None) -> Optional[torch.Tensor]:
    """silu(x Wg^T + bg) * (x Wu^T + bu) for few rows in bfloat16, W = [Wg; Wu]: the fused gate/up
    projection with the SwiGLU in its epilogue, [M, I] (up to 32 rows with X in registers; 17 to 208 with chunks
    of X in LDS where the outputs fill the chip).  None where no kernel applies (more rows, few outputs,
    float32): the caller then runs the projection and the activation.  `row_ss`: x is what `gemm_tail` left (residual * norm weight) and row_ss its
    partial sums of squares: the rows' division by sqrt(mean square + eps) happens in this kernel's
    epilogue (only the kernel with X in registers does that: `gateup_resident_ok`)."""
    M, K = x.shape
    resident = _few_rows(M, K) and K <= 8192
    if row_ss is not None:
        if not (resident and gateup_resident_ok(M, w) and _mfma_operands_ok(x, w, K) and row_ss.dtype == F32
                and row_ss.dim() == 2 and row_ss.shape[1] == TAIL_SS_ROWS and row_ss.is_contiguous() and row_ss.is_cuda):
            raise KernelError("a product with the norm's division in its epilogue needs the few-rows gate/up kernel")
    # (a workgroup takes 64 outputs: with fewer outputs than three quarters of the compute units have workgroups
    # the library is faster - measured with the kernel this one replaced, which cut alike: 2B-family shape, 5,760
    # outputs, 64 rows: 6.40 against 6.07 ms a step)
    tall_min = GATEUP_TALL_MIN_OUTPUTS if GATEUP_TALL_MIN_OUTPUTS >= 0 else 48 * _num_cus(x.device)
    # 17 to 112 rows, and up to 176 where the rows are no multiple of 32 (the vendor library's product is then slow):
    # chunks of X resident in LDS, two workgroups a compute unit (gemm_tall.hip).  Measured at the 8B shape: 48.1 us
    # against 52.9 (X in registers, two row groups) at 32 rows, 53.2 against 57.4 (X through LDS in steps of 256 k, one
    # workgroup a unit: the kernel it replaced) at 64; against the library's product and the activation kernel 57.7 / 66.2 at 96, 66.5 / 81.4 at
    # 112, 71.2 / 69.0 at 128, 76.1 / 85.2 at 144, 75.3 / 72.7 at 160, 82.8 / 90.1 at 176, 86.6 / 75.6 at 192, 90.4 / 83.0 at 208
    tall = (USE_TALL and row_ss is None and max(TALL_MIN_ROWS, 17) <= M <= TALL_MAX_ROWS
            and w.shape[0] // 2 >= tall_min and (M <= TALL_GATEUP_MAX_ROWS or (M % 32 != 0 and M <= 176)))
    if not (USE_GATEUP_SWIGLU and not FORCE_BASIC and x.dtype == BF16 and w.dtype == BF16 and x.is_cuda
            and (resident or tall) and K % 8 == 0 and w.shape[0] % 2 == 0 and w.shape[1] == K
            and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return None
    _dev(x, w, bias)
    I = w.shape[0] // 2
    if bias is not None and (bias.shape != (2 * I,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused gate/up projection")
    if tall:
        return gemm_tall_swiglu(x, w, bias, frag_w)
    out = torch.empty((M, I), dtype=BF16, device=x.device)
    _run("ilm_gemm_gateup_swiglu", out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
         _ptr(bias), M, I, K, _ptr(row_ss), 0 if row_ss is None else row_ss.shape[0], float(eps), _stream())
    return out


def swiglu_gemm(gate_up: torch.Tensor, w: torch.Tensor) -> Optional[torch.Tensor]:
    """(silu(gate) * up) w^T for at most 32 rows [gate | up] in bfloat16, in one kernel: float32 parts
    [P, M, N] for add_rmsnorm.  None when the shapes do not fit (the caller then runs the two kernels)."""
    M, two_k = gate_up.shape
    K = two_k // 2
    N = w.shape[0]
    # (above 32 rows the activation would be recomputed by every workgroup along N: the separate kernel
    # and the product with parts are faster, 38 against 42 us at 64 rows)
    ok = (gate_up.dtype == BF16 and w.dtype == BF16 and not FORCE_BASIC and USE_KSPLIT and M <= max(16, FEW_ROWS)
          and two_k % 2 == 0
          and w.shape[1] == K and K % 8 == 0 and gate_up.stride(1) == 1 and w.stride(1) == 1 and gate_up.stride(0) % 8 == 0
          and w.stride(0) % 8 == 0 and gate_up.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and gate_up.is_cuda)
    if not ok:
        return None
    kb = -(-K // KSPLIT_SPAN)
    parts = torch.empty((kb, M, N), dtype=F32, device=gate_up.device)
    _run("ilm_gemm_ksplit", parts.data_ptr(), _DT[F32], N, M * N, kb, w.data_ptr(), w.stride(0), None, 1.0,
         M, N, K, gate_up.data_ptr(), gate_up.stride(0), 1, _stream())
    return parts


_NUM_CUS: dict = {}


def _num_cus(device) -> int:
    """Compute units of the device (looked up once)."""
    cus = _NUM_CUS.get(device)
    if cus is None:
        cus = _NUM_CUS[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return cus


def bound_pages(need: int) -> int:
    """The block-table width a context of `need` pages is served with: 4, 6, 8, 12, 16, 24, ... (at
    most a third above the need).  The step function records one graph a width, and the attention
    kernels size their grids for it, so an eager step and a replayed one cut their keys alike."""
    width = 4
    while width < need:
        width = width * 3 // 2 if width & (width - 1) == 0 else width * 4 // 3
    return width


def bound_rows(rows: int) -> int:
    """The number of rows a decode step of `rows` requests is served with when it is recorded: 1, 2, 4, 8,
    16, 24, 32, 48, 64, 96, 128, 160, 208, 256, 384, 512, ... (the rest are rows of no request).  The sizes end
    where the products change kernels (16, 32, 64 rows; 208, the last size of the product with chunks of X in LDS), so a
    filled-up step runs the kernels the step itself would run and its recording equals the eager step."""
    for b in (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 160, 208, 256):
        if rows <= b:
            return b
    b = 256
    while b < rows:
        b = b * 3 // 2 if b & (b - 1) == 0 else b * 4 // 3
    return b


def attention_chunks(max_total_len: int, page: int, pairs: int, device) -> tuple:
    """(keys a chunk, chunks) of the chunked single-token attention for `pairs` = tokens x head groups.

    A chunk is a whole number of steps of ATT_STEP keys.  Few tokens: one step a chunk (latency
    counts, the chip is not full anyway).  Up to four steps as long as the launch still has a
    workgroup for every compute unit (fewer partial results to write and merge), and beyond that
    while it still has two for each.  Measured at the 8B head shape, 4096 keys, kernel + merge:
    8 tokens 17.0 us with 256 keys a chunk (128: 18.4, 512: 20.2); 16 tokens 22.4 with 512 (256:
    24.0); 32 tokens 34.3 with 512 (256: 40.0, 1024: 36.5); 64 tokens 57.5 with 1024 (512: 60.5).
    At most ATT_MAX_CHUNKS chunks (one token over 32,768 keys: 128 chunks of 256 keys 14.9 us, 64 of 512 18.1).  The length is first rounded up the way the step function rounds
    its graphs' block tables (`bound_pages`), so that an eager step and a replayed one cut alike."""
    bound = bound_pages(-(-max_total_len // page)) * page
    cus = _num_cus(device)
    steps = -(-bound // ATT_STEP)
    pairs = max(pairs, 1)
    workgroups = lambda per_chunk: pairs * -(-steps // per_chunk)
    per_chunk = 1
    for n in (2, 3, 4):
        if workgroups(n) >= cus:
            per_chunk = n
    while per_chunk >= 4 and 2 * per_chunk <= steps and workgroups(2 * per_chunk) >= 2 * cus:
        per_chunk *= 2
    # More workgroups than the chip holds at once (two a compute unit): they run in rounds, and a last round that is
    # nearly empty costs as much as a full one.  Among chunks of a quarter to twice that length take the one with the
    # least rounds x (steps a chunk + a workgroup's fixed cost, about three quarters of a step) + the chunks' merge.
    # Measured at the 8B head shape, 4096 keys, kernel + merge: 80 tokens 80.7 us with 512 keys a chunk (1024: 91.1),
    # 96 tokens 89.1 with 512 (1024: 95.9), 160 tokens 148.4 with 512 (2048: 170.4), 192 tokens 159.0 with 1024
    # (2048: 174.9); 160 tokens over 8192 keys 267.4 with 1024 (4096: 317.7).
    slots = 2 * cus
    if workgroups(per_chunk) > slots:
        def cost(n):
            return -(-workgroups(n) // slots) * (0.75 + n) + 0.15 * -(-steps // n)
        best = per_chunk
        for n in (per_chunk * 2, per_chunk // 2, per_chunk // 4):
            if 2 <= n <= steps and (cost(n), -n) < (cost(best), -best):
                best = n
        per_chunk = best
    while -(-steps // per_chunk) > ATT_MAX_CHUNKS:
        per_chunk += 1
    span = per_chunk * ATT_STEP
    return span, -(-max_total_len // span)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    seg_of_token: torch.Tensor, positions: torch.Tensor, nh: int, nkv: int, d: int,
                    scale: float, window: int = 0, max_total_len: Optional[int] = None,
                    tiles: Optional[torch.Tensor] = None, single_rows: Optional[torch.Tensor] = None,
                    softcap: float = 0.0, float_weights: bool = False) -> torch.Tensor:
    """Attention of every token over its request's cached keys up to its own position.
    `softcap` > 0: scaled scores pass through softcap * tanh(score / softcap) before the softmax.
    `float_weights`: the softmax weights stay float32 in the second product (the bfloat16 matrix-core kernels round them:
    they are passed over, the plain kernel runs).

    q: rows of T tokens in which head h lies at [h*d, (h+1)*d) (a view into the fused projection is
    fine); caches as the cache manager lays them out; block_tables [R, max_blocks]; `max_total_len`: an
    upper bound of position + 1 over the batch (the matrix-core kernel sizes its key chunks by it;
    without it the plain kernel runs).  `tiles` [n, 2] = (first row, count <= ATT_TILE_TOKENS) lists runs of
    consecutive tokens of one request and `single_rows` the remaining rows; without them every token
    is served on its own.  Returns [T, nh*d]."""
    _dev(q, k_cache, v_cache, block_tables, seg_of_token, positions)
    _i32(block_tables, "block_tables")
    _i32(seg_of_token, "seg_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    if q.stride(1) != 1 or q.shape[1] < nh * d:
        raise KernelError("q rows must be dense and hold all query heads")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError(f"cache dtype {k_cache.dtype} differs from the activations' {q.dtype}")
    page = _check_cache(k_cache, v_cache, nkv, d)
    if seg_of_token.numel() != T or positions.numel() != T or block_tables.dim() != 2:
        raise KernelError("per-token metadata does not match the number of tokens")
    out = torch.empty((T, nh * d), dtype=q.dtype, device=q.device)
    if (q.dtype == BF16 and not FORCE_BASIC and not float_weights and d % 16 == 0 and d <= 128 and page % 16 == 0
            and q.stride(0) % 8 == 0 and max_total_len is not None):
        n_single = T
        rows = None
        if tiles is not None and tiles.numel() > 0:
            # portions of prompts: tiles of consecutive tokens share their keys through LDS
            _i32(tiles, "tiles")
            _run("ilm_attn_tile", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                 block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), tiles.data_ptr(),
                 tiles.numel() // 2, nh, nkv, d, page, block_tables.shape[1], q.stride(0), out.stride(0), float(scale),
                 int(window), float(softcap), _stream())
            if single_rows is None or single_rows.numel() == 0:
                return out
            _i32(single_rows, "single_rows")
            rows, n_single = single_rows, single_rows.numel()
        # (the tokens counted as the recorded steps round them, so that an eager step and a replayed one cut alike)
        span, nsplit = attention_chunks(int(max_total_len), page, bound_rows(n_single) * nkv * (-(-(nh // nkv) // 16)), q.device)
        ws_acc = ws_ml = None
        if nsplit > 1:
            # partial results of the rows served here (not of every token of the step)
            ws_acc = torch.empty((n_single * nh * nsplit * d,), dtype=F32, device=q.device)
            ws_ml = torch.empty((n_single * nh * nsplit * 2,), dtype=F32, device=q.device)
        _run("ilm_attn_mfma", out.data_ptr(), _ptr(ws_acc), _ptr(ws_ml), q.data_ptr(), k_cache.data_ptr(),
             v_cache.data_ptr(), block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), _ptr(rows),
             n_single, nh, nkv, d, page, block_tables.shape[1], q.stride(0), out.stride(0), float(scale), int(window),
             nsplit, span, float(softcap), _stream())
        return out
    bound = block_tables.shape[1] * page if max_total_len is None else min(int(max_total_len), block_tables.shape[1] * page)
    if (q.dtype == F32 and not FORCE_BASIC and d % 16 == 0 and d <= 256 and page % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0 and k_cache.data_ptr() % 16 == 0 and v_cache.data_ptr() % 16 == 0):
        # the 32-bit path: the group's heads side by side on the float matrix instruction.  Few tokens (decoding):
        # one wave a chunk of keys and a fold; many: one wave a token that walks its chunks.  The same bits.
        ws, nchunks = None, 1
        waves = T * nkv * -(-(nh // nkv) // 16)
        if F32_ATTN_SPLIT and waves <= F32_ATTN_SPLIT_WAVES and bound > F32_ATTN_CHUNK:
            nchunks = -(-bound // F32_ATTN_CHUNK)
            ws = torch.empty((T * nh * nchunks * (d + 4),), dtype=F32, device=q.device)
        _run("ilm_attn_f32", out.data_ptr(), _ptr(ws), nchunks, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
             block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), T, nh, nkv, d, page,
             block_tables.shape[1], q.stride(0), out.stride(0), float(scale), int(window), float(softcap), _stream())
        return out
    # The plain kernel.  Few tokens over long contexts (decoding): one wave a chunk of keys and a fold of the
    # partial results, instead of one wave a head; the bits are the same (see attn_basic.hip).
    ws, nchunks = None, 1
    if BASIC_SPLIT and T * nh <= BASIC_SPLIT_WAVES and bound > BASIC_CHUNK:
        nchunks = -(-bound // BASIC_CHUNK)
        ws = torch.empty((T * nh * nchunks * (d + 2),), dtype=F32, device=q.device)
    _run("ilm_attn_basic", out.data_ptr(), _ptr(ws), nchunks, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), T, nh, nkv, d, page, block_tables.shape[1],
         q.stride(0), out.stride(0), float(scale), int(window), _dt(q), float(softcap), _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits)
    if logits.dtype != F32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax takes float32 rows")
    n, V = logits.shape
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _run("ilm_argmax", out.data_ptr(), logits.data_ptr(), n, V, logits.stride(0), _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor) -> torch.Tensor:
    """One token a row; per-row temperature (float32), top_k (int32), top_p (float32), u in [0,1)."""
    _dev(logits, temperature, top_k, top_p, uniform)
    if logits.dtype != F32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample takes float32 rows")
    n, V = logits.shape
    _i32(top_k, "top_k")
    for t, nm in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if t.dtype != F32 or t.numel() != n or not t.is_contiguous():
            raise KernelError(f"{nm} must be float32 with one entry a row")
    if top_k.numel() != n:
        raise KernelError("top_k must have one entry a row")
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _run("ilm_sample", out.data_ptr(), logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
         uniform.data_ptr(), n, V, logits.stride(0), _stream())
    return out


# ---- operands in fragment order (csrc/frag.h): the products of a decode step ------------------------------
FRAG_MAX_ROWS = 64    # most rows of X the fragment-order products take
FRAG_SS_ROWS = 64     # rows of a tile's record of partial sums of squares (ilm_gemm_frag_ss_rows())
USE_FRAG = os.environ.get("INFINILM_AMD_FRAG", "1") == "1" and not FORCE_BASIC
FRAG_TILES = int(os.environ.get("INFINILM_AMD_FRAG_TILES", "2"))   # tiles of W a workgroup (2 or 4)


class FragRows:
    """Activations [rows, width] in bfloat16, stored in fragment order (`data`: a flat int32 buffer)."""
    __slots__ = ("data", "rows", "width")

    def __init__(self, data: torch.Tensor, rows: int, width: int):
        self.data, self.rows, self.width = data, int(rows), int(width)

    @property
    def shape(self):
        return (self.rows, self.width)

    @property
    def dtype(self):
        return BF16

    @property
    def device(self):
        return self.data.device


def frag_rows_empty(rows: int, width: int, device) -> FragRows:
    """An uninitialised fragment-order buffer for [rows, width]; the k beyond the width (up to a multiple of 32)
    are zeros, as the products need them."""
    groups, steps = -(-rows // 16), -(-width // 32)
    if width % 32:
        data = torch.zeros((steps * groups * 64 * 4,), dtype=torch.int32, device=device)
    else:
        data = torch.empty((steps * groups * 64 * 4,), dtype=torch.int32, device=device)
    return FragRows(data, rows, width)


def to_frag(x: torch.Tensor) -> FragRows:
    """Plain bfloat16 rows into fragment order (a kernel of its own: for producers that have no such store)."""
    _dev(x)
    M, K = x.shape
    if x.dtype != BF16 or x.stride(1) != 1 or K % 8 or x.stride(0) % 8 or x.data_ptr() % 16:
        raise KernelError("fragment order takes bfloat16 rows of a multiple of 8 elements, 16-byte aligned")
    out = FragRows(torch.empty((-(-K // 32) * -(-M // 16) * 64 * 4,), dtype=torch.int32, device=x.device), M, K)
    _run("ilm_frag_pack_rows", out.data.data_ptr(), x.data_ptr(), M, K, x.stride(0), _stream())
    return out


def from_frag(f: FragRows) -> torch.Tensor:
    out = torch.empty((f.rows, f.width), dtype=BF16, device=f.data.device)
    _run("ilm_frag_unpack_rows", out.data_ptr(), f.data.data_ptr(), f.rows, f.width, f.width, _stream())
    return out


class FragWeight:
    """A weight [N, K] in fragment order: tiles of 16 rows in the order `rows` names (None: W's own), padded to a
    multiple of 4 tiles; `tiles` counts the real ones."""
    __slots__ = ("data", "N", "K", "tiles", "kind")

    def __init__(self, data, N, K, tiles, kind):
        self.data, self.N, self.K, self.tiles, self.kind = data, N, K, tiles, kind


def frag_weight_ok(w: torch.Tensor) -> bool:
    return (USE_FRAG and w.is_cuda and w.dtype == BF16 and w.dim() == 2 and w.shape[1] % 8 == 0 and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def pack_weight(w: torch.Tensor, kind: str = "plain", **layout) -> FragWeight:
    """`kind`: "plain" (tiles of consecutive rows), "gate_up" (w = [Wg; Wu]: tile pairs (gate rows 16p.., up rows 16p..)),
    "qkv" (nh, nkv, d given: tile pairs (first rows, second rows) of 16 rotation pairs; pair p = head slot p // (d/2),
    dim p % (d/2))."""
    if not frag_weight_ok(w):
        raise KernelError("fragment order takes a bfloat16 weight with rows of a multiple of 8 elements, 16-byte aligned")
    N, K = w.shape
    rows = None
    alloc_to = 4
    if kind == "plain":
        tiles = -(-N // 16)
    elif kind == "gate_up":
        I = N // 2
        it = -(-I // 16)
        idx = torch.arange(it * 16, dtype=torch.int64).view(it, 16)
        g = torch.where(idx < I, idx, torch.full_like(idx, -1))
        u = torch.where(idx < I, idx + I, torch.full_like(idx, -1))
        rows = torch.stack([g, u], dim=1).reshape(-1)
        tiles = 2 * it
    elif kind == "gate_up8":   # tiles of 8 gate rows and the 8 up rows of the same outputs
        I = N // 2
        it = -(-I // 8)
        idx = torch.arange(it * 8, dtype=torch.int64).view(it, 8)
        g = torch.where(idx < I, idx, torch.full_like(idx, -1))
        u = torch.where(idx < I, idx + I, torch.full_like(idx, -1))
        rows = torch.cat([g, u], dim=1).reshape(-1)
        tiles = it
        alloc_to = 8   # a workgroup of the kernel that reads it takes 8 tiles
    elif kind == "qkv":
        nh, nkv, d = layout["nh"], layout["nkv"], layout["d"]
        half = d // 2
        pairs = (nh + 2 * nkv) * half
        pt = -(-pairs // 16)
        p = torch.arange(pt * 16, dtype=torch.int64).view(pt, 16)
        first = (p // half) * d + p % half
        a = torch.where(p < pairs, first, torch.full_like(p, -1))
        b = torch.where(p < pairs, first + half, torch.full_like(p, -1))
        rows = torch.stack([a, b], dim=1).reshape(-1)
        tiles = 2 * pt
    else:
        raise KernelError(f"unknown fragment layout {kind!r}")
    alloc = -(-tiles // alloc_to) * alloc_to
    steps = -(-K // 32)
    data = torch.zeros((alloc * steps * 64 * 4,), dtype=torch.int32, device=w.device)
    rows_dev = None
    if rows is not None:
        rows_dev = rows.to(torch.int32).to(w.device)
    _run("ilm_frag_pack_weight", data.data_ptr(), w.data_ptr(), _ptr(rows_dev), N, K, w.stride(0), tiles, _stream())
    return FragWeight(data, N, K, tiles, kind)


# Rows from which the q/k/v projection of a decode step takes its operands in fragment order (measured at the 8B
# shape: 12.7 against 17.3 us at 32 rows, 16.2 against 22.5 us for the vendor library's product and the rotation
# kernel at 64; up to 16 rows the kernel that keeps X in registers is as fast)
FRAG_QKV_MIN_ROWS = int(os.environ.get("INFINILM_AMD_FRAG_QKV_MIN_ROWS", "17"))


def qkv_frag_ok(rows: int, w: torch.Tensor, d: int, rd: int, width: int) -> bool:
    """Whether the fused q/k/v projection takes `rows` rows in fragment order (see `gemm_frag_rope`)."""
    return (FRAG_QKV_MIN_ROWS <= rows <= FRAG_MAX_ROWS and frag_weight_ok(w) and rd == d and d % 32 == 0 and width % 8 == 0
            and USE_QKV_ROPE)


def _frag_x(x: FragRows, fw: FragWeight) -> None:
    if not isinstance(x, FragRows) or x.width != fw.K or x.rows > FRAG_MAX_ROWS:
        raise KernelError(f"fragment-order product: X {getattr(x, 'shape', None)} does not fit W [{fw.N}, {fw.K}] "
                          f"(at most {FRAG_MAX_ROWS} rows)")


def gemm_frag(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor] = None, alpha: float = 1.0,
              out: str = "bf16", parts: int = 1):
    """alpha (x W^T + bias) of up to 64 rows.  `out`: "bf16" or "f32" rows [M, N]; "parts": float32 [parts, M, N] of a
    K split in `parts` ranges (for add_rmsnorm); "frag": bfloat16 in fragment order."""
    _frag_x(x, fw)
    M, N, K = x.rows, fw.N, fw.K
    steps = -(-K // 32)
    spp = 0
    if out == "parts":
        spp = -(-steps // max(parts, 1))
        spp = -(-spp // 8) * 8 if spp > 8 else spp
        parts = -(-steps // spp)
        res = torch.empty((parts, M, N), dtype=F32, device=x.device)
        kind, ldc, target = 1, N, res
    elif out == "f32":
        res = torch.empty((M, N), dtype=F32, device=x.device)
        kind, ldc, target = 1, N, res
    elif out == "bf16":
        res = torch.empty((M, N), dtype=BF16, device=x.device)
        kind, ldc, target = 0, N, res
    else:
        res = frag_rows_empty(M, N, x.device)
        kind, ldc, target = 2, N, res.data
    if bias is not None and (bias.shape != (N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the product")
    _run("ilm_gemm_frag", target.data_ptr(), ldc, M * N, kind, x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), M, N, K,
         spp, float(alpha), FRAG_TILES, _stream())
    return res


def gemm_frag_swiglu(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor] = None,
                     row_ss: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0) -> FragRows:
    """silu(x Wg^T + bg) * (x Wu^T + bu) in fragment order; `row_ss`: x is what `gemm_frag_tail` left and the rows'
    division by sqrt(mean square + eps) over `norm_width` happens here."""
    _frag_x(x, fw)
    if fw.kind != "gate_up":
        raise KernelError("the SwiGLU epilogue needs a weight packed as gate_up")
    I = fw.N // 2
    if bias is not None and (bias.shape != (2 * I,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused gate/up projection")
    if row_ss is not None and (row_ss.dtype != F32 or row_ss.dim() != 2 or row_ss.shape[1] != FRAG_SS_ROWS or not row_ss.is_contiguous()):
        raise KernelError("partial sums of squares must be float32 [tiles, 64]")
    act = frag_rows_empty(x.rows, I, x.device)
    _run("ilm_gemm_frag_swiglu", act.data.data_ptr(), x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), x.rows, I, fw.K,
         _ptr(row_ss), 0 if row_ss is None else row_ss.shape[0], int(norm_width), float(eps), FRAG_TILES, _stream())
    return act


def gemm_frag_rope(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor], positions: torch.Tensor, cos: torch.Tensor,
                   sin: torch.Tensor, k_cache, v_cache, slots, nh: int, nkv: int, d: int) -> torch.Tensor:
    """The fused q/k/v projection with rotation and cache write; returns the rotated q [M, nh*d]."""
    _frag_x(x, fw)
    if fw.kind != "qkv" or fw.N != (nh + 2 * nkv) * d or d % 32:
        raise KernelError("the rotation epilogue needs a weight packed as qkv with heads in steps of 32")
    M = x.rows
    _i32(positions, "positions")
    if positions.numel() != M:
        raise KernelError("positions must have one entry a row")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or cos.shape[1] != d // 2 \
            or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError(f"rotation tables must be float32 [positions, {d // 2}], got {tuple(cos.shape)}")
    if bias is not None and (bias.shape != (fw.N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused projection")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != BF16 or v_cache.dtype != BF16:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    q = torch.empty((M, nh * d), dtype=BF16, device=x.device)
    _run("ilm_gemm_frag_rope", q.data_ptr(), q.stride(0), x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), M, fw.K,
         positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache) if slots is not None else None,
         _ptr(v_cache) if slots is not None else None, _ptr(slots), nh, nkv, d, page, _stream())
    return q


def gemm_frag_tail(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor], alpha: float, residual: torch.Tensor,
                   norm_w: torch.Tensor):
    """residual += alpha (x W^T + bias) in place; returns (xw, ss): xw = bfloat16(residual * norm_w) in fragment order,
    ss [ceil(N / 16), 64] partial sums of squares of the residual's rows."""
    _frag_x(x, fw)
    M, N = x.rows, fw.N
    if fw.kind != "plain":
        raise KernelError("the tail epilogue needs a weight packed plainly")
    if residual.dtype != F32 or tuple(residual.shape) != (M, N) or residual.stride(1) != 1:
        raise KernelError("the residual stream is a float32 tensor with dense rows of the product's width")
    if norm_w.shape != (N,) or norm_w.dtype not in (BF16, F32) or not norm_w.is_contiguous():
        raise KernelError("the norm's weight does not fit")
    if bias is not None and (bias.shape != (N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the product")
    xw = frag_rows_empty(M, N, x.device)
    ss = torch.empty((-(-N // 16), FRAG_SS_ROWS), dtype=F32, device=x.device)
    _run("ilm_gemm_frag_tail", residual.data_ptr(), residual.stride(0), xw.data.data_ptr(), ss.data_ptr(), x.data.data_ptr(),
         fw.data.data_ptr(), _ptr(bias), norm_w.data_ptr(), 1 if norm_w.dtype == F32 else 0, float(alpha), M, N, fw.K,
         FRAG_TILES, _stream())
    return xw, ss


# ---- mixers with a fixed-size state, and the small steps around them -------------------------------------------------
ACTIVATIONS = {"none": 0, "silu": 1, "sigmoid": 2, "relu2": 3, "gelu_tanh": 4}
SCAN_MAX_KEY_DIM = 512      # most state entries a value column of the recurrence (ilm_decay_scan_max_dk())
SCAN_PIECE = int(os.environ.get("INFINILM_AMD_SCAN_PIECE", "64"))        # tokens a piece of a long segment (0: never cut)
SCAN_PIECE_FROM = int(os.environ.get("INFINILM_AMD_SCAN_PIECE_FROM", "129"))   # segments from this length on are cut
CONV_MAX_TAPS = 8           # most taps of the short convolution (ilm_causal_conv_max_taps())


def activation_code(kind: str) -> int:
    """The kernels' number of an activation's name; raises for a name they do not know (parts call it when they are built)."""
    try:
        return ACTIVATIONS[kind]
    except KeyError:
        raise KernelError(f"unknown activation {kind!r}; known: {sorted(ACTIVATIONS)}") from None


def _rows(x: torch.Tensor, name: str) -> None:
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError(f"{name} must be a matrix with dense rows")


def activation(x: torch.Tensor, kind: str, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """act(x) element by element; x [T, n] with dense rows (a view into wider rows is fine)."""
    _dev(x)
    _rows(x, "x")
    T, n = x.shape
    out = torch.empty((T, n), dtype=out_dtype or x.dtype, device=x.device)
    _run("ilm_unary", out.data_ptr(), x.data_ptr(), T, n, out.stride(0), x.stride(0), activation_code(kind), _dt(out), _dt(x), _stream())
    return out


def linear_attention_inputs(qkv: torch.Tensor, positions: Optional[torch.Tensor], freq: Optional[torch.Tensor], heads: int,
                            dk: int, dv: int, rotary_dims: int, act: str, k_scale: float) -> torch.Tensor:
    """float32 rows [q: heads*dk | k: heads*dk | v: heads*dv] from the fused projection's rows of the same layout:
    an activation on all, q and k turned by position * freq[i] on their first `rotary_dims` entries (entry i paired
    with entry i + rotary_dims/2), k times `k_scale`."""
    _dev(qkv, positions, freq)
    _rows(qkv, "qkv")
    T = qkv.shape[0]
    n = heads * (2 * dk + dv)
    if qkv.shape[1] < n:
        raise KernelError(f"rows of {qkv.shape[1]} do not hold q, k and v of {heads} heads of {dk} / {dv}")
    if rotary_dims:
        if positions is None or freq is None:
            raise KernelError("a rotation needs positions and frequencies")
        _i32(positions, "positions")
        if positions.numel() != T or freq.dtype != F32 or freq.numel() != rotary_dims // 2 or not freq.is_contiguous():
            raise KernelError(f"frequencies must be float32 [{rotary_dims // 2}] and positions one a token")
    out = torch.empty((T, n), dtype=F32, device=qkv.device)
    _run("ilm_lin_prep", out.data_ptr(), qkv.data_ptr(), _ptr(positions), _ptr(freq), T, heads, dk, dv, int(rotary_dims),
         qkv.stride(0), activation_code(act), float(k_scale), _dt(qkv), _stream())
    return out


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, dk: int, dv: int, groups: int,
               pool: torch.Tensor, state_in: torch.Tensor, state_out: torch.Tensor, seg_offsets: torch.Tensor, segments: int,
               decay_h: Optional[torch.Tensor] = None, decay_t: Optional[torch.Tensor] = None,
               kscale_t: Optional[torch.Tensor] = None, skip_h: Optional[torch.Tensor] = None,
               max_len: Optional[int] = None, decay_c: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S_t = a_t S_(t-1) + (b_t k_t) v_t^T, o_t = S_t^T q_t + skip_h v_t for every head of every segment, token by token,
    all in float32.  q, k: [T, groups*dk] (views with one row stride; head h reads group h // (heads/groups)), v [T, heads*dv];
    a per head (`decay_h` [heads]), per token (`decay_t` [T, heads]) or per token, head and key channel (`decay_c`
    [T, heads*dk], float32 rows of one stride: S_t = diag(a_t) S_(t-1) + ...); b `kscale_t` [T, heads] or absent.  `pool`
    [rows, heads, dv, dk] holds the states: segment r starts from row state_in[r] and leaves its state in row state_out[r].
    `max_len`: a bound on the segments' lengths known on the host; from SCAN_PIECE_FROM tokens on, segments are cut
    into pieces of SCAN_PIECE tokens that run side by side (two passes and a combination of the pieces' states; the
    result differs from the single pass by rounding).  Returns o [T, heads*dv]."""
    _dev(q, k, v, pool, state_in, state_out, seg_offsets, decay_h, decay_t, kscale_t, skip_h)
    for t, nm in ((q, "q"), (k, "k"), (v, "v")):
        _rows(t, nm)
        if t.dtype != F32:
            raise KernelError(f"{nm} of the recurrence must be float32")
    T = v.shape[0]
    if q.shape != (T, groups * dk) or k.shape != (T, groups * dk) or v.shape != (T, heads * dv) or q.stride(0) != k.stride(0):
        raise KernelError(f"recurrence operands {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)} do not fit {heads} heads "
                          f"in {groups} groups of {dk} / {dv}")
    if groups <= 0 or heads % groups or dk > SCAN_MAX_KEY_DIM:
        raise KernelError(f"{heads} heads in {groups} groups, key size {dk} (at most {SCAN_MAX_KEY_DIM})")
    if pool.dtype != F32 or not pool.is_contiguous() or tuple(pool.shape[1:]) != (heads, dv, dk):
        raise KernelError(f"the state pool must be float32 [rows, {heads}, {dv}, {dk}], got {tuple(pool.shape)}")
    for t, nm in ((state_in, "state_in"), (state_out, "state_out"), (seg_offsets, "seg_offsets")):
        _i32(t, nm)
    if state_in.numel() < segments or state_out.numel() < segments or seg_offsets.numel() < segments + 1:
        raise KernelError("state rows and offsets must cover every segment")
    for t, shape, nm in ((decay_h, (heads,), "decay_h"), (decay_t, (T, heads), "decay_t"), (kscale_t, (T, heads), "kscale_t"),
                         (skip_h, (heads,), "skip_h")):
        if t is not None and (t.dtype != F32 or tuple(t.shape) != shape or not t.is_contiguous()):
            raise KernelError(f"{nm} must be contiguous float32 {shape}")
    if decay_c is not None:
        _dev(decay_c)
        _rows(decay_c, "decay_c")
        if decay_h is not None or decay_t is not None or decay_c.dtype != F32 or decay_c.shape != (T, heads * dk):
            raise KernelError(f"a decay per channel is float32 [{T}, {heads * dk}] and stands alone")
    elif (decay_h is None) == (decay_t is None):
        raise KernelError("the recurrence takes a decay per head or per token, one of them")
    o = torch.empty((T, heads * dv), dtype=F32, device=v.device)
    piece, ws_state, ws_decay = 0, None, None
    if SCAN_PIECE > 0 and max_len is not None and max_len >= SCAN_PIECE_FROM and T // SCAN_PIECE + int(segments) <= 65535:
        piece = SCAN_PIECE
        slots = T // piece + int(segments)
        ws_state = torch.empty((slots * heads * dv * dk,), dtype=F32, device=v.device)
        ws_decay = torch.empty((slots * heads * (dk if decay_c is not None else 1),), dtype=F32, device=v.device)
    _run("ilm_decay_scan", o.data_ptr(), o.stride(0), q.data_ptr(), k.data_ptr(), q.stride(0), heads // groups, v.data_ptr(),
         v.stride(0), _ptr(decay_h), _ptr(decay_t), _ptr(kscale_t), _ptr(skip_h), pool.data_ptr(), state_in.data_ptr(),
         state_out.data_ptr(), seg_offsets.data_ptr(), int(segments), heads, dk, dv, T, piece, _ptr(ws_state), _ptr(ws_decay),
         _ptr(decay_c), decay_c.stride(0) if decay_c is not None else 0, _stream())
    return o


def sigmoid_root(z: torch.Tensor, tau: float, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 sigmoid(z + bias)^(1/tau), element by element (the decays of a gated recurrence from their raw rows); z [T, n]
    with dense rows, `bias` [n] or None."""
    _dev(z, bias)
    _rows(z, "z")
    T, n = z.shape
    if bias is not None and (bias.shape != (n,) or not bias.is_contiguous()):
        raise KernelError(f"bias must be contiguous [{n}]")
    out = torch.empty((T, n), dtype=F32, device=z.device)
    _run("ilm_sigmoid_root", out.data_ptr(), z.data_ptr(), _ptr(bias), T, n, out.stride(0), z.stride(0), 1.0 / float(tau), _dt(z),
         _dt(bias) if bias is not None else 0, _stream())
    return out


def group_norm_gate(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, groups: int = 1,
                    gate: Optional[torch.Tensor] = None, gate_act: str = "none", gate_before: bool = False,
                    out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """RMS norm of every row in `groups` equal parts (each by its own root mean square, eps inside the root), times
    `weight` [n] if given; `gate` [T, n]: times act(gate), before the norm or after it.  Sums in float32.
    x may come as contiguous parts [P, T, n] that are summed first (a product that was split over K)."""
    _dev(x, weight, gate)
    parts, pstride = 1, 0
    if x.dim() == 3:
        if not x.is_contiguous():
            raise KernelError("parts must be contiguous")
        parts, pstride, x = x.shape[0], x.stride(0), x[0]
    _rows(x, "x")
    T, n = x.shape
    if groups <= 0 or n % groups:
        raise KernelError(f"rows of {n} do not divide into {groups} groups")
    if weight is not None and (weight.shape != (n,) or not weight.is_contiguous()):
        raise KernelError(f"norm weight has shape {tuple(weight.shape)}, expected ({n},)")
    if gate is not None:
        _rows(gate, "gate")
        if gate.shape != (T, n):
            raise KernelError(f"gate {tuple(gate.shape)} does not match {tuple(x.shape)}")
    out = torch.empty((T, n), dtype=out_dtype or x.dtype, device=x.device)
    _run("ilm_group_norm_gate", out.data_ptr(), x.data_ptr(), _ptr(gate), _ptr(weight), T, n, int(groups), x.stride(0),
         gate.stride(0) if gate is not None else 0, out.stride(0), float(eps), activation_code(gate_act), int(bool(gate_before)),
         _dt(out), _dt(x), _dt(gate) if gate is not None else 0, _dt(weight) if weight is not None else 0, parts, pstride,
         _stream())
    return out


def causal_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], pool: torch.Tensor,
                state_in: torch.Tensor, state_out: torch.Tensor, seg_of_token: torch.Tensor, seg_offsets: torch.Tensor,
                segments: int, act: str = "silu") -> torch.Tensor:
    """y[t, c] = act(bias[c] + sum_i weight[c, i] x[t - taps + 1 + i, c]) over the tokens of each segment; what lies
    before a segment's first row comes from its row of `pool` [rows, taps - 1, channels] (float32, oldest first), which
    is then written anew (row state_out[r]).  float32 result [T, channels]."""
    _dev(x, weight, bias, pool, state_in, state_out, seg_of_token, seg_offsets)
    _rows(x, "x")
    T, C = x.shape
    _i32(seg_of_token, "seg_of_token")
    if seg_of_token.numel() != T:
        raise KernelError("seg_of_token must have one entry a token")
    if weight.dim() != 2 or weight.shape[0] != C or not weight.is_contiguous() or not 1 <= weight.shape[1] <= CONV_MAX_TAPS:
        raise KernelError(f"convolution weight {tuple(weight.shape)} must be [{C}, taps <= {CONV_MAX_TAPS}]")
    taps = weight.shape[1]
    if bias is not None and (bias.shape != (C,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
        raise KernelError("convolution bias does not fit its weight")
    if pool.dtype != F32 or not pool.is_contiguous() or tuple(pool.shape[1:]) != (max(taps - 1, 0), C):
        raise KernelError(f"the convolution's state pool must be float32 [rows, {taps - 1}, {C}], got {tuple(pool.shape)}")
    for t, nm in ((state_in, "state_in"), (state_out, "state_out"), (seg_offsets, "seg_offsets")):
        _i32(t, nm)
    if state_in.numel() < segments or state_out.numel() < segments or seg_offsets.numel() < segments + 1:
        raise KernelError("state rows and offsets must cover every segment")
    y = torch.empty((T, C), dtype=F32, device=x.device)
    _run("ilm_causal_conv", y.data_ptr(), x.data_ptr(), weight.data_ptr(), _ptr(bias), pool.data_ptr(), state_in.data_ptr(),
         state_out.data_ptr(), seg_of_token.data_ptr(), seg_offsets.data_ptr(), T, int(segments), C, taps, x.stride(0),
         y.stride(0), activation_code(act), _dt(x), _dt(weight), _stream())
    return y


def ssm_steps(raw: torch.Tensor, bias: torch.Tensor, a_log: torch.Tensor):
    """(dt, decay), float32 [T, heads]: dt = softplus(raw + bias), decay = exp(-exp(a_log) dt)."""
    _dev(raw, bias, a_log)
    _rows(raw, "raw step sizes")
    T, H = raw.shape
    for t, nm in ((bias, "bias"), (a_log, "a_log")):
        if t.dtype != F32 or t.shape != (H,) or not t.is_contiguous():
            raise KernelError(f"{nm} must be contiguous float32 [{H}]")
    dt = torch.empty((T, H), dtype=F32, device=raw.device)
    decay = torch.empty((T, H), dtype=F32, device=raw.device)
    _run("ilm_ssm_steps", dt.data_ptr(), decay.data_ptr(), raw.data_ptr(), bias.data_ptr(), a_log.data_ptr(), T, H,
         raw.stride(0), _dt(raw), _stream())
    return dt, decay


def unit_qk_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, dn: int,
                    normed: bool, eps: float, coef: float, every: int) -> None:
    """Inside the fused rows [T, (nh + 2 nkv) d]: q and k heads divided by their root mean square over their `dn` entries
    that count (if `normed`), q times 1 + coef * ln(floor((position + 1) / every) + 1) (if every > 0); then k and v go
    to the paged cache at `slots` (None: no write)."""
    _dev(qkv, positions, k_cache, v_cache, slots)
    _rows(qkv, "qkv")
    _i32(positions, "positions")
    T = qkv.shape[0]
    if qkv.shape[1] < (nh + 2 * nkv) * d or positions.numel() != T or not 0 < dn <= d:
        raise KernelError("fused rows do not hold the heads, or positions do not match the tokens")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    _run("ilm_unit_qk_kvwrite", qkv.data_ptr(), positions.data_ptr(), _ptr(k_cache) if slots is not None else None,
         _ptr(v_cache) if slots is not None else None, _ptr(slots), T, nh, nkv, d, int(dn), qkv.stride(0), page,
         int(bool(normed)), float(eps), float(coef), int(every), _dt(qkv), _stream())


def weighted_sum(x: torch.Tensor, y: torch.Tensor, a: float, b: float, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """a x + b y, element by element."""
    _dev(x, y)
    if x.shape != y.shape or not x.is_contiguous() or not y.is_contiguous():
        raise KernelError("weighted_sum takes two contiguous tensors of one shape")
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    _run("ilm_weighted_sum", out.data_ptr(), x.data_ptr(), y.data_ptr(), x.numel(), float(a), float(b), _dt(out), _dt(x),
         _dt(y), _stream())
    return out


def norm_add_norm(residual: torch.Tensor, branch: torch.Tensor, branch_weight: torch.Tensor, branch_eps: float, alpha: float,
                  weight: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """residual += alpha * rmsnorm(branch) * branch_weight (in place, float32), then the residual's own RMS norm times
    `weight` as out_dtype: a branch that is normed before it joins the stream, and the norm before the next sublayer,
    in one kernel.  `branch` is [rows, H] or float32 parts [P, rows, H] that are summed first."""
    _dev(residual, branch, branch_weight, weight)
    rows, H = residual.shape
    if residual.dtype != F32 or not residual.is_contiguous():
        raise KernelError("the residual stream is a contiguous float32 tensor")
    parts, pstride = 1, 0
    if branch.dim() == 3:      # float32 parts of a product that was split over K
        parts, pstride = branch.shape[0], branch.stride(0)
    if tuple(branch.shape[-2:]) != (rows, H) or not branch.is_contiguous():
        raise KernelError(f"branch {tuple(branch.shape)} does not match residual {tuple(residual.shape)}")
    for wt in (branch_weight, weight):
        if wt.shape != (H,) or not wt.is_contiguous():
            raise KernelError(f"norm weight has shape {tuple(wt.shape)}, expected ({H},)")
    out = torch.empty((rows, H), dtype=out_dtype, device=residual.device)
    _run("ilm_norm_add_norm", out.data_ptr(), residual.data_ptr(), branch.data_ptr(), branch_weight.data_ptr(), weight.data_ptr(),
         rows, H, float(alpha), float(branch_eps), float(eps), _dt(out), _dt(branch), _dt(branch_weight), _dt(weight), parts, pstride,
         _stream())
    return out


# ---- a sum of several addends into the residual stream + layer norm ---------------------------------
LN_MAX_ADDENDS = 4   # (ilm_add_layernorm_max_addends())


def add_layernorm(residual: torch.Tensor, addends, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float,
                  out_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """residual += sum of scale * addend (in place, float32) over `addends` = [(tensor, scale), ...], then its layer norm
    (x - mean) / sqrt(mean of squared deviations + eps) * weight + bias as out_dtype.  An addend is [rows, H] (float32 or
    bfloat16), contiguous float32 parts [P, rows, H] that are summed in order, or one row [H] added to every row.
    Without `weight` only the sum is done and None returned.  More addends than the kernel takes are summed by a call
    of their own first."""
    _dev(residual, weight, bias)
    rows, H = residual.shape
    if residual.dtype != F32 or not residual.is_contiguous():
        raise KernelError("the residual stream is a contiguous float32 tensor")
    addends = list(addends)
    while len(addends) > LN_MAX_ADDENDS:
        add_layernorm(residual, addends[:LN_MAX_ADDENDS], None, None, eps, out_dtype)
        addends = addends[LN_MAX_ADDENDS:]
    if weight is None and not addends:
        return None
    flat = []
    for t, scale in addends:
        _dev(t)
        parts, pstride, rstride = 1, 0, H
        if t.dim() == 1:
            rstride = 0
        elif t.dim() == 3:
            parts, pstride = t.shape[0], t.stride(0)
        if t.shape[-1] != H or (t.dim() > 1 and t.shape[-2] != rows) or not t.is_contiguous():
            raise KernelError(f"an addend of shape {tuple(t.shape)} does not fit the residual stream {tuple(residual.shape)}")
        flat += [t.data_ptr(), _dt(t), parts, pstride, rstride, float(scale)]
    flat += [None, 0, 0, 0, 0, 0.0] * (LN_MAX_ADDENDS - len(addends))
    out = None
    if weight is not None:
        if weight.shape != (H,) or not weight.is_contiguous() or (bias is not None and (bias.shape != (H,) or bias.dtype != weight.dtype
                                                                                         or not bias.is_contiguous())):
            raise KernelError(f"layer norm weight and bias must be [{H}] of one dtype")
        out = torch.empty((rows, H), dtype=out_dtype, device=residual.device)
    _run("ilm_add_layernorm", _ptr(out), residual.data_ptr(), _ptr(weight), _ptr(bias), rows, H, float(eps), _DT[out_dtype],
         _dt(weight) if weight is not None else 0, len(addends), *flat, _stream())
    return out


# ---- attention with scores mixed over the heads ----------------------------------------------------
def headmix_mfma_ok(nh: int, nkv: int, d: int, page: int, dtype: torch.dtype) -> bool:
    """Whether `headmix_attention` runs its matrix-core kernel for these sizes."""
    return bool(dtype == BF16 and not FORCE_BASIC and USE_HEADMIX_MFMA and _lib().ilm_attn_headmix_mfma_ok(nh, nkv, d, page))


USE_HEADMIX_MFMA = os.environ.get("INFINILM_AMD_HEADMIX_MFMA", "1") == "1"   # 0: always the plain kernel


def qkv_norm_rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, freq: Optional[torch.Tensor], q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                          slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, dn: int, dv: int, rd: int, v_norm: bool,
                          eps: float) -> None:
    """In the fused projection rows [T, (nh + 2 nkv) d]: every q and k head RMS-normed over its first `dn` entries times
    `q_weight` / `k_weight` [dn] (None: no norm), then its entry pairs (2i, 2i + 1), i < rd / 2, turned by position x
    freq[i]; every v head divided by its root mean square over its first `dv` entries (`v_norm`); k and v written to the
    paged cache at `slots` (None: no write).  Entries of a head beyond those that count become zeros."""
    _dev(qkv, positions, freq, q_weight, k_weight, k_cache, v_cache, slots)
    _rows(qkv, "qkv")
    _i32(positions, "positions")
    T = qkv.shape[0]
    if qkv.shape[1] != (nh + 2 * nkv) * d or positions.numel() != T:
        raise KernelError(f"rows of {qkv.shape[1]} do not hold {nh} + 2 x {nkv} heads of {d}")
    if rd and (freq is None or freq.dtype != F32 or freq.numel() != rd // 2 or not freq.is_contiguous()):
        raise KernelError(f"frequencies must be float32 [{rd // 2}]")
    for w in (q_weight, k_weight):
        if w is not None and (w.shape != (dn,) or not w.is_contiguous() or w.dtype != (q_weight.dtype if q_weight is not None else w.dtype)):
            raise KernelError(f"a query/key norm weight must be [{dn}]")
    page = 1
    if slots is not None:
        _i32(slots, "slots")
        if k_cache.dtype != qkv.dtype or slots.numel() != T:
            raise KernelError("cache dtype or slots do not match the rows")
        page = _check_cache(k_cache, v_cache, nkv, d)
    _run("ilm_qkv_norm_rope_kvwrite", qkv.data_ptr(), positions.data_ptr(), _ptr(freq), _ptr(q_weight), _ptr(k_weight),
         _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, _ptr(slots), T, nh, nkv, d,
         int(dn), int(dv), int(rd), int(bool(v_norm)), float(eps), page, qkv.stride(0), _dt(qkv),
         _dt(q_weight) if q_weight is not None else _dt(qkv), _stream())


def headmix_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                      seg_of_token: torch.Tensor, positions: torch.Tensor, nh: int, nkv: int, d: int, dv: int, scale: float,
                      window: int = 0, mix: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                      tiles: Optional[torch.Tensor] = None, single_rows: Optional[torch.Tensor] = None,
                      max_total_len: Optional[int] = None, seg_offsets: Optional[torch.Tensor] = None,
                      keep_first: int = 0, spread_queries: bool = False, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Attention of every token over its request's cached keys (its last `window` positions, or all; with `keep_first` the
    sequence's first that many keys stay seen however far the window has moved) where the scaled
    scores of the heads are mixed before the softmax, s_h = sum_g mix[h, g] raw_g (`mix` float32 [nh, nh] or None),
    and every head's denominator holds one more term exp(sink[h]) (`sink` float32 [nh] or None); with neither it is the
    attention of `paged_attention` with its weights kept in float32 up to the second product.  q, caches, block
    tables as for `paged_attention`; `dv`: the entries of a value head that count.  `tiles` [n, 2] = (first row, count <=
    ATT_TILE_TOKENS) lists runs of consecutive tokens of one request and `single_rows` the remaining rows (without them
    every token is served on its own); the matrix-core kernel (bfloat16, heads of 32 to 128 in steps of 32, 1, 2 or 4
    key/value groups, pages of a multiple of 32) works by them, the plain kernel token by token.  `seg_offsets` (the step's
    first row of every request, and the end of the last): tiles that were cut 8 by 8 from each request's first row are then
    served two at a time.  `spread_queries` (matrix-core sizes only, no `mix`): q comes as [T, nh, nkv, d], every head's query
    against the key row of all groups side by side, as a caller made it.  `out_dtype` float32 (matrix-core sizes only): the result
    in float32.  Returns [T, nh*d]."""
    _dev(q, k_cache, v_cache, block_tables, seg_of_token, positions, mix, sink)
    if spread_queries:
        if mix is not None or tuple(q.shape[1:]) != (nh, nkv, d) or not q.is_contiguous() or not headmix_mfma_ok(nh, nkv, d, k_cache.shape[2], q.dtype):
            raise KernelError("queries spread over the groups are for the matrix-core kernel, [T, heads, groups, d], unmixed")
        spread, q = q, q.view(q.shape[0], -1)
    else:
        spread = None
    if out_dtype not in (None, q.dtype) and not (out_dtype == F32 and headmix_mfma_ok(nh, nkv, d, k_cache.shape[2], q.dtype)):
        raise KernelError("a float32 result of bfloat16 operands comes from the matrix-core kernel alone")
    _i32(block_tables, "block_tables")
    _i32(seg_of_token, "seg_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    if q.stride(1) != 1 or q.shape[1] < nh * d:
        raise KernelError("q rows must be dense and hold all query heads")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError(f"cache dtype {k_cache.dtype} differs from the activations' {q.dtype}")
    page = _check_cache(k_cache, v_cache, nkv, d)
    if seg_of_token.numel() != T or positions.numel() != T or block_tables.dim() != 2:
        raise KernelError("per-token metadata does not match the number of tokens")
    if mix is not None and (mix.dtype != F32 or tuple(mix.shape) != (nh, nh) or not mix.is_contiguous()):
        raise KernelError(f"the heads' mixing matrix must be contiguous float32 [{nh}, {nh}]")
    if sink is not None and (sink.dtype != F32 or tuple(sink.shape) != (nh,) or not sink.is_contiguous()):
        raise KernelError(f"the denominators' extra terms must be contiguous float32 [{nh}]")
    out = torch.empty((T, nh * d), dtype=out_dtype or q.dtype, device=q.device)
    if (q.dtype == BF16 and not FORCE_BASIC and USE_HEADMIX_MFMA and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0
            and _lib().ilm_attn_headmix_mfma_ok(nh, nkv, d, page)):
        # the mixing carried into the queries, then a flash attention on the matrix cores
        if spread is not None:
            qx = spread
        elif mix is None and nkv == 1 and q.stride(0) == nh * d:
            qx = q        # one group and no mixing: the mixed queries are the queries
        else:
            qx = torch.empty((T, nh, nkv, d), dtype=BF16, device=q.device)
            _run("ilm_headmix_queries", qx.data_ptr(), q.data_ptr(), _ptr(mix), T, nh, nkv, d, q.stride(0), _stream())
        n_tiles, n_single, rows = 0, T, None
        if seg_offsets is not None:
            _dev(seg_offsets)
            _i32(seg_offsets, "seg_offsets")
        if tiles is not None and tiles.numel() > 0:
            _i32(tiles, "tiles")
            n_tiles, n_single = tiles.numel() // 2, 0
            if single_rows is not None and single_rows.numel() > 0:
                _i32(single_rows, "single_rows")
                rows, n_single = single_rows, single_rows.numel()
        # single tokens over long windows (decoding): the keys in chunks over more workgroups, and a merge.  The chunks are
        # sized by bounded numbers (rows as recorded steps round them, the block table's width), so an eager step and its
        # recording cut alike.
        ws, nz, chunk = None, 1, 0
        if n_tiles == 0:
            span = block_tables.shape[1] * page
            if max_total_len is not None:
                span = min(span, bound_pages(-(-int(max_total_len) // page)) * page)
            if window > 0:
                span = min(span, int(window) + 64)
            hpw = 1 if d > 64 else (2 if nkv == 4 else 4)      # heads a wave, as the kernel's launcher picks them
            passes = -(-nh // (4 * hpw))
            if nkv == 1 or (nh % 16 == 0 and (nh // nkv) % 16 == 0):   # (heads as the products' columns: 64 heads a workgroup)
                passes = -(-nh // 64)
            want = max(1, (4 * _num_cus(q.device)) // max(1, bound_rows(n_single) * passes))
            chunk = max(128, -(-(-(-span // want)) // 64) * 64)
            nz = -(-span // chunk)
            if nz > 1:
                ws = torch.empty((n_single * nz * nh * (d + 4),), dtype=F32, device=q.device)
            else:
                nz, chunk = 1, 0
        _run("ilm_attn_headmix_mfma", out.data_ptr(), qx.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
             seg_of_token.data_ptr(), positions.data_ptr(), _ptr(tiles) if n_tiles else None, n_tiles, _ptr(rows), n_single,
             _ptr(sink), nh, nkv, d, page, block_tables.shape[1], out.stride(0), float(scale), int(window), _ptr(ws), nz, chunk,
             _ptr(seg_offsets) if n_tiles else None, int(keep_first), int(out.dtype == F32), _stream(),
             label="ilm_attn_headmix_mfma (unmixed)" if mix is None and sink is None else None)
        return out
    _run("ilm_attn_headmix", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
         seg_of_token.data_ptr(), positions.data_ptr(), None, T, _ptr(mix), _ptr(sink), nh, nkv, d, int(dv), page,
         block_tables.shape[1], q.stride(0), out.stride(0), float(scale), int(window), int(keep_first), _dt(q), _stream())
    return out


# ---- attention in maps over shared values ("differential" attention) ---------------------------------------------------
def maps_norm_rope_kvwrite(src: torch.Tensor, q_off: int, k_off: int, v_off: int, positions: torch.Tensor,
                           freq: Optional[torch.Tensor], q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                           k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                           heads: int, kv_heads: int, maps: int, dim: int, vdim: int, rd: int, eps: float,
                           out_dtype: torch.dtype, spread: bool = False) -> torch.Tensor:
    """From rows `src` (float32 or `out_dtype`) that hold [q: heads maps dim] at entry q_off, [k: kv_heads maps dim] at k_off
    and [v: kv_heads vdim] at v_off (k_off < 0: no keys and values in these rows): every q and k unit of `dim` entries
    RMS-normed times `q_weight` / `k_weight` [dim] (None: no norm) and its first `rd` entries turned in the pairs (i, i + rd/2)
    by position x freq[i]; k goes to the paged cache with a head's maps side by side (entry m dim + e of cache heads of d >=
    maps dim), v to the value cache, at `slots` (None: no write).  Returns the queries [T, heads maps dim] as `out_dtype`, or,
    `spread`, as [T, heads maps, kv_heads, d] with zeros everywhere but at a unit's own group and map (what `headmix_attention`
    takes as `spread_queries`)."""
    _dev(src, positions, freq, q_weight, k_weight, k_cache, v_cache, slots)
    _rows(src, "src")
    _i32(positions, "positions")
    T = src.shape[0]
    need = max(q_off + heads * maps * dim, (k_off + kv_heads * maps * dim) if k_off >= 0 else 0, (v_off + kv_heads * vdim) if k_off >= 0 else 0)
    if src.shape[1] < need or positions.numel() != T or src.dtype not in (F32, out_dtype):
        raise KernelError(f"rows of {src.shape[1]} ({src.dtype}) do not hold the queries, keys and values asked for")
    if rd and (freq is None or freq.dtype != F32 or freq.numel() != rd // 2 or not freq.is_contiguous()):
        raise KernelError(f"frequencies must be float32 [{rd // 2}]")
    if k_off >= 0 and (q_weight is None) != (k_weight is None):
        raise KernelError("a norm weight for q and k, or for neither")
    for w in (q_weight, k_weight):
        if w is not None and (tuple(w.shape) != (dim,) or not w.is_contiguous() or w.dtype != q_weight.dtype):
            raise KernelError(f"a query/key norm weight must be [{dim}]")
    page, d = 1, maps * dim
    write = k_off >= 0 and slots is not None
    if k_cache is not None:
        d = k_cache.shape[3]
        page = _check_cache(k_cache, v_cache, kv_heads, d)
    elif write or spread:
        raise KernelError("the cache is needed for its head size")
    if write:
        _i32(slots, "slots")
        if k_cache.dtype != out_dtype or slots.numel() != T:
            raise KernelError("cache dtype or slots do not match the rows")
    q = torch.empty((T, heads * maps, kv_heads, d) if spread else (T, heads * maps * dim), dtype=out_dtype, device=src.device)
    _run("ilm_maps_norm_rope_kvwrite", q.data_ptr(), src.data_ptr(), src.stride(0), int(q_off), int(k_off), int(v_off),
         positions.data_ptr(), _ptr(freq), _ptr(q_weight), _ptr(k_weight), _ptr(k_cache) if write else None,
         _ptr(v_cache) if write else None, _ptr(slots) if write else None, T, int(heads), int(kv_heads), int(maps), int(dim),
         int(vdim), int(d), int(rd), float(eps), page, _dt(src), _DT[out_dtype], _dt(q_weight) if q_weight is not None else _DT[out_dtype],
         int(bool(spread)), _stream())
    return q


USE_MAPS_MFMA = os.environ.get("INFINILM_AMD_MAPS_MFMA", "1") == "1"   # 0: never the two-maps matrix-core kernel


def maps_mfma_ok(heads: int, kv_heads: int, dim: int, vdim: int, d: int, page: int, dtype: torch.dtype) -> bool:
    """Whether `maps_attention_tiles` takes these sizes (bfloat16; maps and cache heads in multiples of 32, pages of a multiple of 32)."""
    return bool(dtype == BF16 and not FORCE_BASIC and USE_MAPS_MFMA and _lib().ilm_attn_maps_mfma_ok(heads, kv_heads, dim, vdim, d, page))


def maps_attention_tiles(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                         seg_of_token: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int,
                         scale: float, window: int, lambda_vectors, diff: float, norm_eps: float, out_scale: float,
                         tiles: Optional[torch.Tensor] = None, single_rows: Optional[torch.Tensor] = None,
                         seg_offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`maps_attention` with two maps on the matrix cores (bfloat16, sizes of `maps_mfma_ok`), a head's two maps in one pass with
    the combination, the norm and the scale in the kernel's epilogue.  `tiles` [n, 2] = (first row, count <= ATT_TILE_TOKENS)
    lists runs of consecutive tokens of one request and `single_rows` the remaining rows (without them every token is served on
    its own); `seg_offsets`: tiles cut 8 by 8 from each request's first row are then served two at a time.  An item's keys are
    walked by one workgroup: for steps of decoded tokens alone over long windows the chunked kernel behind `headmix_attention`
    spreads them wider.  q [T, heads 2 dim] dense; returns [T, heads vdim]."""
    _dev(q, k_cache, v_cache, block_tables, seg_of_token, positions, tiles, single_rows, seg_offsets, *lambda_vectors)
    _i32(block_tables, "block_tables")
    _i32(seg_of_token, "seg_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    if q.dtype != BF16 or not q.is_contiguous() or q.shape[1] != heads * 2 * dim:
        raise KernelError(f"queries must be dense bfloat16 rows of {heads} x 2 x {dim}")
    if k_cache.dtype != BF16 or v_cache.dtype != BF16:
        raise KernelError("the cache must be bfloat16")
    d = k_cache.shape[3] if k_cache.dim() == 4 else 0
    page = _check_cache(k_cache, v_cache, kv_heads, d)
    if not _lib().ilm_attn_maps_mfma_ok(heads, kv_heads, dim, vdim, d, page):
        raise KernelError(f"the two-maps matrix-core kernel does not take {heads} heads in {kv_heads} groups, maps of {dim}, values of {vdim}, "
                          f"cache heads of {d}, pages of {page}")
    if seg_of_token.numel() != T or positions.numel() != T or block_tables.dim() != 2:
        raise KernelError("per-token metadata does not match the number of tokens")
    if len(lambda_vectors) != 4:
        raise KernelError("two maps need the four vectors of their weight")
    for v in lambda_vectors:
        if tuple(v.shape) != (dim,) or not v.is_contiguous() or v.dtype != lambda_vectors[0].dtype:
            raise KernelError(f"the maps' weight vectors must be contiguous [{dim}] of one dtype")
    n_tiles, n_single, rows = 0, T, None
    if seg_offsets is not None:
        _i32(seg_offsets, "seg_offsets")
    if tiles is not None and tiles.numel() > 0:
        _i32(tiles, "tiles")
        n_tiles, n_single = tiles.numel() // 2, 0
        if single_rows is not None and single_rows.numel() > 0:
            _i32(single_rows, "single_rows")
            rows, n_single = single_rows, single_rows.numel()
    out = torch.empty((T, heads * vdim), dtype=BF16, device=q.device)
    _run("ilm_attn_maps_mfma", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
         seg_of_token.data_ptr(), positions.data_ptr(), _ptr(tiles) if n_tiles else None, n_tiles, _ptr(rows), n_single, int(heads),
         int(kv_heads), int(dim), int(vdim), int(d), page, block_tables.shape[1], out.stride(0), float(scale), int(window),
         _ptr(seg_offsets) if n_tiles else None, *[v.data_ptr() for v in lambda_vectors], float(diff), float(norm_eps), float(out_scale),
         _dt(lambda_vectors[0]), _stream())
    return out


def maps_combine(a: torch.Tensor, heads: int, vdim: int, dim: int, lambda_vectors, diff: float, norm_eps: float, out_scale: float,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """From float32 rows [T, heads x 2 x d] that hold every head's two maps' attention results: a_0 - lambda a_1 over the
    first `vdim` entries, lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, divided by its root mean square (norm_eps >= 0), times
    out_scale; [T, heads vdim] as `out_dtype` (bfloat16)."""
    _dev(a, *lambda_vectors)
    T = a.shape[0]
    d = a.shape[1] // (2 * heads)
    if a.dtype != F32 or not a.is_contiguous() or a.shape[1] != heads * 2 * d or vdim > d or out_dtype != BF16:
        raise KernelError("the maps' results are contiguous float32 rows of heads x 2 x d; the combined rows bfloat16")
    for v in lambda_vectors:
        if tuple(v.shape) != (dim,) or not v.is_contiguous() or v.dtype != lambda_vectors[0].dtype:
            raise KernelError(f"the maps' weight vectors must be contiguous [{dim}] of one dtype")
    out = torch.empty((T, heads * vdim), dtype=out_dtype, device=a.device)
    _run("ilm_maps_combine", out.data_ptr(), a.data_ptr(), T, int(heads), int(vdim), int(d), out.stride(0), *[v.data_ptr() for v in lambda_vectors],
         float(diff), float(norm_eps), float(out_scale), int(dim), _dt(lambda_vectors[0]), _stream())
    return out


def maps_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                   seg_of_token: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, maps: int, dim: int, vdim: int,
                   scale: float, window: int = 0, keep_first: int = 0, sink: Optional[torch.Tensor] = None,
                   lambda_vectors=None, diff: float = 0.0, norm_eps: float = -1.0, out_scale: float = 1.0) -> torch.Tensor:
    """Every query head's `maps` softmax attentions over its request's cached keys (the last `window` positions and the first
    `keep_first`, or all), each map against its own part of the key head (entries m dim ..) and all over the same values;
    `sink` float32 [heads]: one more term exp(sink_h) in the denominators.  One map: the attention's result.  Two maps:
    a_0 - lambda a_1 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff from `lambda_vectors` = (lq1, lk1, lq2, lk2), each [dim];
    then, with norm_eps >= 0, divided by its root mean square over the head's vdim entries; times out_scale.  All sums and
    weights float32.  q [T, heads maps dim] dense; returns [T, heads vdim]."""
    _dev(q, k_cache, v_cache, block_tables, seg_of_token, positions, sink)
    _i32(block_tables, "block_tables")
    _i32(seg_of_token, "seg_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    if not q.is_contiguous() or q.shape[1] != heads * maps * dim:
        raise KernelError(f"queries must be dense rows of {heads} x {maps} x {dim}")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError(f"cache dtype {k_cache.dtype} differs from the activations' {q.dtype}")
    d = k_cache.shape[3] if k_cache.dim() == 4 else 0
    page = _check_cache(k_cache, v_cache, kv_heads, d)
    if seg_of_token.numel() != T or positions.numel() != T or block_tables.dim() != 2:
        raise KernelError("per-token metadata does not match the number of tokens")
    if sink is not None and (sink.dtype != F32 or tuple(sink.shape) != (heads,) or not sink.is_contiguous()):
        raise KernelError(f"the denominators' extra terms must be contiguous float32 [{heads}]")
    lv = [None] * 4
    if maps == 2:
        if lambda_vectors is None or len(lambda_vectors) != 4:
            raise KernelError("two maps need the four vectors of their weight")
        lv = list(lambda_vectors)
        _dev(*lv)
        for v in lv:
            if tuple(v.shape) != (dim,) or not v.is_contiguous() or v.dtype != lv[0].dtype:
                raise KernelError(f"the maps' weight vectors must be contiguous [{dim}] of one dtype")
    out = torch.empty((T, heads * vdim), dtype=q.dtype, device=q.device)
    _run("ilm_attn_maps", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
         seg_of_token.data_ptr(), positions.data_ptr(), None, T, int(heads), int(kv_heads), int(maps), int(dim), int(vdim), int(d),
         page, block_tables.shape[1], out.stride(0), float(scale), int(window), int(keep_first), _ptr(sink), _ptr(lv[0]), _ptr(lv[1]),
         _ptr(lv[2]), _ptr(lv[3]), float(diff), float(norm_eps), float(out_scale), _dt(q), _dt(lv[0]) if lv[0] is not None else _dt(q),
         _stream())
    return out


# ---- a selective scan with a decay per channel and state entry -----------------------------------------------------------
SELECTIVE_SCAN_MAX_STATE = 256   # most state entries a channel (ilm_selective_scan_max_state())
SELECTIVE_SCAN_PIECE = int(os.environ.get("INFINILM_AMD_SELECTIVE_SCAN_PIECE", "64"))   # tokens a piece of a long segment (0: never cut)
SELECTIVE_SCAN_PIECE_FROM = 128  # segments from this length on are cut into pieces that run side by side


def selective_scan(x: torch.Tensor, raw_dt: torch.Tensor, dt_bias: torch.Tensor, B: torch.Tensor, C: torch.Tensor, z: torch.Tensor,
                   a_log: torch.Tensor, skip: torch.Tensor, pool: torch.Tensor, state_in: torch.Tensor, state_out: torch.Tensor,
                   seg_offsets: torch.Tensor, segments: int, max_len: Optional[int] = None) -> torch.Tensor:
    """Per channel c and state entry n, token by token from the request's state row: dt = softplus(raw_dt + dt_bias),
    S[c, n] <- exp(-exp(a_log[c, n]) dt_c) S[c, n] + dt_c x_c B_n, y_c = sum_n S[c, n] C_n + skip_c x_c, out = y silu(z).
    x float32 [T, inner]; raw_dt, z [T, inner] and B, C [T, state] in the activations' dtype (views with dense rows; B and C of
    one row stride); a_log float32 [inner, state], skip float32 [inner]; pool float32 [rows, inner, state].  `max_len`: a bound
    on the segments' lengths known on the host; from SELECTIVE_SCAN_PIECE_FROM tokens on, segments are cut into pieces of
    SELECTIVE_SCAN_PIECE tokens that run side by side (the result differs from the single pass by rounding).  Returns
    [T, inner] in the activations' dtype."""
    _dev(x, raw_dt, dt_bias, B, C, z, a_log, skip, pool, state_in, state_out, seg_offsets)
    for t, nm in ((x, "x"), (raw_dt, "raw_dt"), (B, "B"), (C, "C"), (z, "z")):
        _rows(t, nm)
    T, inner = x.shape
    state = B.shape[1]
    dt = raw_dt.dtype
    if x.dtype != F32 or raw_dt.shape != (T, inner) or z.shape != (T, inner) or z.dtype != dt or B.dtype != dt or C.dtype != dt \
            or B.shape != (T, state) or C.shape != (T, state) or B.stride(0) != C.stride(0):
        raise KernelError("the scan's operands do not fit each other")
    if state > SELECTIVE_SCAN_MAX_STATE:
        raise KernelError(f"{state} state entries a channel (at most {SELECTIVE_SCAN_MAX_STATE})")
    if a_log.dtype != F32 or tuple(a_log.shape) != (inner, state) or not a_log.is_contiguous() or skip.dtype != F32 \
            or tuple(skip.shape) != (inner,) or tuple(dt_bias.shape) != (inner,) or not dt_bias.is_contiguous():
        raise KernelError(f"a_log float32 [{inner}, {state}], skip float32 [{inner}], dt_bias [{inner}]")
    if pool.dtype != F32 or not pool.is_contiguous() or tuple(pool.shape[1:]) != (inner, state):
        raise KernelError(f"the state pool must be float32 [rows, {inner}, {state}], got {tuple(pool.shape)}")
    for t, nm in ((state_in, "state_in"), (state_out, "state_out"), (seg_offsets, "seg_offsets")):
        _i32(t, nm)
    if state_in.numel() < segments or state_out.numel() < segments or seg_offsets.numel() < segments + 1:
        raise KernelError("state rows and offsets must cover every segment")
    out = torch.empty((T, inner), dtype=dt, device=x.device)
    piece, max_pieces, ws_state, ws_dt = 0, 0, None, None
    if SELECTIVE_SCAN_PIECE > 0 and max_len is not None and max_len >= SELECTIVE_SCAN_PIECE_FROM:
        piece = SELECTIVE_SCAN_PIECE
        # (the grid holds the pieces of a segment as long as the whole step, not of the longest one now: a recorded step is
        # replayed with other segment lengths; a piece beyond a segment's end leaves at once)
        max_pieces = -(-T // piece)
        slots = T // piece + int(segments)
        if max_pieces <= 65535:
            ws_state = torch.empty((slots * inner * state,), dtype=F32, device=x.device)
            ws_dt = torch.empty((slots * inner,), dtype=F32, device=x.device)
        else:
            piece = max_pieces = 0
    _run("ilm_selective_scan", out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), raw_dt.data_ptr(), raw_dt.stride(0),
         dt_bias.data_ptr(), B.data_ptr(), C.data_ptr(), B.stride(0), z.data_ptr(), z.stride(0), a_log.data_ptr(), skip.data_ptr(),
         pool.data_ptr(), state_in.data_ptr(), state_out.data_ptr(), seg_offsets.data_ptr(), int(segments), inner, state, piece,
         max_pieces, _ptr(ws_state), _ptr(ws_dt), _DT[dt], _dt(dt_bias), _stream())
    return out


# ---- attention over latent rows -------------------------------------------------------------------
def latent_prep(rows: torch.Tensor, qx: torch.Tensor, positions: torch.Tensor, freq: Optional[torch.Tensor], weight: torch.Tensor,
                k_cache: torch.Tensor, v_cache: torch.Tensor, slots: Optional[torch.Tensor], heads: int, dn: int, dr: int, rank: int,
                d: int, eps: float, down_offset: int = -1) -> None:
    """From fused projection rows [q: heads (dn + dr) | down: rank + dr] (`down_offset` >= 0: `down` begins at that entry of a
    row instead, for queries that are made elsewhere; only without rotated entries): the latent c = RMS norm of down[:rank] times
    `weight`, the last dr entries of `down` and of every query head turned in pairs (2i, 2i + 1) by position x freq[i];
    key row [c | turned part | zeros] and value [c | zeros] into the one-head cache of head size d at `slots`; the
    queries' turned parts (and zeros up to d) into qx [T, heads, d] from entry `rank` on."""
    _dev(rows, qx, positions, freq, weight, k_cache, v_cache, slots)
    _rows(rows, "rows")
    _i32(positions, "positions")
    T = rows.shape[0]
    if tuple(qx.shape) != (T, heads, d) or not qx.is_contiguous() or qx.dtype != rows.dtype:
        raise KernelError(f"the attention's query rows must be contiguous [{T}, {heads}, {d}] of the rows' dtype")
    if down_offset >= 0 and dr:
        raise KernelError("rows that hold the latent at an offset of their own have no rotated query entries")
    if (rows.shape[1] != heads * (dn + dr) + rank + dr if down_offset < 0 else rows.shape[1] < down_offset + rank) \
            or weight.shape != (rank,) or not weight.is_contiguous():
        raise KernelError("rows or norm weight do not fit the latent sizes")
    if dr and (freq is None or freq.dtype != F32 or freq.numel() != dr // 2 or not freq.is_contiguous()):
        raise KernelError(f"frequencies must be float32 [{dr // 2}]")
    page = 1
    if slots is not None:
        _i32(slots, "slots")
        if k_cache.dtype != rows.dtype or slots.numel() != T:
            raise KernelError("cache dtype or slots do not match the rows")
        page = _check_cache(k_cache, v_cache, 1, d)
    _run("ilm_latent_prep", rows.data_ptr(), qx.data_ptr(), positions.data_ptr(), _ptr(freq), weight.data_ptr(),
         _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, _ptr(slots), T, heads, dn, dr,
         rank, d, float(eps), page, rows.stride(0), int(down_offset), _dt(rows), _dt(weight), _stream())


HEAD_GEMM_LIBRARY_MIN_ROWS = 33   # rows from which the bfloat16 product per head goes to the vendor library
HEAD_GEMM_MFMA_MAX_ROWS = int(os.environ.get("INFINILM_AMD_HEAD_GEMM_MFMA_MAX_ROWS", "128"))   # rows up to which it takes the matrix-core kernel without LDS (0: never)


def head_gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, h, n] = sum_k x[t, h, k] w[h, k, n]: a product per head.  x [T, H, K] and out [T, H, N] are views with
    a dense last axis; w [H, K, N] is a view one of whose last two axes is dense.  Float sums."""
    _dev(x, w, out)
    T, H, K = x.shape
    N = w.shape[2]
    if tuple(w.shape) != (H, K, N) or tuple(out.shape) != (T, H, N) or x.stride(2) != 1 or out.stride(2) != 1 \
            or x.dtype != w.dtype or (w.stride(1) != 1 and w.stride(2) != 1):
        raise KernelError(f"a product per head of {tuple(x.shape)} x {tuple(w.shape)} -> {tuple(out.shape)} does not fit")
    if (x.dtype == BF16 and out.dtype == BF16 and T <= HEAD_GEMM_MFMA_MAX_ROWS and not FORCE_BASIC and K % 8 == 0
            and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0 and x.data_ptr() % 16 == 0
            and (w.stride(1) != 1 or (w.stride(2) % 8 == 0 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0))):
        # few rows (decoded tokens): a wave a head and 16 outputs on the matrix cores, nothing through LDS
        _run("ilm_head_gemm_mfma", out.data_ptr(), x.data_ptr(), w.data_ptr(), T, N, K, H, x.stride(0), x.stride(1), w.stride(0),
             w.stride(1), w.stride(2), out.stride(0), out.stride(1), _stream())
        return out
    if x.dtype == BF16 and out.dtype == BF16 and T >= HEAD_GEMM_LIBRARY_MIN_ROWS and USE_LIBRARY_GEMM and not FORCE_BASIC:
        with _timed("library_gemm"):
            out.copy_(torch.bmm(x.transpose(0, 1), w).transpose(0, 1))
        return out
    _run("ilm_head_gemm", out.data_ptr(), x.data_ptr(), w.data_ptr(), T, N, K, H, x.stride(0), x.stride(1), w.stride(0),
         w.stride(1), w.stride(2), out.stride(0), out.stride(1), _dt(x), _dt(out), _stream())
    return out


# ---- a residual stream whose branches are gated or normed on their way in -----------------------------------------------
STREAM_PLAIN, STREAM_GATED, STREAM_NORMED = 1, 2, 3
STREAM_MAX_WIDTH = 12288     # widest row of `stream_update` (the row lies in LDS)


def embed_positions(ids: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, position_table: torch.Tensor,
                    scale: float = 1.0) -> torch.Tensor:
    """float32 residual rows scale * table[ids] + position_table[positions]."""
    _dev(ids, positions, table, position_table)
    _i32(ids, "ids")
    _i32(positions, "positions")
    V, H = table.shape
    if position_table.dim() != 2 or position_table.shape[1] != H or position_table.dtype != table.dtype \
            or not table.is_contiguous() or not position_table.is_contiguous():
        raise KernelError("the token table and the position table must be contiguous, of one dtype and one width")
    T = ids.numel()
    if positions.numel() != T:
        raise KernelError("one position a token")
    out = torch.empty((T, H), dtype=F32, device=table.device)
    _run("ilm_embed_pos", out.data_ptr(), ids.data_ptr(), positions.data_ptr(), table.data_ptr(), position_table.data_ptr(), T, H, V,
         position_table.shape[0], float(scale), _dt(table), _stream())
    return out


def stream_update(residual: torch.Tensor, branch: Optional[torch.Tensor] = None, alpha: float = 1.0,
                  gate: Optional[torch.Tensor] = None, gate_bias: Optional[torch.Tensor] = None,
                  branch_weight: Optional[torch.Tensor] = None, branch_eps: float = 0.0,
                  weight: Optional[torch.Tensor] = None, eps: float = 0.0, groups: int = 1,
                  out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """residual += alpha * f(branch) in place (float32), where f(y) = y, y * sigmoid(gate + gate_bias) with `gate` [T, H], or
    y / rms(y) * branch_weight (eps inside the root); the branch may come as contiguous float32 parts [P, T, H] that are
    summed first.  Then, with `out_dtype`: the stream's rows normed in `groups` consecutive equal parts (each by its own root mean
    square) times `weight`, or without a weight the rows themselves, as out_dtype.  Returns that output or None."""
    _dev(residual, branch, gate, gate_bias, branch_weight, weight)
    rows, H = residual.shape
    if residual.dtype != F32 or not residual.is_contiguous():
        raise KernelError("the residual stream is a contiguous float32 tensor")
    if H > STREAM_MAX_WIDTH:
        raise KernelError(f"rows of {H} are wider than the {STREAM_MAX_WIDTH} this kernel holds")
    kind, parts, pstride, ystride = 0, 1, 0, H
    if branch is not None:
        kind = STREAM_GATED if gate is not None else (STREAM_NORMED if branch_weight is not None else STREAM_PLAIN)
        if gate is not None and branch_weight is not None:
            raise KernelError("a branch is gated or normed, not both")
        y = branch
        if y.dim() == 3:
            if not y.is_contiguous() or y.dtype != F32:
                raise KernelError("parts must be contiguous float32")
            parts, pstride, y = y.shape[0], y.stride(0), y[0]
        if tuple(y.shape) != (rows, H) or y.stride(1) != 1:
            raise KernelError(f"a branch of shape {tuple(branch.shape)} does not fit the stream {tuple(residual.shape)}")
        ystride = y.stride(0)
    ws = [t for t in (gate_bias, branch_weight, weight) if t is not None]
    for t in ws:
        if tuple(t.shape) != (H,) or not t.is_contiguous() or t.dtype != ws[0].dtype:
            raise KernelError(f"weights and biases must be contiguous [{H}] of one dtype")
    if gate is not None and (tuple(gate.shape) != (rows, H) or gate.stride(1) != 1):
        raise KernelError("the gate's rows must match the stream's")
    if weight is not None and (groups < 1 or H % groups):
        raise KernelError(f"rows of {H} do not divide into {groups} groups")
    if weight is not None and out_dtype is None:
        raise KernelError("a norm needs an output dtype")
    out = torch.empty((rows, H), dtype=out_dtype, device=residual.device) if out_dtype is not None else None
    if kind == 0 and out is None:
        return None
    _run("ilm_stream_update", _ptr(out), residual.data_ptr(), _ptr(branch), _ptr(gate), _ptr(gate_bias), _ptr(branch_weight), _ptr(weight),
         rows, H, int(groups), kind, float(alpha), float(branch_eps), float(eps), _DT[out_dtype] if out is not None else 0,
         _dt(branch) if branch is not None else 0, _dt(gate) if gate is not None else 0, _dt(ws[0]) if ws else 0, parts, pstride,
         ystride, gate.stride(0) if gate is not None else 0, _stream())
    return out


def embed_gate(z: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """g[t, j] = gelu_tanh(z[t, j]) * table[ids[t], col0 + j] for rows z [T, n]."""
    _dev(z, ids, table)
    _i32(ids, "ids")
    _rows(z, "z")
    T, n = z.shape
    if table.dim() != 2 or not table.is_contiguous() or table.dtype != z.dtype or ids.numel() != T:
        raise KernelError("the table must be contiguous and of the rows' dtype, one id a row")
    out = torch.empty((T, n), dtype=z.dtype, device=z.device)
    _run("ilm_embed_gate", out.data_ptr(), z.data_ptr(), ids.data_ptr(), table.data_ptr(), T, n, table.shape[1], int(col0), z.stride(0),
         _dt(z), _stream())
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap), in place on a contiguous float32 tensor."""
    _dev(x)
    if x.dtype != F32 or not x.is_contiguous():
        raise KernelError("the capped numbers are a contiguous float32 tensor")
    if x.numel():
        _run("ilm_softcap", x.data_ptr(), x.numel(), float(cap), _stream())
    return x


# ---- many small experts of which a token uses a few -----------------------------------------------------------------------
MOE_TILE_ROWS = 64       # rows of one expert a workgroup of the experts' products takes (ilm_moe_tile_rows())
MOE_BIG_TILE_ROWS = 128  # the same for steps of many rows an expert (the bfloat16 matrix-core kernel with tiles of 128 x 128)
MOE_BIG_MIN_ROWS = int(os.environ.get("INFINILM_AMD_MOE_BIG_MIN_ROWS", "96"))   # pairs an expert (on average) from which it runs
MOE_FORCE_PLAIN = os.environ.get("INFINILM_AMD_MOE_PLAIN", "0") == "1"   # 1: the FMA products also in bfloat16
# 1: the plain form's few-rows kernel takes two blocks of 64 outputs a workgroup for large matrices (faster while a step's loads
# were in flight over one step's products only, 175 -> 149 us; with two sets of load registers one block is: 132 against 135 us)
MOE_PLAIN_PAIR = os.environ.get("INFINILM_AMD_MOE_PLAIN_PAIR", "0") == "1"
MOE_WIDE = int(os.environ.get("INFINILM_AMD_MOE_WIDE", "0"))   # 1: tiles of 256 rows of W in the many-rows kernel wherever the outputs fill one (measured slower at the shapes tried)


class ExpertPlan:
    """Where every (token, slot) pair of a step lies once the pairs are ordered by expert."""
    __slots__ = ("ids", "weights", "perm", "inv", "tiles", "n_tiles", "offsets", "max_tiles", "top", "pairs", "tile_rows")


def moe_route(logits: torch.Tensor, experts: int, top: int, big_tiles_ok: bool = False, softmax: bool = False,
              weight_scale: float = 1.0) -> ExpertPlan:
    """From float32 router logits [T, >= experts] (the first `experts` entries of a row count): the `top` experts of every token
    with weight_scale x sigmoid(logit) (or, `softmax`, weight_scale x the logit's softmax over all experts) as their weights, and
    the pairs ordered by expert for `moe_gemm`.  `big_tiles_ok`: the products that
    follow are bfloat16 with every K a multiple of 8, so a step of many pairs an expert may be cut into tiles of 128 rows."""
    _dev(logits)
    if logits.dtype != F32 or logits.dim() != 2 or logits.stride(1) != 1 or logits.shape[1] < experts:
        raise KernelError("router logits are float32 rows that hold every expert")
    T = logits.shape[0]
    P = T * top
    plan = ExpertPlan()
    dev = logits.device
    plan.top, plan.pairs = int(top), P
    plan.ids = torch.empty((T, top), dtype=torch.int32, device=dev)
    plan.weights = torch.empty((T, top), dtype=F32, device=dev)
    _run("ilm_moe_route", plan.ids.data_ptr(), plan.weights.data_ptr(), logits.data_ptr(), T, int(experts), int(top), logits.stride(0),
         int(bool(softmax)), float(weight_scale), _stream())
    plan.tile_rows = MOE_BIG_TILE_ROWS if big_tiles_ok and not MOE_FORCE_PLAIN and P >= MOE_BIG_MIN_ROWS * experts else MOE_TILE_ROWS
    plan.max_tiles = min(P, P // plan.tile_rows + min(experts, P))
    book = torch.empty((experts + 1 + 2 * P + 3 * plan.max_tiles + 1,), dtype=torch.int32, device=dev)
    plan.offsets = book[:experts + 1]
    plan.perm = book[experts + 1:experts + 1 + P]
    plan.inv = book[experts + 1 + P:experts + 1 + 2 * P]
    plan.tiles = book[experts + 1 + 2 * P:experts + 1 + 2 * P + 3 * plan.max_tiles]
    plan.n_tiles = book[-1:]
    _run("ilm_moe_sort", plan.offsets.data_ptr(), plan.perm.data_ptr(), plan.inv.data_ptr(), plan.tiles.data_ptr(), plan.n_tiles.data_ptr(),
         plan.ids.data_ptr(), P, int(experts), plan.max_tiles, plan.tile_rows, _stream())
    return plan


def moe_gemm(x: torch.Tensor, w: torch.Tensor, plan: ExpertPlan, glu: bool, limit: float = 0.0, alpha: float = 1.702,
             gather: bool = False, act: str = "none") -> torch.Tensor:
    """The experts' products over the ordered pairs.  `glu`: x [T, K] are the tokens' rows, w [E, 2 I, K] holds every expert's
    gate rows and then its up rows; a pair's row is its token's row times the pair's weight, and the result [pairs, I] is
    min(gate, limit) * sigmoid(alpha * min(gate, limit)) * (clamp(up, -limit, limit) + 1) in sorted order.  Otherwise x [pairs, K] are rows
    in sorted order (`gather`: the tokens' rows [T, K], from which every pair takes its token's, unweighted) and w [E, N, K]: the
    result is [pairs, N] in sorted order, `act` ("none" or "relu2", the square of relu) applied to it."""
    _dev(x, w)
    _rows(x, "x")
    E, Nw, K = w.shape
    if not w.is_contiguous() or w.dtype != x.dtype or x.shape[1] != K or (glu and Nw % 2):
        raise KernelError(f"experts of shape {tuple(w.shape)} do not fit rows of {tuple(x.shape)}")
    N = Nw // 2 if glu else Nw
    if not glu and not gather and x.shape[0] != plan.pairs:
        raise KernelError("rows in sorted order: one a pair")
    if act not in ("none", "relu2") or (glu and act != "none"):
        raise KernelError(f"the experts' plain product takes no activation or relu2, got {act!r}")
    out = torch.empty((plan.pairs, N), dtype=x.dtype, device=x.device)
    _run("ilm_moe_gemm", out.data_ptr(), N, x.data_ptr(), x.stride(0), plan.perm.data_ptr() if (glu or gather) else None, plan.top,
         plan.weights.data_ptr() if glu else None,
         w.data_ptr(), Nw * K, K, plan.tiles.data_ptr(), plan.n_tiles.data_ptr(), plan.max_tiles, N, K, int(bool(glu)), float(limit),
         float(alpha), 1 if act == "relu2" else 0, _dt(x), int(MOE_FORCE_PLAIN), plan.tile_rows, int(MOE_WIDE) | (2 if MOE_PLAIN_PAIR else 0), _stream(), label="ilm_moe_gemm (gate/up)" if glu else ("ilm_moe_gemm (up)" if gather else "ilm_moe_gemm (down)"))
    return out


def moe_combine(pair_out: torch.Tensor, plan: ExpertPlan, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None, weighted: bool = False) -> torch.Tensor:
    """y[t] = sum over the token's slots of pair_out[place of (t, slot)] (`weighted`: times the pair's weight of the plan, in
    float32) + shared[t] * sigmoid(shared_gate[t]); `shared_gate` is a float32 column (one number a token, any stride; None: the
    shared rows are added as they are)."""
    _dev(pair_out, shared, shared_gate)
    _rows(pair_out, "pair_out")
    P, H = pair_out.shape
    T = P // plan.top
    if P != plan.pairs:
        raise KernelError("one row a pair")
    sg_stride = 0
    if shared is not None:
        if tuple(shared.shape) != (T, H) or not shared.is_contiguous() or shared.dtype != pair_out.dtype:
            raise KernelError("the shared expert's rows must match the tokens'")
        if shared_gate is not None:
            if shared_gate.dtype != F32 or shared_gate.shape[0] != T:
                raise KernelError("the shared expert's gate is one float32 number a token")
            sg_stride = shared_gate.stride(0)
    out = torch.empty((T, H), dtype=pair_out.dtype, device=pair_out.device)
    _run("ilm_moe_combine", out.data_ptr(), pair_out.data_ptr(), plan.inv.data_ptr(), plan.top, _ptr(shared),
         _ptr(shared_gate) if shared is not None else None, sg_stride, T, H, pair_out.stride(0),
         plan.weights.data_ptr() if weighted else None, _dt(pair_out), _stream())
    return out


def glu_clamp(gate_up: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """From fused rows [gate | up]: g = min(gate, limit), u = clamp(up, -limit, limit), g * sigmoid(alpha g) * (u + 1)."""
    _dev(gate_up)
    _rows(gate_up, "gate_up")
    T, n = gate_up.shape
    out = torch.empty((T, n // 2), dtype=gate_up.dtype, device=gate_up.device)
    _run("ilm_glu_clamp", out.data_ptr(), gate_up.data_ptr(), T, n // 2, gate_up.stride(0), float(limit), float(alpha), _dt(gate_up), _stream())
    return out
