"""Python launchers of the HIP kernels: argument checks on the host, then one C call.

Every function takes torch tensors that live on the GPU, checks what the kernel and its
grid assume (device, dtype, contiguity, shapes) and launches on torch's current stream.
There is no fallback: a missing library or a size a kernel does not take raises
`KernelError`.
"""
from __future__ import annotations

import ctypes
from ctypes import c_void_p, c_int, c_float, c_size_t
from typing import Optional

import torch

from .errors import KernelError
from .csrc import build as _build

_P = c_void_p


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _req(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(name: str, *tensors) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError(f"{name}: tensor on {t.device}; kernels run on the GPU only")
        if not t.is_contiguous():
            raise KernelError(f"{name}: tensor of shape {tuple(t.shape)} is not contiguous")


def _is_bf16(t: torch.Tensor, name: str) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise KernelError(f"{name}: dtype {t.dtype} is not supported (float32 or bfloat16)")


def _check(rc: int, name: str) -> None:
    if rc == 0:
        return
    raise KernelError(f"{name}: " + {1: "arguments outside what the kernel takes",
                                     2: "launch failed", 3: "sizes beyond the entry point's fixed scratch"}.get(rc, f"error {rc}"))


_sigs_done = set()


def _fn(module: str, name: str, argtypes):
    lib = _build.load(module)
    f = getattr(lib, name)
    if (module, name) not in _sigs_done:
        f.argtypes = argtypes
        f.restype = c_int
        _sigs_done.add((module, name))
    return f


_device_cus = {}


def device_cus() -> int:
    """Compute units of the current GPU (256 when the runtime does not say)."""
    dev = torch.cuda.current_device()
    if dev not in _device_cus:
        n = int(_fn("elementwise", "br_device_cu_count", [])())
        _device_cus[dev] = n if n > 0 else 256
    return _device_cus[dev]


# ------------------------------------------------------------------ elementwise -----
def embedding(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> None:
    _dev("embedding", table, tokens, out)
    T = tokens.numel()
    V, H = table.shape
    _req(tokens.dtype == torch.int32, "embedding: tokens must be int32")
    _req(out.dtype == torch.float32 and out.shape == (T, H), "embedding: out must be float32 [T, H]")
    f = _fn("elementwise", "br_embedding", [_P, c_int, _P, _P, c_int, c_int, c_int, _P])
    _check(f(_ptr(table), _is_bf16(table, "embedding"), _ptr(tokens), _ptr(out), T, H, V, _stream()), "embedding")


def rmsnorm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None) -> None:
    _dev("rmsnorm", x, w, out, rows)
    H = x.shape[-1]
    R = out.shape[0]
    _req(x.dtype == torch.float32 and w.dtype == torch.float32, "rmsnorm: x and w must be float32")
    _req(w.numel() == H and out.shape[-1] == H, "rmsnorm: widths of x, w and out differ")
    if rows is None:
        _req(x.shape[0] == R, "rmsnorm: out has other rows than x")
    else:
        _req(rows.dtype == torch.int32 and rows.numel() == R, "rmsnorm: rows must be int32 [R]")
    f = _fn("elementwise", "br_rmsnorm", [_P, _P, _P, c_int, _P, c_int, c_int, c_float, _P])
    _check(f(_ptr(x), _ptr(w), _ptr(out), _is_bf16(out, "rmsnorm"), _ptr(rows), R, H, float(eps), _stream()),
           "rmsnorm")


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    _dev("rope_table", positions, inv_freq, cos, sin)
    T, P = positions.numel(), inv_freq.numel()
    _req(positions.dtype == torch.int32 and inv_freq.dtype == torch.float32, "rope_table: dtypes")
    _req(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.numel() >= T * P
         and sin.numel() >= T * P, "rope_table: tables must be float32 [T, P]")
    f = _fn("elementwise", "br_rope_table", [_P, _P, _P, _P, c_int, c_int, _P])
    _check(f(_ptr(positions), _ptr(inv_freq), _ptr(cos), _ptr(sin), T, P, _stream()), "rope_table")


def rope_kv_write(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  positions: torch.Tensor, seq_of_token: torch.Tensor, slots: torch.Tensor,
                  block_table: torch.Tensor, cache: Optional[torch.Tensor], nq: int, nkv: int, hd: int,
                  rotary_dim: int, adjacent: bool, page: int, write_cache: bool) -> None:
    _dev("rope_kv_write", qkv, cos, sin, positions, seq_of_token, slots, block_table, cache)
    T = qkv.shape[0]
    _req(qkv.shape[1] == (nq + 2 * nkv) * hd, "rope_kv_write: qkv width is not (nq + 2 nkv) * head_dim")
    _req(positions.numel() >= T and seq_of_token.numel() >= T, "rope_kv_write: positions shorter than tokens")
    _req(block_table.dim() == 2 and block_table.dtype == torch.int32, "rope_kv_write: block table int32 [slots, pages]")
    if cos is not None:
        _req(cos.numel() >= T * (rotary_dim // 2) and sin is not None, "rope_kv_write: rotary tables too short")
    if write_cache:
        _req(cache is not None and cache.dtype == qkv.dtype, "rope_kv_write: cache dtype differs from activations")
        _req(cache.shape[1:] == (2, nkv, page, hd), "rope_kv_write: cache unit must be [pages, 2, nkv, page, hd]")
    f = _fn("elementwise", "br_rope_kv_write",
            [_P, c_int, _P, _P, _P, _P, _P, _P, c_int, _P] + [c_int] * 8 + [_P])
    _check(f(_ptr(qkv), _is_bf16(qkv, "rope_kv_write"), _ptr(cos), _ptr(sin), _ptr(positions),
             _ptr(seq_of_token), _ptr(slots), _ptr(block_table), block_table.shape[1], _ptr(cache), T, nq, nkv,
             hd, rotary_dim, int(adjacent), page, int(write_cache), _stream()), "rope_kv_write")


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> None:
    _dev("silu_mul", gu, out)
    T, I2 = gu.shape
    _req(I2 % 2 == 0 and out.shape == (T, I2 // 2) and out.dtype == gu.dtype, "silu_mul: out must be [T, I] of gu's dtype")
    f = _fn("elementwise", "br_silu_mul", [_P, _P, c_int, c_int, c_int, _P])
    _check(f(_ptr(gu), _ptr(out), _is_bf16(gu, "silu_mul"), T, I2 // 2, _stream()), "silu_mul")


def residual_add(x: torch.Tensor, y: torch.Tensor) -> None:
    _dev("residual_add", x, y)
    _req(x.dtype == torch.float32 and x.numel() == y.numel(), "residual_add: x float32, same size as y")
    f = _fn("elementwise", "br_residual_add", [_P, _P, c_int, c_size_t, _P])
    _check(f(_ptr(x), _ptr(y), _is_bf16(y, "residual_add"), x.numel(), _stream()), "residual_add")


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    _dev("gather_rows", x, rows, out)
    _req(x.dtype == torch.float32 and out.dtype == torch.float32 and rows.dtype == torch.int32, "gather_rows: dtypes")
    _req(out.shape == (rows.numel(), x.shape[1]), "gather_rows: out must be [R, H]")
    f = _fn("elementwise", "br_gather_rows", [_P, _P, _P, c_int, c_int, _P])
    _check(f(_ptr(x), _ptr(rows), _ptr(out), rows.numel(), x.shape[1], _stream()), "gather_rows")


def convert(a: torch.Tensor, out: torch.Tensor) -> None:
    _dev("convert", a, out)
    _req(a.numel() == out.numel(), "convert: sizes differ")
    if a.dtype == torch.float32 and out.dtype == torch.bfloat16:
        to_bf16 = 1
    elif a.dtype == torch.bfloat16 and out.dtype == torch.float32:
        to_bf16 = 0
    else:
        raise KernelError(f"convert: {a.dtype} -> {out.dtype} is not supported")
    f = _fn("elementwise", "br_convert", [_P, _P, c_int, c_size_t, _P])
    _check(f(_ptr(a), _ptr(out), to_bf16, a.numel(), _stream()), "convert")


# -------------------------------------------------------------- random weights -----
def _random_fill(fn_name: str, out: torch.Tensor, key: int, param: float, first: int) -> None:
    _dev(fn_name, out)
    f = _fn("random_weights", "br_" + fn_name, [_P, c_int, c_size_t, c_size_t, ctypes.c_uint64, c_float, _P])
    _check(f(_ptr(out), _is_bf16(out, fn_name), out.numel(), int(first), int(key) & ((1 << 64) - 1), param, _stream()),
           fn_name)


def random_normal(out: torch.Tensor, key: int, std: float, first: int = 0) -> None:
    """out (flat order) = elements first.. of the normal tensor with this key (see
    weights/random_weights.py for the generator); the scale is float32(std) * 2^-16."""
    import numpy as np
    _random_fill("random_normal", out, key, float(np.float32(std) * np.float32(2.0 ** -16)), first)


def random_ones(out: torch.Tensor, key: int, jitter: float, first: int = 0) -> None:
    """out = 1 + (2u - 1) * jitter with u the generator's uniform number of each element."""
    _random_fill("random_ones", out, key, float(jitter), first)


# ------------------------------------------------------- memory-rate measurements -----
def stream_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst = src, 16 bytes a lane: what a plain copy kernel gets out of this GPU's memory
    (`bench.py` reports it beside the published peak)."""
    _dev("stream_copy", src, dst)
    n = src.numel() * src.element_size()
    _req(n == dst.numel() * dst.element_size() and n % 16 == 0, "stream_copy: equal sizes, a multiple of 16 bytes")
    f = _fn("elementwise", "br_stream_copy", [_P, _P, c_size_t, _P])
    _check(f(_ptr(src), _ptr(dst), n, _stream()), "stream_copy")


def stream_read(src: torch.Tensor, sums: torch.Tensor) -> None:
    """Reads all of `src` once (every workgroup a contiguous region of its own, eight non-temporal
    16-byte loads in flight per lane) and leaves partial sums of its words in `sums` (float32, at
    least 32 per compute unit): the read rate of a kernel that only streams."""
    _dev("stream_read", src, sums)
    n = src.numel() * src.element_size()
    _req(n % 16 == 0 and sums.dtype == torch.float32, "stream_read: a multiple of 16 bytes, float32 sums")
    f = _fn("elementwise", "br_stream_read", [_P, _P, c_int, c_size_t, _P])
    _check(f(_ptr(src), _ptr(sums), sums.numel(), n, _stream()), "stream_read")


# ------------------------------------------------------------------------ GEMM ------
GEMM_SCRATCH_FLOATS = 16 * 1024 * 1024   # 64 MB: room for the partial sums of the products that the bf16 kernels split along k


def weight_blockable(w: torch.Tensor) -> bool:
    """Whether `block_weight` takes this matrix: bfloat16 [N, K] on the device with K in steps of
    128 from 1024 (what every bf16 kernel family that reads the blocked layout takes)."""
    return w.dim() == 2 and w.is_cuda and w.dtype == torch.bfloat16 and w.shape[1] % 128 == 0 and w.shape[1] >= 1024


def weight_block_rows() -> int:
    """Rows of a block of the blocked weight layout (WL_BLOCK_ROWS in csrc/gemm_bf16.hip)."""
    return int(_fn("gemm_bf16", "br_gemm_bf16_block_rows", [])())


def block_weight(w: torch.Tensor, alloc=None) -> torch.Tensor:
    """The matrix [N, K] as blocks [ceil(N / R), K / 128, R, 128], R = `weight_block_rows()` = 16:
    R rows by 128 k are contiguous and a strip of R rows is one run along k; rows are padded
    with zeros to a multiple of R.  The products that stream a weight matrix once per step
    read it faster in this order than 256 bytes from every row.  `gemm`, `gemm_swiglu`,
    `gemm_norm_prepare` and `gemm_norm_scaled` take either form and tell them apart by the
    number of dimensions; N is then the output's width.  `alloc(shape, dtype)` gives the
    memory of the result (default: a new tensor)."""
    if not weight_blockable(w):
        raise KernelError(f"block_weight: {tuple(w.shape)} {w.dtype} on {w.device} is not taken")
    N, K = w.shape
    R = weight_block_rows()
    nb = -(-N // R)
    shape = (nb, K // 128, R, 128)
    out = alloc(shape, w.dtype) if alloc is not None else torch.empty(shape, dtype=w.dtype, device=w.device)
    full = N // R
    if full:
        out[:full].copy_(w[:full * R].view(full, R, K // 128, 128).permute(0, 2, 1, 3))
    if full != nb:
        out[full].zero_()
        out[full, :, :N - full * R].copy_(w[full * R:].view(N - full * R, K // 128, 128).permute(1, 0, 2))
    return out


def unblock_weight(wb: torch.Tensor, N: int) -> torch.Tensor:
    """The rows [N, K] of a blocked matrix (tests, and parts that need rows again)."""
    nb, kb, R = wb.shape[0], wb.shape[1], wb.shape[2]
    return wb.permute(0, 2, 1, 3).reshape(nb * R, kb * 128)[:N].contiguous()


def _weight_dims(name: str, w: torch.Tensor, n_out: int):
    """(N, K, layout) of a weight argument: rows [N, K] (layout 0) or blocks (layout 1, N = n_out)."""
    if w.dim() == 4:
        R = weight_block_rows()
        _req(w.shape[2] == R and w.shape[3] == 128 and w.dtype == torch.bfloat16 and w.is_contiguous()
             and w.shape[0] == -(-n_out // R), f"{name}: blocked weight {tuple(w.shape)} for {n_out} outputs")
        return n_out, w.shape[1] * 128, 1
    _req(w.dim() == 2 and w.is_contiguous(), f"{name}: the weight must be [N, K], dense")
    return w.shape[0], w.shape[1], 0


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, kernel: int = 0,
         scratch: Optional[torch.Tensor] = None) -> None:
    """out[M, N] (+)= a[M, K] @ w[N, K]^T.

    float32 a and w: the true 32-bit kernel (out float32).  bfloat16 a and w: the
    matrix-core kernels with float accumulation; out is bfloat16, or float32 (and may
    then accumulate, which is how a projection adds into the residual stream).
    Rows of `a` and `out` may be strided (a view of a wider buffer); w is contiguous.
    `kernel` forces one bf16 kernel (1, 2: 128x128 and 256x128 tiles staged through
    registers, any shape; 3: skinny, M <= 64; 4, 5, 6: 256x128, 128x256 and 128x128 tiles
    loaded straight into LDS, K in steps of 64; 7: streaming by workgroups that stay, M <= 16
    and K in steps of 128 from 1024; 8: the same for 17 to 64 rows, K in steps of 128; 5 or 6 plus
    16 p: that tile with p runs along k, for measurements; 9: a 64x128 tile loaded straight into
    LDS, M <= 64; 10: a 256x192 tile loaded straight into LDS; 12 to 15: 256x256, 128x256, 256x192 and
    256x224 tiles of four waves, one to a SIMD, K in steps of 64 and output rows in steps of 16 bytes, plus
    16 p for p runs along k); 0 chooses by shape.  A weight from `block_weight` is taken by kernels 4 to 15.
    `scratch` (float32, on the device): with it, a bf16 product of more than 16 rows with too
    few tiles to fill the chip is cut along k into runs that a second kernel sums in a fixed order.
    """
    name = "gemm"
    for t in (a, w, out):
        if not t.is_cuda:
            raise KernelError(f"{name}: tensor on {t.device}; kernels run on the GPU only")
    _req(a.dim() == 2 and out.dim() == 2, "gemm: 2-D tensors")
    M, K = a.shape
    N, wk, wl = _weight_dims(name, w, out.shape[1])
    _req(wk == K and out.shape == (M, N), f"gemm: shapes a{tuple(a.shape)} w{tuple(w.shape)} out{tuple(out.shape)}")
    _req(a.stride(1) == 1 and out.stride(1) == 1, "gemm: rows must be dense")
    lda, ldc = (a.stride(0) if M > 1 else K), (out.stride(0) if M > 1 else N)
    if a.dtype == torch.float32 and w.dtype == torch.float32:
        _req(out.dtype == torch.float32, "gemm: float32 inputs give a float32 output")
        f = _fn("gemm_f32", "br_gemm_f32", [_P, _P, _P, c_int, c_int, c_int, c_size_t, c_size_t, c_int, _P])
        _check(f(_ptr(a), _ptr(w), _ptr(out), M, N, K, lda, ldc, int(accumulate), _stream()), name)
    elif a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        if out.dtype == torch.bfloat16:
            _req(not accumulate, "gemm: accumulation needs a float32 output")
            mode = 0
        elif out.dtype == torch.float32:
            mode = 2 if accumulate else 1
        else:
            raise KernelError(f"gemm: output dtype {out.dtype}")
        if scratch is not None:
            _req(scratch.is_cuda and scratch.dtype == torch.float32 and scratch.is_contiguous(), "gemm: scratch must be float32 on the device")
        f = _fn("gemm_bf16", "br_gemm_bf16_ex",
                [_P, _P, _P, c_int, c_int, c_int, c_size_t, c_size_t, c_int, c_int, _P, c_size_t, c_int, _P])
        _check(f(_ptr(a), _ptr(w), _ptr(out), M, N, K, lda, ldc, mode, kernel, _ptr(scratch),
                 0 if scratch is None else scratch.numel() * 4, wl, _stream()), name)
    else:
        raise KernelError(f"gemm: a is {a.dtype} and w is {w.dtype}; both float32 or both bfloat16")


def gemm_swiglu(a: torch.Tensor, w_gu: torch.Tensor, out: torch.Tensor, kernel: int = 0,
                scratch: Optional[torch.Tensor] = None) -> None:
    """out[M, I] = silu(a @ Wg^T) * (a @ Wu^T) in one bf16 product: `w_gu` [2 I, K] holds
    gate and up rows interleaved in blocks of 16 (see `interleave_gate_up`).  `scratch` as
    for `gemm`."""
    for t in (a, w_gu, out):
        if not t.is_cuda:
            raise KernelError(f"gemm_swiglu: tensor on {t.device}; kernels run on the GPU only")
    _req(a.dtype == w_gu.dtype == out.dtype == torch.bfloat16, "gemm_swiglu: bfloat16 only")
    M, K = a.shape
    N, wk, wl = _weight_dims("gemm_swiglu", w_gu, 2 * out.shape[1])
    _req(N % 16 == 0 and wk == K and out.shape == (M, N // 2), "gemm_swiglu: shapes")
    _req(a.stride(1) == 1 and out.stride(1) == 1, "gemm_swiglu: rows must be dense")
    lda, ldc = (a.stride(0) if M > 1 else K), (out.stride(0) if M > 1 else N // 2)
    f = _fn("gemm_bf16", "br_gemm_bf16_ex",
            [_P, _P, _P, c_int, c_int, c_int, c_size_t, c_size_t, c_int, c_int, _P, c_size_t, c_int, _P])
    if scratch is not None:
        _req(scratch.is_cuda and scratch.dtype == torch.float32 and scratch.is_contiguous(), "gemm_swiglu: scratch must be float32 on the device")
    _check(f(_ptr(a), _ptr(w_gu), _ptr(out), M, N, K, lda, ldc, 3, kernel, _ptr(scratch),
             0 if scratch is None else scratch.numel() * 4, wl, _stream()), "gemm_swiglu")


def gemm_stream_takes(M: int, K: int) -> bool:
    """Whether the streaming products (kernels 7 and 8 of `gemm`, and the two forms below)
    take M rows over K: up to 16 rows with K in steps of 128 from 1024, or 17 to 64 rows with
    K in steps of 128 from 256."""
    return (0 < M <= 16 and K % 128 == 0 and K >= 1024) or (16 < M <= 64 and K % 128 == 0 and K >= 256)


def gemm_tile_choice(M: int, N: int, K: int, mode: int = 0, scratch_floats: int = 0):
    """What a bf16 product of more than 64 rows runs on when its K is a multiple of 64 and its rows and output
    are aligned: (kernel, runs along k, n1).  n1 > 0: the first n1 weight rows go to the 256x256 tile of one
    wave per SIMD in whole rounds over the chip, the rest to `kernel`.  mode: 0 bf16 out, 1 float out,
    2 float out added to, 3 SwiGLU."""
    f = _fn("gemm_bf16", "br_gemm_bf16_tile_choice", [c_int, c_int, c_int, c_int, c_size_t, _P, _P, _P])
    k, p, n1 = c_int(0), c_int(0), c_int(0)
    _check(f(M, N, K, mode, scratch_floats * 4, ctypes.byref(k), ctypes.byref(p), ctypes.byref(n1)), "gemm_tile_choice")
    return k.value, p.value, n1.value


def gemm_wide_parts(M: int, N: int, K: int, scratch_floats: int, accumulate: bool = True) -> int:
    """Into how many runs along k a bf16 product of 17 to 64 rows is cut when it is given that
    much scratch (0: the wide streaming product does not take it)."""
    f = _fn("gemm_bf16", "br_gemm_bf16_wide_parts", [c_int, c_int, c_int, c_int, c_size_t])
    return int(f(M, N, K, 2 if accumulate else 1, scratch_floats * 4))


def gemm_wide_partial(a: torch.Tensor, w: torch.Tensor, n_out: int, scratch: torch.Tensor,
                      ssq: Optional[torch.Tensor] = None, tiles: int = 0, eps: float = 0.0) -> int:
    """The runs of a @ w^T (17 to 64 bfloat16 rows, `n_out` columns) as float sums left in
    `scratch`, [runs][M][n_out], for a consumer that adds them in run order and rounds to bfloat16
    itself: the bits of `gemm` (with `ssq` and `tiles`: of `gemm_norm_scaled`) without the launch
    that adds the runs.  Returns the number of runs, or 0 (nothing launched) where the product
    would not be cut."""
    _dev("gemm_wide_partial", a, w, scratch, ssq)
    M, K = a.shape
    N, wk, wl = _weight_dims("gemm_wide_partial", w, n_out)
    _req(a.dtype == w.dtype == torch.bfloat16 and scratch.dtype == torch.float32 and wk == K and N == n_out,
         "gemm_wide_partial: bfloat16 rows and matrix")
    if not (16 < M <= 64 and gemm_stream_takes(M, K) and a.stride(1) == 1 and a.stride(0) % 8 == 0
            and gemm_wide_parts(M, N, K, scratch.numel()) >= 2):
        return 0
    if ssq is not None:
        _req(ssq.dtype == torch.float32 and tiles > 0 and ssq.numel() >= tiles * SSQ_LD, "gemm_wide_partial: sums of squares")
    f = _fn("gemm_bf16", "br_gemm_bf16_wide_partial",
            [_P, _P, c_int, c_int, c_int, c_size_t, _P, c_int, c_int, c_float, _P, c_size_t, c_int, _P, _P])
    parts = c_int(0)
    _check(f(_ptr(a), _ptr(w), M, N, K, a.stride(0), _ptr(ssq), int(tiles), K, float(eps), _ptr(scratch),
             scratch.numel() * 4, wl, ctypes.byref(parts), _stream()), "gemm_wide_partial")
    return parts.value


SSQ_LD = 64        # row stride of the sums of squares that a product leaves for the next norm (SSQ_LD in csrc/gemm_bf16.hip)


def gemm_norm_prepare(a: torch.Tensor, w: torch.Tensor, x: torch.Tensor, gain: torch.Tensor, xg: torch.Tensor,
                      ssq: torch.Tensor, scratch: Optional[torch.Tensor] = None) -> int:
    """x += a @ w^T (x float32: rows of the residual stream) and, in the same kernels, what
    the RMS norm that reads x next needs: xg = bfloat16(x * gain) and, in ssq[tiles, 64],
    sums of x^2 per row over runs of columns.  Returns the number of tiles; `gemm_norm_scaled`
    takes all three.  Up to 16 rows: N in steps of 16.  17 to 64 rows: N in steps of 256 and
    `scratch` (float32, as for `gemm`) for the product's runs along k.  Raises KernelError for
    anything else."""
    _dev("gemm_norm_prepare", a, w, x, gain, xg, ssq, scratch)
    M, K = a.shape
    N, wk, wl = _weight_dims("gemm_norm_prepare", w, x.shape[1])
    _req(a.dtype == w.dtype == xg.dtype == torch.bfloat16 and x.dtype == gain.dtype == ssq.dtype == torch.float32,
         "gemm_norm_prepare: bfloat16 product into float32 rows")
    _req(gemm_stream_takes(M, K) and N % (16 if M <= 16 else 256) == 0, f"gemm_norm_prepare: {M} rows, N {N}, K {K} are not taken")
    _req(wk == K and x.shape == (M, N) and xg.shape == (M, N) and gain.numel() == N
         and ssq.numel() >= (N // 16) * SSQ_LD, "gemm_norm_prepare: shapes")
    tiles = c_int(0)
    f = _fn("gemm_bf16", "br_gemm_bf16_norm_prepare",
            [_P, _P, _P, c_int, c_int, c_int, c_size_t, c_size_t, _P, _P, c_size_t, _P, ctypes.POINTER(c_int), _P, c_size_t, c_int, _P])
    _check(f(_ptr(a), _ptr(w), _ptr(x), M, N, K, a.stride(0) if M > 1 else K, x.stride(0) if M > 1 else N, _ptr(gain),
             _ptr(xg), xg.stride(0) if M > 1 else N, _ptr(ssq), ctypes.byref(tiles), _ptr(scratch),
             0 if scratch is None else scratch.numel() * 4, wl, _stream()), "gemm_norm_prepare")
    return tiles.value


def gemm_norm_scaled(xg: torch.Tensor, ssq: torch.Tensor, tiles: int, eps: float, w: torch.Tensor, out: torch.Tensor,
                     swiglu: bool = False, scratch: Optional[torch.Tensor] = None) -> None:
    """out = rmsnorm(x) @ w^T from what `gemm_norm_prepare` left: xg = bfloat16(x * gain)
    [M, K], the sums of squares ssq and their number of tiles; 1 / rms multiplies the
    product's sums.  `out` bfloat16 or float32 [M, N]; with `swiglu`, bfloat16 [M, N / 2] as
    `gemm_swiglu`."""
    _dev("gemm_norm_scaled", xg, ssq, w, out, scratch)
    M, K = xg.shape
    N, wk, wl = _weight_dims("gemm_norm_scaled", w, 2 * out.shape[1] if swiglu else out.shape[1])
    _req(xg.dtype == w.dtype == torch.bfloat16 and ssq.dtype == torch.float32, "gemm_norm_scaled: bfloat16 rows and matrix")
    _req(gemm_stream_takes(M, K) and wk == K and tiles > 0 and ssq.numel() >= tiles * SSQ_LD, "gemm_norm_scaled: sizes")
    if swiglu:
        _req(out.dtype == torch.bfloat16 and N % 16 == 0 and out.shape == (M, N // 2), "gemm_norm_scaled: SwiGLU gives bfloat16 [M, N / 2]")
        mode = 3
    else:
        _req(out.shape == (M, N) and out.dtype in (torch.bfloat16, torch.float32), "gemm_norm_scaled: out must be [M, N]")
        mode = 0 if out.dtype == torch.bfloat16 else 1
    f = _fn("gemm_bf16", "br_gemm_bf16_norm_scaled",
            [_P, _P, _P, c_int, c_int, c_int, c_size_t, c_size_t, c_int, _P, c_int, c_int, c_float, _P, c_size_t, c_int, _P])
    _check(f(_ptr(xg), _ptr(w), _ptr(out), M, N, K, xg.stride(0) if M > 1 else K, out.stride(0) if M > 1 else out.shape[1],
             mode, _ptr(ssq), int(tiles), K, float(eps), _ptr(scratch), 0 if scratch is None else scratch.numel() * 4,
             wl, _stream()), "gemm_norm_scaled")


def interleave_gate_up(w_gate: torch.Tensor, w_up: torch.Tensor, alloc=None) -> torch.Tensor:
    """[2 I, K]: blocks of 8 gate rows followed by the 8 up rows of the same outputs.
    `alloc(shape, dtype)` gives the memory of the result (default: a new tensor)."""
    I, K = w_gate.shape
    if I % 8:
        raise KernelError(f"interleave_gate_up: intermediate size {I} is not a multiple of 8")
    out = alloc((2 * I, K), w_gate.dtype) if alloc is not None else torch.empty((2 * I, K), dtype=w_gate.dtype, device=w_gate.device)
    o = out.view(I // 8, 2, 8, K)
    o[:, 0].copy_(w_gate.view(I // 8, 8, K))
    o[:, 1].copy_(w_up.view(I // 8, 8, K))
    return out


# ------------------------------------------------------------------- attention -----
def attention_simple(q: torch.Tensor, q_stride: int, out: torch.Tensor, positions: torch.Tensor,
                     seq_of_token: torch.Tensor, slots: torch.Tensor, block_table: torch.Tensor,
                     cache: torch.Tensor, T: int, nq: int, nkv: int, hd: int, page: int,
                     window: Optional[int], scale: float) -> None:
    _dev("attention_simple", out, positions, seq_of_token, slots, block_table, cache)
    _req(q.is_cuda and q.dtype == cache.dtype == out.dtype, "attention_simple: q, cache and out share a dtype")
    _req(out.shape == (T, nq * hd), "attention_simple: out must be [T, nq * hd]")
    _req(cache.shape[1:] == (2, nkv, page, hd), "attention_simple: cache unit must be [pages, 2, nkv, page, hd]")
    _req(nq % nkv == 0, "attention_simple: heads must be a multiple of kv heads")
    _req(hd <= 512, f"attention_simple: head_dim {hd} above 512 is not supported")
    f = _fn("attention_simple", "br_attn_simple",
            [_P, c_size_t, _P, c_int, _P, _P, _P, _P, c_int, _P] + [c_int] * 6 + [c_float, _P])
    _check(f(_ptr(q), q_stride, _ptr(out), _is_bf16(q, "attention_simple"), _ptr(positions), _ptr(seq_of_token),
             _ptr(slots), _ptr(block_table), block_table.shape[1], _ptr(cache), T, nq, nkv, hd, page,
             int(window or 0), float(scale), _stream()), "attention_simple")


def attention_prefill_bf16(q: torch.Tensor, q_stride: int, out: torch.Tensor, cu_seqlens: torch.Tensor,
                           slots: torch.Tensor, ctx_lens: torch.Tensor, block_table: torch.Tensor,
                           cache: torch.Tensor, B: int, max_new: int, nq: int, nkv: int, hd: int, page: int,
                           window: Optional[int], scale: float, variant: int = 0) -> None:
    """Flash attention on the matrix cores for steps with several tokens per sequence.
    `variant` 1 reads operand fragments straight from the cache, 2 and 3 stage pages in LDS
    through registers (workgroups of 8 and of 4 waves), 4 brings them into an LDS ring by
    direct loads (head sizes 64 and 128), 0 chooses by the head size."""
    _dev("attention_prefill_bf16", out, cu_seqlens, slots, ctx_lens, block_table, cache)
    _req(q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
         "attention_prefill_bf16: bfloat16 only")
    _req(hd % 16 == 0 and hd <= 256, f"attention_prefill_bf16: head_dim {hd} must be a multiple of 16, at most 256")
    _req(page == 64, "attention_prefill_bf16: pages of 64 tokens")
    _req(scale > 0, f"attention_prefill_bf16: the score scale must be positive, not {scale} (the kernels take the row maximum before scaling)")
    _req(cache.shape[1:] == (2, nkv, page, hd), "attention_prefill_bf16: cache unit must be [pages, 2, nkv, page, hd]")
    _req(out.shape[1] == nq * hd and nq % nkv == 0, "attention_prefill_bf16: out must be [T, nq * hd]")
    f = _fn("attention_bf16", "br_attn_prefill_bf16",
            [_P, c_size_t, _P, _P, _P, _P, _P, c_int, _P] + [c_int] * 7 + [c_float, c_int, _P])
    _check(f(_ptr(q), q_stride, _ptr(out), _ptr(cu_seqlens), _ptr(slots), _ptr(ctx_lens), _ptr(block_table),
             block_table.shape[1], _ptr(cache), B, max_new, nq, nkv, hd, page, int(window or 0), float(scale),
             variant, _stream()), "attention_prefill_bf16")


def attention_decode_bf16(q: torch.Tensor, q_stride: int, out: torch.Tensor, slots: torch.Tensor,
                          ctx_lens: torch.Tensor, block_table: torch.Tensor, cache: torch.Tensor, B: int,
                          nq: int, nkv: int, hd: int, page: int, window: Optional[int], scale: float,
                          nsplit: int, part_o: Optional[torch.Tensor], part_ml: Optional[torch.Tensor],
                          variant: int = 0, fuse_rope: bool = False, cos: Optional[torch.Tensor] = None,
                          sin: Optional[torch.Tensor] = None, write_cache: bool = True,
                          run_sums: Optional[torch.Tensor] = None, runs: int = 0) -> None:
    """Attention of one new token per sequence over its pages, cut into `nsplit` runs.
    `variant` forces a kernel: 1 reads operands straight from the cache, 2 brings pages
    through a ring in LDS (head sizes 64 and 128); 0 chooses.

    `fuse_rope` (where `attention_decode_fuses_rope` says so): `q` is the step's raw
    [B, (nq + 2 nkv) * hd] rows; the kernel rotates queries and the new key by `cos` / `sin`
    ([B, hd / 2], pairs (p, p + hd / 2); None = no rotation) and stores key and value of the
    new token in the cache itself (`write_cache`), so `rope_kv_write` is not called.  With
    `run_sums` (float32, `runs` matrices [B, (nq + 2 nkv) * hd] one after another, as
    `gemm_wide_partial` leaves them) the raw rows are the runs' sums, which the kernel adds
    itself; `q` is then not read."""
    _dev("attention_decode_bf16", out, slots, ctx_lens, block_table, cache, part_o, part_ml, run_sums)
    _req(q.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
         "attention_decode_bf16: bfloat16 only")
    _req(hd % 16 == 0 and hd <= 256, f"attention_decode_bf16: head_dim {hd} must be a multiple of 16, at most 256")
    _req(page == 64, "attention_decode_bf16: pages of 64 tokens")
    _req(cache.shape[1:] == (2, nkv, page, hd), "attention_decode_bf16: cache unit must be [pages, 2, nkv, page, hd]")
    _req(out.shape == (B, nq * hd) and nq % nkv == 0, "attention_decode_bf16: out must be [B, nq * hd]")
    if nsplit > 1:
        _req(part_o is not None and part_o.dtype == torch.float32 and part_o.numel() >= B * nq * nsplit * hd
             and part_ml is not None and part_ml.numel() >= B * nq * nsplit * 2,
             "attention_decode_bf16: scratch for the splits is too small")
    f = _fn("attention_bf16", "br_attn_decode_bf16",
            [_P, c_size_t, _P, _P, _P, _P, c_int, _P] + [c_int] * 6 + [c_float, c_int, _P, _P, c_int, c_int, _P, _P,
                                                                      c_int, _P])
    if fuse_rope:
        _req(attention_decode_fuses_rope(hd, nq, nkv, page, block_table.shape[1], nsplit),
             "attention_decode_bf16: rotation and cache write are not fused for these sizes")
        _req(run_sums is not None or q.shape[-1] == (nq + 2 * nkv) * hd,
             "attention_decode_bf16: fused rotation needs the raw q, k, v rows")
        if cos is not None:
            _dev("attention_decode_bf16", cos, sin)
            _req(sin is not None and cos.dtype == sin.dtype == torch.float32 and cos.numel() >= B * (hd // 2)
                 and sin.numel() >= B * (hd // 2), "attention_decode_bf16: rotary tables must be float32 [B, hd / 2]")
    if run_sums is not None:
        _req(fuse_rope and variant in (0, 2) and run_sums.dtype == torch.float32 and 1 <= runs <= 64
             and run_sums.numel() >= runs * B * (nq + 2 * nkv) * hd,
             "attention_decode_bf16: run sums go with the fused rotation, float32 [runs, B, (nq + 2 nkv) * hd]")
        g = _fn("attention_bf16", "br_attn_decode_bf16_runs",
                [_P, c_int, _P, _P, _P, _P, c_int, _P] + [c_int] * 6 + [c_float, c_int, _P, _P, _P, _P, c_int, _P])
        _check(g(_ptr(run_sums), int(runs), _ptr(out), _ptr(slots), _ptr(ctx_lens), _ptr(block_table),
                 block_table.shape[1], _ptr(cache), B, nq, nkv, hd, page, int(window or 0), float(scale), nsplit,
                 _ptr(part_o), _ptr(part_ml), _ptr(cos), _ptr(sin), int(write_cache), _stream()),
               "attention_decode_bf16")
        return
    _check(f(_ptr(q), q_stride, _ptr(out), _ptr(slots), _ptr(ctx_lens), _ptr(block_table), block_table.shape[1],
             _ptr(cache), B, nq, nkv, hd, page, int(window or 0), float(scale), nsplit, _ptr(part_o),
             _ptr(part_ml), int(variant), int(fuse_rope), _ptr(cos) if fuse_rope else None,
             _ptr(sin) if fuse_rope else None, int(write_cache), _stream()), "attention_decode_bf16")


def attention_decode_fuses_rope(hd: int, nq: int, nkv: int, page: int, table_pages: int, nsplit: int) -> bool:
    """Whether `attention_decode_bf16` can do the step's rotation (full head, pairs
    (p, p + hd / 2), or none) and cache write itself: the kernel that brings pages through
    LDS (head sizes 64 and 128, runs of at most 1024 pages), groups of up to 16 heads."""
    return (hd in (64, 128) and page == 64 and nkv > 0 and nq % nkv == 0 and nq // nkv <= 16
            and -(-table_pages // max(1, nsplit)) <= 1024)


# -------------------------------------------------------------------- sampling -----
def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    _dev("argmax", logits, out)
    B, V = logits.shape
    _req(logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= B, "argmax: float32 in, int32 out")
    f = _fn("sampling", "br_argmax", [_P, _P, c_int, c_int, _P])
    _check(f(_ptr(logits), _ptr(out), B, V, _stream()), "argmax")


def argmax_advance(logits: torch.Tensor, out: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor,
                   slots: torch.Tensor, ctx_lens: torch.Tensor) -> None:
    """`argmax`, and for every live row (slot >= 0) the step arrays of the next single-token
    step: tokens[b] = the row's token, positions[b] and ctx_lens[b] one more."""
    _dev("argmax_advance", logits, out, tokens, positions, slots, ctx_lens)
    B, V = logits.shape
    _req(logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= B, "argmax_advance: float32 in, int32 out")
    _req(all(t.dtype == torch.int32 and t.numel() >= B for t in (tokens, positions, slots, ctx_lens)),
         "argmax_advance: the step arrays must be int32 [B]")
    f = _fn("sampling", "br_argmax_advance", [_P, _P, c_int, c_int, _P, _P, _P, _P, _P])
    _check(f(_ptr(logits), _ptr(out), B, V, _ptr(tokens), _ptr(positions), _ptr(slots), _ptr(ctx_lens), _stream()),
           "argmax_advance")


def step_advance(drawn: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                 ctx_lens: torch.Tensor, n: int) -> None:
    """For the first n rows that are live (slot >= 0): tokens[i] = drawn[i], positions[i] and
    ctx_lens[i] one more: the next single-token step's arrays from the tokens a sampler drew."""
    _dev("step_advance", drawn, tokens, positions, slots, ctx_lens)
    _req(all(t.dtype == torch.int32 and t.numel() >= n for t in (drawn, tokens, positions, slots, ctx_lens)),
         "step_advance: int32 arrays of at least n entries")
    f = _fn("sampling", "br_step_advance", [_P, _P, _P, _P, _P, c_int, _P])
    _check(f(_ptr(drawn), _ptr(tokens), _ptr(positions), _ptr(slots), _ptr(ctx_lens), int(n), _stream()), "step_advance")


def sample_prepare(logits, work, bias_off, bias_tok, bias_val, counts, penalty, temperature):
    """work = logits with bias, repetition penalty and temperature applied.  `counts`: the rows'
    histories as a table int32 [B, V] of occurrences per token on the device (None: no history)."""
    _dev("sample_prepare", logits, work, bias_off, bias_tok, bias_val, counts, penalty, temperature)
    B, V = logits.shape
    _req(logits.dtype == torch.float32 and work.dtype == torch.float32 and work.shape == logits.shape, "sample_prepare: float32 [B, V]")
    _req(counts is None or (counts.dtype == torch.int32 and counts.dim() == 2 and counts.shape[0] >= B and counts.shape[1] == V
                            and counts.is_contiguous()), "sample_prepare: counts must be int32 [B, V]")
    f = _fn("sampling", "br_sample_prepare", [_P, _P, c_int, c_int] + [_P] * 7)
    _check(f(_ptr(logits), _ptr(work), B, V, _ptr(bias_off), _ptr(bias_tok), _ptr(bias_val), _ptr(counts), _ptr(penalty),
             _ptr(temperature), _stream()), "sample_prepare")


def sample_count_add(counts, rows, toks, cnts):
    """counts[rows[e], toks[e]] += cnts[e]: puts histories into the table of `sample_prepare`."""
    _dev("sample_count_add", counts, rows, toks, cnts)
    n = rows.numel()
    _req(counts.dtype == torch.int32 and counts.dim() == 2 and all(t.dtype == torch.int32 and t.numel() == n for t in (rows, toks, cnts)),
         "sample_count_add: int32 counts [B, V] and three int32 lists of one length")
    f = _fn("sampling", "br_sample_count_add", [_P, c_int, c_int, _P, _P, _P, c_int, _P])
    _check(f(_ptr(counts), counts.shape[0], counts.shape[1], _ptr(rows), _ptr(toks), _ptr(cnts), n, _stream()), "sample_count_add")


def sample_filter(work, top_k, min_p, top_p, temperature):
    """Top-k, min-p and top-p masks on `work` [B, V] (entries cut become -inf), the reference's
    order and rules (sampling.rs:89-151), the lower index first among equal values; rows of
    temperature 0 are left alone.  Any vocabulary size, any top_k."""
    _dev("sample_filter", work, top_k, min_p, top_p, temperature)
    B, V = work.shape
    _req(work.dtype == torch.float32 and work.is_contiguous() and top_k.dtype == torch.int32
         and min_p.dtype == top_p.dtype == temperature.dtype == torch.float32
         and min(top_k.numel(), min_p.numel(), top_p.numel(), temperature.numel()) >= B,
         "sample_filter: float32 rows, int32 top_k [B], float32 min_p, top_p, temperature [B]")
    f = _fn("sampling", "br_sample_filter", [_P, c_int, c_int, _P, _P, _P, _P, _P])
    _check(f(_ptr(work), B, V, _ptr(top_k), _ptr(min_p), _ptr(top_p), _ptr(temperature), _stream()), "sample_filter")


def sample_filter_sort(work, keys, top_k, min_p, top_p, temperature):
    """The same masks by sorting every row whole and adding the probabilities in that order
    (what tests hold `sample_filter` against).  `keys`: int64 [B, power of two >= V] scratch."""
    _dev("sample_filter_sort", work, keys, top_k, min_p, top_p, temperature)
    B, V = work.shape
    n2 = keys.shape[1]
    _req(keys.dtype == torch.int64 and keys.shape[0] >= B and n2 >= V and n2 & (n2 - 1) == 0 and keys.is_contiguous(),
         "sample_filter_sort: keys must be int64 [B, power of two >= V]")
    f = _fn("sampling", "br_sample_filter_sort", [_P, _P, c_int, c_int, c_int, _P, _P, _P, _P, _P])
    _check(f(_ptr(work), _ptr(keys), B, V, n2, _ptr(top_k), _ptr(min_p), _ptr(top_p), _ptr(temperature), _stream()),
           "sample_filter_sort")


def sample_draw(work, out, temperature, u, counts=None, rng_key=None, rng_draw=None):
    """`counts` (int32 [B, V], optional): the table of `sample_prepare`; the token drawn
    for a row is added to the row's history there.  The rows' uniform numbers stand in `u`
    (float32 [B]), or with `rng_key` (int64 [B]: `sampling.uniform_key` of each request) and
    `rng_draw` (int32 [B]: each request's next draw, moved on by the call) are made by the
    kernel: `sampling.uniform(seed, sequence, draw)` bit for bit."""
    _dev("sample_draw", work, out, temperature, u, counts, rng_key, rng_draw)
    B, V = work.shape
    _req(out.dtype == torch.int32 and temperature.dtype == torch.float32, "sample_draw: dtypes")
    if counts is not None:
        _req(counts.dtype == torch.int32 and counts.shape[0] >= B and counts.shape[1] == V, "sample_draw: counts must be int32 [B, V]")
    if rng_key is not None:
        _req(rng_draw is not None and rng_key.dtype == torch.int64 and rng_draw.dtype == torch.int32
             and rng_key.numel() >= B and rng_draw.numel() >= B, "sample_draw: rng_key int64 [B] and rng_draw int32 [B]")
        f = _fn("sampling", "br_sample_draw_random", [_P, _P, c_int, c_int, _P, _P, _P, _P, _P])
        _check(f(_ptr(work), _ptr(out), B, V, _ptr(temperature), _ptr(rng_key), _ptr(rng_draw), _ptr(counts), _stream()),
               "sample_draw")
        return
    _req(u is not None and u.dtype == torch.float32 and u.numel() >= B, "sample_draw: u must be float32 [B]")
    if counts is None:
        f = _fn("sampling", "br_sample_draw", [_P, _P, c_int, c_int, _P, _P, _P])
        _check(f(_ptr(work), _ptr(out), B, V, _ptr(temperature), _ptr(u), _stream()), "sample_draw")
        return
    f = _fn("sampling", "br_sample_draw_count", [_P, _P, c_int, c_int, _P, _P, _P, _P])
    _check(f(_ptr(work), _ptr(out), B, V, _ptr(temperature), _ptr(u), _ptr(counts), _stream()), "sample_draw")
