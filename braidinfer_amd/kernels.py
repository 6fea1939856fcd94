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
def embedding(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    _dev("embedding", table, tokens, out)
    T = tokens.numel()
    V, H = table.shape
    _req(tokens.dtype == torch.int32, "embedding: tokens must be int32")
    _req(out.dtype == torch.float32 and out.shape == (T, H), "embedding: out must be float32 [T, H]")
    f = _fn("elementwise", "br_embedding", [_P, c_int, _P, _P, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(table), _is_bf16(table, "embedding"), _ptr(tokens), _ptr(out), T, H, V, float(scale), _stream()), "embedding")


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


def layernorm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
              center: bool = True, add: bool = False, then=None) -> None:
    """out = norm(x) * w, or out += norm(x) * w with `add` (float `out`); `center` False: the RMS norm.
    `then` = (w2, out2, eps2, center2), with `add` only: the rows just added to are normed once more,
    out2 = norm2(out) * w2, in the same kernel; with w2 None out2 takes the rows just added to as they are, in its
    own dtype (for a reader that takes the rows without a norm)."""
    _dev("layernorm", x, w, out, rows)
    H = x.shape[-1]
    R = out.shape[0]
    _req(x.dtype == torch.float32 and w.dtype == torch.float32, "layernorm: x and w must be float32")
    _req(w.numel() == H and out.shape[-1] == H, "layernorm: widths of x, w and out differ")
    if rows is None:
        _req(x.shape[0] == R, "layernorm: out has other rows than x")
    else:
        _req(rows.dtype == torch.int32 and rows.numel() == R, "layernorm: rows must be int32 [R]")
    _req(not add or (out.dtype == torch.float32 and rows is None and out.data_ptr() != x.data_ptr()),
         "layernorm: adding needs float rows of their own, without a gather")
    w2 = out2 = None
    eps2, center2 = 0.0, False
    if then is not None:
        w2, out2, eps2, center2 = then
        _dev("layernorm", w2, out2)
        _req(add and (w2 is None or (w2.dtype == torch.float32 and w2.numel() == H)) and out2.shape == (R, H)
             and out2.data_ptr() not in (x.data_ptr(), out.data_ptr()), "layernorm: the second norm takes float weights [H] "
             "and rows [R, H] of their own, behind an add")
    f = _fn("elementwise", "br_layernorm", [_P, _P, _P, c_int, _P, c_int, c_int, c_float, c_int, c_int, _P, _P, c_int,
                                            c_float, c_int, _P])
    _check(f(_ptr(x), _ptr(w), _ptr(out), _is_bf16(out, "layernorm"), _ptr(rows), R, H, float(eps), int(center),
             int(add), _ptr(w2), _ptr(out2), _is_bf16(out2, "layernorm") if out2 is not None else 0, float(eps2),
             int(center2), _stream()), "layernorm")


def scale_(x: torch.Tensor, scale: float) -> None:
    _dev("scale", x)
    _req(x.dtype == torch.float32, "scale: float32 only")
    f = _fn("elementwise", "br_scale", [_P, c_float, c_size_t, _P])
    _check(f(_ptr(x), float(scale), x.numel(), _stream()), "scale")


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


def add_position_rows(x: torch.Tensor, table: torch.Tensor, positions: torch.Tensor) -> None:
    """x[t, :] += table[positions[t], :]: x float [T, H], table [rows, H] float or bfloat16, positions int32 [T]
    (a position outside the table adds nothing; callers refuse such steps on the host)."""
    _dev("add_position_rows", x, table, positions)
    T, H = x.shape
    _req(x.dtype == torch.float32 and table.dim() == 2 and table.shape[1] == H, "add_position_rows: x float32 [T, H], table [rows, H]")
    _req(positions.dtype == torch.int32 and positions.numel() >= T, "add_position_rows: positions int32 [T]")
    f = _fn("elementwise", "br_add_position_rows", [_P, _P, c_int, _P, c_int, c_int, c_int, _P])
    _check(f(_ptr(x), _ptr(table), _is_bf16(table, "add_position_rows"), _ptr(positions), T, H, table.shape[0], _stream()),
           "add_position_rows")


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

# -------------------------------------------- window attention with pooled blocks -----
def _pwa_unit(name: str, unit: torch.Tensor, nkv: int, dk: int, dv: int, page: int) -> None:
    _req(unit.dim() >= 2 and unit[0].numel() == nkv * page * (dk + dv),
         f"{name}: a page of the cache unit must hold {nkv} heads x {page} rows x ({dk} + {dv})")


def pwa_prepare(qkv: torch.Tensor, bias: Optional[torch.Tensor], q_norm: Optional[torch.Tensor],
                k_norm: Optional[torch.Tensor], eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                rotary_dim: int, positions: torch.Tensor, seq_of_token: torch.Tensor, slots: torch.Tensor,
                block_table: torch.Tensor, q_out: torch.Tensor, unit: torch.Tensor, v_first: Optional[torch.Tensor],
                mix: Optional[torch.Tensor], v_role: int, nq: int, nkv: int, dk: int, dv: int, page: int,
                write_cache: bool, values_from_keys: bool = False, q_temp_coef: float = 0.0, q_temp_every: int = 0,
                maps: int = 1, row_ss: Optional[torch.Tensor] = None, pad_queries: bool = True) -> None:
    """Float projection sums [T, nq*dk + nkv*dk + nkv*dv (+ more columns that are not read)] -> queries (normed,
    rotated) in `q_out` and the tokens' keys (normed, rotated) and values in their cache pages.  `v_role` 1 leaves
    the values in `v_first`, 2 mixes them with it by the scalar `mix`.  `values_from_keys`: there are no value
    columns, the keys' sums as projected (before norm and rotation) are the values.  `q_temp_every` > 0: the query
    at position p is multiplied by 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1) behind its norm.
    `maps` > 1: every query and key head is `maps` vectors of dk side by side, each normed and rotated by itself; the
    cache's key rows are maps * dk wide and `q_out` is [T, nq * maps rows of maps * dk], every row one map's query with
    zeros where the other maps' keys lie (the attention kernels then take nq * maps query heads of maps * dk).  `row_ss`
    (float scratch [T, 2]): the norm runs over the token's whole query (key) projection instead of over a head, with
    weights for the whole projection (`q_norm` [nq * maps * dk], `k_norm` [nkv * maps * dk]).  `pad_queries` False: the
    rows of `q_out` are dk wide, without the zeros (for a kernel that takes `maps` itself)."""
    _dev("pwa_prepare", qkv, bias, q_norm, k_norm, cos, sin, positions, seq_of_token, slots, block_table, q_out, unit,
         v_first, mix, row_ss)
    T = qkv.shape[0]
    _req(maps >= 1 and (maps == 1 or not values_from_keys), "pwa_prepare: one or more maps; keys that serve as values have one")
    nqs, nks, kw = nq * maps, nkv * maps, maps * dk
    width = nqs * dk + nks * dk + (0 if values_from_keys else nkv * dv)
    _req(qkv.dtype == torch.float32 and qkv.dim() == 2 and qkv.shape[1] >= width,
         "pwa_prepare: projections must be float32 [T, nq*dk + nkv*(dk+dv) or more]")
    _req(not values_from_keys or (dv == dk and bias is None), "pwa_prepare: values taken from the keys have their width and no bias")
    _req(bias is None or (bias.dtype == torch.float32 and bias.numel() == width), "pwa_prepare: bias float32 of the projections' width")
    _req(q_temp_every >= 0, "pwa_prepare: the query temperature's period must not be negative")
    whole = row_ss is not None
    for nw, heads in ((q_norm, nqs), (k_norm, nks)):
        _req(nw is None or (nw.dtype == torch.float32 and nw.numel() == (heads * dk if whole else dk)),
             "pwa_prepare: norm weights float32 [dk], or of the whole projection with a norm over it")
    _req(not whole or (row_ss.dtype == torch.float32 and row_ss.numel() >= 2 * T and q_norm is not None and k_norm is not None),
         "pwa_prepare: a norm over the whole projection takes float scratch [T, 2] and weights for queries and keys")
    _req(positions.numel() >= T and seq_of_token.numel() >= T, "pwa_prepare: positions shorter than tokens")
    _req(block_table.dim() == 2 and block_table.dtype == torch.int32, "pwa_prepare: block table int32 [slots, pages]")
    _req(q_out.shape == (T, nqs * (kw if pad_queries else dk)) and q_out.dtype == unit.dtype,
         "pwa_prepare: q_out [T, nq*maps rows of maps*dk (or of dk, without the zeros)] of the cache's dtype")
    _pwa_unit("pwa_prepare", unit, nkv, kw, dv, page)
    if rotary_dim:
        _req(cos is not None and sin is not None and cos.dtype == sin.dtype == torch.float32
             and cos.numel() >= T * (rotary_dim // 2) and sin.numel() >= T * (rotary_dim // 2), "pwa_prepare: rotary tables float32 [T, rotary_dim/2]")
    if v_role:
        _req(v_first is not None and v_first.dtype == torch.float32 and v_first.numel() >= T * nkv * dv,
             "pwa_prepare: v_first float32 [T, nkv*dv]")
        _req(v_role != 2 or (mix is not None and mix.dtype == torch.float32 and mix.numel() == 1), "pwa_prepare: mix is one float")
    f = _fn("pooled_attention", "br_pwa_prepare",
            [_P, _P, _P, _P, c_float, _P, _P, c_int, _P, _P, _P, _P, c_int, _P, _P, c_int, _P, _P] + [c_int] * 10 + [c_float, c_int, c_int, _P, c_int, c_int, _P])
    _check(f(_ptr(qkv), _ptr(bias), _ptr(q_norm), _ptr(k_norm), float(eps), _ptr(cos), _ptr(sin), int(rotary_dim),
             _ptr(positions), _ptr(seq_of_token), _ptr(slots), _ptr(block_table), block_table.shape[1], _ptr(q_out),
             _ptr(unit), _is_bf16(unit, "pwa_prepare"), _ptr(v_first), _ptr(mix), int(v_role), T, nq, nkv, dk, dv, page,
             int(write_cache), int(qkv.shape[1]), int(bool(values_from_keys)), float(q_temp_coef), int(q_temp_every),
             int(maps), _ptr(row_ss), dk if whole else 0, int(bool(pad_queries)), _stream()), "pwa_prepare")


def pwa_pair_combine(a: torch.Tensor, out: torch.Tensor, nq: int, dv: int, factor: float, eps: Optional[float],
                     scale: float = 1.0) -> None:
    """Two score maps a head into one output: a [T, nq*2*dv] holds, head by head, the rows a1 and a2 that attention left
    for the head's two maps; out[t, h] = (a1 - factor a2) / sqrt(mean((a1 - factor a2)^2) + eps) * scale over the head's
    dv values (no weight; `eps` None: no norm)."""
    _dev("pwa_pair_combine", a, out)
    T = a.shape[0]
    _req(a.shape == (T, nq * 2 * dv) and out.shape == (T, nq * dv) and a.dtype == out.dtype, "pwa_pair_combine: a [T, nq*2*dv], out [T, nq*dv]")
    _req(0 < dv <= 512 and (eps is None or eps >= 0), "pwa_pair_combine: value widths up to 512, eps not negative")
    f = _fn("pooled_attention", "br_pwa_pair_combine", [_P, _P, c_int, c_int, c_int, c_int, c_float, c_float, c_float, _P])
    _check(f(_ptr(a), _ptr(out), _is_bf16(a, "pwa_pair_combine"), T, nq, dv, float(factor), -1.0 if eps is None else float(eps),
             float(scale), _stream()), "pwa_pair_combine")


def pwa_gate(o: torch.Tensor, gate: torch.Tensor, nq: int, dv: int, per_head: bool, scale: float = 1.0) -> None:
    """o[t, h, i] <- o[t, h, i] * sigmoid(g) * scale in place, g = gate[t, h] (`per_head`) or gate[t, h * dv + i]:
    o [T, nq*dv]; gate a float view [T, nq or nq*dv] whose rows may be strided (the sums of its projection)."""
    _dev("pwa_gate", o)
    T = o.shape[0]
    n = nq if per_head else nq * dv
    _req(o.shape == (T, nq * dv), "pwa_gate: o [T, nq*dv]")
    _req(gate.is_cuda and gate.dtype == torch.float32 and gate.shape == (T, n) and gate.stride(1) == 1,
         "pwa_gate: gate float32 [T, heads] or [T, heads * value width]")
    gs = gate.stride(0) if T > 1 else n
    f = _fn("pooled_attention", "br_pwa_gate", [_P, c_int, _P, c_size_t, c_int, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(o), _is_bf16(o, "pwa_gate"), _ptr(gate), gs, T, nq, dv, int(bool(per_head)), float(scale), _stream()), "pwa_gate")


def pwa_pool(unit: torch.Tensor, block_table: torch.Tensor, pooled: torch.Tensor, pooled_table: torch.Tensor,
             cu_seqlens: torch.Tensor, ctx_lens: torch.Tensor, slots: torch.Tensor, B: int, max_new: int, nkv: int,
             dk: int, dv: int, page: int, pool: int) -> None:
    """Rows of the pooled unit for the blocks of `pool` tokens that this step completed: the means of
    their keys and of their values as the token unit holds them."""
    _dev("pwa_pool", unit, block_table, pooled, pooled_table, cu_seqlens, ctx_lens, slots)
    _req(unit.dtype == pooled.dtype, "pwa_pool: both units share a dtype")
    _pwa_unit("pwa_pool", unit, nkv, dk, dv, page)
    _pwa_unit("pwa_pool", pooled, nkv, dk, dv, page)
    _req(cu_seqlens.numel() >= B + 1 and ctx_lens.numel() >= B and slots.numel() >= B, "pwa_pool: arrays shorter than the batch")
    for tb in (block_table, pooled_table):
        _req(tb.dim() == 2 and tb.dtype == torch.int32, "pwa_pool: block tables int32 [slots, pages]")
    f = _fn("pooled_attention", "br_pwa_pool", [_P, _P, c_int, _P, _P, c_int, _P, _P, _P] + [c_int] * 8 + [_P])
    _check(f(_ptr(unit), _ptr(block_table), block_table.shape[1], _ptr(pooled), _ptr(pooled_table), pooled_table.shape[1],
             _ptr(cu_seqlens), _ptr(ctx_lens), _ptr(slots), _is_bf16(unit, "pwa_pool"), B, max_new, nkv, dk, dv, page, pool,
             _stream()), "pwa_pool")


def _sinks(name: str, sinks: Optional[torch.Tensor], nq: int) -> c_void_p:
    """A learnt sink score per query head (float32 [nq]) for a softmax with a sink; None: the sink's score is 0."""
    if sinks is not None:
        _dev(name, sinks)
        _req(sinks.dtype == torch.float32 and sinks.numel() == nq, f"{name}: sink scores must be float32 [query heads]")
    return _ptr(sinks)


def pwa_attend(q: torch.Tensor, out: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, slots: torch.Tensor,
               block_table: torch.Tensor, unit: torch.Tensor, pooled_table: Optional[torch.Tensor],
               pooled: Optional[torch.Tensor], nq: int, nkv: int, dk: int, dv: int, page: int, size: int, pool: int,
               scale: float, sink: bool, sinks: Optional[torch.Tensor] = None, chunk: int = 0, keep: int = 0,
               softcap: float = 0.0) -> None:
    """One wave per (query, head), float arithmetic: the window's tokens and the pooled blocks before it.  `chunk` > 0:
    a query sees no key before its own run of `chunk` positions (counted from 0); `keep` > 0: it also sees the sequence's
    first `keep` tokens; `softcap` > 0: scores become softcap * tanh(score / softcap)."""
    _dev("pwa_attend", q, out, positions, seq_of_token, slots, block_table, unit, pooled_table, pooled)
    T = q.shape[0]
    _req(q.shape == (T, nq * dk) and out.shape == (T, nq * dv) and q.dtype == out.dtype == unit.dtype,
         "pwa_attend: q [T, nq*dk], out [T, nq*dv], both of the cache's dtype")
    _pwa_unit("pwa_attend", unit, nkv, dk, dv, page)
    if pool:
        _req(pooled is not None and pooled_table is not None and pooled.dtype == unit.dtype, "pwa_attend: pooled unit missing")
        _pwa_unit("pwa_attend", pooled, nkv, dk, dv, page)
    f = _fn("pooled_attention", "br_pwa_attend",
            [_P, _P, c_int, _P, _P, _P, _P, c_int, _P, _P, c_int, _P] + [c_int] * 8 + [c_float, c_int, _P, c_int, c_int, c_float, _P])
    _check(f(_ptr(q), _ptr(out), _is_bf16(q, "pwa_attend"), _ptr(positions), _ptr(seq_of_token), _ptr(slots),
             _ptr(block_table), block_table.shape[1], _ptr(unit), _ptr(pooled_table),
             pooled_table.shape[1] if pooled_table is not None else 0, _ptr(pooled), T, nq, nkv, dk, dv, page, int(size),
             int(pool), float(scale), int(sink), _sinks("pwa_attend", sinks, nq), int(chunk), int(keep), float(softcap),
             _stream()), "pwa_attend")


def pwa_prefill_takes(dtype: torch.dtype, dk: int, dv: int, page: int) -> bool:
    """Whether the matrix-core kernel takes these sizes (else `pwa_attend` does the step)."""
    return dtype == torch.bfloat16 and page == 64 and dk % 8 == 0 and dv % 4 == 0 and 0 < dk <= 256 and 0 < dv <= 256


def pwa_prefill_bf16(q: torch.Tensor, out: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor, ctx_lens: torch.Tensor,
                     block_table: torch.Tensor, unit: torch.Tensor, pooled_table: Optional[torch.Tensor],
                     pooled: Optional[torch.Tensor], B: int, max_new: int, nq: int, nkv: int, dk: int, dv: int, page: int,
                     size: int, pool: int, scale: float, sink: bool, sinks: Optional[torch.Tensor] = None, chunk: int = 0,
                     keep: int = 0, softcap: float = 0.0, maps: int = 1) -> None:
    """Steps of several tokens per sequence on the matrix cores: the same sums as `pwa_attend`, bfloat16 operands,
    float scores and softmax, the weights rounded to bfloat16 for the second product.  `maps` > 1: `nq` counts a token's
    query rows (heads x maps, the map innermost), each `dk` wide (`pwa_prepare` without padding); the cache's key rows hold
    the maps side by side, and query row (h, m) reads elements m * dk .. (m + 1) * dk of them."""
    _dev("pwa_prefill_bf16", q, out, cu_seqlens, slots, ctx_lens, block_table, unit, pooled_table, pooled)
    T = q.shape[0]
    _req(pwa_prefill_takes(q.dtype, dk, dv, page), "pwa_prefill_bf16: bfloat16, pages of 64, key widths in steps of 8 and value "
         "widths in steps of 4 up to 256")
    _req(q.shape == (T, nq * dk) and out.shape == (T, nq * dv) and out.dtype == unit.dtype == torch.bfloat16,
         "pwa_prefill_bf16: q [T, nq*dk], out [T, nq*dv], bfloat16 like the cache")
    _req(cu_seqlens.numel() >= B + 1 and slots.numel() >= B and ctx_lens.numel() >= B, "pwa_prefill_bf16: arrays shorter than the batch")
    _req(maps >= 1 and nq % (nkv * maps) == 0 and (maps == 1 or not pool), "pwa_prefill_bf16: query rows a multiple of kv heads x maps; no pooled rows with maps")
    _pwa_unit("pwa_prefill_bf16", unit, nkv, maps * dk, dv, page)
    if pool:
        _req(pooled is not None and pooled_table is not None and pooled.dtype == unit.dtype, "pwa_prefill_bf16: pooled unit missing")
        _pwa_unit("pwa_prefill_bf16", pooled, nkv, dk, dv, page)
    f = _fn("pooled_attention", "br_pwa_prefill_bf16",
            [_P, _P, _P, _P, _P, _P, c_int, _P, _P, c_int, _P] + [c_int] * 8 + [c_float, c_int, _P, c_int, c_int, c_float, c_int, _P])
    _check(f(_ptr(q), _ptr(out), _ptr(cu_seqlens), _ptr(slots), _ptr(ctx_lens), _ptr(block_table), block_table.shape[1], _ptr(unit),
             _ptr(pooled_table), pooled_table.shape[1] if pooled_table is not None else 0, _ptr(pooled), B, max_new, nq, nkv, dk, dv,
             int(size), int(pool), float(scale), int(sink), _sinks("pwa_prefill_bf16", sinks, nq), int(chunk), int(keep),
             float(softcap), int(maps), _stream()), "pwa_prefill_bf16")


def pwa_decode_takes(dtype: torch.dtype, nq: int, nkv: int, dk: int, dv: int, page: int) -> bool:
    """Whether the matrix-core kernel for single tokens takes these sizes (else `pwa_attend` does the step)."""
    if dtype != torch.bfloat16 or page != 64:
        return False
    f = _build.load("pooled_attention").br_pwa_decode_takes
    f.argtypes, f.restype = [c_int] * 4, c_int
    return bool(f(nq, nkv, dk, dv))


def pwa_decode_bf16(q: torch.Tensor, out: torch.Tensor, slots: torch.Tensor, ctx_lens: torch.Tensor, block_table: torch.Tensor,
                    unit: torch.Tensor, pooled_table: Optional[torch.Tensor], pooled: Optional[torch.Tensor], B: int, nq: int,
                    nkv: int, dk: int, dv: int, page: int, size: int, pool: int, scale: float, sink: bool,
                    sinks: Optional[torch.Tensor] = None, cache_heads: int = 0, chunk: int = 0, keep: int = 0,
                    softcap: float = 0.0) -> None:
    """Steps of one token per sequence on the matrix cores (row b of q is sequence b's token): a workgroup per
    (kv head, sequence) serves all query heads of the kv head.  `cache_heads` (0: nkv): the kv heads the cache holds
    when `nkv` is a multiple of them: the query heads of one cache head are then dealt to several workgroups (many
    query heads over one row a token, whose merge would not fit one workgroup's LDS)."""
    _dev("pwa_decode_bf16", q, out, slots, ctx_lens, block_table, unit, pooled_table, pooled)
    held = cache_heads or nkv
    _req(pwa_decode_takes(q.dtype, nq, nkv, dk, dv, page) and nkv % held == 0, "pwa_decode_bf16: sizes outside what the kernel takes")
    _req(q.shape == (B, nq * dk) and out.shape == (B, nq * dv) and out.dtype == unit.dtype == torch.bfloat16,
         "pwa_decode_bf16: q [B, nq*dk], out [B, nq*dv], bfloat16 like the cache")
    _req(slots.numel() >= B and ctx_lens.numel() >= B, "pwa_decode_bf16: arrays shorter than the batch")
    _pwa_unit("pwa_decode_bf16", unit, held, dk, dv, page)
    if pool:
        _req(pooled is not None and pooled_table is not None and pooled.dtype == unit.dtype, "pwa_decode_bf16: pooled unit missing")
        _pwa_unit("pwa_decode_bf16", pooled, held, dk, dv, page)
    f = _fn("pooled_attention", "br_pwa_decode_bf16", [_P, _P, _P, _P, _P, c_int, _P, _P, c_int, _P] + [c_int] * 7 + [c_float, c_int, _P, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(q), _ptr(out), _ptr(slots), _ptr(ctx_lens), _ptr(block_table), block_table.shape[1], _ptr(unit), _ptr(pooled_table),
             pooled_table.shape[1] if pooled_table is not None else 0, _ptr(pooled), B, nq, nkv, dk, dv, int(size), int(pool),
             float(scale), int(sink), _sinks("pwa_decode_bf16", sinks, nq), int(held), int(chunk), int(keep), float(softcap),
             _stream()), "pwa_decode_bf16")


# ------------------------------------------------------ gated linear recurrence -----
def glr_rows_per_lane(d: int) -> int:
    """Rows of a head's state that one lane of `glr_scan` holds: ceil(d / 16) rounded up to 4, 8, 16 or 32
    (the kernel's own rule, `glr_rpl`; the launcher checks the state's size against it)."""
    r = (int(d) + 15) // 16
    return 4 if r <= 4 else (8 if r <= 8 else (16 if r <= 16 else 32))


def glr_state_shape(H: int, d: int, e: int):
    """A sequence's recurrent state as `glr_scan` keeps it, [H, ceil(e/4), rows per lane, 64]: S[h][r][c] lies in
    column block c // 4 at k = r % rows per lane, lane = 16 (c % 4) + r // rows per lane."""
    return (H, (e + 3) // 4, glr_rows_per_lane(d), 64)


def glr_state_dense(state: torch.Tensor, H: int, d: int, e: int) -> torch.Tensor:
    """One slot's state [H, ceil(e/4), rows per lane, 64] as the plain S [H, d, e] (for tests and inspection)."""
    ncb, rpl = (e + 3) // 4, glr_rows_per_lane(d)
    t = state.reshape(H, ncb, rpl, 4, 16)                  # [h, cb, k, cg, g]
    t = t.permute(0, 4, 2, 1, 3).reshape(H, 16 * rpl, ncb * 4)      # rows r = g * rpl + k, columns c = cb * 4 + cg
    return t[:, :d, :e]


def glr_scan(rows: torch.Tensor, f_bias: Optional[torch.Tensor], lower: Optional[torch.Tensor], out: torch.Tensor,
             state: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor, B: int, H: int, d: int, e: int) -> None:
    """rows [T, 2*H*d + H*e] float, the projections' sums q | f | v; q = silu(.), f = lower + (1 - lower) *
    sigmoid(. + f_bias) are applied on the way.  state [slots, *glr_state_shape]: walks every sequence's new
    tokens in order, writes o [T, H*e] float and leaves the state."""
    _dev("glr_scan", rows, f_bias, lower, out, cu_seqlens, slots)
    T = rows.shape[0]
    _req(state.is_cuda and state.shape[1:] == glr_state_shape(H, d, e) and state[0].is_contiguous(),
         "glr_scan: state [slots, H, ceil(e/4), rows per lane, 64], every slot's dense")
    _req(rows.dtype == out.dtype == state.dtype == torch.float32, "glr_scan: float32 only")
    _req(rows.shape == (T, 2 * H * d + H * e) and out.shape == (T, H * e), "glr_scan: rows [T, 2*H*d + H*e], out [T, H*e]")
    for v in (f_bias, lower):
        _req(v is None or (v.dtype == torch.float32 and v.numel() == H * d), "glr_scan: bias and lower bound float32 [H*d]")
    _req(cu_seqlens.numel() >= B + 1 and slots.numel() >= B, "glr_scan: arrays shorter than the batch")
    _req(d <= 512, f"glr_scan: {d} query channels a head are beyond the kernel's 512")
    f = _fn("gated_recurrence", "br_glr_scan", [_P, _P, _P, _P, _P, _P, _P] + [c_int] * 5 + [c_size_t, _P])
    _check(f(_ptr(rows), _ptr(f_bias), _ptr(lower), _ptr(out), _ptr(state), _ptr(cu_seqlens), _ptr(slots), B, H, d, e,
             rows.shape[1], state.stride(0), _stream()), "glr_scan")


def glr_scan_pieces(rows: torch.Tensor, f_bias: Optional[torch.Tensor], lower: Optional[torch.Tensor], out: torch.Tensor,
                    state: torch.Tensor, slots: torch.Tensor, piece_cu: torch.Tensor, piece_slots: torch.Tensor,
                    piece_state: torch.Tensor, decay: torch.Tensor, B: int, pieces: int, H: int, d: int, e: int) -> None:
    """`glr_scan` of a step of long prompts with every sequence cut into `pieces` pieces that are walked side by
    side (twice: from a zero state, then from their true first states).  `piece_cu` int32 [B*pieces + 1] cuts the
    packed tokens, `piece_slots` int32 [B*pieces] numbers the pieces (-1: a padding sequence's); `piece_state`
    float [B*pieces, *glr_state_shape] and `decay` float [B*pieces, H, 16 * rows per lane] are scratch."""
    _dev("glr_scan_pieces", rows, f_bias, lower, out, slots, piece_cu, piece_slots, piece_state, decay)
    T = rows.shape[0]
    shape = glr_state_shape(H, d, e)
    _req(state.is_cuda and state.shape[1:] == shape and state[0].is_contiguous(), "glr_scan_pieces: state [slots, *glr_state_shape]")
    _req(rows.dtype == out.dtype == state.dtype == piece_state.dtype == decay.dtype == torch.float32, "glr_scan_pieces: float32 only")
    _req(rows.shape == (T, 2 * H * d + H * e) and out.shape == (T, H * e), "glr_scan_pieces: rows [T, 2*H*d + H*e], out [T, H*e]")
    _req(piece_state.shape == (B * pieces,) + tuple(shape) and decay.shape == (B * pieces, H, 16 * glr_rows_per_lane(d)),
         "glr_scan_pieces: scratch of the wrong size")
    _req(piece_cu.dtype == piece_slots.dtype == torch.int32 and piece_cu.numel() == B * pieces + 1 and piece_slots.numel() == B * pieces
         and slots.numel() >= B, "glr_scan_pieces: piece arrays int32 [B*pieces + 1] and [B*pieces]")
    for v in (f_bias, lower):
        _req(v is None or (v.dtype == torch.float32 and v.numel() == H * d), "glr_scan_pieces: bias and lower bound float32 [H*d]")
    f = _fn("gated_recurrence", "br_glr_scan_pieces", [_P] * 10 + [c_int] * 6 + [c_size_t, _P])
    _check(f(_ptr(rows), _ptr(f_bias), _ptr(lower), _ptr(out), _ptr(state), _ptr(slots), _ptr(piece_cu), _ptr(piece_slots),
             _ptr(piece_state), _ptr(decay), B, pieces, H, d, e, rows.shape[1], state.stride(0), _stream()), "glr_scan_pieces")


def head_rmsnorm(o: torch.Tensor, w: Optional[torch.Tensor], out: torch.Tensor, H: int, e: int, eps: float) -> None:
    _dev("head_rmsnorm", o, w, out)
    T = o.shape[0]
    _req(o.dtype == torch.float32 and o.shape == (T, H * e) and out.shape == (T, H * e), "head_rmsnorm: o float32 [T, H*e]")
    _req(w is None or (w.dtype == torch.float32 and w.numel() == e), "head_rmsnorm: weight float32 [e]")
    f = _fn("gated_recurrence", "br_glr_head_norm", [_P, _P, _P, c_int, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(o), _ptr(w), _ptr(out), _is_bf16(out, "head_rmsnorm"), T, H, e, float(eps), _stream()), "head_rmsnorm")


# ------------------------------------------------- decayed recurrence with a bonus -----
def wkv_scan(rows: torch.Tensor, w0: torch.Tensor, bonus: torch.Tensor, out: torch.Tensor, state: torch.Tensor,
             cu_seqlens: torch.Tensor, slots: torch.Tensor, B: int, H: int, d: int, e: int) -> None:
    """rows [T, >= 3*H*d + H*e] float, the projections' sums r | k | v | z (the decay is exp(-exp(z + w0)), made on the
    way); bonus float [H*d].  state [slots, n] float with a slot's first prod(glr_state_shape(H, d, e)) floats its S as
    `glr_scan` keeps it: walks every sequence's new tokens in order, o_t = (S + diag(bonus) k v^T)^T r before
    S <- diag(decay) S + k v^T, writes o [T, H*e] float and leaves the state."""
    _dev("wkv_scan", rows, w0, bonus, out, cu_seqlens, slots)
    T = rows.shape[0]
    need = 1
    for n in glr_state_shape(H, d, e):
        need *= n
    _req(state.is_cuda and state.dim() == 2 and state.shape[1] >= need and state.stride(1) == 1,
         "wkv_scan: state [slots, at least the head states' floats], every slot's dense")
    _req(rows.dtype == out.dtype == state.dtype == torch.float32, "wkv_scan: float32 only")
    _req(rows.dim() == 2 and rows.shape[1] >= 3 * H * d + H * e and out.shape == (T, H * e), "wkv_scan: rows [T, >= 3*H*d + H*e], out [T, H*e]")
    for v in (w0, bonus):
        _req(v.dtype == torch.float32 and v.numel() == H * d, "wkv_scan: w0 and bonus float32 [H*d]")
    _req(cu_seqlens.numel() >= B + 1 and slots.numel() >= B, "wkv_scan: arrays shorter than the batch")
    _req(d <= 512, f"wkv_scan: {d} key channels a head are beyond the kernel's 512")
    f = _fn("gated_recurrence", "br_wkv_scan", [_P, _P, _P, _P, _P, _P, _P] + [c_int] * 5 + [c_size_t, _P])
    _check(f(_ptr(rows), _ptr(w0), _ptr(bonus), _ptr(out), _ptr(state), _ptr(cu_seqlens), _ptr(slots), B, H, d, e,
             rows.shape[1], state.stride(0), _stream()), "wkv_scan")


def wkv_scan_pieces(rows: torch.Tensor, w0: torch.Tensor, bonus: torch.Tensor, out: torch.Tensor, state: torch.Tensor,
                    slots: torch.Tensor, piece_cu: torch.Tensor, piece_slots: torch.Tensor, piece_state: torch.Tensor,
                    decay: torch.Tensor, B: int, pieces: int, H: int, d: int, e: int) -> None:
    """`wkv_scan` of a step of long prompts with every sequence cut into `pieces` pieces that are walked side by side
    (twice: from a zero state, then from their true first states); arrays as for `glr_scan_pieces`."""
    _dev("wkv_scan_pieces", rows, w0, bonus, out, slots, piece_cu, piece_slots, piece_state, decay)
    T = rows.shape[0]
    shape = glr_state_shape(H, d, e)
    need = 1
    for n in shape:
        need *= n
    _req(state.is_cuda and state.dim() == 2 and state.shape[1] >= need and state.stride(1) == 1, "wkv_scan_pieces: state [slots, >= the head states' floats]")
    _req(rows.dtype == out.dtype == state.dtype == piece_state.dtype == decay.dtype == torch.float32, "wkv_scan_pieces: float32 only")
    _req(rows.dim() == 2 and rows.shape[1] >= 3 * H * d + H * e and out.shape == (T, H * e), "wkv_scan_pieces: rows [T, >= 3*H*d + H*e], out [T, H*e]")
    _req(piece_state.shape == (B * pieces,) + tuple(shape) and decay.shape == (B * pieces, H, 16 * glr_rows_per_lane(d)),
         "wkv_scan_pieces: scratch of the wrong size")
    _req(piece_cu.dtype == piece_slots.dtype == torch.int32 and piece_cu.numel() == B * pieces + 1 and piece_slots.numel() == B * pieces
         and slots.numel() >= B, "wkv_scan_pieces: piece arrays int32 [B*pieces + 1] and [B*pieces]")
    for v in (w0, bonus):
        _req(v.dtype == torch.float32 and v.numel() == H * d, "wkv_scan_pieces: w0 and bonus float32 [H*d]")
    f = _fn("gated_recurrence", "br_wkv_scan_pieces", [_P] * 10 + [c_int] * 6 + [c_size_t, _P])
    _check(f(_ptr(rows), _ptr(w0), _ptr(bonus), _ptr(out), _ptr(state), _ptr(slots), _ptr(piece_cu), _ptr(piece_slots),
             _ptr(piece_state), _ptr(decay), B, pieces, H, d, e, rows.shape[1], state.stride(0), _stream()), "wkv_scan_pieces")


def shift_mix(h: torch.Tensor, mu: torch.Tensor, out: torch.Tensor, kept: torch.Tensor, seq_of_token: torch.Tensor,
              cu_seqlens: torch.Tensor, slots: torch.Tensor, B: int, single_tokens: bool) -> None:
    """out[s, t] = h[t] + (h'[t] - h[t]) * mu[s], h' the row of the token before in its sequence, and before a step's
    first token the row its slot keeps (`kept` [slots, >= W] float, a slot's first W floats); every sequence's last
    row is left there.  h and out [n, T, W] have the products' type, mu [n, W] is float."""
    _dev("shift_mix", h, mu, out, seq_of_token, cu_seqlens, slots)
    T, W = h.shape
    n = mu.shape[0]
    _req(mu.dtype == torch.float32 and mu.shape == (n, W) and out.shape == (n, T, W) and out.dtype == h.dtype, "shift_mix: mu float32 [n, W], out [n, T, W] of h's type")
    _req(kept.is_cuda and kept.dtype == torch.float32 and kept.dim() == 2 and kept.shape[1] >= W and kept.stride(1) == 1, "shift_mix: kept float32 [slots, >= W]")
    _req(seq_of_token.numel() >= T and cu_seqlens.numel() >= B + 1 and slots.numel() >= B, "shift_mix: arrays shorter than the step")
    f = _fn("gated_recurrence", "br_shift_mix", [_P, c_int, _P, _P, _P, c_size_t, _P, _P, _P] + [c_int] * 5 + [_P])
    _check(f(_ptr(h), _is_bf16(h, "shift_mix"), _ptr(mu), _ptr(out), _ptr(kept), kept.stride(0), _ptr(seq_of_token), _ptr(cu_seqlens),
             _ptr(slots), T, B, W, n, int(single_tokens), _stream()), "shift_mix")


def head_norm_gate(o: torch.Tensor, w: Optional[torch.Tensor], gate: Optional[torch.Tensor], out: torch.Tensor, H: int, e: int,
                   eps: float, gate_sigmoid: bool = False) -> None:
    """out[t, h, :] = o[t, h, :] / rms * w[h, :] * silu(gate[t, h, :]) (`gate_sigmoid`: sigmoid instead of silu): o float
    [T, H*e], w float [H*e] or None, gate a float view [T, H*e] whose rows may be strided (the sums of its projection) or None."""
    _dev("head_norm_gate", o, w, out)
    T = o.shape[0]
    _req(o.dtype == torch.float32 and o.shape == (T, H * e) and out.shape == (T, H * e), "head_norm_gate: o float32 [T, H*e]")
    _req(w is None or (w.dtype == torch.float32 and w.numel() == H * e), "head_norm_gate: weight float32 [H*e]")
    gs = 0
    if gate is not None:
        _req(gate.is_cuda and gate.dtype == torch.float32 and gate.shape == (T, H * e) and gate.stride(1) == 1, "head_norm_gate: gate float32 [T, H*e]")
        gs = gate.stride(0) if T > 1 else H * e
    f = _fn("gated_recurrence", "br_head_norm_gate", [_P, _P, _P, c_size_t, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P])
    _check(f(_ptr(o), _ptr(w), _ptr(gate), gs, _ptr(out), _is_bf16(out, "head_norm_gate"), T, H, e, float(eps),
             int(bool(gate_sigmoid)), _stream()), "head_norm_gate")


# ------------------------------------------------- recurrences with one decay a head -----
def dr_conv_prepare(rows: torch.Tensor, taps: torch.Tensor, kept: Optional[torch.Tensor], a_log: torch.Tensor,
                    dt_bias: torch.Tensor, seq_of_token: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor,
                    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gb: torch.Tensor, B: int, G: int, H: int, d: int,
                    e: int, taps_t: Optional[torch.Tensor] = None) -> None:
    """rows float [T, >= C + 2 H] with C = 2 G d + H e: the sums q | k | v | b | a of a gated delta rule's projections.
    The first C columns pass a causal convolution over time per channel (taps float [C, n], the last column the current
    token's; `kept` a float view [slots, (n - 1) * C] of every sequence's last inputs, read and then brought up to
    date) and silu; q and k become unit vectors per head (q times d^-1/2); gb [T, 2 H] takes
    g = exp(-exp(a_log) softplus(a + dt_bias)) and beta = sigmoid(b).  `taps_t` float [n, C], the same taps with the channels
    side by side, lets widths that are multiples of 4 go four channels a lane."""
    _dev("dr_conv_prepare", rows, taps, a_log, dt_bias, seq_of_token, cu_seqlens, slots, q, k, v, gb, taps_t)
    T = rows.shape[0]
    C = 2 * G * d + H * e
    n = taps.shape[1] if taps.dim() == 2 else 0
    _req(rows.dtype == torch.float32 and rows.dim() == 2 and rows.shape[1] >= C + 2 * H, "dr_conv_prepare: rows float32 [T, >= C + 2 H]")
    _req(taps.dtype == torch.float32 and taps.shape == (C, n) and 1 <= n <= 16, "dr_conv_prepare: taps float32 [C, 1..16]")
    _req(a_log.dtype == dt_bias.dtype == torch.float32 and a_log.numel() == H and dt_bias.numel() == H, "dr_conv_prepare: A_log and dt_bias float32 [H]")
    _req(q.dtype == k.dtype == v.dtype == gb.dtype == torch.float32 and q.shape == k.shape == (T, G * d) and v.shape == (T, H * e)
         and gb.shape == (T, 2 * H), "dr_conv_prepare: q, k [T, G d], v [T, H e], gb [T, 2 H] float32")
    _req(seq_of_token.numel() >= T and cu_seqlens.numel() >= B + 1 and slots.numel() >= B, "dr_conv_prepare: arrays shorter than the batch")
    ks = 0
    if n > 1:
        _req(kept is not None and kept.is_cuda and kept.dtype == torch.float32 and kept.dim() == 2 and kept.shape[1] == (n - 1) * C
             and kept.stride(1) == 1, "dr_conv_prepare: kept float32 [slots, (n - 1) * C]")
        ks = kept.stride(0)
    _req(taps_t is None or (taps_t.dtype == torch.float32 and taps_t.shape == (n, C) and taps_t.is_contiguous()), "dr_conv_prepare: taps_t float32 [n, C]")
    f = _fn("delta_rule", "br_dr_conv_prepare", [_P, c_int, _P, _P, c_int, _P, c_size_t, _P, _P, _P, _P, _P, _P, _P, _P, _P] + [c_int] * 6 + [_P])
    _check(f(_ptr(rows), int(rows.shape[1]), _ptr(taps), _ptr(taps_t), n, _ptr(kept) if n > 1 else c_void_p(0), ks, _ptr(a_log), _ptr(dt_bias),
             _ptr(seq_of_token), _ptr(cu_seqlens), _ptr(slots), _ptr(q), _ptr(k), _ptr(v), _ptr(gb), T, B, G, H, d, e, _stream()),
           "dr_conv_prepare")


def dr_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gb: Optional[torch.Tensor], decay: Optional[torch.Tensor],
            out: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor, B: int, H: int, G: int,
            d: int, e: int, silu: bool = False) -> None:
    """A walk over every sequence's new tokens with a state S [d, e] a head, float, in `state` [slots, *glr_state_shape]
    (a view whose slots may be strided).  q, k float views [T, G d], v [T, H e] (rows may be strided; head h reads
    q/k head h // (H / G)).  With `gb` [T, 2 H] (g | beta) the gated delta rule
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; else with `decay` [H] S <- decay_h S + k v^T.  o = S^T q after
    the write, into out float [T, H e].  `silu`: q, k, v pass silu on their way in."""
    _dev("dr_scan", gb, decay, out, cu_seqlens, slots)
    T = out.shape[0]
    for name, t, w in (("q", q, G * d), ("k", k, G * d), ("v", v, H * e)):
        _req(t.is_cuda and t.dtype == torch.float32 and t.shape == (T, w) and t.stride(1) == 1, f"dr_scan: {name} float32 [T, {w}]")
    _req(T <= 1 or q.stride(0) == k.stride(0), "dr_scan: q and k rows equally far apart")
    _req((gb is None) != (decay is None), "dr_scan: either g and beta per token or one decay a head")
    _req(gb is None or (gb.dtype == torch.float32 and gb.shape == (T, 2 * H)), "dr_scan: gb float32 [T, 2 H]")
    _req(decay is None or (decay.dtype == torch.float32 and decay.numel() == H), "dr_scan: decay float32 [H]")
    _req(out.dtype == torch.float32 and out.shape == (T, H * e), "dr_scan: out float32 [T, H e]")
    _req(state.is_cuda and state.dtype == torch.float32 and tuple(state.shape[1:]) == tuple(glr_state_shape(H, d, e))
         and state[0].is_contiguous(), "dr_scan: state float32 [slots, H, ceil(e/4), rows per lane, 64], every slot's dense")
    _req(cu_seqlens.numel() >= B + 1 and slots.numel() >= B, "dr_scan: arrays shorter than the batch")
    _req(H % G == 0 and d <= 512, f"dr_scan: {H} heads over {G} key heads of {d} channels (a multiple; at most 512 channels)")
    qs = q.stride(0) if T > 1 else G * d
    vs = v.stride(0) if T > 1 else H * e
    f = _fn("delta_rule", "br_dr_scan", [_P, _P, c_size_t, _P, c_size_t, _P, c_size_t, _P, _P, _P, c_size_t, _P, _P] + [c_int] * 7 + [_P])
    _check(f(_ptr(q), _ptr(k), qs, _ptr(v), vs, _ptr(gb), 2 * H, _ptr(decay), _ptr(out), _ptr(state), state.stride(0),
             _ptr(cu_seqlens), _ptr(slots), B, H, G, d, e, int(gb is not None), int(bool(silu)), _stream()), "dr_scan")


def dr_rotate_rows(q: torch.Tensor, k: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rotary_dim: int,
                   heads: int, d: int, q_mul: float = 1.0, k_mul: float = 1.0) -> None:
    """q and k, float views [T, heads * d] with rows equally far apart, turned in place by their tokens' positions
    (cos, sin float [T, rotary_dim / 2]; channel i < rotary_dim / 2 of a head pairs with channel i + rotary_dim / 2, the
    channels from rotary_dim on pass), then multiplied by `q_mul` and `k_mul`."""
    _dev("dr_rotate_rows", cos, sin)
    T = q.shape[0]
    for name, t in (("q", q), ("k", k)):
        _req(t.is_cuda and t.dtype == torch.float32 and t.shape == (T, heads * d) and t.stride(1) == 1, f"dr_rotate_rows: {name} float32 [T, heads*d]")
    _req(T <= 1 or q.stride(0) == k.stride(0), "dr_rotate_rows: q and k rows equally far apart")
    _req(0 <= rotary_dim <= d and rotary_dim % 2 == 0, "dr_rotate_rows: an even number of rotated channels, at most a head's")
    if rotary_dim:
        _req(cos is not None and sin is not None and cos.dtype == sin.dtype == torch.float32
             and cos.numel() >= T * (rotary_dim // 2) and sin.numel() >= T * (rotary_dim // 2), "dr_rotate_rows: rotary tables float32 [T, rotary_dim/2]")
    f = _fn("delta_rule", "br_dr_rotate_rows", [_P, _P, c_size_t, _P, _P, c_int, c_int, c_int, c_int, c_float, c_float, _P])
    _check(f(_ptr(q), _ptr(k), q.stride(0) if T > 1 else heads * d, _ptr(cos), _ptr(sin), int(rotary_dim), T, heads, d,
             float(q_mul), float(k_mul), _stream()), "dr_rotate_rows")


def silu_rows(x: torch.Tensor) -> None:
    """x <- silu(x) in place: a float view [T, n] whose rows may be strided (some columns of a projection's sums)."""
    _req(x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1, "silu_rows: a float32 view [T, n] with dense rows")
    T, n = x.shape
    f = _fn("delta_rule", "br_silu_rows", [_P, c_size_t, c_int, c_int, _P])
    _check(f(_ptr(x), x.stride(0) if T > 1 else n, T, n, _stream()), "silu_rows")


def dr_scan_pieces(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, out: torch.Tensor, state: torch.Tensor,
                   slots: torch.Tensor, piece_cu: torch.Tensor, piece_slots: torch.Tensor, piece_state: torch.Tensor, B: int,
                   pieces: int, H: int, d: int, e: int, silu: bool = False) -> None:
    """`dr_scan` with one decay a head over a step of long prompts with every sequence cut into `pieces` pieces that are
    walked side by side (twice: from a zero state, then from their true first states).  `piece_cu` int32 [B*pieces + 1]
    cuts the packed tokens, `piece_slots` int32 [B*pieces] numbers the pieces (-1: a padding sequence's); `piece_state`
    float [B*pieces, *glr_state_shape] is scratch."""
    _dev("dr_scan_pieces", decay, out, slots, piece_cu, piece_slots, piece_state)
    T = out.shape[0]
    shape = tuple(glr_state_shape(H, d, e))
    for name, t, w in (("q", q, H * d), ("k", k, H * d), ("v", v, H * e)):
        _req(t.is_cuda and t.dtype == torch.float32 and t.shape == (T, w) and t.stride(1) == 1, f"dr_scan_pieces: {name} float32 [T, {w}]")
    _req(T <= 1 or q.stride(0) == k.stride(0), "dr_scan_pieces: q and k rows equally far apart")
    _req(decay.dtype == torch.float32 and decay.numel() == H, "dr_scan_pieces: decay float32 [H]")
    _req(out.dtype == torch.float32 and out.shape == (T, H * e), "dr_scan_pieces: out float32 [T, H e]")
    _req(state.is_cuda and state.dtype == torch.float32 and tuple(state.shape[1:]) == shape and state[0].is_contiguous(),
         "dr_scan_pieces: state float32 [slots, *glr_state_shape], every slot's dense")
    _req(piece_state.dtype == torch.float32 and piece_state.shape == (B * pieces,) + shape and piece_state.is_contiguous(),
         "dr_scan_pieces: scratch of the wrong size")
    _req(piece_cu.dtype == piece_slots.dtype == torch.int32 and piece_cu.numel() == B * pieces + 1 and piece_slots.numel() == B * pieces
         and slots.numel() >= B, "dr_scan_pieces: piece arrays int32 [B*pieces + 1] and [B*pieces]")
    qs = q.stride(0) if T > 1 else H * d
    vs = v.stride(0) if T > 1 else H * e
    f = _fn("delta_rule", "br_dr_scan_pieces", [_P, _P, c_size_t, _P, c_size_t, _P, _P, _P, c_size_t, _P, _P, _P, _P] + [c_int] * 6 + [_P])
    _check(f(_ptr(q), _ptr(k), qs, _ptr(v), vs, _ptr(decay), _ptr(out), _ptr(state), state.stride(0), _ptr(slots), _ptr(piece_cu),
             _ptr(piece_slots), _ptr(piece_state), B, pieces, H, d, e, int(bool(silu)), _stream()), "dr_scan_pieces")


def tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    _dev("tanh", x, out)
    _req(x.dtype == torch.float32 and x.numel() == out.numel(), "tanh: x float32, out of the same size")
    f = _fn("gated_recurrence", "br_tanh", [_P, _P, c_int, c_size_t, _P])
    _check(f(_ptr(x), _ptr(out), _is_bf16(out, "tanh"), x.numel(), _stream()), "tanh")


# ------------------------------------------------------ attention through a latent -----
def latent_prepare(q: torch.Tensor, dkv: Optional[torch.Tensor], c_weight: Optional[torch.Tensor], eps: float,
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot: int, positions: torch.Tensor,
                   seq_of_token: torch.Tensor, slots: torch.Tensor, block_table: Optional[torch.Tensor],
                   cache: Optional[torch.Tensor], q_plain: torch.Tensor, q_wide: torch.Tensor, H: int, D: int, DR: int, R: int,
                   page: int) -> None:
    """q float [T, H*(D+DR)] and dkv float [T, R+DR] (views whose rows may be strided; dkv None: nothing is kept):
    the normed latent and the rotated shared key part into the token's cache row, the queries' plain parts into
    q_plain [T, H*D] and their rotated parts into q_wide [T, H*(R+DR)] behind each head's first R elements."""
    _dev("latent_prepare", c_weight, cos, sin, positions, seq_of_token, slots, block_table, cache, q_plain, q_wide)
    T = q.shape[0]
    _req(q.is_cuda and q.dtype == torch.float32 and q.shape == (T, H * (D + DR)) and q.stride(1) == 1, "latent_prepare: q float32 [T, H*(D+DR)]")
    _req(q_plain.shape == (T, H * D) and q_wide.shape == (T, H * (R + DR)) and q_plain.dtype == q_wide.dtype, "latent_prepare: q_plain [T, H*D], q_wide [T, H*(R+DR)]")
    if rot:
        _req(cos is not None and sin is not None and cos.numel() >= T * (rot // 2) and sin.numel() >= T * (rot // 2), "latent_prepare: rotary tables too short")
    ds = 0
    if dkv is not None:
        _req(dkv.is_cuda and dkv.dtype == torch.float32 and dkv.shape == (T, R + DR) and dkv.stride(1) == 1, "latent_prepare: dkv float32 [T, R+DR]")
        _req(c_weight is not None and c_weight.dtype == torch.float32 and c_weight.numel() == R, "latent_prepare: the latent's norm weight float32 [R]")
        _req(cache is not None and cache.dtype == q_plain.dtype and cache.dim() == 2 and cache.shape[1] == page * (2 * R + DR),
             "latent_prepare: cache [pages, page * (2 R + DR)] of the products' type")
        _req(block_table is not None and block_table.dim() == 2 and block_table.dtype == torch.int32, "latent_prepare: block table int32 [slots, pages]")
        ds = dkv.stride(0) if T > 1 else R + DR
    f = _fn("latent_attention", "br_latent_prepare",
            [_P, c_size_t, _P, c_size_t, _P, c_float, _P, _P, _P, _P, _P, _P, c_int, _P, _P, _P] + [c_int] * 8 + [_P])
    _check(f(_ptr(q), q.stride(0) if T > 1 else H * (D + DR), _ptr(dkv), ds, _ptr(c_weight), float(eps), _ptr(cos), _ptr(sin),
             _ptr(positions), _ptr(seq_of_token), _ptr(slots), _ptr(block_table), block_table.shape[1] if block_table is not None else 0,
             _ptr(cache), _ptr(q_plain), _ptr(q_wide), _is_bf16(q_plain, "latent_prepare"), T, H, D, DR, R, int(rot), page, _stream()),
           "latent_prepare")


def head_linear(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, h, :] = w[h] a[t, h, :] for every head in one launch: a [T, H, K] and out [T, H, N] may be views of
    wider rows (strides between tokens and heads, dense last dimension); w [H, N, K] dense."""
    _dev("head_linear", w)
    T, H, K = a.shape
    N = w.shape[1]
    _req(a.is_cuda and out.is_cuda and a.dtype == w.dtype == out.dtype, "head_linear: one type, on the device")
    _req(w.shape == (H, N, K) and out.shape == (T, H, N) and a.stride(2) == 1 and out.stride(2) == 1, "head_linear: a [T, H, K], w [H, N, K], out [T, H, N]")
    lda, ldo = (a.stride(0) if T > 1 else H * K), (out.stride(0) if T > 1 else H * N)
    f = _fn("latent_attention", "br_head_linear", [_P, c_size_t, c_size_t, _P, _P, c_size_t, c_size_t] + [c_int] * 5 + [_P])
    _check(f(_ptr(a), lda, a.stride(1) if H > 1 else K, _ptr(w), _ptr(out), ldo, out.stride(1) if H > 1 else N, _is_bf16(a, "head_linear"),
             T, H, N, K, _stream()), "head_linear")


# ---------------------------------------------------------------- routed experts -----
def route_topk(scores: torch.Tensor, bias: Optional[torch.Tensor], chosen: torch.Tensor, share: torch.Tensor, top: int,
               out_scale: float = 1.0) -> None:
    """scores float [T, E] (+ bias [E]): the `top` largest per row (ties to the lower number) into chosen int32 [T, top],
    the softmax over them times `out_scale` into share float [T, top]."""
    _dev("route_topk", scores, bias, chosen, share)
    T, E = scores.shape
    _req(scores.dtype == torch.float32 and (bias is None or (bias.dtype == torch.float32 and bias.numel() == E)), "route_topk: float32 scores and bias")
    _req(chosen.dtype == torch.int32 and chosen.shape == (T, top) and share.dtype == torch.float32 and share.shape == (T, top), "route_topk: chosen int32 and share float32 [T, top]")
    _req(0 < top <= min(E, 64) and E <= 512, f"route_topk: {top} of {E} experts is outside the kernel's sizes (512 experts, 64 chosen)")
    f = _fn("routed_experts", "br_route_topk", [_P, _P, _P, _P, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(scores), _ptr(bias), _ptr(chosen), _ptr(share), T, E, top, float(out_scale), _stream()), "route_topk")


def route_sigmoid(scores: torch.Tensor, correction: Optional[torch.Tensor], chosen: torch.Tensor, share: torch.Tensor, top: int,
                  groups: int = 1, keep: int = 1, out_scale: float = 1.0) -> None:
    """scores float [T, E]: s = sigmoid(scores); the `top` experts with the largest s + correction per row (ties to the
    lower number) into chosen int32 [T, top], their s over the chosen ones' sum (+ 1e-20) times `out_scale` into share
    float [T, top].  `groups` > 1: the experts form that many runs of neighbours, a run scores the sum of its two largest
    s + correction, and only experts of the `keep` best runs can be chosen."""
    _dev("route_sigmoid", scores, correction, chosen, share)
    T, E = scores.shape
    _req(scores.dtype == torch.float32 and (correction is None or (correction.dtype == torch.float32 and correction.numel() == E)),
         "route_sigmoid: float32 scores and correction")
    _req(chosen.dtype == torch.int32 and chosen.shape == (T, top) and share.dtype == torch.float32 and share.shape == (T, top),
         "route_sigmoid: chosen int32 and share float32 [T, top]")
    _req(0 < top <= min(E, 64) and E <= 512, f"route_sigmoid: {top} of {E} experts is outside the kernel's sizes (512 experts, 64 chosen)")
    _req(groups >= 1 and E % groups == 0 and (groups == 1 or (1 <= keep <= groups and keep * (E // groups) >= top)),
         f"route_sigmoid: {groups} runs of experts of which {keep} are kept cannot give {top} of {E} experts")
    f = _fn("routed_experts", "br_route_sigmoid", [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P])
    _check(f(_ptr(scores), _ptr(correction), _ptr(chosen), _ptr(share), T, E, top, int(groups), int(keep), float(out_scale),
             _stream()), "route_sigmoid")


def experts_up(h: torch.Tensor, w_gu: torch.Tensor, chosen: torch.Tensor, y: torch.Tensor) -> None:
    """y[t, s] = silu(W_gate[e] h[t]) * (W_up[e] h[t]) with e = chosen[t, s]; w_gu [E, 2 F, W] holds an expert's gate
    rows, then its up rows; y [T, top, F]."""
    _dev("experts_up", h, w_gu, chosen, y)
    T, W = h.shape
    E, F2, _ = w_gu.shape
    top = chosen.shape[1]
    _req(F2 % 2 == 0 and w_gu.shape == (E, F2, W) and y.shape == (T, top, F2 // 2) and chosen.shape == (T, top) and chosen.dtype == torch.int32, "experts_up: shapes")
    _req(h.dtype == w_gu.dtype == y.dtype, "experts_up: one type for rows and weights")
    _req(W <= 16384, "experts_up: rows wider than 16,384")
    f = _fn("routed_experts", "br_experts_up", [_P, _P, _P, _P] + [c_int] * 5 + [_P])
    _check(f(_ptr(h), _ptr(w_gu), _ptr(chosen), _ptr(y), _is_bf16(h, "experts_up"), T, W, F2 // 2, top, _stream()), "experts_up")


def experts_sort(chosen: torch.Tensor, first: torch.Tensor, order: torch.Tensor, place: torch.Tensor, E: int) -> None:
    """The (token, slot) pairs of chosen [T, top] grouped by expert: first int32 [E + 1], order and place int32 [T * top]."""
    _dev("experts_sort", chosen, first, order, place)
    n = chosen.numel()
    _req(chosen.dtype == first.dtype == order.dtype == place.dtype == torch.int32 and first.numel() == E + 1 and order.numel() == n
         and place.numel() == n, "experts_sort: int32 arrays [E + 1], [pairs], [pairs]")
    f = _fn("routed_experts", "br_experts_sort", [_P, _P, _P, _P, c_int, c_int, _P])
    _check(f(_ptr(chosen), _ptr(first), _ptr(order), _ptr(place), n, E, _stream()), "experts_sort")


def experts_gather(h: torch.Tensor, order: torch.Tensor, rows: torch.Tensor, top: int) -> None:
    """rows[p] = h[order[p] // top]."""
    _dev("experts_gather", h, order, rows)
    n, W = rows.shape
    _req(h.dtype == rows.dtype and h.shape[1] == W and order.dtype == torch.int32 and order.numel() == n, "experts_gather: shapes")
    f = _fn("routed_experts", "br_experts_gather", [_P, _P, _P, c_int, c_int, c_int, c_int, _P])
    _check(f(_ptr(h), _ptr(order), _ptr(rows), _is_bf16(h, "experts_gather"), n, W, top, _stream()), "experts_gather")


def experts_combine(out: torch.Tensor, place: torch.Tensor, share: torch.Tensor, x: torch.Tensor) -> None:
    """x[t] += sum_s share[t, s] * out[place[t * top + s]]; out float [T * top, W]."""
    _dev("experts_combine", out, place, share, x)
    T, top = share.shape
    W = x.shape[1]
    _req(out.dtype == x.dtype == share.dtype == torch.float32 and place.dtype == torch.int32 and out.shape == (T * top, W)
         and x.shape == (T, W) and place.numel() == T * top, "experts_combine: shapes")
    f = _fn("routed_experts", "br_experts_combine", [_P, _P, _P, _P, c_int, c_int, c_int, _P])
    _check(f(_ptr(out), _ptr(place), _ptr(share), _ptr(x), T, W, top, _stream()), "experts_combine")


def experts_down(y: torch.Tensor, w_down: torch.Tensor, chosen: torch.Tensor, share: torch.Tensor, x: torch.Tensor) -> None:
    """x[t] += sum_s share[t, s] * W_down[chosen[t, s]] y[t, s]; w_down [E, W, F], x float [T, W]."""
    _dev("experts_down", y, w_down, chosen, share, x)
    T, top, F = y.shape
    E, W, _ = w_down.shape
    _req(w_down.shape == (E, W, F) and x.shape == (T, W) and x.dtype == torch.float32 and chosen.shape == (T, top) and share.shape == (T, top), "experts_down: shapes")
    _req(y.dtype == w_down.dtype and chosen.dtype == torch.int32 and share.dtype == torch.float32, "experts_down: types")
    _req(top * F <= 16384, "experts_down: more than 16,384 inner elements a token")
    f = _fn("routed_experts", "br_experts_down", [_P, _P, _P, _P, _P] + [c_int] * 5 + [_P])
    _check(f(_ptr(y), _ptr(w_down), _ptr(chosen), _ptr(share), _ptr(x), _is_bf16(y, "experts_down"), T, W, F, top, _stream()), "experts_down")


def experts_grouped_takes(dtype: torch.dtype, W: int, F: int) -> bool:
    """Whether the kernels that read every expert once take these sizes (bfloat16, widths in steps of 8)."""
    return dtype == torch.bfloat16 and W % 8 == 0 and F % 8 == 0


def experts_up_grouped(h: torch.Tensor, w_gu: torch.Tensor, first: torch.Tensor, order: torch.Tensor, y: torch.Tensor, top: int) -> None:
    """y[p] = silu(W_gate[e] h[t]) * (W_up[e] h[t]) for the pairs p of `experts_sort` (t = order[p] // top, e the
    expert whose run holds p); y [pairs, F] in the experts' order."""
    _dev("experts_up_grouped", h, w_gu, first, order, y)
    T, W = h.shape
    E, F2, _ = w_gu.shape
    n = order.numel()
    _req(experts_grouped_takes(h.dtype, W, F2 // 2) and w_gu.dtype == y.dtype == torch.bfloat16, "experts_up_grouped: bfloat16, widths in steps of 8")
    _req(w_gu.shape == (E, F2, W) and y.shape == (n, F2 // 2) and first.numel() == E + 1 and n == T * top
         and first.dtype == order.dtype == torch.int32, "experts_up_grouped: shapes")
    f = _fn("routed_experts", "br_experts_up_grouped", [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P])
    _check(f(_ptr(h), _ptr(w_gu), _ptr(first), _ptr(order), _ptr(y), E, W, F2 // 2, top, _stream()), "experts_up_grouped")


def experts_down_grouped(y: torch.Tensor, w_down: torch.Tensor, first: torch.Tensor, out: torch.Tensor) -> None:
    """out[p] = W_down[e] y[p] (float) for the pairs in the experts' order."""
    _dev("experts_down_grouped", y, w_down, first, out)
    n, F = y.shape
    E, W, _ = w_down.shape
    _req(experts_grouped_takes(y.dtype, W, F) and w_down.dtype == torch.bfloat16 and out.dtype == torch.float32, "experts_down_grouped: types")
    _req(w_down.shape == (E, W, F) and out.shape == (n, W) and first.numel() == E + 1 and first.dtype == torch.int32, "experts_down_grouped: shapes")
    f = _fn("routed_experts", "br_experts_down_grouped", [_P, _P, _P, _P, c_int, c_int, c_int, _P])
    _check(f(_ptr(y), _ptr(w_down), _ptr(first), _ptr(out), E, W, F, _stream()), "experts_down_grouped")


def experts_gemm(a: torch.Tensor, w: torch.Tensor, first: torch.Tensor, out: torch.Tensor) -> None:
    """out[p] = w[e] a[p] for the pairs p of every expert e in the experts' order (`experts_sort`): a [pairs, K] bfloat16
    rows in that order, w [E, N, K] bfloat16, out [pairs, N] bfloat16 or float32; one launch for all experts."""
    _dev("experts_gemm", a, w, first, out)
    n, Kd = a.shape
    E, N, _ = w.shape
    _req(a.dtype == w.dtype == torch.bfloat16 and Kd % 8 == 0 and w.shape == (E, N, Kd) and out.shape == (n, N)
         and first.dtype == torch.int32 and first.numel() == E + 1, "experts_gemm: bfloat16 [pairs, K] x [E, N, K], K in steps of 8")
    f = _fn("routed_experts", "br_experts_gemm", [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P])
    _check(f(_ptr(a), _ptr(w), _ptr(first), _ptr(out), _is_bf16(out, "experts_gemm"), n, E, N, Kd, _stream()), "experts_gemm")


# ------------------------------------------------------------- clamped gated unit -----
def clamped_glu(gu: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, limit: float, alpha: float) -> None:
    """out = g sigmoid(alpha g) (u + 1), g = min(gate + b, limit), u = clamp(up + b, -limit, limit), from the float sums
    gu [T, 2 I] (gate | up) and their biases [2 I]."""
    _dev("clamped_glu", gu, bias, out)
    T, I2 = gu.shape
    _req(gu.dtype == torch.float32 and I2 % 2 == 0 and out.shape == (T, I2 // 2), "clamped_glu: gu float32 [T, 2 I], out [T, I]")
    _req(bias is None or (bias.dtype == torch.float32 and bias.numel() == I2), "clamped_glu: bias float32 [2 I]")
    f = _fn("elementwise", "br_clamped_glu", [_P, _P, _P, c_int, c_int, c_int, c_float, c_float, _P])
    _check(f(_ptr(gu), _ptr(bias), _ptr(out), _is_bf16(out, "clamped_glu"), T, I2 // 2, float(limit), float(alpha), _stream()), "clamped_glu")


def add_bias_rows(x: torch.Tensor, bias: torch.Tensor) -> None:
    _dev("add_bias_rows", x, bias)
    _req(x.dtype == torch.float32 and bias.dtype == torch.float32 and x.dim() == 2 and bias.numel() == x.shape[1], "add_bias_rows: x float32 [T, H], bias float32 [H]")
    f = _fn("elementwise", "br_add_bias_rows", [_P, _P, c_int, c_int, _P])
    _check(f(_ptr(x), _ptr(bias), x.shape[0], x.shape[1], _stream()), "add_bias_rows")


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
