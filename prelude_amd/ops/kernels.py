"""Python faces of the HIP kernels: shape and type checks on the host, then one launch.

Every function works on CUDA (HIP) tensors and launches on torch's current
stream.  Nothing here computes on the CPU or through a torch operator;
``linear`` in bfloat16 for tall inputs calls the library matrix product
(hipBLASLt, directly) where the reference calls its GEMM libraries
(crates/prelude-cuda/src/ops/gemm.rs:35-137).
"""
from __future__ import annotations

from typing import Optional

import torch

from .._native import NativeError, check, kernels

_CODES = {torch.float32: 0, torch.bfloat16: 1}


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise NativeError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle.  Asked for before every launch (a graph capture switches streams), so
    through torch's raw accessor where it has one: the Stream object costs several microseconds to build."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise NativeError("kernel operand is not on the GPU; there is no CPU path")
        if not t.is_contiguous():
            raise NativeError(f"kernel operand of shape {tuple(t.shape)} is not contiguous")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32:
        raise NativeError(f"{name} must be int32, got {t.dtype}")


def _f32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None and t.dtype != torch.float32:
        raise NativeError(f"{name} must be float32, got {t.dtype}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T], table [V, H]."""
    _dev(ids, table)
    _i32(ids, "ids")
    if ids.dim() != 1 or table.dim() != 2:
        raise NativeError(f"embed_gather: ids {tuple(ids.shape)} / table {tuple(table.shape)}")
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
    check(kernels().pa_embed_gather(_stream(), _code(table), _ptr(ids), _ptr(table), _ptr(out), ids.shape[0],
                                    table.shape[1], table.shape[0]))
    return out


def carry_tokens(sampled: torch.Tensor, src: torch.Tensor, dst: torch.Tensor, ids: torch.Tensor) -> None:
    """ids[dst[i]] = sampled[src[i]] where src[i] >= 0; all int32 on the device."""
    _dev(sampled, src, dst, ids)
    for t, name in ((sampled, "sampled"), (src, "src"), (dst, "dst"), (ids, "ids")):
        _i32(t, name)
    if src.shape != dst.shape or src.dim() != 1:
        raise NativeError(f"carry_tokens: src {tuple(src.shape)} / dst {tuple(dst.shape)}")
    check(kernels().pa_carry_tokens(_stream(), _ptr(sampled), _ptr(src), _ptr(dst), _ptr(ids), src.shape[0],
                                    sampled.numel(), ids.numel()))


def zero_fresh_rows(data: torch.Tensor, slots: torch.Tensor, fresh: torch.Tensor) -> None:
    """data[slots[i]] = 0 for every sequence i with fresh[i] != 0 and slots[i] >= 0; data [rows, ...] of a
    4-byte-multiple row size, slots / fresh int32 [B] on the device."""
    _dev(data, slots, fresh)
    _i32(slots, "slots")
    _i32(fresh, "fresh")
    if data.dim() < 1 or slots.shape != fresh.shape or slots.dim() != 1:
        raise NativeError(f"zero_fresh_rows: data {tuple(data.shape)} / slots {tuple(slots.shape)} / fresh {tuple(fresh.shape)}")
    if data.shape[0] == 0 or slots.shape[0] == 0:
        return
    row_bytes = data[0].numel() * data.element_size()
    check(kernels().pa_zero_fresh_rows(_stream(), _ptr(data), row_bytes, _ptr(slots), _ptr(fresh), slots.shape[0],
                                       data.shape[0]))


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last axis of x [T, H] with a float32 weight [H].

    With ``residual`` the norm is taken of x + residual (32-bit sum) and the
    residual tensor receives the sum.  With ``rows`` (int32 [R]) only those
    rows are normed, into a compact [R, H] output, and the residual is read only.
    """
    if isinstance(x, SliceSums):
        return _rmsnorm_slices(x, weight, eps, residual, rows)
    _dev(x, weight, residual, rows)
    _f32(weight, "norm weight")
    if x.dim() != 2 or weight.shape != (x.shape[1],):
        raise NativeError(f"rmsnorm: x {tuple(x.shape)} / weight {tuple(weight.shape)}")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype):
        raise NativeError(f"rmsnorm: residual {tuple(residual.shape)} {residual.dtype} does not match x")
    n = x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=x.device)
    check(kernels().pa_rmsnorm(_stream(), _code(x), _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), n,
                               x.shape[1], float(eps)))
    return out


def _rmsnorm_slices(x, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor],
                    rows: Optional[torch.Tensor]) -> torch.Tensor:
    """``rmsnorm`` of a product that comes as partial sums: the slices are added in order as they are loaded."""
    parts = x.parts
    _dev(parts, weight, residual, rows)
    _f32(weight, "norm weight")
    s, m, h = parts.shape
    if weight.shape != (h,) or h % 4:
        raise NativeError(f"rmsnorm: slices {tuple(parts.shape)} / weight {tuple(weight.shape)}")
    if residual is not None and (tuple(residual.shape) != (m, h) or residual.dtype != x.dtype):
        raise NativeError(f"rmsnorm: residual {tuple(residual.shape)} {residual.dtype} does not match the product")
    n = m
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    out = torch.empty((n, h), dtype=x.dtype, device=parts.device)
    check(kernels().pa_rmsnorm_slices(_stream(), _CODES[x.dtype], _ptr(parts), s, m * h, _ptr(residual), _ptr(weight),
                                      _ptr(out), _ptr(rows), n, h, float(eps)))
    return out


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}   # codes of the kernels' gated epilogues (common.h)


def gate_activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise NativeError(f"gated activation {name!r} is not one of {sorted(GATE_ACTIVATIONS)}") from None


def silu_mul(gate_up: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """act(gate) * up for gate_up [T, 2I] whose columns alternate gate_j, up_j -> [T, I]; ``activation`` is
    ``"silu"`` or ``"gelu_tanh"``, here and in the gated epilogues of the products."""
    act = gate_activation_code(activation)
    _dev(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise NativeError(f"silu_mul: input {tuple(gate_up.shape)} is not [T, 2I]")
    inter = gate_up.shape[1] // 2
    out = torch.empty((gate_up.shape[0], inter), dtype=gate_up.dtype, device=gate_up.device)
    check(kernels().pa_silu_mul(_stream(), _code(gate_up), _ptr(gate_up), _ptr(out), gate_up.shape[0], inter, act))
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    _dev(x, rows)
    _i32(rows, "rows")
    if x.dim() != 2:
        raise NativeError(f"gather_rows: x {tuple(x.shape)}")
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    check(kernels().pa_gather_rows(_stream(), _code(x), _ptr(x), _ptr(rows), _ptr(out), rows.shape[0], x.shape[1]))
    return out


def add_bias_(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    _dev(y, bias)
    _f32(bias, "bias")
    if y.dim() != 2 or bias.shape != (y.shape[1],):
        raise NativeError(f"add_bias: y {tuple(y.shape)} / bias {tuple(bias.shape)}")
    check(kernels().pa_add_bias(_stream(), _code(y), _ptr(y), _ptr(bias), y.shape[0], y.shape[1]))
    return y


def to_f32(x: torch.Tensor) -> torch.Tensor:
    _dev(x)
    if x.dtype == torch.float32:
        return x
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    check(kernels().pa_to_f32(_stream(), _code(x), _ptr(x), _ptr(out), x.numel()))
    return out


def _check_caches(k_cache, v_cache, num_kv_heads, head_dim, dtype, what) -> None:
    """K [pages, nkv, page, hd] and V [pages, nkv, hd, page] of the same pool."""
    ok = (k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4
          and k_cache.shape[0] == v_cache.shape[0] and k_cache.shape[1] == v_cache.shape[1] == num_kv_heads
          and k_cache.shape[3] == v_cache.shape[2] == head_dim and k_cache.shape[2] == v_cache.shape[3]
          and k_cache.dtype == dtype and v_cache.dtype == dtype)
    if not ok:
        raise NativeError(f"{what}: caches must be K [pages, {num_kv_heads}, page, {head_dim}] and "
                          f"V [pages, {num_kv_heads}, {head_dim}, page] of {dtype}")


def qknorm_rope_kv(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                   slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int, eps: float,
                   inv_freq: Optional[torch.Tensor] = None, values_from_keys: bool = False,
                   q_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per-head RMSNorm of Q and K, rotation by position, K and V into the paged cache.

    qkv [T, (nh + 2 nkv) * hd]; returns q [T, nh, hd].  With ``slots`` None
    nothing is written to the cache (then ``num_kv_heads`` may be 0 for a
    Q-only input).  K cache [pages, nkv, page_size, hd], V cache [pages, nkv, hd, page_size].
    ``inv_freq`` (float32 [rotary_dim / 2]) in place of the tables: the kernel takes the angle
    position * inv_freq[j] and its cosine and sine itself.  ``values_from_keys``: qkv is [T, (nh + nkv) * hd]
    and a head's cached value is its key as projected, before norm and rotation.  ``q_scale`` (float32 [nh]): every
    query head times its number, in 32-bit before it is rounded (a temperature per head).
    """
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, v_cache, inv_freq, q_scale)
    _f32(q_scale, "query scales")
    if q_scale is not None and tuple(q_scale.shape) != (num_heads,):
        raise NativeError(f"qknorm_rope_kv: query scales {tuple(q_scale.shape)} for {num_heads} heads")
    _i32(positions, "positions")
    _f32(q_weight, "q_norm weight")
    _f32(k_weight, "k_norm weight")
    _f32(cos, "cos table")
    _f32(sin, "sin table")
    _f32(inv_freq, "rotary frequencies")
    t = qkv.shape[0]
    width = (num_heads + (1 if values_from_keys else 2) * num_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise NativeError(f"qknorm_rope_kv: qkv {tuple(qkv.shape)} is not [T, {width}]")
    if positions.shape != (t,):
        raise NativeError(f"qknorm_rope_kv: positions {tuple(positions.shape)} for {t} tokens")
    for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
        if w is not None and w.shape != (head_dim,):
            raise NativeError(f"qknorm_rope_kv: {nm} weight {tuple(w.shape)} is not [{head_dim}]")
    by_freq = inv_freq is not None or values_from_keys or q_scale is not None
    if q_scale is not None and (cos is not None or sin is not None):
        raise NativeError("qknorm_rope_kv: a scale per query head goes with rotation from the frequencies, not from tables")
    if rotary_dim and inv_freq is not None:
        if cos is not None or sin is not None or tuple(inv_freq.shape) != (rotary_dim // 2,):
            raise NativeError(f"qknorm_rope_kv: frequencies must be [{rotary_dim // 2}] and come without tables")
    elif rotary_dim:
        if values_from_keys:
            raise NativeError("qknorm_rope_kv: values that are the keys are rotated from the frequencies, not from tables")
        if cos is None or sin is None or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rotary_dim // 2:
            raise NativeError(f"qknorm_rope_kv: cos/sin tables must be [positions, {rotary_dim // 2}]")
    page_size = 1
    if slots is not None:
        _i32(slots, "slots")
        if slots.shape != (t,):
            raise NativeError(f"qknorm_rope_kv: slots {tuple(slots.shape)} for {t} tokens")
        _check_caches(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype, "qknorm_rope_kv")
        page_size = k_cache.shape[2]
    q_out = torch.empty((t, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    if by_freq:
        check(kernels().pa_qknorm_rope_kv_freq(_stream(), _code(qkv), _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _ptr(inv_freq),
                                               _ptr(positions), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), t,
                                               num_heads, num_kv_heads, head_dim, rotary_dim, page_size, float(eps),
                                               1 if values_from_keys else 0, _ptr(q_scale)))
        return q_out
    check(kernels().pa_qknorm_rope_kv(_stream(), _code(qkv), _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _ptr(cos),
                                      _ptr(sin), _ptr(positions), _ptr(slots), _ptr(q_out), _ptr(k_cache),
                                      _ptr(v_cache), t, num_heads, num_kv_heads, head_dim, rotary_dim, page_size,
                                      float(eps)))
    return q_out


def gemm_plain(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] @ w[N, K]^T (+ bias) with 32-bit FMA arithmetic in a fixed order."""
    _dev(x, w, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.dtype != w.dtype:
        raise NativeError(f"gemm: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    out_dtype = out_dtype or x.dtype
    m, k = x.shape
    n = w.shape[0]
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm: bias {tuple(bias.shape)} is not [{n}]")
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_plain(_stream(), _code(x), _CODES[out_dtype], _ptr(x), _ptr(w), _ptr(bias), _ptr(out), m, n,
                                  k, k, k, n))
    return out


SKINNY_MAX_ROWS = 16   # above this the library product is faster (the kernel itself takes up to 64) ...
# ... except for small weights in tiles, where the library's 19 us floor is what it takes: (rows, elements) up to
# which the streaming kernel measured faster -- [6144, 2560] and [2560, 4096] to 48 rows (11 against 19 us at 32),
# [6144, 4096] to 32 rows (15 against 19 us); weights beyond that go to the library, as do rows of 8192 columns or
# more -- unless they are very long: [5120, 25600] takes the library 143 to 155 us at 24 to 64 rows, the streaming
# kernel 67 to 118.  Inside a captured step, where no launch waits for the host, the library's floor is 11 us and
# the order is the same: [4096, 1024] takes the streaming kernel 4.6 to 8.0 us at 17 to 64 rows, [6144, 2560] 11.6
# to 14.4 at 17 to 48 rows against 12.5 to 15.5
TILED_LIMITS = ((64, 1 << 23), (48, 1 << 24), (32, 1 << 25))
TILED_LONG_ROWS = 16384


def _tiled_beyond_16(m: int, n: int, k: int) -> bool:
    if k % 8:
        return False
    if k >= TILED_LONG_ROWS:
        return m <= 64
    return k < 8192 and any(m <= rows and n * k <= size for rows, size in TILED_LIMITS)


class TiledWeight:
    """A bfloat16 weight [n, k] laid out in the tiles the weight-streaming kernel reads (``pack_tiles``)."""

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data, self.n, self.k = data, n, k
        self.shape = (n, k)
        self.dtype, self.device = data.dtype, data.device


def pack_tiles(w: torch.Tensor) -> TiledWeight:
    """The weight in tiles of 16 rows x 64 columns, each stored in the order a wavefront's lanes load it."""
    _dev(w)
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise NativeError(f"pack_tiles: w {tuple(w.shape)} {w.dtype}")
    n, k = w.shape
    out = torch.empty(((n + 15) // 16) * ((k + 63) // 64) * 1024, dtype=torch.bfloat16, device=w.device)
    check(kernels().pa_pack_tiles(_stream(), _ptr(w), _ptr(out), n, k))
    return TiledWeight(out, n, k)


WEIGHT_TILES = True   # keep a tiled copy of bfloat16 weights for products of few rows (``set_weight_tiles``)


def set_weight_tiles(on: bool) -> None:
    """Whether ``prepare_weight`` adds the tiled copy (a second copy of the weight in device memory)."""
    global WEIGHT_TILES
    WEIGHT_TILES = bool(on)


class LinearWeight:
    """A matrix [out, in] as the products read it: by rows for many-row products (the library's) and the
    32-bit path, and, for bfloat16, in tiles for the weight-streaming product of few rows."""

    def __init__(self, rows: torch.Tensor, tiles: Optional[TiledWeight] = None):
        self.rows, self.tiles = rows, tiles
        self.shape, self.dtype, self.device = tuple(rows.shape), rows.dtype, rows.device

    def first_rows(self, n: int) -> torch.Tensor:
        """The first n outputs as a plain matrix (a view)."""
        return self.rows[:n]


def prepare_weight(w: torch.Tensor) -> LinearWeight:
    """What a part keeps of a weight it multiplies by: called once when weights are loaded."""
    tiles = None
    if WEIGHT_TILES and w.dtype == torch.bfloat16 and w.is_cuda and w.dim() == 2:
        tiles = pack_tiles(w.contiguous())
    return LinearWeight(w, tiles)


def gemm_skinny(x: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False,
                activation: str = "silu") -> torch.Tensor:
    """x [M <= 64, K] @ w[N, K]^T in bfloat16 on the matrix cores, streaming w once.

    ``w`` is a tensor [N, K] or a ``TiledWeight``.  With
    ``silu_mul_epilogue`` the rows of w alternate gate_j, up_j and the
    result is act(gate) * up, [M, N/2], act being ``activation``."""
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    tiled = isinstance(w, TiledWeight)
    wt = w.data if tiled else w
    _dev(x, wt, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or len(w.shape) != 2 or x.shape[1] != w.shape[1] or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"gemm_skinny: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_skinny: bias {tuple(bias.shape)} is not [{n}]")
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_skinny(_stream(), _CODES[out_dtype], epi, _ptr(x), _ptr(wt),
                                   _ptr(bias), _ptr(out), m, n, k, k, cols, 1 if tiled else 0))
    return out


class SliceSums:
    """A product left as 32-bit partial sums of slices of its inner size, [slices, M, N]: what ``gemm_mid`` gives
    when its reader can add the slices itself (``rmsnorm`` does, as it loads them).  ``materialize()`` adds them
    for any other reader."""

    def __init__(self, parts: torch.Tensor, dtype: torch.dtype):
        self.parts = parts
        self.shape = tuple(parts.shape[1:])
        self.dtype, self.device = dtype, parts.device

    def materialize(self) -> torch.Tensor:
        s, m, n = self.parts.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.device)
        check(kernels().pa_sum_slices(_stream(), _CODES[self.dtype], _ptr(self.parts), _ptr(out), s, m * n))
        return out


def gemm_skinny_sliced(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None, slices: int = 2,
                       waves: int = 0) -> SliceSums:
    """``gemm_skinny`` of up to 16 rows with K cut into slices, each a workgroup of its own a tile, left as 32-bit
    partial sums for a reader that adds them: a narrow weight has too few tiles to give every compute unit work."""
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    m, k = x.shape
    n = w.shape[0]
    if x.dtype != torch.bfloat16 or w.shape[1] != k or not 1 <= m <= 16 or (bias is not None and bias.shape != (n,)):
        raise NativeError(f"gemm_skinny_sliced: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    made = int(kernels().pa_gemm_skinny_slices(k, int(slices)))
    parts = torch.empty((made, m, n), dtype=torch.float32, device=x.device)
    check(kernels().pa_gemm_skinny_sliced(_stream(), _ptr(x), _ptr(w.data), _ptr(bias), _ptr(parts), m, n, k, k, int(slices),
                                          int(waves)))
    return SliceSums(parts, torch.bfloat16)


GEMM_MID_MAX_ROWS = 128
# Where ``linear`` takes the product with X staged in LDS (measured at the shapes of 4B, 8B and 32B models, 17 to
# 128 rows).  Cut into slices, for a reader that adds them, wherever the weight's shape gives two slices or more:
# [2560, 4096] at 64 rows 9.2 against the library's 14.7 us, [2560, 9728] 14.4 against 28, [4096, 12288] 28 against
# 37, [5120, 25600] 50 against 155 (and 73 against 179 at 128 rows).  Uncut for very wide weights with 32-bit output
# (the head; figures at MID_WIDE_MAX_M).  The gated product with its activation in the epilogue: see
# ``linear_silu_mul``.
MID_MIN_SLICES = 2
MID_WIDE_ROWS = 65536
MID_WIDE_MAX_M = 64            # ... for rows of up to MID_WIDE_SHORT_K columns, half of it beyond.  (Alone inside a
#                                captured graph the head is ahead of the library up to 128 rows, 214 against 230 us at
#                                96 rows of 2,560 columns; in the decode step of 112 requests it is not: 7,380 against
#                                7,640 tok/s.  The step decides.)
MID_WIDE_SHORT_K = 4096
MID_SLICED_MIN_ROWS = 9        # ... for rows of MID_SLICED_LONG_K columns or more; 17 otherwise
MID_SLICED_LONG_K = 5120
MID_SLICED_MIN_ROWS_LONG = 8   # rows of TILED_LONG_ROWS columns or more: in slices from here on
# A reader that wants a tensor gets the slices too, added by a kernel of their own, where the pair is still ahead of
# the library: large weights ([10240, 5120] inside a captured step: 24.2 to 26.9 us at 24 to 64 rows against 28.4 to
# 32.4, 33.7 and 38.6 at 96 and 128 rows against 36.1 and 40.4; [6144, 4096] and [6144, 2560] are within a
# microsecond either way and stay with the library)
MID_SUMMED_MIN_ELEMENTS = 40 << 20
MID_PRODUCTS = True    # ``set_mid_products``: off sends these products where they went without this kernel (measurements)


def set_mid_products(on: bool) -> None:
    global MID_PRODUCTS
    MID_PRODUCTS = bool(on)


def gemm_mid_slices(n: int, k: int) -> int:
    """Into how many slices of its inner size ``gemm_mid`` cuts an [n, k] weight for a reader that adds slices."""
    return int(kernels().pa_gemm_mid_slices(int(n), int(k)))


def gemm_mid(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None,
             out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False, slices: int = 1, waves: int = 0,
             activation: str = "silu"):
    """x [M <= 128, K] @ w[N, K]^T from the weight in tiles, X staged through LDS; with ``slices`` > 1 the result
    is a ``SliceSums`` (one 32-bit partial sum per slice of K) instead of a tensor.  ``waves``: wavefronts a
    workgroup (3, 4, 5, 6, 8; 0 lets the launcher choose by the weight's shape; the same bits at every number)."""
    if not isinstance(w, TiledWeight):
        raise NativeError("gemm_mid takes the weight in tiles (pack_tiles)")
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or x.shape[1] != w.k or x.dtype != torch.bfloat16:
        raise NativeError(f"gemm_mid: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    m, k = x.shape
    n = w.n
    out_dtype = out_dtype or torch.bfloat16
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_mid: bias {tuple(bias.shape)} is not [{n}]")
    if slices > 1:
        parts = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        check(kernels().pa_gemm_mid(_stream(), _CODES[out_dtype], 0, _ptr(x), _ptr(w.data), _ptr(bias), None, _ptr(parts),
                                    m, n, k, k, n, slices, waves))
        return SliceSums(parts, out_dtype)
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_mid(_stream(), _CODES[out_dtype], epi, _ptr(x), _ptr(w.data),
                                _ptr(bias), _ptr(out), None, m, n, k, k, cols, 1, waves))
    return out


def gemm_tall(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None, silu_mul_epilogue: bool = False,
              slices: int = 1, shape=(0, 0), activation: str = "silu"):
    """x [M, K] @ w[N, K]^T for any number of rows from the weight in tiles, the output tiled both ways: a
    workgroup owns ``16 * shape[0]`` rows of X and ``64 * shape[1]`` rows of W ((0, 0): the launcher chooses by the
    product's size; the same bits at every shape).  bfloat16 out; with ``slices`` > 1 a ``SliceSums``."""
    if not isinstance(w, TiledWeight):
        raise NativeError("gemm_tall takes the weight in tiles (pack_tiles)")
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or x.shape[1] != w.k or x.dtype != torch.bfloat16:
        raise NativeError(f"gemm_tall: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    m, k = x.shape
    n = w.n
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_tall: bias {tuple(bias.shape)} is not [{n}]")
    if slices > 1:
        parts = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        check(kernels().pa_gemm_tall(_stream(), 0, _ptr(x), _ptr(w.data), _ptr(bias), None, _ptr(parts), m, n, k, k, n,
                                     slices, int(shape[0]), int(shape[1])))
        return SliceSums(parts, torch.bfloat16)
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_tall(_stream(), epi, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out),
                                 None, m, n, k, k, cols, 1, int(shape[0]), int(shape[1])))
    return out


# Where ``linear`` takes the product tiled both ways (``gemm_tall``) beyond the 128 rows of ``gemm_mid``.  Alone, with
# the weights coming from memory, it is ahead of the library for most products of 129 to 320 rows at the shapes of 4B, 8B
# and 32B models ([2560, 9728] at 256 rows in four slices 35.1 against 41.7 us, [4096, 12288] 46.5 against 54.8,
# [5120, 25600] 108 against 261; the gated [19456, 2560] 46.9 against 51.7 with the separate activation kernel); what
# decides is the prompt step it runs in, where the reader of slices pays for them (the norm reads four 32-bit partial
# sums instead of one bfloat16 tensor) -- a whole prompt through 36 layers, same box, library against this kernel:
#  - in four slices for the norm that follows, wide outputs only: hidden 4,096 at 129 / 160 / 192 / 256 rows 7.29 /
#    8.00 / 9.27 / 8.21 against 6.96 / 6.85 / 7.42 / 8.02 ms, level at 320 rows and behind from 384 on; hidden 2,560
#    5.01 / 5.20 / 5.43 / 6.56 against 5.34 / 5.49 / 5.78 / 6.39: the library's.  The very large weights of a 32B
#    model (a [5120, 25600] product alone: 163 against 271 us at 512 rows) up to 576 rows;
#  - the gated product with its activation in the epilogue, rows shorter than 4,096 columns: hidden 2,560 at 129 / 192 /
#    256 rows 5.01 / 5.43 / 6.56 against 4.76 / 5.23 / 6.34 ms, behind from 288 rows on (6.16 against 6.43);
#    [24576, 4096] is the library's at every number of rows (256 rows: 68.2 against 71.9 us);
#  - slices added by a kernel of their own for a reader of tensors (the QKV projection) lost everywhere (hidden
#    2,560 at 256 rows: 6.56 against 8.01 ms) and are not dispatched.
TALL_MAX_ROWS = 256
TALL_SLICED_MIN_N = 4096       # outputs at least this wide go to it in slices for the norm ...
TALL_HUGE_MAX_ROWS = 576       # ... and weights of TALL_HUGE_ELEMENTS up to this many rows
TALL_HUGE_ELEMENTS = 80 << 20        # [5120, 17408] at 384 and 512 rows: 127 and 134 us against the library's 141 and 175
TALL_GATED_MAX_K = 4096
TALL_PRODUCTS = 3              # ``set_tall_products``: which of these products ``gemm_tall`` takes (measurements):
#                                1 in slices for a reader of slices, 2 the gated one


def set_tall_products(on) -> None:
    global TALL_PRODUCTS
    TALL_PRODUCTS = 3 if on is True else int(on)


def _tall_slices(k: int) -> int:
    """Slices of the inner size for ``gemm_tall``: four where every slice still has eight steps of 64 columns."""
    steps = (k + 63) // 64
    for s in (4, 2):
        if steps >= 8 * s and -(-steps // -(-steps // s)) == s:
            return s
    return 1


def _tall_sliced(m: int, n: int, k: int) -> bool:
    if not TALL_PRODUCTS & 1 or m <= GEMM_MID_MAX_ROWS or k % 8 or n % 4 or n < TALL_SLICED_MIN_N:
        return False
    return m <= TALL_MAX_ROWS or (m <= TALL_HUGE_MAX_ROWS and n * k >= TALL_HUGE_ELEMENTS)


LIBRARY_WORKSPACE_BYTES = 76 << 20   # what the library's stream-K kernels may use for partial sums
_library_workspaces: dict = {}


def library_workspace_reserve(device) -> int:
    """Bytes the library product will still allocate on ``device`` at its first call (0 once it has)."""
    return 0 if torch.device(device) in _library_workspaces else LIBRARY_WORKSPACE_BYTES


def gemm_library(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x W^T in bfloat16 with 32-bit accumulation by hipBLASLt, called directly (its plan is kept per shape:
    a call through ``torch.matmul`` costs the host some 20 us, this one 14)."""
    _dev(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"gemm_library: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    ws = _library_workspaces.get(x.device)
    if ws is None:
        ws = _library_workspaces[x.device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_library(_stream(), _ptr(x), _ptr(w), _ptr(out), m, n, k, k, n, _ptr(ws), LIBRARY_WORKSPACE_BYTES))
    return out


def linear(x: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, slices_ok: bool = False):
    """y = x W^T (+ b), W [out, in] as a tensor or a ``LinearWeight``.  float32: our own true 32-bit product.
    bfloat16: few rows our weight-streaming kernel (from the tiled copy if the weight has one), above that the
    library product or, for the shapes they suit, the products with X staged in LDS (``gemm_mid`` to 128 rows,
    ``gemm_tall`` beyond); 32-bit accumulation in all.

    ``slices_ok``: the caller's reader adds slices itself (``rmsnorm`` does): a narrow weight at 17 to 128 rows
    (a wide one beyond, see ``TALL_MAX_ROWS``) then comes back as ``SliceSums`` (the product cut along its inner size, a 32-bit partial sum per slice)
    instead of a tensor."""
    tiles = None
    if isinstance(w, LinearWeight):
        w, tiles = w.rows, w.tiles
    if x.dtype == torch.float32:
        return gemm_plain(x, w, bias, out_dtype)
    _dev(x, w, bias)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"linear: x {x.dtype} / w {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    # what a reader of slices gets from the product with X in LDS: from MID_SLICED_MIN_ROWS rows on where the rows are
    # long (the streaming kernel sums such a row in one workgroup: [2560, 9728] with the norm behind it 20.2 us
    # at 16 rows against 17.7 in four or eight slices, [5120, 25600] 60.4 against 50.6; at 8 rows and fewer it is
    # the other way round), from 17 rows on everywhere
    sliced = (MID_PRODUCTS and slices_ok and tiles is not None and k % 8 == 0 and n % 4 == 0 and m <= GEMM_MID_MAX_ROWS
              and out_dtype in (None, torch.bfloat16)
              and (m > SKINNY_MAX_ROWS or (m >= MID_SLICED_MIN_ROWS and k >= MID_SLICED_LONG_K)
                   # rows of 16,384 columns and more from 8 rows on ([5120, 17408] with the norm behind it 40.0
                   # against 42.6 us at 8 rows, [5120, 25600] 54.3 against 57.9; level at 4 rows)
                   or (m >= MID_SLICED_MIN_ROWS_LONG and k >= TILED_LONG_ROWS)))
    # (with four slices at most this holds just beyond 16 rows too, where eight slices lost to the streaming kernel:
    # with the norm that reads it, at 20 and 24 rows, [2560, 4096] 11.3 and 11.4 us against 12.2 and 13.0, [2048, 2048]
    # 8.7 against 9.0 and 9.2, [5120, 5120] 17.6 and 17.5 against 20.2 and 21.2; [4096, 4096] 14.6 and 14.9 against
    # 13.9 and 14.7 is the one shape the other way round)
    if SKINNY_SLICED and slices_ok and tiles is not None and k % 8 == 0 and n % 4 == 0 and out_dtype in (None, torch.bfloat16):
        s = _skinny_slices(m, n, k)
        if s > 1:
            return gemm_skinny_sliced(x, tiles, bias, slices=s, waves=8)
    if sliced:
        s = gemm_mid_slices(n, k)
        if s >= MID_MIN_SLICES:
            return gemm_mid(x, tiles, bias, slices=s)
    if m <= SKINNY_MAX_ROWS and k % 8 == 0:
        # a large weight whose reader wants a tensor, 9 to 16 rows: [10240, 5120] 22.5 us against the streaming
        # kernel's 27.5 at 12 rows (22.9 against 22.3 at 8); [7168, 5120] is the streaming kernel's (15.4 against 20.8)
        if (MID_PRODUCTS and tiles is not None and m >= MID_SLICED_MIN_ROWS and bias is None and n % 4 == 0
                and out_dtype in (None, torch.bfloat16) and n * k >= MID_SUMMED_MIN_ELEMENTS and k < TILED_LONG_ROWS):
            return gemm_mid(x, tiles)
        return gemm_skinny(x, tiles if tiles is not None and m <= 16 else w, bias, out_dtype)
    if (MID_PRODUCTS and tiles is not None and bias is None and k % 8 == 0 and n % 4 == 0 and m <= GEMM_MID_MAX_ROWS
            and out_dtype in (None, torch.bfloat16) and n * k >= MID_SUMMED_MIN_ELEMENTS and k < TILED_LONG_ROWS):
        s = gemm_mid_slices(n, k)
        if s >= MID_MIN_SLICES:
            return gemm_mid(x, tiles, slices=s).materialize()
    if MID_PRODUCTS and tiles is not None and k % 8 == 0 and m <= GEMM_MID_MAX_ROWS:
        if n >= MID_WIDE_ROWS and m <= (MID_WIDE_MAX_M if k <= MID_WIDE_SHORT_K else MID_WIDE_MAX_M // 2):
            return gemm_mid(x, tiles, bias, out_dtype)
    if tiles is not None and _tiled_beyond_16(m, w.shape[0], k):
        return gemm_skinny(x, tiles, bias, out_dtype)
    if tiles is not None and slices_ok and out_dtype in (None, torch.bfloat16) and _tall_sliced(m, n, k):
        s = _tall_slices(k)
        if s > 1:
            return gemm_tall(x, tiles, bias, slices=s)
    if k % 8:
        # rows that are no multiple of 16 bytes: neither the streaming kernel's loads nor the library's fast
        # kernels take them; the plain product does (bfloat16 in, 32-bit sums), and only odd toy sizes come here
        return gemm_plain(x, w, bias, out_dtype)
    y = gemm_library(x, w)
    if bias is not None:
        add_bias_(y, bias)
    if out_dtype is not None and out_dtype != y.dtype:
        y = to_f32(y)
    return y


# A narrow weight has too few tiles of 16 rows to give every compute unit a workgroup of the streaming kernel (160
# for 2,560 outputs, 64 for 1,024): for a reader of slices K is cut so that there are 256 to 480 workgroups.  Measured
# with the norm behind it, inside a graph, against what was dispatched before (us): [2560, 9728] in three slices
# 16.0 -> 14.9 at 6 rows, 16.8 -> 15.0 at 8, 16.5 -> 15.5 at 10, level at 4 and 12 and behind at 1, 2 and 16;
# [2048, 6144] in two 9.7 -> 8.9 at one row, 10.5 -> 9.5 at 8, 11.0 -> 9.9 at 16; [1024, 3072] in four 7.0 -> 6.5,
# 7.8 -> 7.0, 8.8 -> 7.3; [1024, 2048] in four 6.5 -> 6.3, 7.2 -> 6.8, 7.8 -> 7.0; nothing for [2048, 2048], [4096, 4096],
# [5120, 8192], and for [5120, 5120] at 6 to 8 rows only.
# (most tiles, slices, least k-steps, rows from, rows to)
SKINNY_SLICED_SHAPES = ((64, 4, 32, 1, 16), (128, 2, 64, 1, 16), (160, 3, 128, 4, 12))
SKINNY_SLICED = True    # ``set_skinny_sliced``: off sends these products where they went before (measurements)


def set_skinny_sliced(on: bool) -> None:
    global SKINNY_SLICED
    SKINNY_SLICED = bool(on)


def _skinny_slices(m: int, n: int, k: int) -> int:
    tiles, steps = (n + 15) // 16, (k + 63) // 64
    if k >= TILED_LONG_ROWS:      # rows this long have rules of their own (MID_SLICED_MIN_ROWS_LONG), measured at their shapes
        return 1
    for most_tiles, slices, least_steps, rows_from, rows_to in SKINNY_SLICED_SHAPES:
        if tiles <= most_tiles:
            return slices if steps >= least_steps and rows_from <= m <= rows_to else 1
    return 1


def as_tensor(x):
    """A product that may have come back as ``SliceSums``, as a tensor."""
    return x.materialize() if isinstance(x, SliceSums) else x


def set_skinny_max_rows(n: int) -> None:
    """Up to how many rows ``linear`` uses the weight-streaming kernel (for measurements)."""
    global SKINNY_MAX_ROWS
    SKINNY_MAX_ROWS = max(0, min(int(n), 64))


# The gated product keeps its activation in the streaming kernel's epilogue, which saves the library's separate
# SiLU*up kernel: measured in the decode step, that is the faster way up to 24 rows for [19456, 2560] (5.76 against
# 5.79 ms a step at 24 rows, 6.76 against 6.71 at 32) and up to 32 rows for [24576, 4096] (6.94 against 7.26 ms at
# 24 rows, 7.98 against 8.18 at 32); for [51200, 5120] the library with the separate kernel is ahead from 12 rows on
# Beyond 16 rows the product with X staged in LDS takes it, activation in its epilogue too: [19456, 2560] 20.3 us at
# 32 rows, 22.9 at 64 and 33.0 at 128 against the library's 27.3, 31.0 and 35.3 with the separate kernel (the
# streaming kernel: 30 and 47 at 32 and 64); [24576, 4096] 37.6 at 64 rows against 47.7; [51200, 5120] stays with the
# library (110 against 105 at 64 rows, 163 against 119 at 128).  The bounds below are for weights without tiles
# for that kernel to read, and for measurements with it switched off.
# Up to 16 rows the two kernels are close: [19456, 2560] takes the product with X in LDS 19.4 us at any number of rows
# and the streaming kernel 18.7 at one row, 20.0 at 8, 23.2 at 16; [24576, 4096] 35.0 against 35.8 to 36.7
GATED_MID_MIN_ROWS = 8         # ... for rows shorter than GATED_TILED_LONG_K columns; 1 for longer ones
GATED_TILED_ROWS = 24          # ... and 32 for rows of GATED_TILED_LONG_K columns or more
GATED_TILED_LONG_K = 4096
GATED_TILED_ELEMENTS = 1 << 27
# ... a [34816, 5120] weight too, up to 96 rows (63.4 against the streaming kernel's 70.7 us at 16 rows, 65.3 against
# the library's 79.3 at 20, 75.0 against 85.8 at 48, 95.9 against 97.1 at 96; 116.9 against 101.6 at 128), while
# [51200, 5120] is the library's from 12 rows on
GATED_LARGE_ELEMENTS = 200 << 20
GATED_LARGE_MAX_ROWS = 96
# ... and below this size the streaming kernel keeps 8 rows ([12288, 2048] 10.8 against 12.1 us, [6144, 1024] 4.8
# against 5.5; from 12 rows on the product with X in LDS is level or ahead)
GATED_SMALL_ELEMENTS = 40 << 20


def _gated_tiled(m: int, n: int, k: int) -> bool:
    return n * k <= GATED_TILED_ELEMENTS and k < 8192 and (m <= GATED_TILED_ROWS or (m <= 32 and k >= GATED_TILED_LONG_K))


def linear_gated(x: torch.Tensor, w, activation: str = "silu") -> torch.Tensor:
    """act(x Wg^T) * (x Wu^T) for a weight [2I, K] whose rows alternate gate_j, up_j; ``activation`` is ``"silu"``
    or ``"gelu_tanh"`` (the same kernels, another epilogue code)."""
    gate_activation_code(activation)
    m, k = x.shape
    if x.dtype == torch.bfloat16 and k % 8 == 0:
        tiles = w.tiles if isinstance(w, LinearWeight) else None
        if m <= SKINNY_MAX_ROWS:
            first = 1 if k >= GATED_TILED_LONG_K else GATED_MID_MIN_ROWS
            if tiles is not None and tiles.n * k < GATED_SMALL_ELEMENTS:
                first = GATED_MID_MIN_ROWS + 1
            elif tiles is not None and tiles.n * k > GATED_TILED_ELEMENTS:
                first = MID_SLICED_MIN_ROWS
            if MID_PRODUCTS and tiles is not None and tiles.n * k <= GATED_LARGE_ELEMENTS and m >= first:
                return gemm_mid(x, tiles, silu_mul_epilogue=True, activation=activation)
            if isinstance(w, LinearWeight):
                w = tiles if tiles is not None and m <= 16 else w.rows
            return gemm_skinny(x, w, silu_mul_epilogue=True, activation=activation)
        if MID_PRODUCTS and tiles is not None and (
                (m <= GEMM_MID_MAX_ROWS and tiles.n * k <= GATED_TILED_ELEMENTS)
                or (m <= GATED_LARGE_MAX_ROWS and tiles.n * k <= GATED_LARGE_ELEMENTS)):
            return gemm_mid(x, tiles, silu_mul_epilogue=True, activation=activation)
        if tiles is not None and _gated_tiled(m, tiles.n, k):
            return gemm_skinny(x, tiles, silu_mul_epilogue=True, activation=activation)
        if (TALL_PRODUCTS & 2 and tiles is not None and GEMM_MID_MAX_ROWS < m <= TALL_MAX_ROWS and k < TALL_GATED_MAX_K
                and tiles.n % 2 == 0):
            return gemm_tall(x, tiles, silu_mul_epilogue=True, activation=activation)
    return silu_mul(linear(x, w), activation)


# The residual add and RMSNorm in front of the gated product, inside that product (``gemm_mid`` stages X through LDS
# once per workgroup, and there are a few hundred workgroups, so adding the residual and multiplying by the gain as
# it stages costs little; the row's scale is applied to the finished sums): one kernel less in a decode step's layer.
# For up to 16 rows whose mixer output comes as a tensor, and weights of 40 M to 200 M elements: measured against
# the two kernels apart it gains 1.3 to 3 us at [19456, 2560], 2.3 to 3.8 us at [24576, 4096], 2.5 us up to 8 rows
# at [34816, 5120] (nothing at 12 rows, and it loses 1.5 us at 16), and loses 0.3 to 1.6 us at [6144, 1024] and
# [12288, 2048], where the streaming kernel is the better product.
NORMED_GATED = True              # ``set_normed_gated``: off runs the norm and the product apart (measurements)
NORMED_GATED_MAX_ROWS = 16
NORMED_GATED_MAX_ROWS_LARGE = 12   # ... for weights of more than GATED_TILED_ELEMENTS elements


def set_normed_gated(on: bool) -> None:
    global NORMED_GATED
    NORMED_GATED = bool(on)


def gated_after_norm_supported(x, residual, w, activation: str = "silu") -> bool:
    """Whether ``linear_gated_after_norm`` takes these operands (else: the norm, then ``linear_gated``)."""
    if not (NORMED_GATED and MID_PRODUCTS and isinstance(x, torch.Tensor) and isinstance(residual, torch.Tensor)
            and isinstance(w, LinearWeight) and w.tiles is not None and activation in GATE_ACTIVATIONS):
        return False
    m, k = x.shape
    return (x.dtype == torch.bfloat16 and residual.dtype == torch.bfloat16 and residual.shape == x.shape and x.is_contiguous()
            and residual.is_contiguous() and k % 8 == 0 and w.tiles.n % 2 == 0
            and GATED_SMALL_ELEMENTS <= w.tiles.n * k <= GATED_LARGE_ELEMENTS
            and 1 <= m <= (NORMED_GATED_MAX_ROWS if w.tiles.n * k <= GATED_TILED_ELEMENTS else NORMED_GATED_MAX_ROWS_LARGE))


def linear_gated_after_norm(x: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor, eps: float, w,
                            activation: str = "silu", waves: int = 0):
    """(residual + x rounded once, act(h Wg^T) * (h Wu^T)) for h = rmsnorm(residual + x; gain, eps): the residual add,
    the norm and the gated product in one kernel.  The new residual is a tensor of its own."""
    _dev(x, residual, gain, w.tiles.data)
    _f32(gain, "gain")
    m, k = x.shape
    n = w.tiles.n
    if gain.shape != (k,) or w.tiles.k != k:
        raise NativeError(f"linear_gated_after_norm: x {tuple(x.shape)} / gain {tuple(gain.shape)} / w {w.tiles.shape}")
    res_out = torch.empty_like(residual)
    out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_mid_normed(_stream(), 1 + gate_activation_code(activation), _ptr(x), _ptr(residual), _ptr(gain),
                                       float(eps), _ptr(res_out), _ptr(w.tiles.data), _ptr(out), m, n, k, k, n // 2, int(waves)))
    return res_out, out


def linear_silu_mul(x: torch.Tensor, w) -> torch.Tensor:
    """``linear_gated`` with SiLU, the reference's own feed-forward (crates/prelude-core/src/models/qwen3.rs:429-447)."""
    return linear_gated(x, w, "silu")


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      seq_of_token: torch.Tensor, positions: torch.Tensor, window: int, scale: float,
                      softcap: float = 0.0, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Paged causal attention, any mix of portions and decode tokens.  ``sink`` (float32 [heads], here and in
    ``attention``): a head's softmax divides by sum_j exp(score_j) + exp(sink_h), a term that brings no value.  ``softcap`` > 0 (here and in the other
    attention entry points) bends every scaled score to ``softcap * tanh(score / softcap)`` before the softmax;
    0, the default, leaves the scores alone (the same bits as without the parameter).

    q [T, nh, hd]; K cache [pages, nkv, page, hd], V cache [pages, nkv, hd, page]; block_table int32 [B, stride];
    seq_of_token / positions int32 [T].  window 0 = all keys.
    """
    _dev(q, k_cache, v_cache, block_table, seq_of_token, positions)
    _i32(block_table, "block_table")
    _i32(seq_of_token, "seq_of_token")
    _i32(positions, "positions")
    if q.dim() != 3:
        raise NativeError(f"attention: q {tuple(q.shape)} is not [T, heads, head_dim]")
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1] if k_cache is not None and k_cache.dim() == 4 else -1, hd, q.dtype,
                  "attention")
    if seq_of_token.shape != (t,) or positions.shape != (t,) or block_table.dim() != 2:
        raise NativeError("attention: index arrays do not match the number of tokens")
    out = torch.empty_like(q)
    if sink is not None:
        _check_sinks(sink, nh)
        check(kernels().pa_attn_generic_sink(_stream(), _code(q), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                             block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out), t, nh,
                                             k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale),
                                             float(softcap), _ptr(sink)))
        return out
    check(kernels().pa_attn_generic(_stream(), _code(q), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                    block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out), t, nh,
                                    k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale), float(softcap)))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Index of the largest logit per row (lowest index among equals); logits float32 [R, V] -> int32 [R]."""
    _dev(logits)
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise NativeError(f"argmax: logits {tuple(logits.shape)}")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    words = kernels().pa_argmax_scratch(logits.shape[0], logits.shape[1])
    scratch = torch.empty((words,), dtype=torch.float32, device=logits.device) if words else None
    check(kernels().pa_argmax(_stream(), _ptr(logits), _ptr(out), _ptr(scratch), logits.shape[0], logits.shape[1]))
    return out


# Keys per split of the decode kernel: fixed, so which keys a split sums never depends on the batch.  (The order in
# which a split's steps are added does, in the last bits: grids of 769 to 1,536 workgroups run with two wavefronts a
# workgroup instead of four.  Steps of the same size on the same side of those limits give the same bits.)
DECODE_SPLIT_KEYS = 256
DECODE_CONTEXT_STEP = 1024   # the longest context of a step counts rounded up to this many tokens (whole pages)


def decode_context_bound(max_context: int, page_size: int) -> int:
    """The longest context of a step of single tokens, rounded up: the number of splits the decode kernels are
    launched for follows this bound and not the context itself, and so do the choices that follow the grid's size
    (wavefronts a workgroup, groups of the merge), which change a sum's last bits.  A step replayed from a graph
    knows only such a bound (the width of its block tables); with the same rounding a step run directly is launched
    alike and gives the same bits.

    Contexts of up to one split (256 keys) are a class of their own: one split needs no workspace and no merge, a
    launch less per layer where a whole step is a few hundred short kernels (a 28-layer model at 128 to 160 tokens of
    context: 233 launches a step with the merge, 205 without)."""
    first = max(1, DECODE_SPLIT_KEYS // page_size) * page_size
    if max_context <= first:
        return first
    step = max(1, DECODE_CONTEXT_STEP // page_size) * page_size
    return -(-max(int(max_context), 1) // step) * step


def _decode_splits(max_context: int, window: int, page_size: int) -> int:
    bound = decode_context_bound(max_context, page_size)
    if bound <= DECODE_SPLIT_KEYS:
        return 1            # every context lies in the first split, window or not
    span = min(bound, window + DECODE_SPLIT_KEYS) if window else bound
    return max(1, -(-span // DECODE_SPLIT_KEYS) + (1 if window else 0))


def mfma_attention_supported(head_dim: int, page_size: int) -> bool:
    return bool(kernels().pa_attn_mfma_supports(int(head_dim), int(page_size)))


def attention_decode(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out, max_context: int,
                     window: int, scale: float, every_seq: bool = False, softcap: float = 0.0,
                     sink: Optional[torch.Tensor] = None) -> None:
    """Matrix-core attention for the sequences ``seq_ids`` (each feeding one token); writes their rows of ``out``.
    ``every_seq``: ``seq_ids`` is 0, 1, .. (a step of single tokens only); the kernels then count for themselves
    instead of reading it, which is one trip to memory less before their first key."""
    _dev(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out)
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1], hd, torch.bfloat16, "attention_decode")
    n = seq_ids.shape[0]
    if n == 0:
        return
    max_splits = _decode_splits(max_context, window, k_cache.shape[2])
    words = kernels().pa_attn_decode_workspace(n, nh, hd, max_splits)
    ws = torch.empty((max(words, 1),), dtype=torch.float32, device=q.device)
    if sink is not None:
        _check_sinks(sink, nh)
        check(kernels().pa_attn_decode_sink(_stream(), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                            block_table.shape[1], None if every_seq else _ptr(seq_ids), _ptr(cu_q),
                                            _ptr(context_lens), _ptr(out), _ptr(ws), n, nh, k_cache.shape[1], hd,
                                            k_cache.shape[2], int(window), float(scale), float(softcap), _ptr(sink),
                                            DECODE_SPLIT_KEYS, max_splits))
        return
    check(kernels().pa_attn_decode(_stream(), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                   block_table.shape[1], None if every_seq else _ptr(seq_ids), _ptr(cu_q),
                                   _ptr(context_lens), _ptr(out),
                                   _ptr(ws), n, nh, k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale),
                                   float(softcap), DECODE_SPLIT_KEYS, max_splits))


def _check_sinks(sink: torch.Tensor, heads: int) -> None:
    _dev(sink)
    _f32(sink, "sinks")
    if tuple(sink.shape) != (heads,):
        raise NativeError(f"attention: sinks {tuple(sink.shape)} for {heads} heads")


def attention_decode_fused_supported(nh: int, nkv: int, hd: int, rot: int, page_size: int) -> bool:
    return bool(kernels().pa_attn_decode_fused_supports(int(nh), int(nkv), int(hd), int(rot), int(page_size)))


def attention_decode_fused(qkv, q_weight, k_weight, cos, sin, slots, eps: float, k_cache, v_cache,
                           block_table, seq_ids, cu_q, context_lens, nh: int, max_context: int, window: int,
                           scale: float, every_seq: bool = False, softcap: float = 0.0) -> torch.Tensor:
    """``qknorm_rope_kv`` and ``attention_decode`` in one kernel, for a step in which every sequence feeds one
    token: takes the merged projection [T, (nh + 2 nkv) * hd], writes the tokens' keys and values into the caches
    and returns the attention output [T, nh, hd].  A token's position is its sequence's context length less one.
    ``every_seq``: as in ``attention_decode``."""
    _dev(qkv, q_weight, k_weight, cos, sin, slots, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens)
    nkv, page, hd = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    _check_caches(k_cache, v_cache, nkv, hd, torch.bfloat16, "attention_decode_fused")
    t = qkv.shape[0]
    if qkv.dtype != torch.bfloat16 or qkv.dim() != 2 or qkv.shape[1] != (nh + 2 * nkv) * hd or not qkv.is_contiguous():
        raise NativeError(f"attention_decode_fused: qkv {tuple(qkv.shape)} {qkv.dtype} for nh={nh} nkv={nkv} hd={hd}")
    _f32(q_weight, "q_weight")
    _f32(k_weight, "k_weight")
    _f32(cos, "cos")
    _f32(sin, "sin")
    _i32(slots, "slots")
    if cos.shape[1] != hd // 2 or sin.shape != cos.shape or slots.shape[0] != t:
        raise NativeError("attention_decode_fused: rotary tables or slots do not match the tokens")
    out = torch.empty((t, nh, hd), dtype=torch.bfloat16, device=qkv.device)
    n = seq_ids.shape[0]
    if n == 0:
        return out
    max_splits = _decode_splits(max_context, window, page)
    words = kernels().pa_attn_decode_workspace(n, nh, hd, max_splits)
    ws = torch.empty((max(words, 1),), dtype=torch.float32, device=qkv.device)
    check(kernels().pa_attn_decode_fused(_stream(), _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin),
                                         _ptr(slots), float(eps), _ptr(k_cache), _ptr(v_cache),
                                         _ptr(block_table), block_table.shape[1],
                                         None if every_seq else _ptr(seq_ids), _ptr(cu_q),
                                         _ptr(context_lens), _ptr(out), _ptr(ws), n, nh, nkv, hd, page, int(window),
                                         float(scale), float(softcap), DECODE_SPLIT_KEYS, max_splits))
    return out


def attention_prefill(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out, max_q_len: int,
                      window: int, scale: float, cut=None, min_prefix: int = 0, softcap: float = 0.0,
                      sink: Optional[torch.Tensor] = None) -> None:
    """Matrix-core attention for the sequences ``seq_ids`` (portions of several tokens); writes their rows of ``out``.

    ``min_prefix`` is the fewest keys any of the sequences has before its portion: a hint for how the launcher
    cuts the work (portions far into their contexts need no pairing of early and late tiles).
    ``cut`` (tests and measurements) fixes the cut instead: ``(paired, heads a wavefront, head groups a
    workgroup, staged)``, -1 for the launcher's choice."""
    _dev(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out)
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1], hd, torch.bfloat16, "attention_prefill")
    n = seq_ids.shape[0]
    if n == 0:
        return
    args = (_stream(), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(seq_ids),
            _ptr(cu_q), _ptr(context_lens), _ptr(out), n, int(max_q_len), int(min_prefix), nh, k_cache.shape[1], hd,
            k_cache.shape[2], int(window), float(scale), float(softcap))
    if sink is not None:
        if cut is not None:
            raise NativeError("attention_prefill: a given cut and a sink do not go together")
        _check_sinks(sink, nh)
        check(kernels().pa_attn_prefill_sink(*args, _ptr(sink)))
    elif cut is None:
        check(kernels().pa_attn_prefill(*args))
    else:
        check(kernels().pa_attn_prefill_cut(*args, *(int(c) for c in cut)))


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, step, window: int,
              scale: float, softcap: float = 0.0, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of one step over one cache group; picks the kernel for the sizes at hand.

    ``group`` is the step's ``GroupStep`` of the cache group, ``step`` the ``StepBatch``.
    bfloat16 with a head_dim and page size the matrix-core kernels take: single
    tokens go to the split decode kernel, portions to the prefill kernel.
    Everything else (float32, other sizes) goes to the generic kernel.
    """
    if q.dtype == torch.bfloat16 and step.decode_seqs is not None \
            and mfma_attention_supported(q.shape[2], k_cache.shape[2]):
        out = torch.empty_like(q)
        if step.n_decode:
            attention_decode(q, k_cache, v_cache, group.block_table, step.decode_seqs, step.cu_q, step.context_lens,
                             out, step.max_decode_context, window, scale,
                             every_seq=step.n_prefill == 0 and step.n_decode == step.num_seqs, softcap=softcap, sink=sink)
        if step.n_prefill:
            attention_prefill(q, k_cache, v_cache, group.block_table, step.prefill_seqs, step.cu_q, step.context_lens,
                              out, step.max_prefill_q, window, scale, min_prefix=step.min_prefill_prefix, softcap=softcap,
                              sink=sink)
        return out
    return attention_generic(q, k_cache, v_cache, group.block_table, step.seq_of_token, step.positions, window, scale,
                             softcap, sink)


def logprobs(logits: torch.Tensor, ids: torch.Tensor, k: int = 0):
    """Log-probabilities under softmax(logits[r]) of the tokens ``ids`` [R] (int32; negative = none, gives 0).

    Returns ``(lp [R] float32, top)``; with ``k`` > 0, ``top`` is ``(values [R, cap], indices [R, cap], count [R])``:
    the entries among each row's k largest with their log-probabilities, ties at the k-th value included, in no
    particular order (the caller sorts the few there are); else ``None``.
    """
    _dev(logits, ids)
    _f32(logits, "logits")
    _i32(ids, "ids")
    if logits.dim() != 2 or ids.shape != (logits.shape[0],):
        raise NativeError(f"logprobs: logits {tuple(logits.shape)} / ids {tuple(ids.shape)}")
    r, vocab = logits.shape
    k = int(k)
    lp = torch.empty(r, dtype=torch.float32, device=logits.device)
    top = None
    cap = 0
    if k > 0:
        cap = min(vocab, k + 32)
        top = (torch.empty((r, cap), dtype=torch.float32, device=logits.device),
               torch.empty((r, cap), dtype=torch.int32, device=logits.device),
               torch.empty(r, dtype=torch.int32, device=logits.device))
    check(kernels().pa_logprobs(_stream(), _ptr(logits), _ptr(ids), _ptr(lp), _ptr(top[0]) if top else None,
                                _ptr(top[1]) if top else None, _ptr(top[2]) if top else None, r, vocab, k, cap))
    return lp, top


SAMPLE_WIDE_FROM = 32768   # rows this long are sampled with every pass spread over the chip,
SAMPLE_WIDE_ROWS = 32      # up to this many at a time (more rows fill the chip with a workgroup each)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, any_top_k: bool = True, any_top_p: bool = True,
           wide: Optional[bool] = None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; per-row float32 temperature / top_p / uniform and int32 top_k.

    temperature < 1e-7: argmax.  Else a draw from softmax(logits / T) kept to the
    top_k largest (0 = all) and the shortest descending prefix of mass top_p
    (>= 1 = all), by inverse CDF in index order at uniform[r] in [0, 1).

    ``any_top_k`` / ``any_top_p`` false promise that no row has one, which spares long rows the passes of
    that search.  ``wide`` picks the kernel (one workgroup a row, or rows cut into slices over many
    workgroups); by default it follows the row length.  Both give the same token except where 32-bit
    rounding of the sums decides between neighbours.
    """
    _dev(logits, temperature, top_k, top_p, uniform)
    _f32(logits, "logits")
    _f32(temperature, "temperature")
    _f32(top_p, "top_p")
    _f32(uniform, "uniform")
    _i32(top_k, "top_k")
    r = logits.shape[0]
    if logits.dim() != 2 or any(t.shape != (r,) for t in (temperature, top_k, top_p, uniform)):
        raise NativeError("sample: per-row parameters do not match the rows of logits")
    out = torch.empty((r,), dtype=torch.int32, device=logits.device)
    vocab = logits.shape[1]
    if wide is None:
        wide = vocab >= SAMPLE_WIDE_FROM and r <= SAMPLE_WIDE_ROWS
    if wide and r > 0:
        ws = torch.empty(int(kernels().pa_sample_wide_workspace(r, vocab)), dtype=torch.uint8, device=logits.device)
        check(kernels().pa_sample_wide(_stream(), _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                       _ptr(uniform), _ptr(out), _ptr(ws), r, vocab,
                                       (1 if any_top_k else 0) | (2 if any_top_p else 0)))
        return out
    check(kernels().pa_sample(_stream(), _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
                              _ptr(out), r, vocab))
    return out


# ---------------------------------------------------------------------------
# A residual stream kept in 32-bit
def rmsnorm_wide(x, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
                 rows: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``rmsnorm`` for a float32 residual [T, H] beside x [T, H] of the engine's type (or a ``SliceSums``): the sum
    is taken and kept in 32-bit (the residual receives it unrounded, unless ``rows``), the output is of x's type."""
    parts = x.parts if isinstance(x, SliceSums) else None
    xt = None if parts is not None else x
    _dev(xt, parts, weight, residual, rows)
    _f32(weight, "norm weight")
    _f32(residual, "residual")
    if x is None:
        # nothing waits to be added: the norm of the stream's wanted rows alone, in ``out_dtype``
        if residual is None or rows is None or out_dtype is None:
            raise NativeError("rmsnorm_wide: without x it norms rows of the residual and needs residual, rows and out_dtype")
        _i32(rows, "rows")
        out = torch.empty((rows.shape[0], residual.shape[1]), dtype=out_dtype, device=weight.device)
        check(kernels().pa_rmsnorm_wide(_stream(), _CODES[out_dtype], None, None, 0, 0, _ptr(residual), _ptr(weight), _ptr(out),
                                        _ptr(rows), rows.shape[0], residual.shape[1], float(eps)))
        return out
    m, h = x.shape
    if weight.shape != (h,) or (residual is not None and tuple(residual.shape) != (m, h)):
        raise NativeError(f"rmsnorm_wide: x {tuple(x.shape)} / weight {tuple(weight.shape)} / residual "
                          f"{None if residual is None else tuple(residual.shape)}")
    n = m
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    out = torch.empty((n, h), dtype=x.dtype, device=weight.device)
    check(kernels().pa_rmsnorm_wide(_stream(), _CODES[x.dtype], _ptr(xt), _ptr(parts),
                                    0 if parts is None else parts.shape[0], m * h, _ptr(residual), _ptr(weight), _ptr(out),
                                    _ptr(rows), n, h, float(eps)))
    return out


def rmsnorm_branch(y, weight: torch.Tensor, eps: float, residual: torch.Tensor,
                   copy_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """residual += y / sqrt(mean(y^2) + eps) * weight, in 32-bit and in place: a branch's output normed and added to
    the stream.  y [T, H] of the engine's type or a ``SliceSums``; residual float32 [T, H].  Returns the new residual
    rounded to ``copy_dtype`` (what the next branch multiplies with), or None when that is float32 itself."""
    parts = y.parts if isinstance(y, SliceSums) else None
    yt = None if parts is not None else y
    _dev(yt, parts, weight, residual)
    _f32(weight, "norm weight")
    _f32(residual, "residual")
    m, h = y.shape
    if weight.shape != (h,) or tuple(residual.shape) != (m, h):
        raise NativeError(f"rmsnorm_branch: y {tuple(y.shape)} / weight {tuple(weight.shape)} / residual {tuple(residual.shape)}")
    copy = None
    if copy_dtype is not None and copy_dtype != torch.float32:
        if copy_dtype != y.dtype:
            raise NativeError(f"rmsnorm_branch: a copy of {copy_dtype} beside a branch of {y.dtype}")
        copy = torch.empty((m, h), dtype=copy_dtype, device=residual.device)
    check(kernels().pa_rmsnorm_branch(_stream(), _CODES[y.dtype], _ptr(yt), _ptr(parts), 0 if parts is None else parts.shape[0],
                                      m * h, _ptr(residual), _ptr(weight), _ptr(copy), m, h, float(eps)))
    return copy


def gated_rmsnorm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """out = o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate) over rows; o float32 [T, N]; gate [T, N] of the engine's
    type, a view whose rows may lie inside a wider tensor (columns contiguous); the output is of the gate's type."""
    _dev(o, weight)
    _f32(o, "gated_rmsnorm input")
    _f32(weight, "norm weight")
    if not gate.is_cuda or gate.dim() != 2 or gate.stride(1) != 1 or o.dim() != 2 or gate.shape != o.shape \
            or weight.shape != (o.shape[1],):
        raise NativeError(f"gated_rmsnorm: o {tuple(o.shape)} / gate {tuple(gate.shape)} strides {gate.stride()} / weight "
                          f"{tuple(weight.shape)}")
    out = torch.empty(o.shape, dtype=gate.dtype, device=o.device)
    check(kernels().pa_gated_rmsnorm(_stream(), _code(gate), _ptr(o), gate.data_ptr(), gate.stride(0), _ptr(weight), _ptr(out),
                                     o.shape[0], o.shape[1], float(eps)))
    return out


LIGHTNING_ACTIVATIONS = {None: 0, "none": 0, "silu": 1}


LIGHTNING_CHUNK = 64       # tokens a chunk of the chunked form; portions of more tokens go to it (bfloat16 engine)


def lightning_attention(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, decay: torch.Tensor, state: torch.Tensor,
                        step, heads: int, dim: int, vdim: int, activation: Optional[str] = "silu",
                        chunk: Optional[int] = None) -> torch.Tensor:
    """Linear attention with a decaying state: per head S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.

    qkv [T, width]: a token's queries [heads, dim], keys [heads, dim] and values [heads, vdim] start at columns
    ``q_off``, ``k_off``, ``v_off`` and pass through ``activation``; decay float32 [heads]; state float32
    [slots, heads, dim, vdim], read and left by the step's sequences through ``step.state_slots``.  Returns
    float32 [T, heads, vdim].

    ``chunk``: portions of more tokens are cut into chunks of that many that run side by side (three passes; the
    sums are the same up to rounding, in another order); 0: every sequence token by token, whose sums do not depend
    on how a prompt was cut.  None: ``LIGHTNING_CHUNK`` for a bfloat16 engine, 0 for a 32-bit one."""
    _dev(qkv, decay, state)
    _f32(decay, "decays")
    _f32(state, "state")
    t = qkv.shape[0]
    if qkv.dim() != 2 or tuple(decay.shape) != (heads,) or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim) \
            or max(q_off, k_off) + heads * dim > qkv.shape[1] or v_off + heads * vdim > qkv.shape[1]:
        raise NativeError(f"lightning_attention: qkv {tuple(qkv.shape)} / decay {tuple(decay.shape)} / state {tuple(state.shape)} "
                          f"for {heads} heads of {dim} and {vdim}")
    if activation not in LIGHTNING_ACTIVATIONS:
        raise NativeError(f"lightning_attention: activation {activation!r} is not one of {sorted(map(str, LIGHTNING_ACTIVATIONS))}")
    if chunk is None:
        chunk = LIGHTNING_CHUNK if qkv.dtype == torch.bfloat16 else 0
    chunked = chunk > 0 and step.n_prefill > 0 and step.max_prefill_q > chunk
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qkv.device)
    args = (_code(qkv), _ptr(qkv), qkv.shape[1], int(q_off), int(k_off), int(v_off), _ptr(decay), _ptr(state),
            _ptr(step.state_slots), _ptr(step.cu_q))
    act = LIGHTNING_ACTIVATIONS[activation]
    # single tokens (decode) have a small kernel of their own; the portions go to the general one
    singles = getattr(step, "n_decode", 0) > 0
    if singles:
        check(kernels().pa_lightning_step(_stream(), *args, _ptr(out), step.num_seqs, heads, dim, vdim, act))
    if step.n_prefill > 0 or not singles:
        check(kernels().pa_lightning_attn(_stream(), *args, _ptr(out), step.num_seqs, t, heads, dim, vdim, act,
                                          int(chunk) if chunked else 0, 2 if singles else 0))
    if chunked:
        words = kernels().pa_lightning_attn_workspace(step.n_prefill, t, heads, dim, vdim, int(chunk))
        work = torch.empty((max(words, 1),), dtype=torch.float32, device=qkv.device)
        check(kernels().pa_lightning_attn_chunked(_stream(), *args, _ptr(step.prefill_seqs), _ptr(out), _ptr(work),
                                                  step.n_prefill, t, int(step.max_prefill_q), heads, dim, vdim, act, int(chunk)))
    return out


def clamped_gate(gate_up: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """gate_up [T, 2I] with columns alternating gate_j, up_j -> [T, I]: g = min(g, limit), u = clamp(u, -limit, limit),
    g * sigmoid(alpha * g) * (u + 1), in 32-bit."""
    _dev(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise NativeError(f"clamped_gate: input {tuple(gate_up.shape)} is not [T, 2I]")
    inter = gate_up.shape[1] // 2
    out = torch.empty((gate_up.shape[0], inter), dtype=gate_up.dtype, device=gate_up.device)
    check(kernels().pa_clamped_gate(_stream(), _code(gate_up), _ptr(gate_up), _ptr(out), gate_up.shape[0], inter,
                                    float(limit), float(alpha)))
    return out


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    _dev(x)
    out = torch.empty_like(x)
    check(kernels().pa_relu_squared(_stream(), _code(x), _ptr(x), _ptr(out), x.numel()))
    return out


# ---------------------------------------------------------------------------
# Attention through a latent
def latent_prep(down: torch.Tensor, q_weight: torch.Tensor, c_weight: torch.Tensor, inv_freq: Optional[torch.Tensor],
                positions: torch.Tensor, slots: Optional[torch.Tensor], cache: Optional[torch.Tensor], q_rank: int,
                rank: int, rot: int, rot_dims: int, eps: float, cache_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The merged down projection [T, q_rank + rank + rot]: returns the normed query latent [T, q_rank]; writes the
    normed latent and the rotated shared key part of every token into ``cache`` [pages, page, rank + rot] at ``slots``,
    and the latent once more into ``cache_t`` [pages, rank, page] where the cache keeps that copy."""
    _dev(q_weight, c_weight, inv_freq, positions, slots, cache, cache_t)   # ``down`` may be rows of a wider tensor
    if not down.is_cuda:
        raise NativeError("latent_prep: the projection is not on the device")
    _f32(q_weight, "query latent norm weight")
    _f32(c_weight, "latent norm weight")
    _f32(inv_freq, "rotary frequencies")
    _i32(positions, "positions")
    t = down.shape[0]
    if down.dim() != 2 or down.shape[1] != q_rank + rank + rot or down.stride(1) != 1 or q_weight.shape != (q_rank,) or \
            c_weight.shape != (rank,):
        raise NativeError(f"latent_prep: input {tuple(down.shape)} for parts {q_rank} + {rank} + {rot}")
    if positions.shape != (t,) or (rot_dims and (inv_freq is None or inv_freq.shape != (rot_dims // 2,))):
        raise NativeError("latent_prep: positions or rotary frequencies do not match")
    if slots is not None:
        _i32(slots, "slots")
        if slots.shape != (t,) or cache is None or cache.dim() != 3 or cache.shape[2] != rank + rot or cache.dtype != down.dtype:
            raise NativeError(f"latent_prep: cache must be [pages, page, {rank + rot}] of {down.dtype}")
        if cache_t is not None and (cache_t.dtype != cache.dtype or tuple(cache_t.shape) != (cache.shape[0], rank, cache.shape[1])):
            raise NativeError(f"latent_prep: the transposed copy must be [pages, {rank}, page] of {cache.dtype}")
    cq = torch.empty((t, q_rank), dtype=down.dtype, device=down.device)
    caching = slots is not None
    check(kernels().pa_latent_prep(_stream(), _code(down), down.data_ptr(), _ptr(q_weight), _ptr(c_weight), _ptr(inv_freq),
                                   _ptr(positions), _ptr(slots), _ptr(cq), _ptr(cache) if caching else None,
                                   _ptr(cache_t) if caching else None, cache.shape[1] if caching else 0, t,
                                   q_rank, rank, rot, rot_dims, float(eps), down.stride(0)))
    return cq


def rotate_pairs(x: torch.Tensor, out: torch.Tensor, inv_freq: Optional[torch.Tensor], positions: torch.Tensor, in_off: int,
                 out_off: int, width: int, rot_dims: int) -> None:
    """x [T, heads, a] -> out [T, heads, b]: ``width`` elements from ``in_off`` of every head to ``out_off``, the first
    ``rot_dims`` of them rotated in pairs (2i, 2i+1) by position * inv_freq[i]."""
    _dev(x, out, inv_freq, positions)
    _f32(inv_freq, "rotary frequencies")
    _i32(positions, "positions")
    if x.dim() != 3 or out.dim() != 3 or x.shape[:2] != out.shape[:2] or x.dtype != out.dtype or positions.shape != (x.shape[0],):
        raise NativeError(f"rotate_pairs: x {tuple(x.shape)} / out {tuple(out.shape)}")
    if rot_dims and (inv_freq is None or inv_freq.shape != (rot_dims // 2,)):
        raise NativeError("rotate_pairs: rotary frequencies do not match the rotated width")
    check(kernels().pa_rotate_pairs(_stream(), _code(x), _ptr(x), _ptr(out), _ptr(inv_freq), _ptr(positions), x.shape[0],
                                    x.shape[1], x.shape[2], int(in_off), out.shape[2], int(out_off), int(width), int(rot_dims)))


class GroupedWeight:
    """A weight per group (expert, head), [groups, out, in], as the grouped products read it: for bfloat16 with rows
    of whole 16-byte pieces as it stands (``nk``: the matrix cores take it so), else transposed to [groups, in, out]
    (``kn``: the vector-ALU product reads its column beside its neighbours')."""

    def __init__(self, w: torch.Tensor):
        if w.dim() != 3:
            raise NativeError(f"grouped weight {tuple(w.shape)} is not [groups, out, in]")
        self.groups, self.n, self.k = (int(d) for d in w.shape)
        self.dtype, self.device = w.dtype, w.device
        self.nk = self.kn = None
        if w.dtype == torch.bfloat16 and self.k % 8 == 0:
            self.nk = w.contiguous()
        else:
            self.kn = w.transpose(1, 2).contiguous()


def head_linear(x: torch.Tensor, w: GroupedWeight, out: torch.Tensor, x_off: int = 0, out_off: int = 0) -> None:
    """out[t, h, out_off : out_off + n] = W[h] x[t, h, x_off : x_off + k] for x [T, heads, a], out [T, heads, b] and a
    weight per head ``w`` [heads, n, k]."""
    k, n = w.k, w.n
    wt = w.nk if w.nk is not None else w.kn
    _dev(x, wt, out)
    if (x.dim() != 3 or out.dim() != 3 or x.shape[:2] != out.shape[:2] or w.groups != x.shape[1]
            or not (x.dtype == w.dtype == out.dtype) or x_off + k > x.shape[2] or out_off + n > out.shape[2]):
        raise NativeError(f"head_linear: x {tuple(x.shape)} / w [{w.groups}, {n}, {k}] / out {tuple(out.shape)}")
    el = x.element_size()
    strides = (x.shape[1] * x.shape[2], x.shape[2], out.shape[1] * out.shape[2], out.shape[2])
    if w.nk is not None and x.shape[2] % 8 == 0 and x_off % 8 == 0:
        check(kernels().pa_head_linear_mfma(_stream(), x.data_ptr() + x_off * el, _ptr(wt), out.data_ptr() + out_off * el,
                                            x.shape[0], x.shape[1], k, n, *strides))
        return
    if w.kn is None:
        w.kn = w.nk.transpose(1, 2).contiguous()     # rows of x that are no whole 16-byte pieces: the other product, once
    check(kernels().pa_head_linear(_stream(), _code(x), x.data_ptr() + x_off * el, _ptr(w.kn), out.data_ptr() + out_off * el,
                                   x.shape[0], x.shape[1], k, n, *strides))


def latent_gather(cache: torch.Tensor, block_table: torch.Tensor, seq: torch.Tensor, pos: torch.Tensor, rank: int) -> torch.Tensor:
    """The latents of the cached positions (seq[i], pos[i]) back out of their pages, [N, rank]: the first ``rank``
    elements of each cached vector (``cache`` [pages, page, width])."""
    _dev(cache, block_table, seq, pos)
    _i32(block_table, "block_table")
    _i32(seq, "sequences")
    _i32(pos, "positions")
    if cache.dim() != 3 or not 0 < rank <= cache.shape[2] or seq.shape != pos.shape or seq.dim() != 1 or block_table.dim() != 2:
        raise NativeError(f"latent_gather: cache {tuple(cache.shape)} / rank {rank} / rows {tuple(seq.shape)}")
    out = torch.empty((seq.shape[0], rank), dtype=cache.dtype, device=cache.device)
    check(kernels().pa_latent_gather(_stream(), _code(cache), _ptr(cache), _ptr(block_table), block_table.shape[1], _ptr(seq), _ptr(pos),
                                     _ptr(out), seq.shape[0], int(rank), cache.shape[2], cache.shape[1]))
    return out


def latent_attention_generic(q: torch.Tensor, cache: torch.Tensor, sink: Optional[torch.Tensor], block_table: torch.Tensor,
                             seq_of_token: torch.Tensor, positions: torch.Tensor, rank: int, window: int,
                             scale: float) -> torch.Tensor:
    """Causal attention of q [T, heads, rank + rot] over cached latents [pages, page, rank + rot] (the value of a key
    is its first ``rank`` elements), with ``sink`` [heads] joining each head's softmax denominator as exp(sink_h);
    returns [T, heads, rank].  32-bit arithmetic; any mix of portions and single tokens."""
    _dev(q, cache, sink, block_table, seq_of_token, positions)
    _f32(sink, "sink")
    _i32(block_table, "block_table")
    _i32(seq_of_token, "seq_of_token")
    _i32(positions, "positions")
    t, nh, dk = q.shape
    if cache.dim() != 3 or cache.shape[2] != dk or cache.dtype != q.dtype or not 0 < rank <= dk:
        raise NativeError(f"latent_attention: q {tuple(q.shape)} / cache {tuple(cache.shape)} / rank {rank}")
    if seq_of_token.shape != (t,) or positions.shape != (t,) or block_table.dim() != 2 or (sink is not None and sink.shape != (nh,)):
        raise NativeError("latent_attention: index arrays or sinks do not match")
    out = torch.empty((t, nh, rank), dtype=q.dtype, device=q.device)
    check(kernels().pa_latent_attn(_stream(), _code(q), _ptr(q), _ptr(cache), _ptr(sink), _ptr(block_table),
                                   block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out), t, nh, int(rank),
                                   dk - int(rank), cache.shape[1], int(window), float(scale)))
    return out


# ---------------------------------------------------------------------------
# Experts
class ExpertOrder:
    """A step's (token, choice) entries put in the order of their experts: ``offsets`` [E + 1], ``order`` [entries]
    (position -> entry), ``place`` [entries] (entry -> position), all int32 on the device."""

    def __init__(self, offsets, order, place, entries: int, experts: int, top: int):
        self.offsets, self.order, self.place = offsets, order, place
        self.entries, self.experts, self.top = entries, experts, top


def moe_choices_by_table(token_ids: torch.Tensor, table: torch.Tensor, experts: int) -> torch.Tensor:
    """choice[t * top + j] = table[token_ids[t], j]: experts by token id, no router."""
    _dev(token_ids, table)
    _i32(token_ids, "token ids")
    _i32(table, "expert table")
    if token_ids.dim() != 1 or table.dim() != 2:
        raise NativeError(f"moe_choices_by_table: ids {tuple(token_ids.shape)} / table {tuple(table.shape)}")
    t, top = token_ids.shape[0], table.shape[1]
    choice = torch.empty(t * top, dtype=torch.int32, device=table.device)
    check(kernels().pa_moe_choices_by_table(_stream(), _ptr(token_ids), _ptr(table), _ptr(choice), t, top, table.shape[0],
                                            int(experts)))
    return choice


NARROW_MAX_COLUMNS = 256
NARROW_FEW_ROWS = 64     # up to here (all it takes) the weight-streaming product, 32-bit result from its own sums: it puts
#                          the whole chip on the weight where the kernel for narrow outputs has a workgroup per 16 rows


def linear_narrow_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x W^T for a weight of few rows with a 32-bit result from 32-bit sums, whatever the number of rows of x: a
    router's scores (the library's product would round them to bfloat16).  float32: the plain product.  bfloat16:
    few rows the weight-streaming kernel, more the matrix-core kernel for narrow outputs; sizes neither takes
    (rows of no whole 16-byte pieces, more than ``NARROW_MAX_COLUMNS`` columns) go to the plain product too."""
    _dev(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.dtype != w.dtype:
        raise NativeError(f"linear_narrow_f32: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    if x.dtype != torch.bfloat16 or k % 8 or n > NARROW_MAX_COLUMNS:
        return gemm_plain(x, w, None, torch.float32)
    if m <= NARROW_FEW_ROWS:
        return gemm_skinny(x, w, None, torch.float32)
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    check(kernels().pa_gemm_narrow(_stream(), _ptr(x), _ptr(w), _ptr(out), m, n, k, k, n))
    return out


def moe_route(logits: torch.Tensor, experts: int, top: int, scale: float, correction: Optional[torch.Tensor] = None,
              gate_col: int = -1, bias: Optional[torch.Tensor] = None, by_logit: bool = False):
    """A router's choices: logits float32 [T, >= experts]; s = softmax over the first ``experts`` columns; the ``top``
    experts with the largest s + correction are chosen and weighted s / (sum of the chosen s + 1e-20) * scale.
    Returns (choice int32 [T * top], weights float32 [T * top], gate float32 [T] or None): the gate is the sigmoid of
    column ``gate_col`` of the same rows, for a shared expert.  ``bias`` (float32 [experts]) is added to the logits
    first.  ``by_logit``: the choice goes by the logits themselves (no correction) and the weights are the softmax over
    the chosen logits alone, times scale."""
    _dev(logits, correction, bias)
    _f32(bias, "router bias")
    if bias is not None and tuple(bias.shape) != (experts,):
        raise NativeError(f"moe_route: bias {tuple(bias.shape)} for {experts} experts")
    if by_logit and correction is not None:
        raise NativeError("moe_route: a choice by the logits takes no correction")
    _f32(logits, "router logits")
    _f32(correction, "router correction")
    if logits.dim() != 2 or logits.shape[1] < experts or (correction is not None and tuple(correction.shape) != (experts,)):
        raise NativeError(f"moe_route: logits {tuple(logits.shape)} for {experts} experts")
    t = logits.shape[0]
    choice = torch.empty(t * top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(t * top, dtype=torch.float32, device=logits.device)
    gate = torch.empty(t, dtype=torch.float32, device=logits.device) if gate_col >= 0 else None
    check(kernels().pa_moe_route(_stream(), _ptr(logits), logits.shape[1], _ptr(correction), _ptr(choice), _ptr(weights),
                                 _ptr(gate), t, int(experts), int(top), float(scale), int(gate_col), _ptr(bias),
                                 1 if by_logit else 0))
    return choice, weights, gate


def moe_order(choice: torch.Tensor, experts: int, top: int) -> ExpertOrder:
    _dev(choice)
    _i32(choice, "choices")
    n = choice.shape[0]
    ints = torch.empty(2 * experts + 1 + 2 * n, dtype=torch.int32, device=choice.device)
    counts, offsets = ints[:experts], ints[experts: 2 * experts + 1]
    order, place = ints[2 * experts + 1: 2 * experts + 1 + n], ints[2 * experts + 1 + n:]
    check(kernels().pa_moe_order(_stream(), _ptr(choice), n, int(experts), _ptr(counts), _ptr(offsets), _ptr(order), _ptr(place)))
    return ExpertOrder(offsets, order, place, n, int(experts), int(top))


def moe_linear(x: torch.Tensor, w: GroupedWeight, eo: ExpertOrder, from_tokens: bool, relu_squared_epilogue: bool = False,
               out_dtype: Optional[torch.dtype] = None, clamped_gate_epilogue: Optional[tuple] = None,
               silu_gate_epilogue: bool = False) -> torch.Tensor:
    """y[p] = act(W[expert of p] x[row of p]) over the ordered positions p; ``w`` [experts, n, k];
    ``from_tokens``: x holds a row per token (position p reads its token's), else a row per position.
    ``clamped_gate_epilogue`` = (limit, alpha): the weights' rows alternate gate_j, up_j and the result is the
    clamped gated pair of ``clamped_gate``, [entries, n / 2] (in the matrix-core product's epilogue; a kernel of
    its own behind the other product).  ``silu_gate_epilogue``: the same rows, the plain gated pair
    silu(gate_j) * up_j."""
    wt = w.nk if w.nk is not None else w.kn
    _dev(x, wt)
    k, n = w.k, w.n
    rows = eo.entries // eo.top if from_tokens else eo.entries
    if x.dim() != 2 or tuple(x.shape) != (rows, k) or w.groups != eo.experts or x.dtype != w.dtype:
        raise NativeError(f"moe_linear: x {tuple(x.shape)} {x.dtype} / w [{w.groups}, {n}, {k}] {w.dtype} for {eo.entries} entries")
    gated = clamped_gate_epilogue is not None or silu_gate_epilogue
    if gated and (relu_squared_epilogue or n % 2 or (clamped_gate_epilogue is not None and silu_gate_epilogue)):
        raise NativeError(f"moe_linear: gated pairs over {n} outputs, or two activations at once")
    out_dtype = out_dtype or x.dtype
    fused = gated and w.nk is not None
    y = torch.empty((eo.entries, n // 2 if fused else n), dtype=out_dtype, device=x.device)
    act = (3 if silu_gate_epilogue else 2) if fused else (1 if relu_squared_epilogue else 0)
    args = (_ptr(x), _ptr(wt), _ptr(y), _ptr(eo.offsets), _ptr(eo.order), eo.entries, eo.experts, eo.top, k, n,
            1 if from_tokens else 0, act)
    if w.nk is not None:
        limit, alpha = clamped_gate_epilogue if (fused and clamped_gate_epilogue is not None) else (0.0, 0.0)
        check(kernels().pa_moe_linear_mfma(_stream(), _CODES[out_dtype], *args, float(limit), float(alpha)))
        return y
    check(kernels().pa_moe_linear(_stream(), _code(x), _code(wt), _CODES[out_dtype], *args))
    if clamped_gate_epilogue is not None:
        return clamped_gate(y, *clamped_gate_epilogue)
    if silu_gate_epilogue:
        return silu_mul(y)
    return y


def moe_combine(y: torch.Tensor, eo: ExpertOrder, weight: float, base: Optional[torch.Tensor], out_dtype: torch.dtype,
                weights: Optional[torch.Tensor] = None, base_scale: Optional[torch.Tensor] = None,
                into: Optional[torch.Tensor] = None, other: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """out[t] = b[t] * base[t] + sum_j w * y[place[t * top + j]] in ascending j; y float32 [entries, H]; ``weights``
    float32 [entries] per entry, else ``weight`` for all; ``base_scale`` float32 [T] gives b, else 1.  With ``into`` (a
    32-bit stream [T, H]) the sum is not rounded and written but added in place, ``into[t] += other[t] + sum`` (``other``
    of ``out_dtype`` or None: another branch's output, added to this one first), and nothing is returned."""
    _dev(y, base, weights, base_scale, into, other)
    _f32(into, "stream")
    _f32(y, "expert outputs")
    _f32(weights, "entry weights")
    _f32(base_scale, "base scale")
    t = eo.entries // eo.top
    h = y.shape[1]
    if y.shape[0] != eo.entries or (base is not None and (tuple(base.shape) != (t, h) or base.dtype != out_dtype)):
        raise NativeError(f"moe_combine: y {tuple(y.shape)} / base {None if base is None else tuple(base.shape)}")
    if into is not None:
        if tuple(into.shape) != (t, h) or (other is not None and (tuple(other.shape) != (t, h) or other.dtype != out_dtype)):
            raise NativeError(f"moe_combine: stream {tuple(into.shape)} / other {None if other is None else tuple(other.shape)}")
    elif other is not None:
        raise NativeError("moe_combine: another branch's output goes with a stream to add to")
    out = torch.empty((t, h), dtype=out_dtype, device=y.device) if into is None else None
    check(kernels().pa_moe_combine(_stream(), _CODES[out_dtype], _ptr(y), _ptr(eo.place), _ptr(weights), float(weight), _ptr(base),
                                   _ptr(base_scale), _ptr(out), t, eo.top, h, _ptr(into), _ptr(other)))
    return out


LATENT_MAX_WIDTH = 1024   # rank + rot of a cached latent vector the attention kernels take


# Keys a split, for steps of single tokens.  Two kernels take them.  Few sequences (fewer than LATENT_WAVE_SPLITS_FROM
# tiles of 16 heads): a split is a workgroup of the staged kernel, whose loads of a block all go out at once (8
# sequences of 4,096 keys: 41.6 us against 54 the other way).  Many: a split is a wavefront that reads the cache
# directly, four a workgroup (32 sequences: 95 us against 115; 64: 167 against 224; 8 of 32,768 keys: 171 against 234;
# one of 32,768 keys in 1,024 splits of a block each: 130 us, which is why a single sequence stays with the staged kernel).
# Either way a workgroup walks its keys block by block and a compute unit holds one workgroup, so the shortest split
# that still leaves the launch within one round of the chip (LATENT_SPLIT_WORKGROUPS workgroups) is the fastest.
LATENT_SPLIT_KEYS = (64, 128, 256)
LATENT_WAVE_SPLIT_KEYS = (32, 64, 128, 256)
LATENT_SPLIT_WORKGROUPS = 256
LATENT_WAVE_SPLITS_FROM = 24      # ... or where the staged kernel's longest splits no longer fit one round
LATENT_MAX_SPLITS = 4096     # what the merge kernel takes; contexts beyond 4,096 splits of 256 keys get longer splits


def latent_split_plan(n_seqs: int, max_context: int, heads: int = 16):
    """(keys a split, whether a split is a wavefront) for a step of ``n_seqs`` single tokens."""
    head_tiles = -(-int(heads) // 16)
    per_wave = (n_seqs * head_tiles >= LATENT_WAVE_SPLITS_FROM
                or n_seqs * -(-int(max_context) // LATENT_SPLIT_KEYS[-1]) > LATENT_SPLIT_WORKGROUPS)
    for keys in (LATENT_WAVE_SPLIT_KEYS if per_wave else LATENT_SPLIT_KEYS):
        splits = -(-int(max_context) // keys)
        groups = n_seqs * head_tiles * -(-splits // 4) if per_wave else n_seqs * splits
        if splits <= LATENT_MAX_SPLITS and groups <= LATENT_SPLIT_WORKGROUPS:
            return keys, per_wave
    keys = LATENT_SPLIT_KEYS[-1]
    while -(-int(max_context) // keys) > LATENT_MAX_SPLITS:
        keys *= 2
    return keys, per_wave


def latent_split_keys(n_seqs: int, max_context: int, heads: int = 16) -> int:
    return latent_split_plan(n_seqs, max_context, heads)[0]


def latent_attention_mfma_supported(rank: int, rot: int, page_size: int) -> bool:
    return bool(kernels().pa_latent_attn_mfma_supports(int(rank), int(rot), int(page_size)))


def latent_attention_mfma(q: torch.Tensor, cache: torch.Tensor, cache_t: torch.Tensor, sink: Optional[torch.Tensor], block_table: torch.Tensor,
                          seq_ids: Optional[torch.Tensor], n_seqs: int, cu_q: torch.Tensor, context_lens: torch.Tensor,
                          out: torch.Tensor, max_q_len: int, rank: int, window: int, scale: float,
                          max_context: int = 0, per_wave: Optional[bool] = None) -> None:
    """The matrix-core kernel for the sequences ``seq_ids`` (None: all ``n_seqs`` of the step); writes their rows of
    ``out`` [T, heads, rank].  ``max_context`` > 0 with ``max_q_len`` 1 cuts the keys into splits of
    ``latent_split_plan`` keys whose partials a second kernel merges: what fills the chip when every sequence feeds one
    token.  ``per_wave`` (tests and measurements) fixes which of the two kernels takes the splits."""
    _dev(q, cache, cache_t, sink, block_table, seq_ids, cu_q, context_lens, out)
    _f32(sink, "sink")
    t, nh, dk = q.shape
    if cache_t is None or cache_t.dtype != torch.bfloat16 or tuple(cache_t.shape) != (cache.shape[0], rank, cache.shape[1]):
        raise NativeError(f"latent_attention_mfma: the transposed copy must be [pages, {rank}, page] of bfloat16")
    if q.dtype != torch.bfloat16 or cache.dtype != torch.bfloat16 or cache.dim() != 3 or cache.shape[2] != dk \
            or tuple(out.shape) != (t, nh, rank) or out.dtype != torch.bfloat16 or (sink is not None and sink.shape != (nh,)):
        raise NativeError(f"latent_attention_mfma: q {tuple(q.shape)} {q.dtype} / cache {tuple(cache.shape)} / out {tuple(out.shape)}")
    if n_seqs == 0:
        return
    splits, ws = 1, None
    split_keys, planned = latent_split_plan(n_seqs, max_context, nh)
    per_wave = planned if per_wave is None else bool(per_wave)
    if max_q_len == 1 and max_context > split_keys:
        splits = -(-int(max_context) // split_keys)
        ws = torch.empty(int(kernels().pa_latent_attn_mfma_workspace(n_seqs, nh, rank, splits)), dtype=torch.float32, device=q.device)
    check(kernels().pa_latent_attn_mfma(_stream(), _ptr(q), _ptr(cache), _ptr(cache_t), _ptr(sink), _ptr(block_table), block_table.shape[1],
                                        _ptr(seq_ids), _ptr(cu_q), _ptr(context_lens), _ptr(out), _ptr(ws), int(n_seqs),
                                        int(max_q_len), nh, int(rank), dk - int(rank), cache.shape[1], int(window), float(scale),
                                        split_keys, splits, 1 if per_wave else 0))


def latent_attention(q: torch.Tensor, cache: torch.Tensor, sink: Optional[torch.Tensor], group, step, rank: int,
                     window: int, scale: float, cache_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of one step over a cache of latents; picks the kernel for the sizes at hand (``group``: the
    step's ``GroupStep`` of the cache group, ``step``: the ``StepBatch``).  bfloat16 with sizes the matrix-core
    kernel takes: single tokens in splits of their keys, portions a launch of their own; everything else
    (float32, other sizes) the kernel on the vector ALU."""
    if (q.dtype == torch.bfloat16 and cache_t is not None and step.decode_seqs is not None and scale > 0
            and latent_attention_mfma_supported(rank, q.shape[2] - rank, cache.shape[1])):
        out = torch.empty((q.shape[0], q.shape[1], rank), dtype=q.dtype, device=q.device)
        if step.n_decode:
            every = step.n_prefill == 0 and step.n_decode == step.num_seqs
            latent_attention_mfma(q, cache, cache_t, sink, group.block_table, None if every else step.decode_seqs, step.n_decode,
                                  step.cu_q, step.context_lens, out, 1, rank, window, scale, max_context=step.max_decode_context)
        if step.n_prefill:
            latent_attention_mfma(q, cache, cache_t, sink, group.block_table, step.prefill_seqs, step.n_prefill, step.cu_q,
                                  step.context_lens, out, step.max_prefill_q, rank, window, scale)
        return out
    return latent_attention_generic(q, cache, sink, group.block_table, step.seq_of_token, step.positions, rank, window, scale)


def linear_clamped_gate(x: torch.Tensor, w, limit: float, alpha: float) -> torch.Tensor:
    """The clamped gated pair of ``clamped_gate`` over x W^T for a weight [2I, K] whose rows alternate gate_j, up_j."""
    return clamped_gate(linear(x, w), limit, alpha)


# ---------------------------------------------------------------------------
# Statistics over parts of a row
def group_norm_step(residual: torch.Tensor, groups: int, eps: float, y: Optional[torch.Tensor] = None,
                    w_add: Optional[torch.Tensor] = None, w_out: Optional[torch.Tensor] = None,
                    out_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One step around a 32-bit stream ``residual`` [T, H], with the RMS norm in groups (the row in ``groups`` equal
    consecutive parts, each over its own sqrt(mean(part^2) + eps)):

    with ``y`` [T, H] and ``w_add``: residual += norm(y) * w_add, in place;
    with ``w_out``: returns norm(residual) * w_out in ``out_dtype`` (the next branch's input), of the rows ``rows``
    alone when given (which goes without ``y``)."""
    _dev(residual, y, w_add, w_out, rows)
    _f32(residual, "residual")
    _f32(w_add, "norm weight")
    _f32(w_out, "norm weight")
    if residual.dim() != 2 or not residual.is_contiguous():
        raise NativeError(f"group_norm_step: the stream {tuple(residual.shape)} is not a contiguous [T, H]")
    m, h = residual.shape
    if y is not None and (tuple(y.shape) != (m, h) or w_add is None or tuple(w_add.shape) != (h,) or not y.is_contiguous()):
        raise NativeError(f"group_norm_step: branch {tuple(y.shape)} / weight beside a stream {tuple(residual.shape)}")
    if w_out is not None and tuple(w_out.shape) != (h,):
        raise NativeError(f"group_norm_step: weight {tuple(w_out.shape)} for rows of {h}")
    n, out = m, None
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    if w_out is not None:
        dt = out_dtype if out_dtype is not None else (y.dtype if y is not None else torch.float32)
        if y is not None and dt != y.dtype:
            raise NativeError(f"group_norm_step: an output of {dt} beside a branch of {y.dtype}")
        out = torch.empty((n, h), dtype=dt, device=residual.device)
    code = _CODES[out.dtype] if out is not None else _code(y)
    check(kernels().pa_group_norm_step(_stream(), code, _ptr(y), _ptr(w_add), _ptr(residual), _ptr(w_out), _ptr(out), _ptr(rows),
                                       n, h, int(groups), float(eps)))
    return out


def poly_norm(x: torch.Tensor, coeff: torch.Tensor, eps: float, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e over rows, z = x (+ bias), powers element by element, N(u) = u over
    sqrt(mean(u^2) + eps); ``coeff`` float32 (a, b, c, e) on the device."""
    _dev(x, coeff, bias)
    _f32(coeff, "coefficients")
    _f32(bias, "bias")
    if x.dim() != 2 or not x.is_contiguous() or tuple(coeff.shape) != (4,) or (bias is not None and tuple(bias.shape) != (x.shape[1],)):
        raise NativeError(f"poly_norm: x {tuple(x.shape)} / coefficients {tuple(coeff.shape)}")
    out = torch.empty_like(x)
    check(kernels().pa_poly_norm(_stream(), _code(x), _ptr(x), _ptr(bias), _ptr(coeff), _ptr(out), x.shape[0], x.shape[1], float(eps)))
    return out


HEAD_GATES = {"sigmoid": 0, "silu": 1}


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], eps: float, gate_activation: str = "sigmoid",
                   out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """o float32 [T, heads, vdim]: every head over its own sqrt(mean^2 + eps), times ``weight`` (float32 [vdim], shared by
    the heads; None: none), times act(gate) (``gate`` [T, heads * vdim] of the engine's type, rows may lie inside a
    wider tensor), times ``scale``.  Written to ``out`` (rows may lie inside a wider tensor) or a fresh [T, heads * vdim]."""
    _dev(o, weight)
    _f32(o, "head_norm_gate input")
    _f32(weight, "norm weight")
    if o.dim() != 3 or not o.is_contiguous():
        raise NativeError(f"head_norm_gate: o {tuple(o.shape)} is not a contiguous [T, heads, vdim]")
    t, heads, vdim = o.shape
    if gate_activation not in HEAD_GATES:
        raise NativeError(f"head_norm_gate: gate activation {gate_activation!r} is not one of {sorted(HEAD_GATES)}")
    if not gate.is_cuda or gate.dim() != 2 or gate.stride(1) != 1 or tuple(gate.shape) != (t, heads * vdim) or \
            (weight is not None and tuple(weight.shape) != (vdim,)):
        raise NativeError(f"head_norm_gate: gate {tuple(gate.shape)} / weight for o {tuple(o.shape)}")
    if out is None:
        out = torch.empty((t, heads * vdim), dtype=gate.dtype, device=o.device)
    elif out.dtype != gate.dtype or tuple(out.shape) != (t, heads * vdim) or out.stride(1) != 1:
        raise NativeError(f"head_norm_gate: out {tuple(out.shape)} {out.dtype}")
    if t:
        check(kernels().pa_head_norm_gate(_stream(), _code(gate), _ptr(o), gate.data_ptr(), gate.stride(0), _ptr(weight),
                                          out.data_ptr(), out.stride(0), t, heads, vdim, float(eps), HEAD_GATES[gate_activation],
                                          float(scale)))
    return out


# ---------------------------------------------------------------------------
# Attention with a window that keeps first tokens, a bias by distance and a gate a head
def qkv_prepare(p: torch.Tensor, q_off: int, k_off: int, v_off: int, q_weight: Optional[torch.Tensor],
                k_weight: Optional[torch.Tensor], slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                v_cache: Optional[torch.Tensor], nh: int, nkv: int, hd: int, vd: int, eps: float) -> torch.Tensor:
    """From the merged projection ``p`` [T, width] (rows may lie inside a wider tensor): the queries [T, nh, hd], with
    ``q_weight`` (float32 [nh * hd]) brought to unit RMS over the whole projection and multiplied by it; keys (the
    same with ``k_weight``) and values written to the caches at ``slots`` (None: queries only)."""
    _dev(p, q_weight, k_weight, slots, k_cache, v_cache)
    _f32(q_weight, "query norm weight")
    _f32(k_weight, "key norm weight")
    if p.dim() != 2 or p.stride(1) != 1:
        raise NativeError(f"qkv_prepare: projection {tuple(p.shape)} with strides {p.stride()}")
    t = p.shape[0]
    if (q_weight is not None and tuple(q_weight.shape) != (nh * hd,)) or (k_weight is not None and tuple(k_weight.shape) != (nkv * hd,)):
        raise NativeError("qkv_prepare: a norm weight does not have its projection's size")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if slots.shape != (t,) or k_cache is None or v_cache is None or k_cache.dtype != p.dtype or v_cache.dtype != p.dtype or \
                tuple(k_cache.shape[1:]) != (nkv, k_cache.shape[2], hd) or tuple(v_cache.shape) != (k_cache.shape[0], nkv, vd, k_cache.shape[2]):
            raise NativeError(f"qkv_prepare: caches {None if k_cache is None else tuple(k_cache.shape)} / "
                              f"{None if v_cache is None else tuple(v_cache.shape)} for {nkv} heads of {hd} and {vd}")
        page = k_cache.shape[2]
    q = torch.empty((t, nh, hd), dtype=p.dtype, device=p.device)
    if t:
        check(kernels().pa_qkv_prepare(_stream(), _code(p), p.data_ptr(), p.stride(0), int(q_off), int(k_off), int(v_off),
                                       _ptr(q_weight), _ptr(k_weight), _ptr(slots), _ptr(q), _ptr(k_cache) if slots is not None else None,
                                       _ptr(v_cache) if slots is not None else None, t, nh, nkv, hd, vd, page, float(eps)))
    return q


def attention_masked_mfma_supported(hd: int, vd: int, page_size: int) -> bool:
    """Whether ``attention_masked`` runs these widths on the matrix cores (bfloat16)."""
    return bool(kernels().pa_attn_masked_mfma_supports(int(hd), int(vd), int(page_size)))


def attention_masked(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, step, window: int, keep_first: int,
                     scale: float, softcap: float = 0.0, slopes: Optional[torch.Tensor] = None,
                     sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
    """Paged causal attention of one step over one cache group, any mix of portions and single tokens.  The query at
    i sees the key at j <= i when i - j < ``window`` (0: no window) or j < ``keep_first``.  score = q.k * scale, bent
    to cap * tanh(score / cap) for ``softcap`` > 0, less ``slopes``[h] * (i - j); ``sink`` [heads] joins the softmax's
    denominator; ``gate`` [T, heads] (rows may lie inside a wider tensor): a head's output times sigmoid(gate), and
    ``out_scale``, before rounding.  q [T, nh, hd]; K cache [pages, nkv, page, hd]; V cache [pages, nkv, vd, page].
    Returns (or fills ``out``, whose rows may lie inside a wider tensor) [T, nh * vd].

    bfloat16 with keys and values of one width the matrix cores take (32, 64, 96, 128) and pages of a power of two runs
    on the matrix cores: portions as tiles of 64 tokens, a single token's keys dealt out to a workgroup's wavefronts.
    Everything else (32-bit, other sizes) runs on the vector units, a wavefront a (token, head)."""
    _dev(q, k_cache, v_cache, slopes, sink)
    if q.dim() != 3 or not q.is_contiguous() or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise NativeError(f"attention_masked: q {tuple(q.shape)} / caches")
    t, nh, hd = q.shape
    pages, nkv, page, khd = k_cache.shape
    nv, vd = v_cache.shape[1], v_cache.shape[2]   # fewer value heads than key heads: key head k goes with value head k mod nv
    if khd != hd or tuple(v_cache.shape) != (pages, nv, vd, page) or nkv % nv or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise NativeError(f"attention_masked: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for q {tuple(q.shape)} {q.dtype}")
    for name, v in (("slopes", slopes), ("sink", sink)):
        if v is not None:
            _f32(v, name)
            if tuple(v.shape) != (nh,):
                raise NativeError(f"attention_masked: {name} {tuple(v.shape)} for {nh} heads")
    if gate is not None and (not gate.is_cuda or gate.dtype != q.dtype or gate.dim() != 2 or tuple(gate.shape) != (t, nh) or gate.stride(1) != 1):
        raise NativeError(f"attention_masked: gate {tuple(gate.shape)} {gate.dtype} for {t} tokens of {nh} heads")
    if out is None:
        out = torch.empty((t, nh * vd), dtype=q.dtype, device=q.device)
    elif out.dtype != q.dtype or tuple(out.shape) != (t, nh * vd) or out.stride(1) != 1:
        raise NativeError(f"attention_masked: out {tuple(out.shape)} {out.dtype}")
    if t:
        check(kernels().pa_attn_masked(_stream(), _code(q), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(group.block_table),
                                       group.block_table.shape[1], _ptr(step.seq_of_token), _ptr(step.positions), out.data_ptr(),
                                       out.stride(0), t, nh, nkv, hd, vd, page, int(window), int(keep_first), float(scale),
                                       float(softcap), _ptr(slopes), _ptr(sink), gate.data_ptr() if gate is not None else None,
                                       gate.stride(0) if gate is not None else 0, float(out_scale), _ptr(getattr(step, "cu_q", None)),
                                       _ptr(getattr(step, "context_lens", None)), int(getattr(step, "num_seqs", 0)),
                                       int(getattr(step, "max_q_len", 0) or getattr(step, "max_prefill_q", 0) or 1), nv))
    return out


# ---------------------------------------------------------------------------
# The gated delta rule; rotation in front of a recurrence
def delta_prepare(p: torch.Tensor, off: int, b_off: int, conv_weight: torch.Tensor, conv_state: torch.Tensor, a: torch.Tensor,
                  a_off: int, a_log: torch.Tensor, dt_bias: torch.Tensor, step, heads: int, kvh: int, d: int, e: int):
    """What stands in front of the gated delta rule.  ``p`` [T, width] holds from column ``off`` the channels
    [q | k | v] (q, k: ``kvh`` heads of ``d``; v: ``heads`` heads of ``e``) and at ``b_off`` one gate input a head.
    Every channel passes a causal convolution (``conv_weight`` float32 [channels, taps], the last tap the token's
    own; the inputs before the step come from ``conv_state`` float32 [slots, channels, taps - 1], which then moves
    on) and SiLU; q and k become unit vectors per head, q also times d^(-1/2).  Returns 32-bit
    (x [T, channels], decay [T, heads, d] = exp(-exp(a_log_h) softplus(a + dt_bias)) from ``a`` [T, .] at column
    ``a_off``, beta [T, heads] = sigmoid of the gate input)."""
    _dev(p, conv_weight, conv_state, a, a_log, dt_bias)
    for name, v in (("convolution weight", conv_weight), ("convolution state", conv_state), ("A_log", a_log), ("dt_bias", dt_bias)):
        _f32(v, name)
    t = p.shape[0]
    c = 2 * kvh * d + heads * e
    taps = conv_weight.shape[1] if conv_weight.dim() == 2 else 0
    if p.dim() != 2 or p.stride(1) != 1 or a.dim() != 2 or a.stride(1) != 1 or a.dtype != p.dtype or a.shape[0] != t or \
            tuple(conv_weight.shape) != (c, taps) or conv_state.dim() != 3 or tuple(conv_state.shape[1:]) != (c, max(taps - 1, 0)) or \
            tuple(a_log.shape) != (heads,) or tuple(dt_bias.shape) != (heads * d,) or not conv_state.is_contiguous():
        raise NativeError(f"delta_prepare: p {tuple(p.shape)} / conv {tuple(conv_weight.shape)} / state {tuple(conv_state.shape)} / "
                          f"a {tuple(a.shape)} for {heads} heads ({kvh} of keys) of {d} and {e}")
    x = torch.empty((t, c), dtype=torch.float32, device=p.device)
    decay = torch.empty((t, heads, d), dtype=torch.float32, device=p.device)
    beta = torch.empty((t, heads), dtype=torch.float32, device=p.device)
    if t:
        check(kernels().pa_delta_prepare(_stream(), _code(p), p.data_ptr(), p.stride(0), int(off), int(b_off), _ptr(conv_weight), taps,
                                         _ptr(conv_state), _ptr(step.seq_of_token), _ptr(step.cu_q), _ptr(step.state_slots),
                                         a.data_ptr(), a.stride(0), int(a_off), _ptr(a_log), _ptr(dt_bias), _ptr(x), _ptr(decay),
                                         _ptr(beta), t, step.num_seqs, heads, kvh, d, e))
    return x, decay, beta


def gated_delta(x: torch.Tensor, decay: torch.Tensor, beta: torch.Tensor, state: torch.Tensor, step, heads: int, kvh: int,
                d: int, e: int) -> torch.Tensor:
    """The gated delta rule over the step's sequences, token by token: per head S <- diag(g) S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q.  ``x``, ``decay``, ``beta`` as ``delta_prepare`` returns them; ``state`` float32
    [slots, heads, d, e], read and left through ``step.state_slots``.  Returns float32 [T, heads, e]."""
    _dev(x, decay, beta, state)
    for name, v in (("x", x), ("decay", decay), ("beta", beta), ("state", state)):
        _f32(v, name)
    t = x.shape[0]
    if tuple(x.shape) != (t, 2 * kvh * d + heads * e) or tuple(decay.shape) != (t, heads, d) or tuple(beta.shape) != (t, heads) or \
            state.dim() != 4 or tuple(state.shape[1:]) != (heads, d, e) or not state.is_contiguous():
        raise NativeError(f"gated_delta: x {tuple(x.shape)} / decay {tuple(decay.shape)} / beta {tuple(beta.shape)} / state {tuple(state.shape)}")
    out = torch.empty((t, heads, e), dtype=torch.float32, device=x.device)
    if t:
        check(kernels().pa_gated_delta(_stream(), _ptr(x), _ptr(decay), _ptr(beta), _ptr(state), _ptr(step.state_slots), _ptr(step.cu_q),
                                       _ptr(out), step.num_seqs, heads, kvh, d, e))
    return out


def rotate_halves_f32(p: torch.Tensor, q_off: int, k_off: int, v_off: int, inv_freq: Optional[torch.Tensor],
                      positions: torch.Tensor, heads: int, d: int, e: int, rot: int, k_scale: float = 1.0) -> torch.Tensor:
    """From ``p`` [T, width]: queries and keys (``heads`` heads of ``d`` from ``q_off`` and ``k_off``) with the first
    ``rot`` dimensions of every head turned, dimension i with i + rot / 2, by position * inv_freq[i], the keys then times
    ``k_scale``; values (``heads`` heads of ``e`` from ``v_off``) as they are.  All in 32-bit:
    returns float32 [T, 2 * heads * d + heads * e] = [q | k | v]."""
    _dev(p, inv_freq, positions)
    _f32(inv_freq, "rotary frequencies")
    _i32(positions, "positions")
    t = p.shape[0]
    if p.dim() != 2 or p.stride(1) != 1 or positions.shape != (t,) or (rot and (inv_freq is None or tuple(inv_freq.shape) != (rot // 2,))):
        raise NativeError(f"rotate_halves: p {tuple(p.shape)} / positions / frequencies for {rot} turned dimensions")
    out = torch.empty((t, 2 * heads * d + heads * e), dtype=torch.float32, device=p.device)
    if t:
        check(kernels().pa_rotate_halves_f32(_stream(), _code(p), p.data_ptr(), p.stride(0), int(q_off), int(k_off), int(v_off),
                                             _ptr(inv_freq), _ptr(positions), _ptr(out), t, heads, d, e, int(rot), float(k_scale)))
    return out


# ---------------------------------------------------------------------------
# Parts around a 32-bit stream, in front of and behind attention
def pair_embed(ids: torch.Tensor, step, prev_state: torch.Tensor, table: torch.Tensor, pair: torch.Tensor, buckets: int,
               mul_prev: int, mul_cur: int, scale: float) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale + pair[(prev * mul_prev + ids[t] * mul_cur) mod buckets] in 32-bit, [T, H]; a
    sequence's first token (position 0) reads row ``buckets`` of ``pair``.  The token before a portion's first comes
    from ``prev_state`` (int32 [slots, 1], the step's ``state_slots``), which then takes the portion's last token."""
    _dev(ids, table, pair, prev_state, step.positions, step.seq_of_token, step.cu_q, step.state_slots)
    _i32(ids, "ids")
    _i32(prev_state, "previous tokens")
    t, h = ids.shape[0], table.shape[1]
    if ids.dim() != 1 or table.dim() != 2 or tuple(pair.shape) != (buckets + 1, h) or pair.dtype != table.dtype:
        raise NativeError(f"pair_embed: ids {tuple(ids.shape)} / table {tuple(table.shape)} / pair {tuple(pair.shape)} for {buckets} buckets")
    out = torch.empty((t, h), dtype=torch.float32, device=table.device)
    check(kernels().pa_pair_embed(_stream(), _code(table), _ptr(ids), _ptr(step.positions), _ptr(step.seq_of_token), _ptr(step.cu_q),
                                  _ptr(step.state_slots), _ptr(prev_state), _ptr(table), _ptr(pair), _ptr(out), t, h, table.shape[0],
                                  int(buckets), int(mul_prev), int(mul_cur), float(scale)))
    return out


def time_conv_add(h: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], step) -> torch.Tensor:
    """h + conv(h) with conv(h)_t = sum_j w[j] h_(t - taps + 1 + j) over time within each sequence, zeros before its
    start.  h [T, C]; ``weight`` float32 [taps, C] (a tap's weights side by side: the stored [C, taps] transposed);
    ``state`` float32 [slots, taps - 1, C]: a request's last taps - 1 inputs, read for the places before the portion and
    moved on afterwards."""
    _dev(h, weight, state, step.seq_of_token, step.cu_q, step.state_slots)
    _f32(weight, "convolution weight")
    _f32(state, "carried inputs")
    t, c = h.shape
    taps = weight.shape[0]
    if weight.dim() != 2 or weight.shape[1] != c or not h.is_contiguous() or \
            (taps > 1 and (state is None or tuple(state.shape[1:]) != (taps - 1, c))):
        raise NativeError(f"time_conv_add: h {tuple(h.shape)} / weight {tuple(weight.shape)} / state "
                          f"{None if state is None else tuple(state.shape)}")
    out = torch.empty_like(h)
    # a step of single tokens alone: every thread moves its sequence's carried inputs on itself, no second launch
    check(kernels().pa_time_conv_add(_stream(), _code(h), _ptr(h), _ptr(weight), _ptr(state), _ptr(step.seq_of_token), _ptr(step.cu_q),
                                     _ptr(step.state_slots), _ptr(out), t, int(step.num_seqs), c, taps,
                                     1 if int(getattr(step, "max_q_len", 0)) == 1 else 0))
    return out


def stream_add_row_(x: torch.Tensor, row: torch.Tensor) -> torch.Tensor:
    """x[t] += row for every row of a 32-bit stream x [T, H], in place."""
    _dev(x, row)
    _f32(x, "stream")
    _f32(row, "row")
    if x.dim() != 2 or tuple(row.shape) != (x.shape[1],) or not x.is_contiguous() or not row.is_contiguous():
        raise NativeError(f"stream_add_row: x {tuple(x.shape)} / row {tuple(row.shape)}")
    check(kernels().pa_stream_add_row(_stream(), _ptr(x), _ptr(row), x.shape[0], x.shape[1]))
    return x


def stream_add_branches_(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += a + b (the branches' sum first, in 32-bit) for a 32-bit stream x [T, H], in place."""
    _dev(x, a, b)
    _f32(x, "stream")
    if a.shape != x.shape or not a.is_contiguous() or not x.is_contiguous() or \
            (b is not None and (b.shape != x.shape or b.dtype != a.dtype or not b.is_contiguous())):
        raise NativeError(f"stream_add_branches: x {tuple(x.shape)} / a {tuple(a.shape)} / b {None if b is None else tuple(b.shape)}")
    check(kernels().pa_stream_add_branches(_stream(), _code(a), _ptr(x), _ptr(a), _ptr(b), x.numel()))
    return x


def qkv_rope_prepare(p: torch.Tensor, q_off: int, k_off: int, v_off: int, inv_freq: Optional[torch.Tensor], positions: torch.Tensor,
                     slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], nq: int,
                     nk: int, nv: int, hd: int, vd: int, rot: int, pairs: bool, q_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From the merged projection ``p`` [T, width]: the queries [T, nq, hd]; ``nk`` key heads of ``hd`` into K
    [pages, nk, page, hd] and ``nv`` value heads of ``vd`` into V [pages, nv, vd, page] at ``slots`` (None: queries
    only).  The first ``rot`` dimensions of every query and key head are turned by position * inv_freq[i], dimension i
    with i + rot / 2, or with ``pairs`` 2i with 2i + 1; ``q_scale`` [nq]: a number per query head."""
    _dev(p, inv_freq, positions, slots, k_cache, v_cache, q_scale)
    _f32(inv_freq, "rotary frequencies")
    _f32(q_scale, "query scales")
    _i32(positions, "positions")
    if p.dim() != 2 or p.stride(1) != 1:
        raise NativeError(f"qkv_rope_prepare: projection {tuple(p.shape)} with strides {p.stride()}")
    t = p.shape[0]
    if rot and (inv_freq is None or tuple(inv_freq.shape) != (rot // 2,)):
        raise NativeError(f"qkv_rope_prepare: frequencies must be [{rot // 2}]")
    if q_scale is not None and tuple(q_scale.shape) != (nq,):
        raise NativeError(f"qkv_rope_prepare: query scales {tuple(q_scale.shape)} for {nq} heads")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if slots.shape != (t,) or k_cache is None or v_cache is None or k_cache.dtype != p.dtype or v_cache.dtype != p.dtype or \
                tuple(k_cache.shape[1:]) != (nk, k_cache.shape[2], hd) or tuple(v_cache.shape) != (k_cache.shape[0], nv, vd, k_cache.shape[2]):
            raise NativeError(f"qkv_rope_prepare: caches {None if k_cache is None else tuple(k_cache.shape)} / "
                              f"{None if v_cache is None else tuple(v_cache.shape)} for {nk} key heads of {hd} and {nv} value heads of {vd}")
        page = k_cache.shape[2]
    q = torch.empty((t, nq, hd), dtype=p.dtype, device=p.device) if nq else None   # no query heads: keys and values alone
    if t:
        caching = slots is not None
        check(kernels().pa_qkv_rope_prepare(_stream(), _code(p), p.data_ptr(), p.stride(0), int(q_off), int(k_off), int(v_off),
                                            _ptr(inv_freq), _ptr(positions), _ptr(slots), _ptr(q_scale), _ptr(q),
                                            _ptr(k_cache) if caching else None, _ptr(v_cache) if caching else None, t, nq, nk, nv,
                                            hd, vd, int(rot), 1 if pairs else 0, page))
    return q


def diff_combine(a: torch.Tensor, heads: int, lam: float, eps: float, scale: float) -> torch.Tensor:
    """a [T, 2 * heads * vd] (the first maps' outputs of all heads, then the second maps') -> [T, heads * vd]:
    u = a1 - lam * a2 per head, over its own sqrt(mean(u^2) + eps), times ``scale``."""
    _dev(a)
    if a.dim() != 2 or a.shape[1] % (2 * heads) or not a.is_contiguous():
        raise NativeError(f"diff_combine: a {tuple(a.shape)} for {heads} heads")
    vd = a.shape[1] // (2 * heads)
    out = torch.empty((a.shape[0], heads * vd), dtype=a.dtype, device=a.device)
    check(kernels().pa_diff_combine(_stream(), _code(a), _ptr(a), _ptr(out), a.shape[0], heads, vd, float(lam), float(eps), float(scale)))
    return out


def sigmoid_gate(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """o * sigmoid(gate), element by element; both [T, N], rows may lie inside wider tensors."""
    if not (o.is_cuda and gate.is_cuda):
        raise NativeError("sigmoid_gate: an operand is not on the device")
    if o.dim() != 2 or o.shape != gate.shape or o.dtype != gate.dtype or o.stride(1) != 1 or gate.stride(1) != 1:
        raise NativeError(f"sigmoid_gate: o {tuple(o.shape)} {o.dtype} / gate {tuple(gate.shape)} {gate.dtype}")
    out = torch.empty(o.shape, dtype=o.dtype, device=o.device)
    check(kernels().pa_sigmoid_gate(_stream(), _code(o), o.data_ptr(), o.stride(0), gate.data_ptr(), gate.stride(0), _ptr(out),
                                    o.shape[0], o.shape[1]))
    return out


def cap_logits_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) for 32-bit logits, in place."""
    _dev(x)
    _f32(x, "logits")
    if not x.is_contiguous():
        raise NativeError("cap_logits: the logits are not contiguous")
    check(kernels().pa_cap_logits(_stream(), _ptr(x), x.numel(), float(cap)))
    return x
